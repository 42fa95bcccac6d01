// sumcheck_kernels.hpp -- the sumcheck prover's round kernel for gfx950, generated per statement.
//
// One launch does, for every pair i of the tables being summed,
//   [FOLD]  bind the previous round's variable: read four entries per table, write the two folded
//           entries lo + r (hi - lo) (src/sumcheck.lisp:84-104), and use them as the pair;
//   sums    for every group g of the statement (a product of tables) and each of its evaluation
//           points X:  acc[g, X] += LOW[l] * prod_{t in g} line_t(X),  line_t(X) = lo + X (hi - lo),
//           i = h |LOW| + l  (src/sumcheck.lisp:230-257), unreduced in 96-bit accumulators;
//   then reduces the accumulators over the workgroup (cross-lane, then LDS), multiplies by HIGH[h]
//   and writes one partial per workgroup.  A second small kernel adds the partials.
//
// The statement is a compile-time descriptor (StmtDesc) when the kernel was generated for it, or a
// run-time one interpreted by the same code (the fallback for statements without a generated kernel).
// Tables, weights and outputs are canonical residues; the sums come out scaled by a power of 1/R
// (R = 2^32) that the host removes: a group of degree d carries R^-d.
#pragma once
// (a run-time compilation of these kernels has the runtime's declarations built in and no host headers)
#if !defined(__HIPCC_RTC__)
#include <hip/hip_runtime.h>

#include <stddef.h>
#include <type_traits>
#endif

#include "dev_transcript.hpp"
#include "field.hpp"
#include "stmtdesc.hpp"

namespace exh {

// StmtDesc and the limits MAXT, MAXG, ... come from stmtdesc.hpp
constexpr int MAXROUNDS = 48;  // rounds of one device-driven sumcheck (a count of them fits six bits)
constexpr int MAXPTS = 7;      // wire points of a device-driven round message
constexpr int MAXTAIL = 16;    // rounds the tail kernel can take

// The control block of a device-driven sumcheck, in device memory: the transcript state, the current
// fold challenge, the launch's completion counter and the logs the host reads back at the end.
struct Ctrl {
  DevB3S tr;
  uint32_t r_mont[8];
  uint32_t round;    // rounds completed
  uint32_t gave_up;  // set by a workgroup of a grid launch whose wait for the others ran out: the proof is void
  uint32_t pad[2];
  uint32_t msg[MAXROUNDS][MAXPTS * 8];
  uint32_t chal[MAXROUNDS][8];
  uint32_t finals[MAXT * 8];  // entry 0 of every table once a single entry is left
};
template <int D>
struct RoundArgs {
  const uint32_t *in[MAXT];  // the tables read: 4 entries per pair when folding, else 2
  uint32_t *out[MAXT];       // folded tables written (FOLD)
  const uint32_t *low;       // |LOW| = 2^low_bits EXTs
  const uint32_t *high;      // n_high EXTs
  uint32_t *partials;        // [gridDim.x][nacc][D]
  uint64_t n_pairs;          // pairs summed (after the fold)
  uint32_t low_bits;
  uint32_t pairs_per_thread;
  uint32_t deferred;         // every workgroup's pairs share one h: HIGH[h] applied once per workgroup
  uint32_t do_sums;
  uint32_t r_mont[D];        // the fold challenge, times R (host-driven rounds)
  Ctrl *ctrl;                // device-driven rounds: the fold challenge is read from here (else null)
  uint32_t pstride;          // words per workgroup partial (a power of two >= nacc * D)
  uint32_t double_fold;      // base tables, folded by challenges 0 and 1 at once (8 entries -> 2 per pair)
  // device-driven rounds: the round's sums meet in counted totals and the last workgroup to arrive sends the
  // message and draws the challenge itself (see RoundTotals); totals null: one partial row per workgroup
  unsigned long long *totals;  // [groups][pstride], zero before the launch
  uint32_t *arrivals;          // workgroups that have added their sums, zero before the launch
  uint32_t groups, points, spin_limit;
  const uint32_t *mtilde, *c0;  // the round's message map and constant terms
  const uint32_t *consts;       // a statement in direct form: its constant slots (EXTs, Montgomery form)
};

// How the workgroups of a streaming launch finish a round without another launch.  Every workgroup adds its sums
// into the totals of its group (workgroup w: group w % groups) with integer atomics that also count the
// contribution in the word's top 16 bits, then takes a ticket; the workgroup with the last ticket polls the words
// until each carries its group's full count -- the data travels inside the atomics, so no fence is needed and
// nobody reads memory another workgroup wrote with plain stores -- and goes on to the message, the transcript step
// and the next challenge, which the next launch reads from the control block.
struct RoundTotals {
  unsigned long long *totals;
  uint32_t *arrivals;
  uint32_t groups, pstride, spin_limit;
};
constexpr int TOTALS_POLLS = 8;  // words a thread of the elected workgroup polls: groups * width <= 8 * BLOCK

// The rounds below 2^18 pairs, with the tables resident in LDS: no global memory round trip separates a
// round's sums, its transcript step and its fold.  With one workgroup (the last rounds) everything
// stays on one compute unit; with a grid (the rounds before them) every workgroup keeps a contiguous
// slice of every table, the round's sums meet in global totals (integer atomics that count their
// contributions), and every workgroup runs the same transcript step, so each knows the next challenge.
// The grid must be resident at once: the host launches at most one workgroup per compute unit.
constexpr uint32_t TAIL_LDS_BYTES = 32768;        // LDS given to the tables of the one-workgroup launch
constexpr uint32_t SLICE_LDS_BYTES = 128 * 1024;  // and to a workgroup's slices in the grid launch
template <int D>
struct TailArgs {
  const uint32_t *in[MAXT];  // tables of `entries` entries each; base (stride 1) when in_base
  uint32_t *out;             // where the folded tables go: table t at t * final_entries * D
  const uint32_t *weights;   // base of the weight tables
  uint64_t low_off[MAXTAIL], high_off[MAXTAIL];  // in EXTs, per round
  uint32_t low_bits[MAXTAIL];
  uint32_t entries;          // per table, over all workgroups
  uint32_t in_base;
  uint32_t first_fold;       // fold by ctrl's challenge while loading
  uint32_t rounds;           // rounds summed here; a fold follows each
  uint32_t first_round;      // index of the first of them
  uint32_t capacity;         // entries per table in a workgroup's LDS
  uint32_t lds_bytes;        // T * capacity * D * 4
  uint32_t points;
  Ctrl *ctrl;
  const uint32_t *mtilde;
  const uint32_t *c0;        // [rounds][points][D]
  unsigned long long *totals;  // grid launch: [rounds][groups][pstride] counted sums, zeroed by the host
  uint32_t pstride;
  uint32_t groups;           // workgroup w adds into group w % groups
  uint32_t spin_limit;       // polls of a total before giving up
  // the last launch of a device-driven loop (one workgroup): it ends by copying the control block into pinned
  // host memory and raising host_log[host_flag_at] to host_seq, so that the host needs neither a copy nor a wait
  // on the stream to read the logs (null: it does both)
  uint32_t *host_log;
  uint32_t host_flag_at, host_seq;
  const uint32_t *consts;  // a statement in direct form: its constant slots (EXTs, Montgomery form)
  // A session whose every round runs in this one launch builds its weight tables itself, in LDS behind the tables
  // (no set-up launch): `factors` holds (r_v R, (1 - r_v) R) for the eq point's n_vars variables; round jj's LOW
  // table covers the low_bits[jj] variables from first_round + jj + 1 on, its HIGH table the rest.  Null: the
  // tables are read from `weights`.
  const uint32_t *factors;
  uint32_t n_vars;
};

template <int D>
__device__ __forceinline__ Ext<D> load_ext(const uint32_t *p) {
  Ext<D> e;
  if constexpr (D == 4) {
    uint4 v = *reinterpret_cast<const uint4 *>(p);
    e.c[0] = v.x, e.c[1] = v.y, e.c[2] = v.z, e.c[3] = v.w;
  } else {
    uint4 v = *reinterpret_cast<const uint4 *>(p), u = *reinterpret_cast<const uint4 *>(p + 4);
    e.c[0] = v.x, e.c[1] = v.y, e.c[2] = v.z, e.c[3] = v.w;
    e.c[4] = u.x, e.c[5] = u.y, e.c[6] = u.z, e.c[7] = u.w;
  }
  return e;
}
template <int D>
__device__ __forceinline__ void store_ext(uint32_t *p, const Ext<D> &e) {
  *reinterpret_cast<uint4 *>(p) = make_uint4(e.c[0], e.c[1], e.c[2], e.c[3]);
  if constexpr (D == 8) *reinterpret_cast<uint4 *>(p + 4) = make_uint4(e.c[4], e.c[5], e.c[6], e.c[7]);
}

// lo + r (hi - lo) for base values: r_mont * (hi - lo) is exact, lo joins coordinate 0
template <int D>
__device__ __forceinline__ Ext<D> fold_base(uint32_t lo, uint32_t hi, const Ext<D> &r_mont) {
  Ext<D> o = ext_scale_mont<D>(r_mont, fsub(hi, lo));
  o.c[0] = fadd(o.c[0], lo);
  return o;
}
template <int D>
__device__ __forceinline__ Ext<D> fold_ext(const Ext<D> &lo, const Ext<D> &hi, const Ext<D> &r_mont) {
  // r is the second operand: its tripled wrap coefficients are the same for every entry of the launch
  return ext_add<D>(lo, ext_mul_mont<D>(ext_sub<D>(hi, lo), r_mont));
}

// ---- the per-pair work: all groups at all their points.  V is uint32_t (base mode) or Ext<D>.
template <int D>
__device__ __forceinline__ uint32_t v_add(uint32_t a, uint32_t b) { return fadd(a, b); }
template <int D>
__device__ __forceinline__ Ext<D> v_add(const Ext<D> &a, const Ext<D> &b) { return ext_add<D>(a, b); }
template <int D>
__device__ __forceinline__ uint32_t v_sub(uint32_t a, uint32_t b) { return fsub(a, b); }
template <int D>
__device__ __forceinline__ Ext<D> v_sub(const Ext<D> &a, const Ext<D> &b) { return ext_sub<D>(a, b); }
template <int D>
__device__ __forceinline__ uint32_t v_mul(uint32_t a, uint32_t b) { return mont_mul(a, b); }
template <int D>
__device__ __forceinline__ Ext<D> v_mul(const Ext<D> &a, const Ext<D> &b) { return ext_mul_mont<D>(a, b); }
template <int D>
__device__ __forceinline__ void v_weigh(Acc96 *acc, const Ext<D> &w, uint32_t v) { ext_scale_acc<D>(acc, w, v); }
template <int D>
__device__ __forceinline__ void v_weigh(Acc96 *acc, const Ext<D> &w, const Ext<D> &v) {
  ext_mul_acc<D>(acc, v, w);  // the weight second: its tripled wrap coefficients are shared by the pair's points
}

// integer multiples and integer offsets, for the linear forms
template <int D>
__device__ __forceinline__ uint32_t v_scale(uint32_t a, uint32_t c, uint32_t c_mont) {
  return c == 1 ? a : c == P - 1 ? fneg(a) : mont_mul(a, c_mont);
}
template <int D>
__device__ __forceinline__ Ext<D> v_scale(const Ext<D> &a, uint32_t c, uint32_t c_mont) {
  Ext<D> o;
#pragma unroll
  for (int k = 0; k < D; k++) o.c[k] = v_scale<D>(a.c[k], c, c_mont);
  return o;
}
template <int D>
__device__ __forceinline__ uint32_t v_offset(uint32_t a, uint32_t k) { return fadd(a, k); }
template <int D>
__device__ __forceinline__ Ext<D> v_offset(Ext<D> a, uint32_t k) {
  a.c[0] = fadd(a.c[0], k);
  return a;
}

// helpers of the weighted first factor (never reached with base values)
template <int D, class V>
__device__ __forceinline__ V v_of(const Ext<D> &w) {
  if constexpr (std::is_same<V, uint32_t>::value)
    return w.c[0];
  else
    return w;
}
template <int D>
__device__ __forceinline__ void v_mul_acc(Acc96 *acc, uint32_t a, uint32_t b) { acc_mad(acc[0], a, b); }
template <int D>
__device__ __forceinline__ void v_mul_acc(Acc96 *acc, const Ext<D> &a, const Ext<D> &b) { ext_mul_acc<D>(acc, a, b); }

// A statement too wide for accumulators per table group comes in direct form: its descriptor's type carries an
// evaluator of the written form (generated code) and a flag, and the accumulators are the wire points.
template <class T>
struct is_direct {
  template <class U>
  static char test(decltype(U::direct) *);
  template <class U>
  static long test(...);
  static constexpr bool value = sizeof(test<T>(nullptr)) == sizeof(char);
};

// The pair's contribution for a statement in direct form: the tables' lines in Montgomery form (so that sums and
// products of any shape stay in one scale), the form evaluated at each wire point X = 0, 2, 3, ..., and w times
// that value added to the point's accumulator.  The loop over the points is kept a loop: the evaluator is long,
// and one copy of it per kernel keeps compile times and code size in hand; the accumulators stay in registers
// because each is named by a constant inside the switch.
template <int D, class V, class Desc, int PARTS, int PART>
__device__ __forceinline__ void accumulate_direct(const Desc &d, const V *lo, const V *hi, const Ext<D> &w,
                                                  Acc96 (*acc)[D], const uint32_t *kc) {
  Ext<D> at0[MAXT], slope[MAXT];
#pragma unroll
  for (int t = 0; t < MAXT; t++)
    if (t < d.T) {
      if constexpr (std::is_same<V, uint32_t>::value) {
        at0[t] = ext_lift<D>(mont_mul(lo[t], R2));
        slope[t] = ext_lift<D>(mont_mul(fsub(hi[t], lo[t]), R2));
      } else {
        at0[t] = ext_scale_mont<D>(lo[t], R2);
        slope[t] = ext_scale_mont<D>(ext_sub<D>(hi[t], lo[t]), R2);
      }
    }
#pragma unroll 1
  for (int k = PART; k < d.nacc; k += PARTS) {
    const uint32_t x_mont = mont_mul(k == 0 ? 0u : (uint32_t)k + 1u, R2);
    Ext<D> t[MAXT];
#pragma unroll
    for (int i = 0; i < MAXT; i++)
      if (i < d.T) t[i] = ext_add<D>(at0[i], ext_scale_mont<D>(slope[i], x_mont));
    const Ext<D> f = Desc::template eval<D>(t, kc);
    switch (k) {
      case 0: ext_mul_acc<D>(acc[0], f, w); break;
      case 1: ext_mul_acc<D>(acc[1], f, w); break;
      case 2: ext_mul_acc<D>(acc[2], f, w); break;
      case 3: ext_mul_acc<D>(acc[3], f, w); break;
      case 4: ext_mul_acc<D>(acc[4], f, w); break;
      default: ext_mul_acc<D>(acc[5], f, w); break;
    }
  }
}

// With PARTS > 1 only the accumulators a with a % PARTS == PART are computed (a compile-time constant: with the
// part as a run-time value, uniform as it is, the compiler folds the parts' branches into one path that indexes
// the accumulators by it, and they move from registers to scratch memory): the last rounds, with a pair per lane
// and lanes to spare, give each of a workgroup's wavefronts a share of a pair's accumulators, so that a round
// waits for a quarter of the products.
template <int D, class V, class Desc, int PARTS = 1, int PART = 0>
__device__ __forceinline__ void accumulate_pair(const Desc &d, const V *lo, const V *hi, const Ext<D> &w,
                                                Acc96 (*acc)[D], const uint32_t *kc = nullptr) {
  if constexpr (is_direct<Desc>::value) {
    accumulate_direct<D, V, Desc, PARTS, PART>(d, lo, hi, w, acc, kc);
    return;
  }
  V cur[MAXT], slope[MAXT];
#pragma unroll
  for (int t = 0; t < MAXT; t++)
    if (t < d.T) {
      cur[t] = lo[t];
      slope[t] = v_sub<D>(hi[t], lo[t]);
    }
  // the linear forms are lines too: value at 0 from the tables' values at 0 plus the offset, slope
  // from the tables' slopes
#pragma unroll
  for (int v = 0; v < MAXV; v++)
    if (v < d.NV) {
      V c0 = v_scale<D>(cur[d.vtab[v][0]], d.vcoef[v][0], d.vcoefm[v][0]);
      V s0 = v_scale<D>(slope[d.vtab[v][0]], d.vcoef[v][0], d.vcoefm[v][0]);
#pragma unroll
      for (int k = 1; k < MAXVT; k++)
        if (k < d.vn[v]) {
          c0 = v_add<D>(c0, v_scale<D>(cur[d.vtab[v][k]], d.vcoef[v][k], d.vcoefm[v][k]));
          s0 = v_add<D>(s0, v_scale<D>(slope[d.vtab[v][k]], d.vcoef[v][k], d.vcoefm[v][k]));
        }
      cur[d.T + v] = v_offset<D>(c0, d.vconst[v]);
      slope[d.T + v] = s0;
    }
  // A group evaluated at three points or more carries the weight on its first factor: w * factor is a
  // line too (two products per pair), and each point then needs one product fewer.  Extension values
  // only: in the base field the products are cheap and the weight is the one extension operation.
  constexpr bool EXT = !std::is_same<V, uint32_t>::value;
  V wcur[MAXG], wslope[MAXG];
#pragma unroll
  for (int g = 0; g < MAXG; g++)
    if (g < d.G && EXT && d.nev[g] >= 3 && d.deg[g] >= 2) {
      wcur[g] = v_mul<D>(cur[d.tab[g][0]], v_of<D, V>(w));
      wslope[g] = v_mul<D>(slope[d.tab[g][0]], v_of<D, V>(w));
    }
#pragma unroll
  for (int x = 0; x <= MAXX; x++) {
    if (x <= d.maxx) {
      if (x >= 1) {
#pragma unroll
        for (int t = 0; t < MAXT; t++) {
          if (x == 1 && t < d.T)
            cur[t] = hi[t];
          else if (t < d.T + d.NV)
            cur[t] = v_add<D>(cur[t], slope[t]);
        }
#pragma unroll
        for (int g = 0; g < MAXG; g++)
          if (g < d.G && EXT && d.nev[g] >= 3 && d.deg[g] >= 2) wcur[g] = v_add<D>(wcur[g], wslope[g]);
      }
      int a = 0;
#pragma unroll
      for (int g = 0; g < MAXG; g++) {
        if (g < d.G) {
#pragma unroll
          for (int k = 0; k < MAXEV; k++) {
            if (k < d.nev[g]) {
              if (d.ev[g][k] == x && (PARTS == 1 || a % PARTS == PART)) {
                // the product of the factors but the last; the last goes with the accumulation
                const bool pre = EXT && d.nev[g] >= 3 && d.deg[g] >= 2;
                V prod = pre ? wcur[g] : cur[d.tab[g][0]];
#pragma unroll
                for (int j = 1; j < MAXDEG; j++)
                  if (j < d.deg[g] - (pre ? 1 : 0)) prod = v_mul<D>(prod, cur[d.tab[g][j]]);
                if constexpr (EXT)
                  v_mul_acc<D>(acc[a], prod, pre ? cur[d.tab[g][d.deg[g] - 1]] : v_of<D, V>(w));
                else
                  v_weigh<D>(acc[a], w, prod);
              }
              a++;
            }
          }
        }
      }
    }
  }
}

// A workgroup barrier that orders LDS traffic only: what the threads of a workgroup hand each other in these
// kernels lives in LDS, and a full barrier would also wait for every global access in flight (the weights fetched
// a round ahead, the rows on their way to the host).
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// cross-lane sum of a canonical value over the 64 lanes of a wavefront: four DPP butterfly steps inside
// each row of 16 lanes (no LDS traffic), then the four row sums through read-lane
#define EXH_DPP(v, ctrl) ((uint32_t)__builtin_amdgcn_update_dpp(0, (int)(v), (ctrl), 0xf, 0xf, false))
__device__ __forceinline__ uint32_t wave_sum(uint32_t v) {
  v = fadd(v, EXH_DPP(v, 0xB1));   // quad_perm [1,0,3,2]
  v = fadd(v, EXH_DPP(v, 0x4E));   // quad_perm [2,3,0,1]
  v = fadd(v, EXH_DPP(v, 0x141));  // row_half_mirror
  v = fadd(v, EXH_DPP(v, 0x140));  // row_mirror
  uint32_t a = (uint32_t)__builtin_amdgcn_readlane((int)v, 0), b = (uint32_t)__builtin_amdgcn_readlane((int)v, 16);
  uint32_t c = (uint32_t)__builtin_amdgcn_readlane((int)v, 32), d = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
  return fadd(fadd(a, b), fadd(c, d));
}

// eq((r0, r1), b) for b = 0..3 (bit 0 of b goes with r0), in Montgomery form: the weights that bind two
// variables of a base table at once, entry <- sum_b e[b] * T[4 x + b] (BIND-PREFIX, src/sumcheck.lisp:496-510)
template <int D>
struct BindWeights {
  Ext<D> e[4];
};
template <int D>
__device__ __forceinline__ BindWeights<D> bind_weights(const Ext<D> &r0_mont, const Ext<D> &r1_mont) {
  BindWeights<D> w;
  w.e[3] = ext_mul_mont<D>(r0_mont, r1_mont);  // r0 r1 R
  w.e[1] = ext_sub<D>(r0_mont, w.e[3]);        // r0 (1 - r1) R
  w.e[2] = ext_sub<D>(r1_mont, w.e[3]);        // (1 - r0) r1 R
  Ext<D> one = ext_lift<D>(R1);
  w.e[0] = ext_add<D>(ext_sub<D>(ext_sub<D>(one, r0_mont), r1_mont), w.e[3]);
  return w;
}
// sum_b e[b] * v[b], exact: four products per coordinate, one reduction
template <int D>
__device__ __forceinline__ Ext<D> bind4(const BindWeights<D> &w, uint32_t v0, uint32_t v1, uint32_t v2, uint32_t v3) {
  Ext<D> o;
#pragma unroll
  for (int c = 0; c < D; c++)
    o.c[c] = mont_reduce4((uint64_t)w.e[0].c[c] * v0 + (uint64_t)w.e[1].c[c] * v1 + (uint64_t)w.e[2].c[c] * v2 +
                          (uint64_t)w.e[3].c[c] * v3);
  return o;
}

// the pair (lo, hi) of every table at pair index i, folding first when FOLD (FOLD2: base tables folded
// twice at once by the bind weights)
template <int D, bool IN_BASE, bool FOLD, class V, class Desc, bool FOLD2 = false>
__device__ __forceinline__ void load_pair(const Desc &d, const uint32_t *const *in, uint32_t *const *out, uint64_t i,
                                          const Ext<D> &r, V *lo, V *hi, const BindWeights<D> *bw = nullptr) {
#pragma unroll
  for (int t = 0; t < MAXT; t++) {
    if (t < d.T) {
      if constexpr (FOLD2) {
        const uint4 *p = reinterpret_cast<const uint4 *>(in[t] + 8 * i);
        uint4 e = p[0], f = p[1];
        lo[t] = bind4<D>(*bw, e.x, e.y, e.z, e.w);
        hi[t] = bind4<D>(*bw, f.x, f.y, f.z, f.w);
      } else if constexpr (FOLD && IN_BASE) {
        uint4 e = *reinterpret_cast<const uint4 *>(in[t] + 4 * i);
        lo[t] = fold_base<D>(e.x, e.y, r);
        hi[t] = fold_base<D>(e.z, e.w, r);
      } else if constexpr (FOLD) {
        const uint32_t *p = in[t] + 4 * i * D;
        lo[t] = fold_ext<D>(load_ext<D>(p), load_ext<D>(p + D), r);
        hi[t] = fold_ext<D>(load_ext<D>(p + 2 * D), load_ext<D>(p + 3 * D), r);
      } else if constexpr (IN_BASE) {
        uint2 e = *reinterpret_cast<const uint2 *>(in[t] + 2 * i);
        lo[t] = e.x;
        hi[t] = e.y;
      } else {
        const uint32_t *p = in[t] + 2 * i * D;
        lo[t] = load_ext<D>(p);
        hi[t] = load_ext<D>(p + D);
      }
      if constexpr (FOLD) {
        store_ext<D>(out[t] + 2 * i * D, lo[t]);
        store_ext<D>(out[t] + (2 * i + 1) * D, hi[t]);
      }
    }
  }
}

// The same in two steps, so that a pair's loads can be issued one pair ahead of its arithmetic: the words as
// they lie in memory (QUADS 16-byte quads per table), then the pair from them.
template <int D, bool IN_BASE, bool FOLD, bool FOLD2>
constexpr int raw_quads() {
  return FOLD2 ? 2 : (FOLD && IN_BASE) ? 1 : FOLD ? D : IN_BASE ? 1 : D / 2;
}
template <int D, bool IN_BASE, bool FOLD, bool FOLD2, int Q, class Desc>
__device__ __forceinline__ void fetch_raw(const Desc &d, const uint32_t *const *in, uint64_t i, uint4 (*raw)[Q]) {
#pragma unroll
  for (int t = 0; t < MAXT; t++) {
    if (t < d.T) {
      if constexpr (!FOLD2 && !FOLD && IN_BASE) {
        uint2 e = *reinterpret_cast<const uint2 *>(in[t] + 2 * i);
        raw[t][0] = make_uint4(e.x, e.y, 0u, 0u);
      } else {
        // words per pair: 8 (FOLD2), 4 (base, folding), 4 D (extension, folding), 2 D (extension)
        const uint4 *p = reinterpret_cast<const uint4 *>(in[t]) + (uint64_t)Q * i;
#pragma unroll
        for (int q = 0; q < Q; q++) raw[t][q] = p[q];
      }
    }
  }
}
template <int D>
__device__ __forceinline__ Ext<D> ext_from_quads(const uint4 *q) {
  Ext<D> e;
  e.c[0] = q[0].x, e.c[1] = q[0].y, e.c[2] = q[0].z, e.c[3] = q[0].w;
  if constexpr (D == 8) e.c[4] = q[1].x, e.c[5] = q[1].y, e.c[6] = q[1].z, e.c[7] = q[1].w;
  return e;
}
template <int D, bool IN_BASE, bool FOLD, class V, bool FOLD2, int Q, class Desc>
__device__ __forceinline__ void pair_from_raw(const Desc &d, const uint4 (*raw)[Q], uint32_t *const *out, uint64_t i,
                                              const Ext<D> &r, V *lo, V *hi, const BindWeights<D> *bw) {
#pragma unroll
  for (int t = 0; t < MAXT; t++) {
    if (t < d.T) {
      if constexpr (FOLD2) {
        const uint4 e = raw[t][0], f = raw[t][1];
        lo[t] = bind4<D>(*bw, e.x, e.y, e.z, e.w);
        hi[t] = bind4<D>(*bw, f.x, f.y, f.z, f.w);
      } else if constexpr (FOLD && IN_BASE) {
        const uint4 e = raw[t][0];
        lo[t] = fold_base<D>(e.x, e.y, r);
        hi[t] = fold_base<D>(e.z, e.w, r);
      } else if constexpr (FOLD) {
        constexpr int E = D / 4;  // quads per element
        lo[t] = fold_ext<D>(ext_from_quads<D>(raw[t]), ext_from_quads<D>(raw[t] + E), r);
        hi[t] = fold_ext<D>(ext_from_quads<D>(raw[t] + 2 * E), ext_from_quads<D>(raw[t] + 3 * E), r);
      } else if constexpr (IN_BASE) {
        lo[t] = raw[t][0].x;
        hi[t] = raw[t][0].y;
      } else {
        constexpr int E = D / 4;
        lo[t] = ext_from_quads<D>(raw[t]);
        hi[t] = ext_from_quads<D>(raw[t] + E);
      }
      if constexpr (FOLD) {
        store_ext<D>(out[t] + 2 * i * D, lo[t]);
        store_ext<D>(out[t] + (2 * i + 1) * D, hi[t]);
      }
    }
  }
}

// the value of lane (l ^ M) of the wavefront
template <int M>
__device__ __forceinline__ uint32_t lane_xor(uint32_t v) {
  if constexpr (M == 1)
    return EXH_DPP(v, 0xB1);  // quad_perm [1,0,3,2]
  else if constexpr (M == 2)
    return EXH_DPP(v, 0x4E);  // quad_perm [2,3,0,1]
  else if constexpr (M == 8)
    return EXH_DPP(v, 0x128);  // row_ror:8
  else if constexpr (M == 4 || M == 16)
    return (uint32_t)__builtin_amdgcn_ds_swizzle((int)v, (M << 10) | 0x1f);  // xor within 32 lanes
  else
    return (uint32_t)__builtin_amdgcn_ds_bpermute((int)(((threadIdx.x & 63) ^ 32) << 2), (int)v);
}

// One step of the transposing reduction: the 2 * H values a lane holds become H, each the sum over
// the lane pair (l, l ^ M); lanes with bit M clear keep the lower half of the values, the others the
// upper half.
template <int M, int H>
__device__ __forceinline__ void halve_step(uint32_t *a) {
  const bool upper = (threadIdx.x & M) != 0;
#pragma unroll
  for (int k = 0; k < H; k++) {
    uint32_t keep = upper ? a[k + H] : a[k], send = upper ? a[k] : a[k + H];
    a[k] = fadd(keep, lane_xor<M>(send));
  }
}

// The wavefront's sums of W = 8, 16 or 32 values per lane, value k given by val(k): afterwards lane l
// holds the sum over all 64 lanes of value bitrev(l mod W).  About 2 W cross-lane operations instead of
// the 6 W of one reduction tree per value.  The first step consumes the values as they are produced, so
// only W / 2 are live at once.
template <int W, class F>
__device__ __forceinline__ uint32_t wave_sums_transposed(F val) {
  uint32_t a[W / 2];
  const bool upper = (threadIdx.x & 1) != 0;
#pragma unroll
  for (int k = 0; k < W / 2; k++) {
    uint32_t lo = val(k), hi = val(k + W / 2);
    a[k] = fadd(upper ? hi : lo, lane_xor<1>(upper ? lo : hi));
  }
  if constexpr (W == 32) {
    halve_step<2, 8>(a), halve_step<4, 4>(a), halve_step<8, 2>(a), halve_step<16, 1>(a);
  } else if constexpr (W == 16) {
    halve_step<2, 4>(a), halve_step<4, 2>(a), halve_step<8, 1>(a);
    a[0] = fadd(a[0], lane_xor<16>(a[0]));
  } else {
    halve_step<2, 2>(a), halve_step<4, 1>(a);
    a[0] = fadd(a[0], lane_xor<8>(a[0]));
    a[0] = fadd(a[0], lane_xor<16>(a[0]));
  }
  return fadd(a[0], lane_xor<32>(a[0]));
}

// accumulator words [first, first + W) of the lane, reduced mod p (zero beyond the statement's), summed
// over the wavefront and left in lds_row[first ..]
template <int D, int W, class Desc>
__device__ __forceinline__ void chunk_sums(const Desc &d, Acc96 (*acc)[D], int first, uint32_t *lds_row) {
  const uint32_t total = wave_sums_transposed<W>([&](int k) -> uint32_t {
    const int o = first + k;
    return o < d.nacc * D ? acc_reduce(acc[o / D][o % D]) : 0u;
  });
  const uint32_t l = threadIdx.x & 63;
  constexpr int BITS = W == 32 ? 5 : W == 16 ? 4 : 3;
  uint32_t idx = 0;
#pragma unroll
  for (int b = 0; b < BITS; b++) idx |= ((l >> b) & 1u) << (BITS - 1 - b);
  if (l < W && first + idx < (uint32_t)d.nacc * D) lds_row[first + idx] = total;
}

// The workgroup's sums of every accumulator, reduced mod p, into sums[nacc * D] (LDS); all threads call.
// TRANSPOSED picks the cross-lane scheme: the transposing reduction is the shorter path (the latency-bound
// LDS-resident rounds use it), one tree per value keeps fewer registers live (the streaming round kernels,
// whose occupancy it would cost, use that).
template <int D, bool TRANSPOSED, class Desc>
__device__ __forceinline__ void block_sums(const Desc &d, Acc96 (*acc)[D], uint32_t (*lds)[MAXACC * D],
                                           uint32_t *sums) {
  const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if constexpr (TRANSPOSED) {
    if (d.nacc * D <= 8)
      chunk_sums<D, 8>(d, acc, 0, lds[wave]);
    else if (d.nacc * D <= 16)
      chunk_sums<D, 16>(d, acc, 0, lds[wave]);
    else {
#pragma unroll
      for (int first = 0; first < MAXACC * D; first += 32)
        if (first < d.nacc * D) chunk_sums<D, 32>(d, acc, first, lds[wave]);
    }
  } else {
#pragma unroll
    for (int a = 0; a < MAXACC; a++) {
      if (a < d.nacc) {
#pragma unroll
        for (int c = 0; c < D; c++) {
          uint32_t v = wave_sum(acc_reduce(acc[a][c]));
          if (lane == 0) lds[wave][a * D + c] = v;
        }
      }
    }
  }
  lds_barrier();
  for (uint32_t o = tid; o < (uint32_t)d.nacc * D; o += BLOCK) {
    uint32_t v = lds[0][o];
#pragma unroll
    for (int wv = 1; wv < BLOCK / 64; wv++) v = fadd(v, lds[wv][o]);
    sums[o] = v;
  }
  lds_barrier();
}

// The wavefront's sums of the accumulators a = PART, PART + PARTS, ... (the ones accumulate_pair<.., PARTS> fills
// on the wavefront that has this part), reduced mod p, into sums[a * D ..] (LDS).  Every word of sums is written
// by one wavefront.
template <int D, int PART, int PARTS, int W, class Desc>
__device__ __forceinline__ void part_chunk_sums(const Desc &d, Acc96 (*acc)[D], int first, int count, uint32_t *sums) {
  const uint32_t total = wave_sums_transposed<W>([&](int k) -> uint32_t {
    const int o = first + k, q = o / D;
    return PARTS * q + PART < MAXACC && q < count ? acc_reduce(acc[(PARTS * q + PART) % MAXACC][o % D]) : 0u;
  });
  const uint32_t l = threadIdx.x & 63;
  constexpr int BITS = W == 32 ? 5 : W == 16 ? 4 : 3;
  uint32_t idx = 0;
#pragma unroll
  for (int b = 0; b < BITS; b++) idx |= ((l >> b) & 1u) << (BITS - 1 - b);
  const uint32_t o = first + idx;
  if (l < W && o < (uint32_t)count * D) sums[(PARTS * (o / D) + PART) * D + o % D] = total;
}
template <int D, int PART, int PARTS, class Desc>
__device__ __forceinline__ void part_wave_sums(const Desc &d, Acc96 (*acc)[D], uint32_t *sums) {
  const int count = (d.nacc - PART + PARTS - 1) / PARTS;  // accumulators of this part
  if (count <= 0) return;
  if (count * D <= 8)
    part_chunk_sums<D, PART, PARTS, 8>(d, acc, 0, count, sums);
  else if (count * D <= 16)
    part_chunk_sums<D, PART, PARTS, 16>(d, acc, 0, count, sums);
  else {
#pragma unroll
    for (int first = 0; first < ((MAXACC + PARTS - 1) / PARTS) * D; first += 32)
      if (first < count * D) part_chunk_sums<D, PART, PARTS, 32>(d, acc, first, count, sums);
  }
}

// From the round's accumulator sums (LDS, nacc * D words, scaled as the kernels leave them) to the round
// message, through the transcript, to the next challenge: rows = mtilde * sums + c0
// (ROUND-MESSAGE, src/sumcheck.lisp:313-317), send = absorb the rows (src/transcript.lisp:116-128),
// r = challenge (src/transcript.lisp:174-176).  All threads of the workgroup call; scratch is LDS.
struct EpilogueLds {
  alignas(16) uint32_t prod[MAXPTS * MAXACC * 8];
  uint32_t msg[MAXPTS * 8];
  uint32_t chal[8];
  uint32_t r_mont[8];
  uint32_t ring[RING_WORDS];
  // staged copies (filled by the caller when it passes staged = true)
  uint32_t state[sizeof(DevB3S) / 4];
  uint32_t round;
  alignas(16) uint32_t mtilde[MAXPTS * MAXACC * 8];
  alignas(16) uint32_t c0[MAXPTS * 8];
};

template <int D>
__device__ __forceinline__ void round_message(const uint32_t *sums, uint32_t nacc, uint32_t points,
                                              const uint32_t *mtilde, const uint32_t *c0, EpilogueLds *e) {
  const uint32_t tid = threadIdx.x, nthreads = blockDim.x;
  for (uint32_t u = tid; u < points * nacc; u += nthreads) {
    uint32_t a = u % nacc;
    Ext<D> m = load_ext<D>(mtilde + (size_t)u * D), sv;
#pragma unroll
    for (int c = 0; c < D; c++) sv.c[c] = sums[a * D + c];
    Ext<D> pr = ext_mul_mont<D>(m, sv);
#pragma unroll
    for (int c = 0; c < D; c++) e->prod[u * D + c] = pr.c[c];
  }
  lds_barrier();
  for (uint32_t o = tid; o < points * D; o += nthreads) {
    uint32_t k = o / D, c = o % D, v = c0[o];
    for (uint32_t a = 0; a < nacc; a++) v = fadd(v, e->prod[(k * nacc + a) * D + c]);
    e->msg[o] = v;
  }
  lds_barrier();
}

// the first wavefront's part: send the message, draw the challenge, log both (every lane the same steps)
// With `publish` (an LDS word), the challenge times R is in e->r_mont and *publish = round + 1 as soon as it is
// drawn, before the transcript absorbs the squeeze's bytes: the workgroup's other wavefronts wait for that word
// instead of a barrier and begin the fold while this one finishes the transcript's bookkeeping.
template <int D>
__device__ __forceinline__ void transcript_step(RunB3S &tr, Ctrl *ctrl, uint32_t round, uint32_t points,
                                                EpilogueLds *e, bool log = true, uint32_t *publish = nullptr,
                                                PendingAppend *pending = nullptr) {
  const uint32_t tid = threadIdx.x;
  if (pending) rb3s_flush(tr, *pending);
  dev_absorb_words(tr, e->msg, points * D);
  dev_challenge(tr, D, e->chal, [&] {
    if (tid < (uint32_t)D) e->r_mont[tid] = to_mont(e->chal[tid]);
    __builtin_amdgcn_wave_barrier();
    if (publish && tid == 0) __hip_atomic_store(publish, round + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  }, pending);
  if (log)
    for (uint32_t o = tid; o < points * D; o += 64) ctrl->msg[round][o] = e->msg[o];
  if (log && tid < (uint32_t)D) ctrl->chal[round][tid] = e->chal[tid], ctrl->r_mont[tid] = e->r_mont[tid];
}

template <int D>
__device__ __forceinline__ void round_epilogue(Ctrl *ctrl, const uint32_t *sums, uint32_t nacc, uint32_t points,
                                               const uint32_t *mtilde, const uint32_t *c0, EpilogueLds *e,
                                               bool staged = false) {
  const uint32_t tid = threadIdx.x;
  round_message<D>(sums, nacc, points, mtilde, c0, e);
  if (tid < 64) {
    const uint32_t round = staged ? e->round : ctrl->round;
    RunB3S tr;
    rb3s_load(tr, e->ring, staged ? reinterpret_cast<const DevB3S *>(e->state) : &ctrl->tr);
    transcript_step<D>(tr, ctrl, round, points, e);
    rb3s_store(tr, &ctrl->tr);
    if (tid == 0) ctrl->round = round + 1;
  }
}

// All threads of the workgroup call with its sums (canonical, `width` words) in `mine` (LDS).  True in the one
// workgroup that arrived last, which then holds the sums over all workgroups in `sums` (LDS, width words);
// *ok is false when a word did not complete within the spin limit.  scratch: groups * width words of LDS.
// A launch may add only the words [add_first, add_first + add_count) (the passes of the base-field sweep share one
// set of totals, a pass per range of words); the workgroup whose ticket is last_ticket is the elected one.
// G: the workgroups that add to every word (the launch's grid, or the part of it that sums).
__device__ __forceinline__ bool add_and_elect(const RoundTotals &rt, const uint32_t *mine, uint32_t width,
                                              uint32_t *scratch, uint32_t *sums, bool *ok, uint32_t add_first,
                                              uint32_t add_count, uint32_t last_ticket, uint32_t G) {
  __shared__ uint32_t ticket;
  const uint32_t tid = threadIdx.x, wg = blockIdx.x, NG = rt.groups;
  for (uint32_t o = add_first + tid; o < add_first + add_count; o += blockDim.x)
    __hip_atomic_fetch_add(rt.totals + (size_t)(wg % NG) * rt.pstride + o, ((unsigned long long)1 << 48) + mine[o],
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (tid == 0) ticket = __hip_atomic_fetch_add(rt.arrivals, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  *ok = true;
  if (ticket != last_ticket) return false;
  // every word this thread answers for is requested before any is looked at (one trip to memory for all), from a
  // clamped address so that no load hangs on a condition
  const uint32_t nwords = NG * width;
  unsigned long long v[TOTALS_POLLS];
  uint32_t pending = 0;
#pragma unroll
  for (int k = 0; k < TOTALS_POLLS; k++)
    if (tid + k * blockDim.x < nwords) pending |= 1u << k;
  uint32_t polls = 0;
  int complete = 1;
  while (pending) {
#pragma unroll
    for (int k = 0; k < TOTALS_POLLS; k++) {
      const uint32_t u = tid + k * blockDim.x, at = u < nwords ? u : 0;
      v[k] = __hip_atomic_load(rt.totals + (size_t)(at / width) * rt.pstride + at % width, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
    }
#pragma unroll
    for (int k = 0; k < TOTALS_POLLS; k++) {
      const uint32_t u = tid + k * blockDim.x, g = u / width;
      const uint32_t expect = (G - g + NG - 1) / NG;  // workgroups w < G with w % NG == g
      if (((pending >> k) & 1u) && (uint32_t)(v[k] >> 48) == expect) {
        scratch[u] = f_canonical((double)(v[k] & (((unsigned long long)1 << 48) - 1)));  // exact below 2^53
        pending &= ~(1u << k);
      }
    }
    if (pending) {
      if (++polls > rt.spin_limit) {
        complete = 0;
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
  }
  if (!__syncthreads_and(complete)) {
    *ok = false;
    return true;
  }
  for (uint32_t o = tid; o < width; o += blockDim.x) {
    uint32_t t = 0;
    for (uint32_t g = 0; g < NG; g++) t = fadd(t, scratch[g * width + o]);
    sums[o] = t;
  }
  __syncthreads();
  return true;
}

// One workgroup's share of a round: pairs [block * tile, (block + 1) * tile) with tile = BLOCK *
// pairs_per_thread, folded first when FOLD, summed into the workgroup's partial row.
template <int D>
struct RoundShape {
  const uint32_t *low, *high;
  uint64_t n_pairs;
  uint32_t low_bits, pairs_per_thread;
  bool deferred, do_sums;
  // device-driven rounds (totals non-null): see RoundTotals
  RoundTotals totals;
  uint32_t points;
  const uint32_t *mtilde, *c0;
  Ctrl *ctrl;
  const uint32_t *consts;
};

template <int D, bool IN_BASE, bool FOLD, class Desc, bool FOLD2 = false, bool GENERATED = false>
__device__ __forceinline__ void round_core(const Desc &d, const uint32_t *const *in, uint32_t *const *out,
                                           const RoundShape<D> &sh, const Ext<D> &r, uint32_t block,
                                           uint32_t *partial_row, const BindWeights<D> *bw = nullptr) {
  constexpr bool BASE_MODE = IN_BASE && !FOLD;  // the pair's values are base-field
  using V = typename std::conditional<BASE_MODE, uint32_t, Ext<D>>::type;
  const uint32_t tid = threadIdx.x;
  const uint64_t tile = (uint64_t)BLOCK * sh.pairs_per_thread;
  const uint64_t tile_start = (uint64_t)block * tile;
  const uint64_t low_mask = ((uint64_t)1 << sh.low_bits) - 1;

  Acc96 acc[MAXACC][D];
#pragma unroll
  for (int a = 0; a < MAXACC; a++)
#pragma unroll
    for (int c = 0; c < D; c++) acc_zero(acc[a][c]);

  // With a statement known at compile time and D = 4 the next pair's words are fetched before this pair's
  // arithmetic (two workgroups per compute unit leave the registers for it, and too few wavefronts to hide the
  // loads behind one another); the interpreter and D = 8 keep the plain order.
  // (nor does a statement in direct form: it is wide, and its tables' words ahead would not fit the registers)
  constexpr bool AHEAD = GENERATED && D == 4 && !is_direct<Desc>::value;
  if constexpr (AHEAD) {
    constexpr int Q = raw_quads<D, IN_BASE, FOLD, FOLD2>();
    uint4 raw[MAXT][Q], ahead[MAXT][Q];
    if (tile_start + tid < sh.n_pairs) fetch_raw<D, IN_BASE, FOLD, FOLD2, Q>(d, in, tile_start + tid, raw);
    for (uint32_t k = 0; k < sh.pairs_per_thread; k++) {
      const uint64_t i = tile_start + (uint64_t)k * BLOCK + tid;
      if (i >= sh.n_pairs) break;
      const bool more = k + 1 < sh.pairs_per_thread && i + BLOCK < sh.n_pairs;
      if (more) fetch_raw<D, IN_BASE, FOLD, FOLD2, Q>(d, in, i + BLOCK, ahead);
      Ext<D> w;
      if (sh.do_sums) w = load_ext<D>(sh.low + (i & low_mask) * D);
      V lo[MAXT], hi[MAXT];
      pair_from_raw<D, IN_BASE, FOLD, V, FOLD2, Q>(d, raw, out, i, r, lo, hi, bw);
      if (sh.do_sums) {
        if (!sh.deferred) w = ext_mul_mont<D>(w, load_ext<D>(sh.high + (i >> sh.low_bits) * D));
        accumulate_pair<D, V>(d, lo, hi, w, acc, sh.consts);
      }
      if (more) {
#pragma unroll
        for (int t = 0; t < MAXT; t++)
          if (t < d.T) {
#pragma unroll
            for (int q = 0; q < Q; q++) raw[t][q] = ahead[t][q];
          }
      }
    }
  } else {
    for (uint32_t k = 0; k < sh.pairs_per_thread; k++) {
      const uint64_t i = tile_start + (uint64_t)k * BLOCK + tid;
      if (i >= sh.n_pairs) break;
      V lo[MAXT], hi[MAXT];
      load_pair<D, IN_BASE, FOLD, V, Desc, FOLD2>(d, in, out, i, r, lo, hi, bw);
      if (sh.do_sums) {
        Ext<D> w = load_ext<D>(sh.low + (i & low_mask) * D);
        if (!sh.deferred) w = ext_mul_mont<D>(w, load_ext<D>(sh.high + (i >> sh.low_bits) * D));
        accumulate_pair<D, V>(d, lo, hi, w, acc, sh.consts);
      }
    }
  }
  if (!sh.do_sums) return;

  __shared__ uint32_t lds[BLOCK / 64][MAXACC * D];
  __shared__ uint32_t sums[MAXACC * D];
  // a device-driven round: what the elected workgroup's serial part reads from memory (the transcript's state, the
  // message map, the constant terms) is requested by every workgroup here, ahead of the reduction that hides the
  // trip; the one elected later finds it in its LDS
  constexpr int PRE = (MAXPTS * MAXACC * 8 + BLOCK - 1) / BLOCK;
  uint32_t pre_map[PRE], pre_c0 = 0, pre_state = 0, pre_round = 0;
  if (sh.totals.totals) {
    const uint32_t map_words = sh.points * (uint32_t)d.nacc * D;
#pragma unroll
    for (int k = 0; k < PRE; k++) {
      const uint32_t u = tid + k * BLOCK;
      pre_map[k] = sh.mtilde[u < map_words ? u : 0];
    }
    pre_c0 = sh.c0[tid < sh.points * D ? tid : 0];
    pre_state = reinterpret_cast<const uint32_t *>(&sh.ctrl->tr)[tid < sizeof(DevB3S) / 4 ? tid : 0];
    pre_round = sh.ctrl->round;
  }
  block_sums<D, false>(d, acc, lds, sums);
  Ext<D> s;
  if (tid < (uint32_t)d.nacc) {
#pragma unroll
    for (int c = 0; c < D; c++) s.c[c] = sums[tid * D + c];
    if (sh.deferred) s = ext_mul_mont<D>(s, load_ext<D>(sh.high + (tile_start >> sh.low_bits) * D));
  }
  if (!sh.totals.totals) {
    if (tid < (uint32_t)d.nacc) store_ext<D>(partial_row + tid * D, s);
    return;
  }
  // the device-driven round: totals, and in the last workgroup to arrive the message and the challenge
  __shared__ EpilogueLds epi;
  __syncthreads();
  if (tid < (uint32_t)d.nacc) {
#pragma unroll
    for (int c = 0; c < D; c++) sums[tid * D + c] = s.c[c];
  }
  {
    const uint32_t map_words = sh.points * (uint32_t)d.nacc * D;
#pragma unroll
    for (int k = 0; k < PRE; k++)
      if (tid + k * BLOCK < map_words) epi.mtilde[tid + k * BLOCK] = pre_map[k];
    if (tid < sh.points * D) epi.c0[tid] = pre_c0;
    if (tid < sizeof(DevB3S) / 4) epi.state[tid] = pre_state;
    if (tid == 0) epi.round = pre_round;
  }
  __syncthreads();
  bool ok;
  const uint32_t width = (uint32_t)d.nacc * D;
  if (!add_and_elect(sh.totals, sums, width, epi.prod, sums, &ok, 0, width, gridDim.x - 1, gridDim.x)) return;
  if (!ok) {
    if (tid == 0) __hip_atomic_store(&sh.ctrl->gave_up, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return;
  }
  round_epilogue<D>(sh.ctrl, sums, (uint32_t)d.nacc, sh.points, epi.mtilde, epi.c0, &epi, true);
}

template <int D, bool IN_BASE, bool FOLD, class Desc, bool FOLD2 = false, bool GENERATED = false>
__device__ __forceinline__ void round_body(const Desc &d, const RoundArgs<D> &args) {
  Ext<D> r = ext_zero<D>();
  if constexpr (FOLD2) {  // challenge 0 from the log, challenge 1 is the latest
    Ext<D> r0, r1;
#pragma unroll
    for (int c = 0; c < D; c++) r0.c[c] = to_mont(args.ctrl->chal[0][c]), r1.c[c] = args.ctrl->r_mont[c];
    BindWeights<D> bw = bind_weights<D>(r0, r1);
    RoundShape<D> sh{args.low, args.high, args.n_pairs, args.low_bits, args.pairs_per_thread, args.deferred != 0,
                     args.do_sums != 0, RoundTotals{args.totals, args.arrivals, args.groups, args.pstride, args.spin_limit},
                     args.points, args.mtilde, args.c0, args.ctrl, args.consts};
    round_core<D, true, true, Desc, true, GENERATED>(d, args.in, args.out, sh, r, blockIdx.x,
                                          args.partials + (uint64_t)blockIdx.x * args.pstride, &bw);
    return;
  }
  if constexpr (FOLD) {
    const uint32_t *rp = args.ctrl ? args.ctrl->r_mont : args.r_mont;
#pragma unroll
    for (int c = 0; c < D; c++) r.c[c] = rp[c];
  }
  RoundShape<D> sh{args.low, args.high, args.n_pairs, args.low_bits, args.pairs_per_thread, args.deferred != 0,
                   args.do_sums != 0, RoundTotals{args.totals, args.arrivals, args.groups, args.pstride, args.spin_limit},
                   args.points, args.mtilde, args.c0, args.ctrl, args.consts};
  round_core<D, IN_BASE, FOLD, Desc, false, GENERATED>(d, args.in, args.out, sh, r, blockIdx.x,
                               args.partials + (uint64_t)blockIdx.x * args.pstride);
}

// The round's second launch when the device drives the loop: one workgroup adds the partials, forms the
// message, runs the transcript and leaves the next challenge in ctrl.  (A last-workgroup-done scheme
// inside the round kernel needs a device-scope fence per workgroup, which on this part writes back the
// XCD's whole L2 and costs more than a launch.)
// sums[o] = sum over the workgroups' partial rows of word o (o < width <= blockDim.x): thread t takes column
// t % width of the rows t / width, t / width + groups, ... with groups = blockDim.x / width, so that all
// threads share the rows whatever the row stride; sixteen loads in flight per thread.
// All threads of the workgroup call; scratch holds blockDim.x words.
__device__ __forceinline__ void sum_partials(const uint32_t *partials, uint32_t nblocks, uint32_t ps, uint32_t width,
                                             uint32_t *scratch, uint32_t *sums) {
  const uint32_t tid = threadIdx.x, nthreads = blockDim.x;
  const uint32_t groups = width ? nthreads / width : 0, col = width ? tid % width : 0, row0 = width ? tid / width : 0;
  // sixteen loads in flight per thread and trip to memory, the last batch's rows beyond the end masked off (a loop
  // over single rows behind full batches would be a trip to memory per row)
  uint32_t v[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  if (row0 < groups) {
    const uint32_t *p = partials + col;
    for (uint32_t b = row0; b < nblocks; b += 16 * groups) {
      uint32_t x[16];
#pragma unroll
      for (int q = 0; q < 16; q++) {
        const uint32_t row = b + q * groups;
        x[q] = row < nblocks ? p[(uint64_t)row * ps] : 0u;
      }
#pragma unroll
      for (int q = 0; q < 16; q++) v[q & 7] = fadd(v[q & 7], x[q]);
    }
  }
  __syncthreads();
  scratch[tid] = fadd(fadd(fadd(v[0], v[1]), fadd(v[2], v[3])), fadd(fadd(v[4], v[5]), fadd(v[6], v[7])));
  __syncthreads();
  if (tid < width) {
    uint32_t total = scratch[tid];
    for (uint32_t g = 1; g < groups; g++) total = fadd(total, scratch[g * width + tid]);
    sums[tid] = total;
  }
  __syncthreads();
}

struct EpilogueArgs {
  const uint32_t *partials;
  uint32_t nblocks, pstride, nacc, points;
  const uint32_t *mtilde, *c0;
  Ctrl *ctrl;
};

constexpr int EPI_BLOCK = 1024;

template <int D>
__global__ __launch_bounds__(EPI_BLOCK) void epilogue_kernel(EpilogueArgs args) {
  __shared__ uint32_t scratch[EPI_BLOCK];
  __shared__ uint32_t sums[MAXACC * D];
  __shared__ EpilogueLds epi;
  const uint32_t tid = threadIdx.x, width = args.nacc * D, ps = args.pstride;
  // everything the serial part needs from global memory is requested first, so that its latency
  // overlaps the partial sums: the transcript state, the message map and the constant terms
  if (tid < sizeof(DevB3S) / 4) epi.state[tid] = reinterpret_cast<const uint32_t *>(&args.ctrl->tr)[tid];
  if (tid == 64) epi.round = args.ctrl->round;
  for (uint32_t u = tid; u < args.points * width; u += EPI_BLOCK) epi.mtilde[u] = args.mtilde[u];
  for (uint32_t u = tid; u < args.points * D; u += EPI_BLOCK) epi.c0[u] = args.c0[u];
  sum_partials(args.partials, args.nblocks, ps, width, scratch, sums);
  round_epilogue<D>(args.ctrl, sums, args.nacc, args.points, epi.mtilde, epi.c0, &epi, true);
}

// A small round's sums on one wavefront: the accumulators PART, PART + 4, ... of the lane's pair, summed over the
// wavefront into sums (LDS).  The accumulators are this function's own, so that they live in registers.
template <int D, int PART, int PARTS, class Desc>
__device__ __forceinline__ void small_round_sums(const Desc &d, const Ext<D> *lo, const Ext<D> *hi, const Ext<D> &w,
                                                 uint32_t *sums, const uint32_t *kc) {
  Acc96 acc[MAXACC][D];
#pragma unroll
  for (int a = 0; a < MAXACC; a++)
#pragma unroll
    for (int c = 0; c < D; c++) acc_zero(acc[a][c]);
  accumulate_pair<D, Ext<D>, Desc, PARTS, PART>(d, lo, hi, w, acc, kc);
  part_wave_sums<D, PART, PARTS>(d, acc, sums);
}

// Load (folding or lifting on the way in) into LDS, then per round sums -> message -> challenge -> fold
// on the slice this workgroup holds: entries [w * E, (w + 1) * E) of every table, E = entries / grid.
// A grid launch ends when its rounds are done and leaves the slices in `out` for the one-workgroup
// launch that follows; that one ends with the finals.
template <int D, class Desc>
__device__ __forceinline__ void tail_body(const Desc &d, const TailArgs<D> &args) {
  extern __shared__ __align__(16) uint32_t tail_tables[];  // [T][capacity][D]
  __shared__ uint32_t lds[BLOCK / 64][MAXACC * D];
  __shared__ uint32_t sums[MAXACC * D];
  __shared__ EpilogueLds epi;
  __shared__ uint32_t c0s[MAXTAIL * MAXPTS * D];
  __shared__ uint32_t ready_round;  // rounds whose challenge the first wavefront has published, counted from the proof's first
  const uint32_t tid = threadIdx.x, cap = args.capacity, G = gridDim.x, wg = blockIdx.x;
  if (tid == 0) ready_round = 0;
  const uint32_t width = (uint32_t)d.nacc * D;
  if (args.ctrl->round != args.first_round) return;  // an earlier launch gave up: leave the count as it is
  RunB3S tr;
  PendingAppend pending{0, 0};  // (the first wavefront's)
  if (tid < 64) rb3s_load(tr, epi.ring, &args.ctrl->tr);
  uint32_t entries = (args.first_fold ? args.entries / 2 : args.entries) / G;  // of this workgroup's slice
  {
    Ext<D> r = ext_zero<D>();
    if (args.first_fold) {
#pragma unroll
      for (int c = 0; c < D; c++) r.c[c] = args.ctrl->r_mont[c];
    }
#pragma unroll
    for (int t = 0; t < MAXT; t++) {
      if (t < d.T) {
        const uint32_t *in = args.in[t];
        for (uint32_t x = tid; x < entries; x += BLOCK) {
          const uint64_t gx = (uint64_t)wg * entries + x;  // index after the fold on the way in
          Ext<D> v;
          if (args.in_base) {
            if (args.first_fold) {
              uint2 e = *reinterpret_cast<const uint2 *>(in + 2 * gx);
              v = fold_base<D>(e.x, e.y, r);
            } else {
              v = ext_zero<D>();
              v.c[0] = in[gx];
            }
          } else if (args.first_fold) {
            v = fold_ext<D>(load_ext<D>(in + 2 * gx * D), load_ext<D>(in + (2 * gx + 1) * D), r);
          } else {
            v = load_ext<D>(in + gx * D);
          }
          store_ext<D>(tail_tables + ((size_t)t * cap + x) * D, v);
        }
      }
    }
    for (uint32_t u = tid; u < args.points * width; u += BLOCK) epi.mtilde[u] = args.mtilde[u];
    for (uint32_t u = tid; u < args.rounds * args.points * D; u += BLOCK) c0s[u] = args.c0[u];
  }
  // The session's own weight tables (see TailArgs::factors), in LDS behind the tables: the factors first, then
  // per round its LOW and its HIGH table.  An entry is a chain of at most n_vars products, one entry per thread
  // and trip: entry x of a table over the variables [first, first + bits) is prod_b (x_b ? r_b : 1 - r_b).
  const bool own_weights = args.factors != nullptr;
  uint32_t *const own_factors = tail_tables + (size_t)d.T * cap * D;
  uint32_t *const own_tables = own_factors + (size_t)2 * args.n_vars * D;
  auto own_high_bits = [&](uint32_t jj) { return args.n_vars - (args.first_round + jj + 1) - args.low_bits[jj]; };
  auto own_at = [&](uint32_t jj, bool high) {  // where round jj's LOW (HIGH) table begins, in elements
    uint32_t at = 0;
    for (uint32_t q = 0; q < jj; q++) at += (1u << args.low_bits[q]) + (1u << own_high_bits(q));
    return high ? at + (1u << args.low_bits[jj]) : at;
  };
  if (own_weights) {
    for (uint32_t u = tid; u < 2 * args.n_vars * D; u += BLOCK) own_factors[u] = args.factors[u];
    __syncthreads();
    const uint32_t total = own_at(args.rounds, false);
    for (uint32_t u = tid; u < total; u += BLOCK) {
      uint32_t jj = 0, start = 0, first = 0, bits = 0;
      for (;; jj++) {  // (u < total: the scan ends inside the rounds)
        const uint32_t lb = args.low_bits[jj], hb = own_high_bits(jj);
        if (u < start + (1u << lb)) {
          first = args.first_round + jj + 1, bits = lb;
          break;
        }
        start += 1u << lb;
        if (u < start + (1u << hb)) {
          first = args.first_round + jj + 1 + lb, bits = hb;
          break;
        }
        start += 1u << hb;
      }
      const uint32_t x = u - start;
      Ext<D> e = ext_lift<D>(1);
      for (uint32_t b = 0; b < bits; b++)
        e = ext_mul_mont<D>(e, load_ext<D>(own_factors + ((size_t)(first + b) * 2 + (((x >> b) & 1) ? 0 : 1)) * D));
      store_ext<D>(own_tables + (size_t)u * D, e);
    }
    __syncthreads();
  }
  // the weight factors of this thread's first pair of a round, fetched one round ahead
  Ext<D> wl = ext_zero<D>(), wh = ext_zero<D>();
  // (a round of at most 64 pairs runs with a pair per lane on all four wavefronts, each computing a share of the
  // pair's accumulators)
  const uint32_t lane = tid & 63, wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
  // (every thread loads, from a clamped index: a load under a condition has to be merged with the old value as soon
  // as it is issued, which turns the prefetch into a wait for memory at the end of every round)
  auto fetch_weight = [&](uint32_t jj, uint32_t pairs) {
    const uint32_t me = pairs <= 64 ? lane : tid;
    const uint64_t i = (uint64_t)wg * pairs + (me < pairs ? me : pairs - 1);
    if (own_weights) {
      wl = load_ext<D>(own_tables + (size_t)(own_at(jj, false) + (uint32_t)(i & (((uint64_t)1 << args.low_bits[jj]) - 1))) * D);
      wh = load_ext<D>(own_tables + (size_t)(own_at(jj, true) + (uint32_t)(i >> args.low_bits[jj])) * D);
      return;
    }
    wl = load_ext<D>(args.weights + (args.low_off[jj] + (i & (((uint64_t)1 << args.low_bits[jj]) - 1))) * D);
    wh = load_ext<D>(args.weights + (args.high_off[jj] + (i >> args.low_bits[jj])) * D);
  };
  // a fold of `count` outputs by r, a table per wavefront, in place: the lanes run in lockstep, so every read of
  // a chunk of 64 comes before its writes, and those land below what later chunks read
  auto fold_small = [&](const Ext<D> &r, uint32_t count) {
#pragma unroll
    for (int t = 0; t < MAXT; t++)
      if (t < d.T && (uint32_t)((t + 1) & 3) == wave) {  // (the first wavefront, late from the transcript, last)
        for (uint32_t x = lane; x < count; x += 64) {
          const uint32_t *p = tail_tables + ((size_t)t * cap + 2 * x) * D;
          const Ext<D> folded = fold_ext<D>(load_ext<D>(p), load_ext<D>(p + D), r);
          store_ext<D>(tail_tables + ((size_t)t * cap + x) * D, folded);
        }
      }
  };
  fetch_weight(0, entries / 2);
  __syncthreads();
  for (uint32_t jj = 0; jj < args.rounds; jj++) {
    const uint32_t pairs = entries / 2;
    const bool small = pairs <= 64 && BLOCK == 256;
    {  // the round's sums
      if (small) {  // each wavefront its own share of the pair's accumulators, in code of its own
        Ext<D> lo[MAXT], hi[MAXT];
        const uint32_t at = lane < pairs ? lane : 0;
#pragma unroll
        for (int t = 0; t < MAXT; t++)
          if (t < d.T) {
            const uint32_t *p = tail_tables + ((size_t)t * cap + 2 * at) * D;
            lo[t] = load_ext<D>(p);
            hi[t] = load_ext<D>(p + D);
          }
        Ext<D> ww = ext_mul_mont<D>(wl, wh);
        if (lane >= pairs) ww = ext_zero<D>();  // lanes without a pair add nothing
        if (jj + 1 < args.rounds) fetch_weight(jj + 1, pairs / 2);
        // three wavefronts share the accumulators; the first, which ran the transcript, meanwhile absorbs what the
        // last squeeze left to absorb (a compression every other round): nobody waits for that any more
        if (wave == 0)
          rb3s_flush(tr, pending);
        else if (wave == 1)
          small_round_sums<D, 0, 3>(d, lo, hi, ww, sums, args.consts);
        else if (wave == 2)
          small_round_sums<D, 1, 3>(d, lo, hi, ww, sums, args.consts);
        else
          small_round_sums<D, 2, 3>(d, lo, hi, ww, sums, args.consts);
        lds_barrier();
      } else {
        Acc96 acc[MAXACC][D];
#pragma unroll
        for (int a = 0; a < MAXACC; a++)
#pragma unroll
          for (int c = 0; c < D; c++) acc_zero(acc[a][c]);
        for (uint32_t i = tid; i < pairs; i += BLOCK) {
          Ext<D> lo[MAXT], hi[MAXT];
#pragma unroll
          for (int t = 0; t < MAXT; t++)
            if (t < d.T) {
              const uint32_t *p = tail_tables + ((size_t)t * cap + 2 * i) * D;
              lo[t] = load_ext<D>(p);
              hi[t] = load_ext<D>(p + D);
            }
          if (i >= BLOCK) {  // beyond the prefetched pair (never with the session's own tables: one launch's
                             // rounds have a pair per thread at most)
            const uint64_t gi = (uint64_t)wg * pairs + i;
            wl = load_ext<D>(args.weights + (args.low_off[jj] + (gi & (((uint64_t)1 << args.low_bits[jj]) - 1))) * D);
            wh = load_ext<D>(args.weights + (args.high_off[jj] + (gi >> args.low_bits[jj])) * D);
          }
          accumulate_pair<D, Ext<D>>(d, lo, hi, ext_mul_mont<D>(wl, wh), acc, args.consts);
        }
        if (jj + 1 < args.rounds) fetch_weight(jj + 1, pairs / 2);
        block_sums<D, true>(d, acc, lds, sums);
      }
      if (G > 1) {
        // The round's sums over all workgroups.  Each workgroup adds its sums into its group's totals,
        // one integer atomic per word that also counts the contribution in the word's top 16 bits; a
        // word whose count equals the group's size is complete, so readers poll the words themselves:
        // nothing else is exchanged (the tables live in LDS), and no fence or separate barrier is needed.
        // Groups keep the atomics on one address few.
        const uint32_t NG = args.groups, gsize = G / NG;
        unsigned long long *totals = args.totals + (size_t)jj * NG * args.pstride;
        for (uint32_t o = tid; o < width; o += BLOCK)
          __hip_atomic_fetch_add(totals + (size_t)(wg % NG) * args.pstride + o, ((unsigned long long)1 << 48) + sums[o],
                                 __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        int complete = 1;
        for (uint32_t u = tid; u < NG * width; u += BLOCK) {
          const unsigned long long *word = totals + (size_t)(u / width) * args.pstride + u % width;
          unsigned long long v;
          uint32_t polls = 0;
          while (((v = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) >> 48) != gsize) {
            if (++polls > args.spin_limit) {  // the grid is not all there: give up, the host sees the round count
              complete = 0;
              break;
            }
            __builtin_amdgcn_s_sleep(1);
          }
          epi.prod[u] = f_canonical((double)(v & (((unsigned long long)1 << 48) - 1)));  // exact below 2^53
        }
        if (!__syncthreads_and(complete)) {
          // leave a mark: the others may have seen this workgroup's sums and go on to publish the rounds, but
          // its slice is never written
          if (tid == 0) __hip_atomic_store(&args.ctrl->gave_up, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          return;
        }
        for (uint32_t o = tid; o < width; o += BLOCK) {
          uint32_t v = 0;
          for (uint32_t g = 0; g < NG; g++) v = fadd(v, epi.prod[g * width + o]);
          sums[o] = v;
        }
        lds_barrier();
      }
    }
    {  // the message, the challenge, the fold
      round_message<D>(sums, (uint32_t)d.nacc, args.points, epi.mtilde, c0s + (size_t)jj * args.points * D, &epi);
      // the first wavefront publishes the challenge the moment it is drawn and finishes the transcript's step while
      // the others, which wait for that word alone, are already folding
      if (tid < 64) {
        transcript_step<D>(tr, args.ctrl, args.first_round + jj, args.points, &epi, wg == 0, &ready_round, &pending);
      } else {
        while (__hip_atomic_load(&ready_round, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) != args.first_round + jj + 1)
          __builtin_amdgcn_s_sleep(1);
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      Ext<D> r;
#pragma unroll
      for (int c = 0; c < D; c++) r.c[c] = epi.r_mont[c];
      if (small) {
        fold_small(r, pairs);
        lds_barrier();
      }
      // fold in place, 256 entries at a time in ascending order: a chunk's reads come before its writes,
      // and its writes land below everything a later chunk reads
      for (uint32_t base = 0; base < pairs && !small; base += BLOCK) {
        const uint32_t x = base + tid;
        Ext<D> folded[MAXT];
        if (x < pairs) {
#pragma unroll
          for (int t = 0; t < MAXT; t++)
            if (t < d.T) {
              const uint32_t *p = tail_tables + ((size_t)t * cap + 2 * x) * D;
              folded[t] = fold_ext<D>(load_ext<D>(p), load_ext<D>(p + D), r);
            }
        }
        lds_barrier();
        if (x < pairs) {
#pragma unroll
          for (int t = 0; t < MAXT; t++)
            if (t < d.T) store_ext<D>(tail_tables + ((size_t)t * cap + x) * D, folded[t]);
        }
        lds_barrier();
      }
    }
    entries = pairs;
  }
#pragma unroll
  for (int t = 0; t < MAXT; t++)
    if (t < d.T)
      for (uint32_t x = tid; x < entries; x += BLOCK)
        store_ext<D>(args.out + (((size_t)t * G + wg) * entries + x) * D,
                     load_ext<D>(tail_tables + ((size_t)t * cap + x) * D));
  if (G == 1 && entries == 1 && tid < (uint32_t)d.T * D)  // the finals travel with the logs
    args.ctrl->finals[tid] = tail_tables[(size_t)(tid / D) * cap * D + tid % D];
  if (tid < 64) rb3s_flush(tr, pending);
  if (wg == 0 && tid < 64) {
    rb3s_store(tr, &args.ctrl->tr);
    if (tid == 0) args.ctrl->round = args.first_round + args.rounds;
  }
  if (args.host_log && G == 1) {
    __syncthreads();
    // every word through the L2 (this workgroup wrote some of them a moment ago, other launches the rest); of
    // the logs only what the rounds filled: the head, points * D words of a round's message, D of its challenge
    const uint32_t *words = reinterpret_cast<const uint32_t *>(args.ctrl);
    auto deliver = [&](uint32_t at) {
      args.host_log[at] = __hip_atomic_load(words + at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };
    const uint32_t all_rounds = args.first_round + args.rounds, mw = args.points * D;
    for (uint32_t u = tid; u < offsetof(Ctrl, msg) / 4; u += BLOCK) deliver(u);
    for (uint32_t u = tid; u < all_rounds * mw; u += BLOCK)
      deliver((uint32_t)(offsetof(Ctrl, msg) / 4) + (u / mw) * (MAXPTS * 8) + u % mw);
    for (uint32_t u = tid; u < all_rounds * D; u += BLOCK)
      deliver((uint32_t)(offsetof(Ctrl, chal) / 4) + (u / D) * 8 + u % D);
    for (uint32_t u = tid; u < (uint32_t)d.T * D; u += BLOCK) deliver((uint32_t)(offsetof(Ctrl, finals) / 4) + u);
    __threadfence_system();
    __syncthreads();
    if (tid == 0) {
      __hip_atomic_store(args.host_log + args.host_flag_at, args.host_seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
  }
}

// ---- rounds 0 and 1 from one sweep of the base tables.  A pair of round 1 is four base entries per table:
// the value at (X0, X1) is bilinear in them, u(X1) + X0 v(X1) with base-field u, v.  A group of degree d is
// therefore a polynomial of degree d in X0 with base-field coefficients at every X1, and the kernel sums,
// weighted by round 1's weights, its values on a grid ("slots"):
//   (point e, node m):  X1 = the group's e-th evaluation point, X0 = m in 0..d     -- round 1, whose epilogue
//                       interpolates in X0 at the challenge r0,
//   (extra e):          X1 = 1, X0 = the e-th evaluation point                     -- round 0: its sum at X0 is
//                       eq(w1, 0) * slot(X1 = 0, X0) + eq(w1, 1) * slot(X1 = 1, X0), the weight of variable 1
//                       being the one factor round 0's weights have beyond round 1's.
// All products are base-field; no folded table is written; round 2 folds twice.  A launch covers the slots
// [PASS * SPP, (PASS + 1) * SPP) so the accumulators stay in registers.
// The epilogue of that sweep, both rounds by one workgroup: slot sums -> round 0's accumulator sums -> its
// message, through the transcript, to r0 -> the Lagrange basis at r0 -> round 1's accumulator sums -> its
// message and r1.  The statement's shape comes as run-time arrays.
struct NodesEpilogueArgs {
  EpilogueArgs e;            // c0 points at round 0's rows, round 1's follow
  const uint32_t *eq1;       // eq(w1, 1) and eq(w1, 0) as two elements, Montgomery form; null: both weights 1
  uint32_t groups, slots;
  uint32_t deg[MAXG], nev[MAXG];
  uint8_t ev[MAXG][MAXEV];
  uint32_t inv_den[(MAXDEG + 1) * (MAXDEG + 1)];  // [deg][m]: 1 / prod_{q != m, q <= deg} (m - q), Montgomery form
};

template <int D>
struct NodesArgs {
  const uint32_t *in[MAXT];  // base tables
  const uint32_t *low, *high;
  uint64_t n_pairs;          // pairs of round 1: four base entries each
  uint32_t low_bits, pairs_per_thread, deferred;
  // the slot sums of all passes meet in one set of counted totals (slot s at word s * D), and the last workgroup
  // of the last pass to arrive runs the two rounds' epilogue itself (see RoundTotals)
  RoundTotals totals;
  uint32_t passes;
  NodesEpilogueArgs epi;
};

// A 64-bit accumulator of 32 x 32-bit products kept below p 2^32 by a conditional subtraction of p from its high
// word after every product: acc < p 2^32, the product of a canonical weight and a residue below 2^32 is below
// p 2^32 as well, so the sum is below 2^64, and min(hi, hi - p) brings it back (hi < p: hi - p wraps above hi).
// Eight registers per slot at F_p^4 where the 96-bit form takes twelve, for one more (cheap) instruction per word.
__device__ __forceinline__ void lazy_mad(uint64_t &acc, uint32_t w, uint32_t v) {
  acc = (uint64_t)w * v + acc;
  const uint32_t hi = (uint32_t)(acc >> 32);
  acc = ((uint64_t)umin32(hi, hi - P) << 32) | (uint32_t)acc;
}
__device__ __forceinline__ uint32_t lazy_reduce(uint64_t acc) {
  Acc96 a;
  a.lo = acc, a.hi = 0;
  return acc_reduce(a);
}

// the LDS of the two rounds' epilogue
template <int D>
struct NodesEpilogueLds {
  uint32_t slot_sums[MAXACC * D];
  uint32_t sums[MAXACC * D];
  uint32_t basis[(MAXDEG + 1) * (MAXDEG + 1) * D];  // [deg][node]: Lagrange basis at r0, Montgomery form
  // the statement's shape: indexed by lane-dependent values out of the kernel's arguments, every access would be
  // a load from memory with the next one waiting behind it
  uint32_t s_deg[MAXG], s_nev[MAXG], s_inv_den[(MAXDEG + 1) * (MAXDEG + 1)];
  uint8_t s_ev[MAXG][MAXEV];
  EpilogueLds epi;
};

// everything the epilogue reads from memory, into LDS (all threads call; a barrier must follow before use)
template <int D>
__device__ __forceinline__ void nodes_epilogue_stage(const NodesEpilogueArgs &args, NodesEpilogueLds<D> &L) {
  const uint32_t tid = threadIdx.x, nthreads = blockDim.x, points = args.e.points, nacc = args.e.nacc;
  if (tid < MAXG) L.s_deg[tid] = args.deg[tid], L.s_nev[tid] = args.nev[tid];
  if (tid < MAXG * MAXEV) L.s_ev[tid / MAXEV][tid % MAXEV] = args.ev[tid / MAXEV][tid % MAXEV];
  if (tid < (MAXDEG + 1) * (MAXDEG + 1)) L.s_inv_den[tid] = args.inv_den[tid];
  if (tid < sizeof(DevB3S) / 4) L.epi.state[tid] = reinterpret_cast<const uint32_t *>(&args.e.ctrl->tr)[tid];
  for (uint32_t u = tid; u < points * nacc * D; u += nthreads) L.epi.mtilde[u] = args.e.mtilde[u];
  for (uint32_t u = tid; u < points * D; u += nthreads) L.epi.c0[u] = args.e.c0[u];
}

// from the slot sums (L.slot_sums) to both rounds' messages and challenges; all threads of the workgroup call
template <int D>
__device__ __forceinline__ void nodes_epilogue_body(const NodesEpilogueArgs &args, NodesEpilogueLds<D> &L) {
  const uint32_t tid = threadIdx.x, nthreads = blockDim.x, points = args.e.points, nacc = args.e.nacc;
  EpilogueLds &epi = L.epi;
  auto slot = [&](uint32_t index) {
    Ext<D> v;
#pragma unroll
    for (int c = 0; c < D; c++) v.c[c] = L.slot_sums[index * D + c];
    return v;
  };
  auto row_of = [&](uint32_t g, uint32_t x) {  // the index of X among group g's points, or nev
    uint32_t at = L.s_nev[g];
    for (uint32_t e = 0; e < L.s_nev[g]; e++)
      if (L.s_ev[g][e] == x) at = e;
    return at;
  };
  // accumulator tid is point e of group g, whose slots start at `base` (every thread finds its own, so that the
  // accumulators' sums below run side by side on the lanes of one wavefront)
  uint32_t g = 0, e = 0, base = 0;
  bool mine = false;
  {
    uint32_t a = 0;
    for (uint32_t k = 0; k < args.groups && !mine; k++) {
      const uint32_t nev = L.s_nev[k];
      if (tid < a + nev) {
        g = k, e = tid - a, mine = true;
      } else {
        a += nev;
        base += nev * (L.s_deg[k] + 1) + (row_of(k, 1) < nev ? 0 : nev);
      }
    }
  }
  // ---- round 0: accumulator (g, e) = eq(w1, 0) * slot(X1 = 0, node ev_e) + eq(w1, 1) * slot(X1 = 1, node ev_e)
  if (mine) {
    const uint32_t deg = L.s_deg[g], nev = L.s_nev[g], row0 = row_of(g, 0), row1 = row_of(g, 1);
    const uint32_t node = L.s_ev[g][e];
    Ext<D> at0 = slot(base + row0 * (deg + 1) + node);
    Ext<D> at1 = row1 < nev ? slot(base + row1 * (deg + 1) + node) : slot(base + nev * (deg + 1) + e);
    if (args.eq1) {
      at1 = ext_mul_mont<D>(at1, load_ext<D>(args.eq1));
      at0 = ext_mul_mont<D>(at0, load_ext<D>(args.eq1 + D));
    }
    const Ext<D> total = ext_add<D>(at0, at1);
#pragma unroll
    for (int c = 0; c < D; c++) L.sums[tid * D + c] = total.c[c];
  }
  __syncthreads();
  round_message<D>(L.sums, nacc, points, epi.mtilde, epi.c0, &epi);
  RunB3S tr;
  if (tid < 64) {
    rb3s_load(tr, epi.ring, reinterpret_cast<const DevB3S *>(epi.state));
    transcript_step<D>(tr, args.e.ctrl, 0, points, &epi);
  }
  __syncthreads();
  // ---- round 1: the basis of nodes 0..deg at r0, L_m = prod_{q != m} (r0 - q) / (m - q)
  for (uint32_t u = tid; u < points * D; u += nthreads) epi.c0[u] = args.e.c0[points * D + u];
  if (tid < (MAXDEG + 1) * (MAXDEG + 1)) {
    const uint32_t deg = tid / (MAXDEG + 1), m = tid % (MAXDEG + 1);
    if (deg >= 1 && m <= deg) {
      Ext<D> r0, acc = ext_lift<D>(R1);  // 1 in Montgomery form
#pragma unroll
      for (int c = 0; c < D; c++) r0.c[c] = epi.r_mont[c];
      for (uint32_t q = 0; q <= deg; q++) {
        if (q == m) continue;
        Ext<D> f = r0;
        f.c[0] = fsub(f.c[0], to_mont(q));  // (r0 - q) R
        acc = ext_mul_mont<D>(acc, f);
      }
      acc = ext_scale_mont<D>(acc, L.s_inv_den[tid]);
#pragma unroll
      for (int c = 0; c < D; c++) L.basis[tid * D + c] = acc.c[c];
    }
  }
  __syncthreads();
  // accumulator (g, e) = sum over nodes of basis * slot
  if (mine) {
    const uint32_t deg = L.s_deg[g];
    Ext<D> total = ext_zero<D>();
    for (uint32_t m = 0; m <= deg; m++) {
      Ext<D> lb;
#pragma unroll
      for (int c = 0; c < D; c++) lb.c[c] = L.basis[(deg * (MAXDEG + 1) + m) * D + c];
      total = ext_add<D>(total, ext_mul_mont<D>(lb, slot(base + e * (deg + 1) + m)));
    }
#pragma unroll
    for (int c = 0; c < D; c++) L.sums[tid * D + c] = total.c[c];
  }
  __syncthreads();
  round_message<D>(L.sums, nacc, points, epi.mtilde, epi.c0, &epi);
  if (tid < 64) {
    transcript_step<D>(tr, args.e.ctrl, 1, points, &epi);
    rb3s_store(tr, &args.e.ctrl->tr);
    if (tid == 0) args.e.ctrl->round = 2;
  }
}

// the slot sums: lines and products in double precision (field.hpp), weighted sums in integers
template <int D, int PASS, int SPP, class Desc>
__device__ __forceinline__ void nodes_body(const Desc &d, const NodesArgs<D> &args) {
  // magnitudes, in units of p: a table line's ends < 1, a linear form < 5 (MAXVT terms and the constant),
  // the step between X points < 10, so at X <= 7 a line's end < 65 and its slope < 52, a node's value
  // < 65 + 6 * 52 = 377; a product of two < 377^2 p^2 < 2^80 and its quotient by p < 2^49.
  static_assert(MAXVT <= 4 && MAXX <= 7 && MAXDEG <= 6, "the bounds of the double-precision products");
  const uint32_t tid = threadIdx.x;
  const uint64_t tile = (uint64_t)BLOCK * args.pairs_per_thread, tile_start = (uint64_t)blockIdx.x * tile;
  const uint64_t low_mask = ((uint64_t)1 << args.low_bits) - 1;
  // the weighted sums themselves are integer: one 32 x 32 -> 64 multiply-add per word into a lazily reduced
  // 64-bit sum (lazy_mad)
  uint64_t acc[SPP][D];
#pragma unroll
  for (int a = 0; a < SPP; a++)
#pragma unroll
    for (int c = 0; c < D; c++) acc[a][c] = 0;

  // the loads run PREFETCH pairs ahead of the arithmetic: few waves fit beside the accumulators
  constexpr int PREFETCH = 2;
  uint4 ahead[PREFETCH][MAXT];
  Ext<D> wahead[PREFETCH];
  auto fetch = [&](uint32_t k, uint4 *e, Ext<D> &w) {
    const uint64_t i = tile_start + (uint64_t)k * BLOCK + tid;
    if (k < args.pairs_per_thread && i < args.n_pairs) {
#pragma unroll
      for (int t = 0; t < MAXT; t++)
        if (t < d.T) e[t] = *reinterpret_cast<const uint4 *>(args.in[t] + 4 * i);
      w = load_ext<D>(args.low + (i & low_mask) * D);
    }
  };
#pragma unroll
  for (int a = 0; a < PREFETCH; a++) fetch(a, ahead[a], wahead[a]);

  for (uint32_t k = 0; k < args.pairs_per_thread; k++) {
    const uint64_t i = tile_start + (uint64_t)k * BLOCK + tid;
    if (i >= args.n_pairs) break;
    // per factor: the line in r0 at X = 0 (u0 + r0 v0) and at X = 1 (u1 + r0 v1)
    double cu[MAXT], cv[MAXT], du[MAXT], dv[MAXT], u1[MAXT], v1[MAXT];
#pragma unroll
    for (int t = 0; t < MAXT; t++)
      if (t < d.T) {
        const uint4 e = ahead[0][t];
        cu[t] = (double)e.x, cv[t] = (double)e.y - cu[t], u1[t] = (double)e.z, v1[t] = (double)e.w - u1[t];
      }
    Ext<D> we = wahead[0];
#pragma unroll
    for (int a = 0; a + 1 < PREFETCH; a++) {
#pragma unroll
      for (int t = 0; t < MAXT; t++)
        if (t < d.T) ahead[a][t] = ahead[a + 1][t];
      wahead[a] = wahead[a + 1];
    }
    fetch(k + PREFETCH, ahead[PREFETCH - 1], wahead[PREFETCH - 1]);
#pragma unroll
    for (int v = 0; v < MAXV; v++)
      if (v < d.NV) {  // a linear form of the tables: the same combination of the lines
        double a0 = (double)d.vconst[v], b0 = 0, a1 = a0, b1 = 0;
#pragma unroll
        for (int q = 0; q < MAXVT; q++)
          if (q < d.vn[v]) {
            const int t = d.vtab[v][q];
            a0 += f_scale(cu[t], d.vcoef[v][q]), b0 += f_scale(cv[t], d.vcoef[v][q]);
            a1 += f_scale(u1[t], d.vcoef[v][q]), b1 += f_scale(v1[t], d.vcoef[v][q]);
          }
        cu[d.T + v] = a0, cv[d.T + v] = b0, u1[d.T + v] = a1, v1[d.T + v] = b1;
      }
#pragma unroll
    for (int t = 0; t < MAXT; t++)
      if (t < d.T + d.NV) du[t] = u1[t] - cu[t], dv[t] = v1[t] - cv[t];
    if (!args.deferred) we = ext_mul_mont<D>(we, load_ext<D>(args.high + (i >> args.low_bits) * D));

    int slot = 0;  // numbered group by group (point by point, node by node, then the extras) -- visited X1-major
#pragma unroll
    for (int x = 0; x <= MAXX; x++) {
      if (x <= d.maxx || x == 1) {
        if (x >= 1) {
#pragma unroll
          for (int t = 0; t < MAXT; t++)
            if (t < d.T + d.NV) {
              if (x == 1)
                cu[t] = u1[t], cv[t] = v1[t];
              else
                cu[t] += du[t], cv[t] += dv[t];
            }
        }
        int base = 0;  // first slot of group g
#pragma unroll
        for (int g = 0; g < MAXG; g++) {
          if (g < d.G) {
            const int e = ev_index(d, g, x);  // an evaluation point's row, or at X1 = 1 the row of extras
            if (e >= 0 || x == 1) {
              double val[MAXDEG];
#pragma unroll
              for (int j = 0; j < MAXDEG; j++)
                if (j < d.deg[g]) val[j] = cu[d.tab[g][j]];
#pragma unroll
              for (int m = 0; m <= MAXDEG; m++) {
                if (m <= d.deg[g]) {
                  if (e >= 0)
                    slot = base + e * (d.deg[g] + 1) + m;
                  else  // only the nodes that are evaluation points
                    slot = ev_index(d, g, m) < 0 ? -1 : base + d.nev[g] * (d.deg[g] + 1) + ev_index(d, g, m);
                  if (slot >= PASS * SPP && slot < (PASS + 1) * SPP) {
                    double prod = val[0];
#pragma unroll
                    for (int j = 1; j < MAXDEG; j++)
                      if (j < d.deg[g]) prod = f_mul(prod, val[j]);
                    if (d.deg[g] == 1) prod = f_reduce(prod);
                    const uint32_t pv = f_residue32(prod);
#pragma unroll
                    for (int c = 0; c < D; c++) lazy_mad(acc[slot - PASS * SPP][c], we.c[c], pv);
                  }
#pragma unroll
                  for (int j = 0; j < MAXDEG; j++)
                    if (j < d.deg[g]) val[j] += cv[d.tab[g][j]];
                }
              }
            }
            base += group_slots(d, g);
          }
        }
      }
    }
    (void)slot;
  }

  // the workgroup's sums of this launch's slots, HIGH applied once when deferred
  constexpr int WORDS = SPP * D, CHUNKS = (WORDS + 31) / 32;
  __shared__ uint32_t lds[BLOCK / 64][CHUNKS * 32];
  __shared__ NodesEpilogueLds<D> L;
  const uint32_t lane = tid & 63, wave = tid >> 6;
  nodes_epilogue_stage<D>(args.epi, L);  // (the loads' trip hides behind the reduction below)
  {  // the wavefront's sums, 32 words at a time by the transposing reduction
    uint32_t idx = 0;
#pragma unroll
    for (int b = 0; b < 5; b++) idx |= ((lane >> b) & 1u) << (4 - b);
#pragma unroll
    for (int first = 0; first < WORDS; first += 32) {
      const uint32_t total = wave_sums_transposed<32>([&](int k) -> uint32_t {
        const int o = first + k;
        return o < WORDS ? lazy_reduce(acc[o / D][o % D]) : 0u;
      });
      if (lane < 32) lds[wave][first + idx] = total;
    }
  }
  __syncthreads();
  const int total = node_slots(d);
  const bool mine = tid < SPP && PASS * SPP + (int)tid < total;
  Ext<D> sum = ext_zero<D>();
  if (mine) {
    // The sums above are of w * (the plain product of the group's factors); the integer kernels' products
    // carry 1/R per multiplication, which the epilogue's constants expect: times R^(1 - degree) here.
    int base = 0, deg = 1;
    for (int g = 0; g < d.G; g++) {
      if (PASS * SPP + (int)tid >= base) deg = d.deg[g];
      base += group_slots(d, g);
    }
    uint32_t fix = R1;  // mont_mul(v, fix) = v R^(1 - degree)
    for (int q = 1; q < deg; q++) fix = mont_mul(fix, 1u);
#pragma unroll
    for (int c = 0; c < D; c++) {
      uint32_t v = lds[0][tid * D + c];
#pragma unroll
      for (int wv = 1; wv < BLOCK / 64; wv++) v = fadd(v, lds[wv][tid * D + c]);
      sum.c[c] = mont_mul(v, fix);
    }
    if (args.deferred) sum = ext_mul_mont<D>(sum, load_ext<D>(args.high + (tile_start >> args.low_bits) * D));
  }
  // the slot sums of all workgroups and passes, and in the last workgroup of the last pass both rounds' epilogue
  if (mine) {
#pragma unroll
    for (int c = 0; c < D; c++) L.sums[(PASS * SPP + tid) * D + c] = sum.c[c];
  }
  __syncthreads();
  const int here = total - PASS * SPP < SPP ? total - PASS * SPP : SPP;  // slots of this pass
  bool ok;
  if (!add_and_elect(args.totals, L.sums, (uint32_t)total * D, L.epi.prod, L.slot_sums, &ok, (uint32_t)(PASS * SPP * D),
                     (uint32_t)(here > 0 ? here : 0) * D, args.passes * gridDim.x - 1, gridDim.x))
    return;
  if (!ok) {
    if (tid == 0) __hip_atomic_store(&args.epi.e.ctrl->gave_up, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return;
  }
  nodes_epilogue_body<D>(args.epi, L);
}

// a kernel generated for one statement: S::d is its descriptor, known at compile time
template <int D, bool IN_BASE, bool FOLD, class S>
__global__ __launch_bounds__(BLOCK) __attribute__((amdgpu_waves_per_eu(2, 2))) void round_kernel(RoundArgs<D> args) {
  round_body<D, IN_BASE, FOLD, decltype(S::d), false, true>(S::d, args);
}
template <int D, class S>
__global__ __launch_bounds__(BLOCK) __attribute__((amdgpu_waves_per_eu(1, 1))) void tail_kernel(TailArgs<D> args) {
  tail_body<D>(S::d, args);
}
// (the same with half the registers: a statement in direct form at F_p^8 needs more than the 512 either way, and the
// compiler's use of the upper half of the register file for 64-bit values that it also spills has been seen to end
// in registers it then rejects)
template <int D, class S>
__global__ __launch_bounds__(BLOCK) __attribute__((amdgpu_waves_per_eu(2, 2))) void tail_kernel_narrow(TailArgs<D> args) {
  tail_body<D>(S::d, args);
}
template <int D, class S>
__global__ __launch_bounds__(BLOCK) __attribute__((amdgpu_waves_per_eu(2, 2))) void round_kernel_fold2(RoundArgs<D> args) {
  round_body<D, true, true, decltype(S::d), true, true>(S::d, args);
}
template <int D, class S, int PASS, int SPP>
__global__ __launch_bounds__(BLOCK) void nodes_kernel(NodesArgs<D> args) {
  nodes_body<D, PASS, SPP>(S::d, args);
}

// the interpreter: the same bodies over a run-time descriptor
template <int D, bool IN_BASE, bool FOLD>
__global__ __launch_bounds__(BLOCK) void round_kernel_interp(RoundArgs<D> args, StmtDesc d) {
  round_body<D, IN_BASE, FOLD>(d, args);
}
template <int D>
__global__ __launch_bounds__(BLOCK) void tail_kernel_interp(TailArgs<D> args, StmtDesc d) {
  tail_body<D>(d, args);
}

}  // namespace exh
