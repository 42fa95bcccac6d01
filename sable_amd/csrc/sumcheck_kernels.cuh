// sumcheck_kernels.cuh -- the sumcheck prover's round kernel for gfx950, generated per statement.
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
#include <hip/hip_runtime.h>

#include <type_traits>

#include "field.cuh"
#include "stmtdesc.hpp"

namespace exh {

// StmtDesc and the limits MAXT, MAXG, ... come from stmtdesc.hpp
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
  uint32_t r_mont[D];        // the fold challenge, times R
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
  return ext_add<D>(lo, ext_mul_mont<D>(r_mont, ext_sub<D>(hi, lo)));
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
__device__ __forceinline__ void v_weigh(Acc96 *acc, const Ext<D> &w, const Ext<D> &v) { ext_mul_acc<D>(acc, w, v); }

template <int D, class V, class Desc>
__device__ __forceinline__ void accumulate_pair(const Desc &d, const V *lo, const V *hi, const Ext<D> &w,
                                                Acc96 (*acc)[D]) {
  V cur[MAXT], slope[MAXT];
#pragma unroll
  for (int t = 0; t < MAXT; t++)
    if (t < d.T) {
      cur[t] = lo[t];
      slope[t] = v_sub<D>(hi[t], lo[t]);
    }
#pragma unroll
  for (int x = 0; x <= MAXX; x++) {
    if (x <= d.maxx) {
      if (x == 1) {
#pragma unroll
        for (int t = 0; t < MAXT; t++)
          if (t < d.T) cur[t] = hi[t];
      } else if (x >= 2) {
#pragma unroll
        for (int t = 0; t < MAXT; t++)
          if (t < d.T) cur[t] = v_add<D>(cur[t], slope[t]);
      }
      int a = 0;
#pragma unroll
      for (int g = 0; g < MAXG; g++) {
        if (g < d.G) {
#pragma unroll
          for (int k = 0; k < MAXEV; k++) {
            if (k < d.nev[g]) {
              if (d.ev[g][k] == x) {
                V prod = cur[d.tab[g][0]];
#pragma unroll
                for (int j = 1; j < MAXDEG; j++)
                  if (j < d.deg[g]) prod = v_mul<D>(prod, cur[d.tab[g][j]]);
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

// cross-lane sum of a canonical value over the 64 lanes of a wavefront
__device__ __forceinline__ uint32_t wave_sum(uint32_t v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fadd(v, (uint32_t)__shfl_xor((int)v, off, 64));
  return v;
}

template <int D, bool IN_BASE, bool FOLD, class Desc>
__device__ __forceinline__ void round_body(const Desc &d, const RoundArgs<D> &args) {
  constexpr bool BASE_MODE = IN_BASE && !FOLD;  // the pair's values are base-field
  using V = typename std::conditional<BASE_MODE, uint32_t, Ext<D>>::type;
  const uint32_t tid = threadIdx.x;
  const uint64_t tile = (uint64_t)BLOCK * args.pairs_per_thread;
  const uint64_t tile_start = (uint64_t)blockIdx.x * tile;
  const uint64_t low_mask = ((uint64_t)1 << args.low_bits) - 1;

  Acc96 acc[MAXACC][D];
#pragma unroll
  for (int a = 0; a < MAXACC; a++)
#pragma unroll
    for (int c = 0; c < D; c++) acc_zero(acc[a][c]);

  Ext<D> r;
  if constexpr (FOLD) {
#pragma unroll
    for (int c = 0; c < D; c++) r.c[c] = args.r_mont[c];
  }

  for (uint32_t k = 0; k < args.pairs_per_thread; k++) {
    const uint64_t i = tile_start + (uint64_t)k * BLOCK + tid;
    if (i >= args.n_pairs) break;
    V lo[MAXT], hi[MAXT];
#pragma unroll
    for (int t = 0; t < MAXT; t++) {
      if (t < d.T) {
        if constexpr (FOLD && IN_BASE) {
          uint4 e = *reinterpret_cast<const uint4 *>(args.in[t] + 4 * i);
          lo[t] = fold_base<D>(e.x, e.y, r);
          hi[t] = fold_base<D>(e.z, e.w, r);
        } else if constexpr (FOLD) {
          const uint32_t *p = args.in[t] + 4 * i * D;
          lo[t] = fold_ext<D>(load_ext<D>(p), load_ext<D>(p + D), r);
          hi[t] = fold_ext<D>(load_ext<D>(p + 2 * D), load_ext<D>(p + 3 * D), r);
        } else if constexpr (IN_BASE) {
          uint2 e = *reinterpret_cast<const uint2 *>(args.in[t] + 2 * i);
          lo[t] = e.x;
          hi[t] = e.y;
        } else {
          const uint32_t *p = args.in[t] + 2 * i * D;
          lo[t] = load_ext<D>(p);
          hi[t] = load_ext<D>(p + D);
        }
        if constexpr (FOLD) {
          store_ext<D>(args.out[t] + 2 * i * D, lo[t]);
          store_ext<D>(args.out[t] + (2 * i + 1) * D, hi[t]);
        }
      }
    }
    if (args.do_sums) {
      Ext<D> w = load_ext<D>(args.low + (i & low_mask) * D);
      if (!args.deferred) w = ext_mul_mont<D>(w, load_ext<D>(args.high + (i >> args.low_bits) * D));
      accumulate_pair<D, V>(d, lo, hi, w, acc);
    }
  }
  if (!args.do_sums) return;

  // reduce: thread -> wavefront -> workgroup
  __shared__ uint32_t lds[BLOCK / 64][MAXACC * D];
  const uint32_t lane = tid & 63, wave = tid >> 6;
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
  __syncthreads();
  if (tid < (uint32_t)d.nacc) {
    Ext<D> s;
#pragma unroll
    for (int c = 0; c < D; c++) {
      uint32_t v = lds[0][tid * D + c];
#pragma unroll
      for (int wv = 1; wv < BLOCK / 64; wv++) v = fadd(v, lds[wv][tid * D + c]);
      s.c[c] = v;
    }
    if (args.deferred) s = ext_mul_mont<D>(s, load_ext<D>(args.high + (tile_start >> args.low_bits) * D));
    store_ext<D>(args.partials + ((uint64_t)blockIdx.x * d.nacc + tid) * D, s);
  }
}

// a kernel generated for one statement: S::d is its descriptor, known at compile time
template <int D, bool IN_BASE, bool FOLD, class S>
__global__ __launch_bounds__(BLOCK) void round_kernel(RoundArgs<D> args) {
  round_body<D, IN_BASE, FOLD>(S::d, args);
}

// the interpreter: the same body over a run-time descriptor
template <int D, bool IN_BASE, bool FOLD>
__global__ __launch_bounds__(BLOCK) void round_kernel_interp(RoundArgs<D> args, StmtDesc d) {
  round_body<D, IN_BASE, FOLD>(d, args);
}

typedef void (*RoundLauncher)(const void *args, int D, bool in_base, bool fold, uint32_t grid, hipStream_t stream);

}  // namespace exh
