// commit.hip -- see commit.hpp.
#include "commit.hpp"

#include <array>

#include <string.h>

#include <algorithm>
#include <atomic>
#include <map>
#include <vector>

#include "blake3.hpp"
#include "context.hpp"
#include "hostfield.hpp"
#include "sumcheck.hpp"
#include "sumcheck_kernels.hpp"

namespace exh {

// ------------------------------------------------------------------ twiddle tables of a domain
// Level l of the 2^n tables (src/rs.lisp:44-55) holds x_s = w_n^(2^l bitrev_{n-1-l}(s)) for the
// 2^(n-1-l) position pairs of the level-l codeword.  Both x (for the encoder's butterflies) and
// 1/(2x) (for folding) are kept on the device, levels concatenated: x as the plain residue, 1/(2x) in Montgomery form.
struct Domain {
  int n = 0;
  uint32_t *tw = nullptr, *tw_inv2 = nullptr;
  uint64_t off[32];
};
static std::map<int, Domain> g_domains;

struct LevelOffsets {
  uint64_t off[32];
  int levels, n;
};

__device__ __forceinline__ uint32_t bitrev_dev(uint32_t v, int bits) { return bits ? __brev(v) >> (32 - bits) : 0; }

// pw: w_n^e for e < 4096, then w_n^(4096 e) for e < 4096 (Montgomery form); pw_inv the same for
// the inverse root times 1/2 folded into the first table
__global__ __launch_bounds__(BLOCK) void twiddle_kernel(LevelOffsets lv, const uint32_t *pw, const uint32_t *pw_inv,
                                                        uint32_t *tw, uint32_t *tw_inv2, uint64_t total) {
  uint64_t gid = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
  if (gid >= total) return;
  int l = 0;
  while (l + 1 < lv.levels && gid >= lv.off[l + 1]) l++;
  uint32_t s = (uint32_t)(gid - lv.off[l]);
  uint32_t e = bitrev_dev(s, lv.n - 1 - l) << l;  // exponent of w_n, below 2^(n-1)
  // mont_mul of two Montgomery-form values is the Montgomery form of the product
  // (the encoder multiplies in double precision and takes the plain residue, the fold the Montgomery form)
  tw[gid] = mont_mul(mont_mul(pw[e & 4095], pw[4096 + (e >> 12)]), 1);
  tw_inv2[gid] = mont_mul(pw_inv[e & 4095], pw_inv[4096 + (e >> 12)]);
}

static int get_domain(int n, Domain **out) {
  auto it = g_domains.find(n);
  if (it != g_domains.end()) {
    *out = &it->second;
    return OK;
  }
  Context &c = ctx();
  Domain d;
  d.n = n;
  int levels = n - 1 > 1 ? n - 1 : 1;
  uint64_t total = 0, len = (uint64_t)1 << (n - 1);
  LevelOffsets lv;
  memset(&lv, 0, sizeof(lv));
  for (int l = 0; l < levels; l++, len /= 2) {
    d.off[l] = lv.off[l] = total;
    total += len;
  }
  lv.levels = levels;
  lv.n = n;
  uint32_t w = fpow(3, (uint64_t)(P - 1) >> n), winv = finv(w);
  std::vector<uint32_t> pw(8192), pwi(8192);
  uint32_t x = 1, xi = INV2;  // the 1/2 of 1/(2x) rides on the low table
  for (int e = 0; e < 4096; e++) {
    pw[e] = to_mont(x), pwi[e] = to_mont(xi);
    x = fmul(x, w), xi = fmul(xi, winv);
  }
  uint32_t w4096 = fpow(w, 4096), wi4096 = fpow(winv, 4096);
  x = 1, xi = 1;
  for (int e = 0; e < 4096; e++) {
    pw[4096 + e] = to_mont(x), pwi[4096 + e] = to_mont(xi);
    x = fmul(x, w4096), xi = fmul(xi, wi4096);
  }
  uint32_t *d_pw = nullptr;
  EXH_HIP(hipMalloc((void **)&d_pw, 2 * 8192 * 4));
  EXH_HIP(hipMemcpy(d_pw, pw.data(), 8192 * 4, hipMemcpyHostToDevice));
  EXH_HIP(hipMemcpy(d_pw + 8192, pwi.data(), 8192 * 4, hipMemcpyHostToDevice));
  EXH_HIP(hipMalloc((void **)&d.tw, total * 4));
  EXH_HIP(hipMalloc((void **)&d.tw_inv2, total * 4));
  uint32_t grid = (uint32_t)((total + BLOCK - 1) / BLOCK);
  hipLaunchKernelGGL(twiddle_kernel, dim3(grid), dim3(BLOCK), 0, c.stream, lv, d_pw, d_pw + 8192, d.tw, d.tw_inv2,
                     total);
  EXH_HIP(hipGetLastError());
  EXH_HIP(hipStreamSynchronize(c.stream));
  EXH_HIP(hipFree(d_pw));
  g_domains[n] = d;
  *out = &g_domains[n];
  return OK;
}

// ------------------------------------------------------------------ the encoder
// One pass of the butterflies (src/rs.lisp:60-73) for the stages b = b_hi .. b_lo over tiles held
// in LDS.  An index is (top | mid | low) with mid the bits b_lo..b_hi; a workgroup takes one top,
// all 2^S mids and C consecutive lows (C = tile / 2^S), so its loads are segments of C words and
// every butterfly of these stages stays inside the tile.  With `first` the input is the message
// m, read as m || m (src/rs.lisp:81).
//
// Inside the tile the stages run four at a time in registers: a thread gathers the 16 elements that
// differ in the four stage bits, does the 32 butterflies, and scatters them back, so LDS and the
// workgroup barrier are touched once per four stages.  The tile is padded by one element per 16 so that
// the strided gathers fall on distinct banks.
// A tile is 2^12 elements, 16 per thread: a domain of 2^24 takes three passes (6 + 5 + 12 stages) with
// global segments of at least 64 words.
// The butterflies run in double precision (field.hpp), eight instructions each where Montgomery arithmetic takes
// about twenty (the multiplies issue at the same rate either way): a product by a twiddle is six operations and
// leaves a residue within about p/2 of zero, and the sum and the difference that follow are one operation each
// with no reduction, exact as long as the values stay integers below 2^53: a tile's elements start below p and
// grow by less than 0.57 p per stage, so after a pass's twelve stages at most they are below 8 p, and a product
// with a twiddle below 2^65.  The tile in LDS therefore holds doubles; a pass ends by writing canonical residues.
// The passes are bound by their instructions all the same (some 330 per thread and round of four stages, the
// vector units busy nine tenths of the time): both columns of 2^24 take 64 + 56 + 92 us, against 300 us with
// Montgomery products and the tile fetched word by word.
constexpr int NTT_TILE_BITS = 12;
constexpr int NTT_BLOCK = 256;
constexpr int NTT_MAX_UPPER_STAGES = 7;  // per pass above the last: segments of 2^(12-7) words at least
static_assert(NTT_TILE_BITS <= 12, "a pass's stages, the bound on the lazily reduced values");
static_assert((1 << NTT_TILE_BITS) == 16 * NTT_BLOCK, "a thread moves a whole tile's sixteen words as four vectors");
__device__ __forceinline__ uint32_t ntt_pad(uint32_t e) { return e + (e >> 4); }
constexpr uint32_t ntt_lds_bytes(int tile_bits) {
  return (((uint32_t)1 << tile_bits) + ((uint32_t)1 << tile_bits >> 4) + 1) * 8;
}

// R stages d_lo .. d_lo + R - 1 of the pass (stage d pairs tile indices differing in bit cbits + d).  A thread
// takes groups of 2^R elements, its number of groups known at compile time for a FULL tile (2^NTT_TILE_BITS): the
// twiddles of all its groups are then fetched before the first butterfly, one wait for memory per round where a
// loop over the groups has one per group.  (Deriving a group's 2^R - 1 twiddles from one table entry, by squarings
// and products with fixed roots of unity, was measured: the passes are bound by their instructions, and fourteen
// more products per thirty-two butterflies cost more than the fetches.)
template <int R, bool FULL>
__device__ __forceinline__ void ntt_round(double *lds, uint32_t tile, int cbits, int d_lo, int b_lo, int b_hi,
                                          uint64_t top, const uint32_t *__restrict__ tw, const LevelOffsets &lv) {
  constexpr int GROUPS = FULL ? ((1 << NTT_TILE_BITS) >> R) / NTT_BLOCK : 1;
  const int p = cbits + d_lo;
  // a FULL tile's rounds have p = 0 or p >= 4 (a pass above the last keeps 2^cbits >= 32 consecutive indices, the
  // last one runs its twelve stages four at a time): a group's padded positions are then evenly spaced
  const uint32_t spacing = (1u << p) + ((1u << p) >> 4);
  for (uint32_t g0 = threadIdx.x; g0 < (tile >> R); g0 += GROUPS * NTT_BLOCK) {
    uint32_t t[GROUPS][(1 << R) - 1];
    // the twiddles of stage d_lo + s: 2^(R-1-s) of them, index (top | mid above the stage bit)
#pragma unroll
    for (int it = 0; it < GROUPS; it++) {
      const uint32_t upper = (g0 + it * NTT_BLOCK) >> p;
#pragma unroll
      for (int s = R - 1; s >= 0; s--) {
        const int b = b_lo + d_lo + s;
        const uint32_t *level = tw + lv.off[b] + ((top << (b_hi - b)) | ((uint64_t)upper << (R - 1 - s)));
#pragma unroll
        for (int jh = 0; jh < (1 << (R - 1 - s)); jh++) t[it][(1 << (R - 1 - s)) - 1 + jh] = level[jh];
      }
    }
#pragma unroll
    for (int it = 0; it < GROUPS; it++) {
      const uint32_t g = g0 + it * NTT_BLOCK, upper = g >> p, e_base = (upper << (p + R)) | (g & ((1u << p) - 1));
      double *const group = lds + ntt_pad(e_base);
      auto at = [&](int j) -> double & { return FULL ? group[j * spacing] : lds[ntt_pad(e_base | ((uint32_t)j << p))]; };
      double v[1 << R];
#pragma unroll
      for (int j = 0; j < (1 << R); j++) v[j] = at(j);
#pragma unroll
      for (int s = R - 1; s >= 0; s--) {
#pragma unroll
        for (int jh = 0; jh < (1 << (R - 1 - s)); jh++) {
          const double x = (double)t[it][(1 << (R - 1 - s)) - 1 + jh];
#pragma unroll
          for (int jl = 0; jl < (1 << s); jl++) {
            const int j = (jh << (s + 1)) | jl;
            const double a = v[j], tc = f_mul(x, v[j + (1 << s)]);
            v[j] = a + tc;
            v[j + (1 << s)] = a - tc;
          }
        }
      }
#pragma unroll
      for (int j = 0; j < (1 << R); j++) at(j) = v[j];
    }
  }
}

// FULL: the tile is 2^NTT_TILE_BITS words and `in`, `out` and the columns' strides are multiples of 16 bytes: a
// thread moves its sixteen words as four vectors of four consecutive ones (a segment of consecutive indices is a
// multiple of four long, or the tile is one segment), all four fetches in flight at once.
template <bool FULL>
__global__ __launch_bounds__(NTT_BLOCK) __attribute__((amdgpu_waves_per_eu(5, 8))) void ntt_pass_kernel(
    const uint32_t *in, uint32_t *out, int n, int b_hi, int b_lo, int tile_bits,
    const uint32_t *__restrict__ tw, LevelOffsets lv, int first, uint64_t in_stride, uint64_t out_stride) {
  extern __shared__ double lds[];  // 2^tile_bits elements plus one per 16
  const int S = b_hi - b_lo + 1, cbits = tile_bits - S;
  const uint32_t tile = 1u << tile_bits, C = 1u << cbits;
  in += (uint64_t)blockIdx.y * in_stride;
  out += (uint64_t)blockIdx.y * out_stride;
  const uint64_t chunks_per_top = ((uint64_t)1 << b_lo) >> cbits;
  const uint64_t top = blockIdx.x / chunks_per_top, chunk = blockIdx.x % chunks_per_top;
  const uint64_t base = (top << (b_hi + 1)) | (chunk << cbits);
  const uint64_t msg_mask = ((uint64_t)1 << (n - 1)) - 1;
  auto global_index = [&](uint32_t e) { return base | ((uint64_t)(e >> cbits) << b_lo) | (e & (C - 1)); };
  if (FULL) {
    uint4 w[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const uint64_t g = global_index(4 * (threadIdx.x + k * NTT_BLOCK));
      w[k] = *reinterpret_cast<const uint4 *>(in + (first ? g & msg_mask : g));
    }
#pragma unroll
    for (int k = 0; k < 4; k++) {
      double *at = lds + ntt_pad(4 * (threadIdx.x + k * NTT_BLOCK));  // (four elements never straddle a pad)
      at[0] = (double)w[k].x, at[1] = (double)w[k].y, at[2] = (double)w[k].z, at[3] = (double)w[k].w;
    }
  } else {
    for (uint32_t e = threadIdx.x; e < tile; e += NTT_BLOCK) {
      const uint64_t g = global_index(e);
      lds[ntt_pad(e)] = (double)(first ? in[g & msg_mask] : in[g]);
    }
  }
  __syncthreads();
  for (int d_hi = S - 1; d_hi >= 0;) {
    const int R = d_hi + 1 < 4 ? d_hi + 1 : 4, d_lo = d_hi - R + 1;
    if (R == 4)
      ntt_round<4, FULL>(lds, tile, cbits, d_lo, b_lo, b_hi, top, tw, lv);
    else if (R == 3)
      ntt_round<3, FULL>(lds, tile, cbits, d_lo, b_lo, b_hi, top, tw, lv);
    else if (R == 2)
      ntt_round<2, FULL>(lds, tile, cbits, d_lo, b_lo, b_hi, top, tw, lv);
    else
      ntt_round<1, FULL>(lds, tile, cbits, d_lo, b_lo, b_hi, top, tw, lv);
    __syncthreads();
    d_hi = d_lo - 1;
  }
  if (FULL) {
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const uint32_t e = 4 * (threadIdx.x + k * NTT_BLOCK);
      const double *at = lds + ntt_pad(e);
      *reinterpret_cast<uint4 *>(out + global_index(e)) =
          make_uint4(f_canonical(at[0]), f_canonical(at[1]), f_canonical(at[2]), f_canonical(at[3]));
    }
  } else {
    for (uint32_t e = threadIdx.x; e < tile; e += NTT_BLOCK) out[global_index(e)] = f_canonical(lds[ntt_pad(e)]);
  }
}

// m || m for the degenerate domains with no butterfly stage
__global__ void dup_kernel(const uint32_t *in, uint32_t *out, uint64_t half, uint64_t in_stride, uint64_t out_stride) {
  uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid < 2 * half) out[blockIdx.y * out_stride + gid] = in[blockIdx.y * in_stride + (gid % half)];
}

int rs_encode_columns(const uint32_t *d_messages, int ncols, int c, uint32_t *d_codewords) {
  Context &cx = ctx();
  int status = cx.require();
  if (status) return status;
  int n = c + 1;
  uint64_t len = (uint64_t)1 << n;
  if (n < 2) {
    hipLaunchKernelGGL(dup_kernel, dim3(1, ncols), dim3(64), 0, cx.stream, d_messages, d_codewords, len / 2, len / 2, len);
    EXH_HIP(hipGetLastError());
    return OK;
  }
  Domain *dom;
  if ((status = get_domain(n, &dom))) return status;
  LevelOffsets lv;
  memset(&lv, 0, sizeof(lv));
  lv.levels = n - 1, lv.n = n;
  for (int l = 0; l < n - 1; l++) lv.off[l] = dom->off[l];
  int tile_bits = n - 1 < NTT_TILE_BITS ? n - 1 : NTT_TILE_BITS;  // a tile never spans two tops
  const uint32_t lds_bytes = ntt_lds_bytes(tile_bits);
  // whole tiles whose words move four at a time: every address and stride a multiple of 16 bytes, segments of
  // consecutive indices at least four long (a pass above the last has 2^(tile_bits - stages) >= 32 of them)
  const bool full = tile_bits == NTT_TILE_BITS && (reinterpret_cast<uintptr_t>(d_messages) & 15) == 0 &&
                    (reinterpret_cast<uintptr_t>(d_codewords) & 15) == 0;
  static_assert(NTT_TILE_BITS - NTT_MAX_UPPER_STAGES >= 2, "segments of four words at least");
  // stages n-2 .. 0: the last pass takes the low tile_bits stages, earlier passes share the rest
  int b = n - 2;
  bool first = true;
  while (b >= 0) {
    int b_lo;
    if (b < tile_bits)
      b_lo = 0;
    else {
      int remaining = b - tile_bits + 1;  // stages above the last pass
      int take = remaining > NTT_MAX_UPPER_STAGES
                     ? (remaining > 2 * NTT_MAX_UPPER_STAGES ? NTT_MAX_UPPER_STAGES : (remaining + 1) / 2)
                     : remaining;
      b_lo = b - take + 1;
    }
    uint32_t grid = (uint32_t)(len >> tile_bits);
    hipLaunchKernelGGL(full ? ntt_pass_kernel<true> : ntt_pass_kernel<false>, dim3(grid, ncols), dim3(NTT_BLOCK),
                       lds_bytes, cx.stream, first ? d_messages : d_codewords, d_codewords, n, b, b_lo, tile_bits,
                       dom->tw, lv, first ? 1 : 0, first ? len / 2 : len, len);
    first = false;
    b = b_lo - 1;
  }
  EXH_HIP(hipGetLastError());
  return OK;
}

// ------------------------------------------------------------------ codeword folding
// pair (a, b) at twiddle x: f0 = (a + b)/2, f1 = (a - b)/(2x), out = f0 + r (f1 - f0)
template <int D>
__global__ __launch_bounds__(BLOCK) void rs_fold_kernel(const uint32_t *cw, const uint32_t *tw_inv2, uint32_t *out,
                                                        uint64_t m, RoundArgs<D> args) {
  uint64_t s = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
  if (s >= m) return;
  Ext<D> r;
#pragma unroll
  for (int c = 0; c < D; c++) r.c[c] = args.r_mont[c];
  Ext<D> a = load_ext<D>(cw + 2 * s * D), b = load_ext<D>(cw + (2 * s + 1) * D);
  Ext<D> f0 = ext_scale_mont<D>(ext_add<D>(a, b), mont_mul(INV2, R2));
  Ext<D> f1 = ext_scale_mont<D>(ext_sub<D>(a, b), tw_inv2[s]);
  store_ext<D>(out + s * D, ext_add<D>(f0, ext_mul_mont<D>(r, ext_sub<D>(f1, f0))));
}

static int rs_fold_launch(int D, uint64_t m, const uint32_t *tw_inv2_level, const uint32_t *d_cw, const uint32_t *r,
                          uint32_t *d_out) {
  Context &c = ctx();
  uint32_t grid = (uint32_t)((m + BLOCK - 1) / BLOCK);
  if (D == 4) {
    RoundArgs<4> a;
    memset(&a, 0, sizeof(a));
    for (int k = 0; k < 4; k++) a.r_mont[k] = to_mont(r[k] % P);
    hipLaunchKernelGGL(rs_fold_kernel<4>, dim3(grid), dim3(BLOCK), 0, c.stream, d_cw, tw_inv2_level, d_out, m, a);
  } else {
    RoundArgs<8> a;
    memset(&a, 0, sizeof(a));
    for (int k = 0; k < 8; k++) a.r_mont[k] = to_mont(r[k] % P);
    hipLaunchKernelGGL(rs_fold_kernel<8>, dim3(grid), dim3(BLOCK), 0, c.stream, d_cw, tw_inv2_level, d_out, m, a);
  }
  EXH_HIP(hipGetLastError());
  return OK;
}

int rs_fold_device(int D, uint64_t m, int n_domain, int level, const uint32_t *d_cw, const uint32_t *r, uint32_t *d_out) {
  int status = ctx().require();
  if (status) return status;
  Domain *dom;
  if ((status = get_domain(n_domain, &dom))) return status;
  return rs_fold_launch(D, m, dom->tw_inv2 + dom->off[level], d_cw, r, d_out);
}

// ------------------------------------------------------------------ COMBINE-COLUMNS (src/pcs.lisp:434-441)
// g[x] = sum_k coefficient_k * column_k[x]: base columns (column k at cols + k * len), extension coefficients,
// the table BaseFold opens.  One pass: 4 ncols bytes read and 4 D written per x, one x per thread (four per
// thread measured a third slower: the 128-byte strides between lanes' stores).  The coefficients arrive as
// kernel arguments in Montgomery form, so a reduction of four products gives their exact sum.
constexpr int COMBINE_COLS = 32;  // columns whose coefficients travel as kernel arguments; more take the other kernel
template <int D>
struct CombineArgs {
  uint32_t coef_mont[COMBINE_COLS][D];
};
template <int D>
__global__ __launch_bounds__(BLOCK) void combine_columns_kernel(const uint32_t *cols, uint64_t len, int ncols,
                                                                CombineArgs<D> a, uint32_t *out, int accumulate) {
  const uint64_t x = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
  if (x >= len) return;
  Ext<D> g = accumulate ? load_ext<D>(out + x * D) : ext_zero<D>();
  for (int k0 = 0; k0 < ncols; k0 += 4) {  // four columns per reduction: 4 p^2 < 2^64
    uint32_t val[4];
#pragma unroll
    for (int q = 0; q < 4; q++) val[q] = k0 + q < ncols ? cols[(uint64_t)(k0 + q) * len + x] : 0u;
#pragma unroll
    for (int c = 0; c < D; c++) {
      uint64_t t = 0;
#pragma unroll
      for (int q = 0; q < 4; q++) t += (uint64_t)(k0 + q < ncols ? a.coef_mont[k0 + q][c] : 0u) * val[q];
      g.c[c] = fadd(g.c[c], mont_reduce4(t));
    }
  }
  store_ext<D>(out + x * D, g);  // (non-temporal stores measured a third slower)
}

// The same sum for many columns in one pass: the output stays in registers across all of them instead of being
// read and written again every 32 columns.  The coefficients (Montgomery form, padded with zeros to a multiple of
// eight columns) come from device memory at addresses every lane shares, eight columns' loads are in flight at
// once, and a lane walks the columns at its own x.
template <int D>
__global__ __launch_bounds__(BLOCK) void combine_columns_many_kernel(const uint32_t *__restrict__ cols, uint64_t len,
                                                                     int ncols, const uint32_t *__restrict__ coef_mont,
                                                                     uint32_t *__restrict__ out) {
  const uint64_t x = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
  if (x >= len) return;
  Ext<D> g = ext_zero<D>();
  for (int k0 = 0; k0 < ncols; k0 += 8) {
    uint32_t val[8];
#pragma unroll
    for (int q = 0; q < 8; q++) {  // a column past the last is read again with a zero coefficient
      const int k = k0 + q < ncols ? k0 + q : ncols - 1;
      val[q] = cols[(uint64_t)k * len + x];
    }
#pragma unroll
    for (int half = 0; half < 2; half++) {  // four columns per reduction: 4 p^2 < 2^64
      const uint32_t *cf = coef_mont + (size_t)(k0 + 4 * half) * D;
#pragma unroll
      for (int c = 0; c < D; c++) {
        uint64_t t = 0;
#pragma unroll
        for (int q = 0; q < 4; q++) t += (uint64_t)cf[q * D + c] * val[4 * half + q];
        g.c[c] = fadd(g.c[c], mont_reduce4(t));
      }
    }
  }
  store_ext<D>(out + x * D, g);
}

template <int D>
static int combine_many_launch(const uint32_t *d_cols, int ncols, uint64_t len, const uint32_t *coef, uint32_t *d_out) {
  Context &c = ctx();
  const int padded = (ncols + 7) / 8 * 8;
  std::vector<uint32_t> cm((size_t)padded * D, 0u);
  for (size_t i = 0; i < (size_t)ncols * D; i++) cm[i] = to_mont(coef[i] % P);
  uint32_t *d_coef = (uint32_t *)c.pool.alloc(cm.size() * 4);
  if (!d_coef) {
    set_error("device-out-of-memory: combine-columns coefficients");
    return E_NOMEM;
  }
  struct Release {
    Pool &pool;
    void *ptr;
    ~Release() { pool.release(ptr); }
  } release{c.pool, d_coef};
  // (from pageable memory: the call returns once the words are staged, so `cm` may go)
  EXH_HIP(hipMemcpyAsync(d_coef, cm.data(), cm.size() * 4, hipMemcpyHostToDevice, c.stream));
  uint32_t grid = (uint32_t)((len + BLOCK - 1) / BLOCK);
  hipLaunchKernelGGL((combine_columns_many_kernel<D>), dim3(grid), dim3(BLOCK), 0, c.stream, d_cols, len, ncols, d_coef,
                     d_out);
  EXH_HIP(hipGetLastError());
  return OK;
}

template <int D>
static int combine_launch(const uint32_t *d_cols, int ncols, uint64_t len, const uint32_t *coef, uint32_t *d_out) {
  Context &c = ctx();
  if (ncols > COMBINE_COLS) return combine_many_launch<D>(d_cols, ncols, len, coef, d_out);
  for (int first = 0; first < ncols; first += COMBINE_COLS) {
    const int count = ncols - first < COMBINE_COLS ? ncols - first : COMBINE_COLS;
    CombineArgs<D> a;
    memset(&a, 0, sizeof(a));
    for (int k = 0; k < count; k++)
      for (int cc = 0; cc < D; cc++) a.coef_mont[k][cc] = to_mont(coef[(size_t)(first + k) * D + cc] % P);
    const uint32_t *cols = d_cols + (uint64_t)first * len;
    uint32_t grid = (uint32_t)((len + BLOCK - 1) / BLOCK);
    hipLaunchKernelGGL((combine_columns_kernel<D>), dim3(grid), dim3(BLOCK), 0, c.stream, cols, len, count, a, d_out,
                       first > 0 ? 1 : 0);
  }
  EXH_HIP(hipGetLastError());
  return OK;
}

int combine_columns_device(int D, const uint32_t *d_cols, int ncols, uint64_t len, const uint32_t *coef,
                           uint32_t *d_out) {
  int status = ctx().require();
  if (status) return status;
  ctx().prof_begin("combine_columns", 0, len * (4 * (uint64_t)ncols + 4 * (uint64_t)D));
  status = D == 4 ? combine_launch<4>(d_cols, ncols, len, coef, d_out) : combine_launch<8>(d_cols, ncols, len, coef, d_out);
  ctx().prof_end();
  return status;
}

// ------------------------------------------------------------------ Merkle trees
// LEAF-DIGEST (src/pcs.lisp:44-52) of leaf l of ncols codewords: one row of 4 symbols per column,
// rows hashed 64 at a time and chained h = BLAKE3(h || d).
__device__ __forceinline__ void column_leaf_digest(const uint32_t *cw, int ncols, uint64_t cw_len, uint64_t l,
                                                   uint32_t h[8]) {
  uint32_t d[8], m[16];
  bool have = false;
  for (int start = 0; start < ncols; start += 64) {
    int rows = ncols - start < 64 ? ncols - start : 64;
    int nblocks = (rows + 3) / 4;
    b3_iv(d);
    for (int b = 0; b < nblocks; b++) {
      int have_rows = rows - 4 * b < 4 ? rows - 4 * b : 4;
#pragma unroll
      for (int k = 0; k < 4; k++) {
        uint4 v = make_uint4(0, 0, 0, 0);
        if (k < have_rows) v = *reinterpret_cast<const uint4 *>(cw + (uint64_t)(start + 4 * b + k) * cw_len + 4 * l);
        m[4 * k] = v.x, m[4 * k + 1] = v.y, m[4 * k + 2] = v.z, m[4 * k + 3] = v.w;
      }
      uint32_t flags = (b == 0 ? B3_CHUNK_START : 0u) | (b == nblocks - 1 ? (B3_CHUNK_END | B3_ROOT) : 0u);
      b3_compress(d, m, 0, (uint32_t)(16 * have_rows), flags, d, 0);
    }
    if (have)
      b3_node(h, d, h);
    else {
#pragma unroll
      for (int i = 0; i < 8; i++) h[i] = d[i];
      have = true;
    }
  }
}

// leaf l of an oracle codeword of EXT8s: one row per coordinate, symbols 4l..4l+3
// (ORACLE-ROWS, src/pcs.lisp:577-579): 128 bytes, two blocks
__device__ __forceinline__ void oracle_leaf_digest(const uint32_t *cw, uint64_t l, uint32_t h[8]) {
  uint32_t sym[4][8];
#pragma unroll
  for (int s = 0; s < 4; s++) {
    Ext<8> e = load_ext<8>(cw + (4 * l + s) * 8);
#pragma unroll
    for (int d = 0; d < 8; d++) sym[s][d] = e.c[d];
  }
  uint32_t m[16];
  b3_iv(h);
#pragma unroll
  for (int b = 0; b < 2; b++) {
#pragma unroll
    for (int k = 0; k < 4; k++)
#pragma unroll
      for (int s = 0; s < 4; s++) m[4 * k + s] = sym[s][4 * b + k];
    uint32_t flags = b == 0 ? B3_CHUNK_START : (B3_CHUNK_END | B3_ROOT);
    b3_compress(h, m, 0, 64, flags, h, 0);
  }
}

__device__ __forceinline__ void store_digest(uint32_t *p, const uint32_t h[8]) {
  uint4 *o = reinterpret_cast<uint4 *>(p);
  o[0] = make_uint4(h[0], h[1], h[2], h[3]);
  o[1] = make_uint4(h[4], h[5], h[6], h[7]);
}
__device__ __forceinline__ void load_digest(const uint32_t *p, uint32_t h[8]) {
  const uint4 *i = reinterpret_cast<const uint4 *>(p);
  uint4 a = i[0], b = i[1];
  h[0] = a.x, h[1] = a.y, h[2] = a.z, h[3] = a.w, h[4] = b.x, h[5] = b.y, h[6] = b.z, h[7] = b.w;
}

// Up to `height` levels of nodes above 2 * BLOCK consecutive nodes of `level` (n of them), node =
// BLAKE3(left || right) (src/pcs.lisp:54-55, 64-77), every level written behind the one below
// (level k + 1 starts 8 * n_k words after level k) and carried to the next step through LDS.
// LEAVES 0: `level` holds digests; 1: the bottom nodes are the leaf digests of ncols codewords
// (written too); 2: of an oracle codeword.
template <int LEAVES>
__global__ __launch_bounds__(BLOCK) void subtree_kernel(uint32_t *level, uint64_t n, int height, const uint32_t *cw,
                                                        int ncols, uint64_t cw_len) {
  __shared__ uint32_t lds[BLOCK][9];  // a digest per row, padded against bank conflicts
  const uint32_t t = threadIdx.x;
  uint64_t first = (uint64_t)blockIdx.x * BLOCK;  // this workgroup's first node of the level being written
  uint64_t count = n / 2;                         // nodes of that level
  uint32_t *out = level + 8 * n;
  uint32_t left[8], right[8], h[8];
  if (first + t < count) {
    const uint64_t c0 = 2 * (first + t);
    if (LEAVES == 0) {
      load_digest(level + 8 * c0, left);
      load_digest(level + 8 * (c0 + 1), right);
    } else {
      if (LEAVES == 1) {
        column_leaf_digest(cw, ncols, cw_len, c0, left);
        column_leaf_digest(cw, ncols, cw_len, c0 + 1, right);
      } else {
        oracle_leaf_digest(cw, c0, left);
        oracle_leaf_digest(cw, c0 + 1, right);
      }
      store_digest(level + 8 * c0, left);
      store_digest(level + 8 * (c0 + 1), right);
    }
    b3_node(left, right, h);
    store_digest(out + 8 * (first + t), h);
#pragma unroll
    for (int i = 0; i < 8; i++) lds[t][i] = h[i];
  }
  uint32_t width = BLOCK;  // nodes of the current level held by this workgroup (when full)
  for (int s = 1; s < height; s++) {
    __syncthreads();
    out += 8 * count;
    count /= 2, first /= 2, width /= 2;
    const bool active = t < width && first + t < count;
    if (active) {
#pragma unroll
      for (int i = 0; i < 8; i++) left[i] = lds[2 * t][i], right[i] = lds[2 * t + 1][i];
      b3_node(left, right, h);
      store_digest(out + 8 * (first + t), h);
    }
    __syncthreads();
    if (active) {
#pragma unroll
      for (int i = 0; i < 8; i++) lds[t][i] = h[i];
    }
  }
}

// a tree of a single leaf: its digest is the whole tree
template <int LEAVES>
__global__ void single_leaf_kernel(uint32_t *level, const uint32_t *cw, int ncols, uint64_t cw_len) {
  if (threadIdx.x || blockIdx.x) return;
  uint32_t h[8];
  if (LEAVES == 1)
    column_leaf_digest(cw, ncols, cw_len, 0, h);
  else
    oracle_leaf_digest(cw, 0, h);
  store_digest(level, h);
}

static int cap_level_of(uint64_t leaves) {  // src/pcs.lisp:57-59
  int il = 0;
  for (uint64_t v = leaves; v; v >>= 1) il++;
  return il - 1 - 7 > 0 ? il - 1 - 7 : 0;
}

// Every level of the tree at d_levels (leaves first), a few launches of up to nine levels each; the
// leaf digests are computed by the first launch (leaves 1: ncols codewords, 2: an oracle codeword) or
// already there (0).  A single leaf (no node above it) is hashed by the same kernel's bottom step.
static int merkle_tree_launch(uint32_t *d_levels, uint64_t nleaves, int leaves, const uint32_t *cw, int ncols,
                              uint64_t cw_len, uint64_t *cap_rows, uint64_t *cap_off_words) {
  Context &c = ctx();
  uint32_t *level = d_levels;
  uint64_t n = nleaves;
  int lc = cap_level_of(nleaves);
  uint64_t cap_off = 0;
  for (int l = 0; l < lc; l++) cap_off += 8 * (nleaves >> l);
  if (nleaves == 1 && leaves == 1)
    hipLaunchKernelGGL(single_leaf_kernel<1>, dim3(1), dim3(64), 0, c.stream, level, cw, ncols, cw_len);
  if (nleaves == 1 && leaves == 2)
    hipLaunchKernelGGL(single_leaf_kernel<2>, dim3(1), dim3(64), 0, c.stream, level, cw, ncols, cw_len);
  while (n > 1) {
    int height = 0;
    // The launch that hashes the leaves climbs few levels: above the leaves every level halves the threads at work
    // and costs a whole compression's latency, so a workgroup of a tall launch idles most of its life (measured at
    // 2^22 leaves: 246 us with nine levels in the first launch, 198 us with five, 175 us with three; five leaves the
    // fewest launches above -- over digests only, nine levels each -- and the shortest commit, 0.51 against 0.55 ms).
    static const int leaf_height = getenv("EXH_MERKLE_LEAF_HEIGHT") ? atoi(getenv("EXH_MERKLE_LEAF_HEIGHT")) : 5;
    const int max_height = leaves != 0 ? leaf_height : 9;
    for (uint64_t v = n; v > 1 && height < max_height; v >>= 1) height++;
    uint32_t grid = (uint32_t)((n / 2 + BLOCK - 1) / BLOCK);
    c.prof_begin(leaves == 1 ? "merkle_leaves" : leaves == 2 ? "merkle_oracle_leaves" : "merkle_levels", 0,
                 (leaves == 1 ? (uint64_t)ncols * 16 * n : leaves == 2 ? 128 * n : 0) + 64 * n);
    if (leaves == 1)
      hipLaunchKernelGGL(subtree_kernel<1>, dim3(grid), dim3(BLOCK), 0, c.stream, level, n, height, cw, ncols, cw_len);
    else if (leaves == 2)
      hipLaunchKernelGGL(subtree_kernel<2>, dim3(grid), dim3(BLOCK), 0, c.stream, level, n, height, cw, ncols, cw_len);
    else
      hipLaunchKernelGGL(subtree_kernel<0>, dim3(grid), dim3(BLOCK), 0, c.stream, level, n, height, cw, ncols, cw_len);
    c.prof_end();
    leaves = 0;
    for (int s = 0; s < height; s++) {
      level += 8 * n;
      n /= 2;
    }
  }
  EXH_HIP(hipGetLastError());
  *cap_rows = nleaves >> lc;
  *cap_off_words = cap_off;
  return OK;
}
__global__ void deliver_kernel(const uint32_t *src, uint32_t words, unsigned long long *host_dst, uint32_t seq);
static bool await_words(Context &c, const volatile unsigned long long *w, size_t n, uint32_t seq, uint32_t *out);
constexpr size_t CAP_PIN = 32768 + 40 * 40;  // (BaseFold's first cap slot: a commitment and an opening never overlap)

static int merkle_tree_device(uint32_t *d_levels, uint64_t nleaves, int leaves, const uint32_t *cw, int ncols,
                              uint64_t cw_len, uint8_t *cap, uint64_t *cap_rows) {
  Context &c = ctx();
  uint64_t cap_off = 0;
  int status = merkle_tree_launch(d_levels, nleaves, leaves, cw, ncols, cw_len, cap_rows, &cap_off);
  if (status) return status;
  // The cap comes to the host as the oracles' caps of BaseFold do: a small launch writes its words into pinned
  // memory, each with the delivery's number in its upper half, and the host polls them -- no copy to set up and no
  // wait on the stream to wake from (15 us of a commitment).
  if (*cap_rows <= 128 && c.host_pinned_dev && !c.profiling) {
    if (++c.log_seq == 0) ++c.log_seq;
    const uint32_t seq = c.log_seq, words = (uint32_t)(8 * *cap_rows);
    hipLaunchKernelGGL(deliver_kernel, dim3(1), dim3(BLOCK), 0, c.stream, d_levels + cap_off, words,
                       reinterpret_cast<unsigned long long *>(c.host_pinned_dev + CAP_PIN), seq);
    EXH_HIP(hipGetLastError());
    std::vector<uint32_t> cap_words(words);
    if (!await_words(c, reinterpret_cast<const volatile unsigned long long *>(c.host_pinned + CAP_PIN), words, seq,
                     cap_words.data())) {
      set_error("device-error: a commitment's cap did not arrive");
      return E_DEVICE;
    }
    memcpy(cap, cap_words.data(), 4 * (size_t)words);
    return OK;
  }
  EXH_HIP(hipMemcpyAsync(cap, d_levels + cap_off, 32 * *cap_rows, hipMemcpyDeviceToHost, c.stream));
  EXH_HIP(hipStreamSynchronize(c.stream));
  return OK;
}

int merkle_commit_columns(const uint32_t *d_codewords, int ncols, int c, uint32_t *d_levels, uint8_t *cap,
                          uint64_t *cap_rows) {
  Context &cx = ctx();
  int status = cx.require();
  if (status) return status;
  uint64_t nleaves = (uint64_t)1 << (c - 1), cw_len = (uint64_t)1 << (c + 1);
  return merkle_tree_device(d_levels, nleaves, 1, d_codewords, ncols, cw_len, cap, cap_rows);
}

// ---- trees of mixed height (src/pcs.lisp:64-77): a shorter class's leaf digests are hashed into the level of the
// taller class's tree that has as many nodes, node = H(H(left, right), injected).  One launch per level (these
// trees sit beside the large single-class ones, whose levels go nine to a launch).
__global__ __launch_bounds__(BLOCK) void node_level_kernel(const uint32_t *below, uint32_t *level, uint64_t count,
                                                           const uint32_t *inj0, const uint32_t *inj1) {
  const uint64_t i = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
  if (i >= count) return;
  uint32_t left[8], right[8], h[8], t[8];
  load_digest(below + 16 * i, left);
  load_digest(below + 16 * i + 8, right);
  b3_node(left, right, h);
  if (inj0) {
    load_digest(inj0 + 8 * i, right);
    b3_node(h, right, t);
#pragma unroll
    for (int k = 0; k < 8; k++) h[k] = t[k];
  }
  if (inj1) {
    load_digest(inj1 + 8 * i, right);
    b3_node(h, right, t);
#pragma unroll
    for (int k = 0; k < 8; k++) h[k] = t[k];
  }
  store_digest(level + 8 * i, h);
}

int merkle_levels_injected_device(const uint32_t *d_leaves, uint64_t nleaves, int ninj, const int *inj_level,
                                  const uint32_t *const *d_inj, uint32_t *d_levels) {
  Context &c = ctx();
  int status = c.require();
  if (status) return status;
  if (nleaves == 0 || (nleaves & (nleaves - 1))) {
    set_error("invalid-parameter: a tree has a power of two of leaves");
    return E_PARAM;
  }
  EXH_HIP(hipMemcpyAsync(d_levels, d_leaves, nleaves * 32, hipMemcpyDeviceToDevice, c.stream));
  uint32_t *below = d_levels;
  uint64_t n = nleaves;
  for (int l = 1; n > 1; l++) {
    uint32_t *level = below + 8 * n;
    n /= 2;
    const uint32_t *inj[2] = {nullptr, nullptr};
    int found = 0;
    for (int k = 0; k < ninj; k++)
      if (inj_level[k] == l) {
        if (found == 2) {
          set_error("invalid-parameter: at most two classes are injected into one level");
          return E_PARAM;
        }
        inj[found++] = d_inj[k];
      }
    hipLaunchKernelGGL(node_level_kernel, dim3((uint32_t)((n + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, c.stream, below,
                       level, n, inj[0], inj[1]);
    below = level;
  }
  EXH_HIP(hipGetLastError());
  return OK;
}

// ------------------------------------------------------------------ BaseFold
// DOT-PAIRS (src/pcs.lisp:473-483) for the three parities at once: sums over pairs of
// pick(tt) pick(et), pick = even entry, odd entry, 2 odd - even.  Partials per workgroup.
__global__ __launch_bounds__(BLOCK) void dot_pairs_kernel(const uint32_t *tt, const uint32_t *et, uint64_t n_pairs,
                                                          uint32_t *partials) {
  Acc96 acc[3][8];
#pragma unroll
  for (int k = 0; k < 3; k++)
#pragma unroll
    for (int c = 0; c < 8; c++) acc_zero(acc[k][c]);
  for (uint64_t i = (uint64_t)blockIdx.x * BLOCK + threadIdx.x; i < n_pairs; i += (uint64_t)gridDim.x * BLOCK) {
    Ext<8> t0 = load_ext<8>(tt + 2 * i * 8), t1 = load_ext<8>(tt + (2 * i + 1) * 8);
    Ext<8> e0 = load_ext<8>(et + 2 * i * 8), e1 = load_ext<8>(et + (2 * i + 1) * 8);
    ext_mul_acc<8>(acc[0], t0, e0);
    ext_mul_acc<8>(acc[1], t1, e1);
    Ext<8> t2 = ext_sub<8>(ext_add<8>(t1, t1), t0), e2 = ext_sub<8>(ext_add<8>(e1, e1), e0);
    ext_mul_acc<8>(acc[2], t2, e2);
  }
  __shared__ uint32_t lds[BLOCK / 64][24];
  const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int k = 0; k < 3; k++)
#pragma unroll
    for (int c = 0; c < 8; c++) {
      uint32_t v = wave_sum(acc_reduce(acc[k][c]));
      if (lane == 0) lds[wave][k * 8 + c] = v;
    }
  __syncthreads();
  if (threadIdx.x < 24) {
    uint32_t v = lds[0][threadIdx.x];
    for (int w = 1; w < BLOCK / 64; w++) v = fadd(v, lds[w][threadIdx.x]);
    partials[(uint64_t)blockIdx.x * 24 + threadIdx.x] = v;
  }
}

__global__ __launch_bounds__(BLOCK) void sum_columns_kernel(const uint32_t *partials, uint32_t nblocks, uint32_t width,
                                                            uint32_t *sums) {
  __shared__ uint32_t lds[BLOCK / 64];
  uint32_t o = blockIdx.x, v = 0;
  for (uint32_t b = threadIdx.x; b < nblocks; b += BLOCK) v = fadd(v, partials[(uint64_t)b * width + o]);
  v = wave_sum(v);
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < BLOCK / 64; w++) v = fadd(v, lds[w]);
    sums[o] = v;
  }
}

// out[x] = h[x] + scale * column[x] over extension tables (h null: zero): the opening's table per class is the
// sum of its units' columns, each times the unit's scalar (src/pcs.lisp:709-716)
template <int D>
__global__ __launch_bounds__(BLOCK) void scale_add_kernel(const uint32_t *h, const uint32_t *column, uint32_t *out,
                                                          uint64_t len, RoundArgs<D> args) {
  uint64_t i = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
  if (i >= len) return;
  Ext<D> sc;
#pragma unroll
  for (int c = 0; c < D; c++) sc.c[c] = args.r_mont[c];
  Ext<D> v = ext_mul_mont<D>(sc, load_ext<D>(column + i * D));
  if (h) v = ext_add<D>(v, load_ext<D>(h + i * D));
  store_ext<D>(out + i * D, v);
}
template <int D>
static void scale_add_launch(const uint32_t *h, const uint32_t *column, uint32_t *out, uint64_t len,
                             const uint32_t *scale) {
  RoundArgs<D> a;
  memset(&a, 0, sizeof(a));
  for (int k = 0; k < D; k++) a.r_mont[k] = to_mont(scale[k] % P);
  uint32_t grid = (uint32_t)((len + BLOCK - 1) / BLOCK);
  hipLaunchKernelGGL(scale_add_kernel<D>, dim3(grid), dim3(BLOCK), 0, ctx().stream, h, column, out, len, a);
}
int scale_add_device(int D, const uint32_t *d_h, const uint32_t *d_column, uint64_t len, const uint32_t *scale,
                     uint32_t *d_out) {
  int status = ctx().require();
  if (status) return status;
  if (D == 4)
    scale_add_launch<4>(d_h, d_column, d_out, len, scale);
  else
    scale_add_launch<8>(d_h, d_column, d_out, len, scale);
  EXH_HIP(hipGetLastError());
  return OK;
}

// DOT-PAIRS of two device tables of len EXT8s for the three parities: out[parity][8] on the host (one wait)
int dot_pairs_device(const uint32_t *d_e, const uint32_t *d_v, uint64_t len, uint32_t *out) {
  Context &c = ctx();
  int status = c.require();
  if (status) return status;
  const uint64_t n_pairs = len / 2;
  const uint32_t grid = (uint32_t)std::min<uint64_t>((n_pairs + BLOCK - 1) / BLOCK, 1024);
  uint32_t *scratch = (uint32_t *)c.pool.alloc(((size_t)grid * 24 + 24) * 4);
  if (!scratch) {
    set_error("device-out-of-memory: dot-pairs partial sums");
    return E_NOMEM;
  }
  uint32_t *sums = scratch + (size_t)grid * 24;
  hipLaunchKernelGGL(dot_pairs_kernel, dim3(grid), dim3(BLOCK), 0, c.stream, d_e, d_v, n_pairs, scratch);
  hipLaunchKernelGGL(sum_columns_kernel, dim3(24), dim3(BLOCK), 0, c.stream, scratch, grid, 24u, sums);
  EXH_HIP(hipMemcpyAsync(out, sums, 96, hipMemcpyDeviceToHost, c.stream));
  EXH_HIP(hipStreamSynchronize(c.stream));
  c.pool.release(scratch);
  return OK;
}

// ---- DOT-PAIRS once more for callers that must not allocate: the workgroups' partial sums live in a static
// device array instead of a pooled buffer, and the 24 words of the result come back through the pinned host
// buffer the context has held since exh_init.  The array's name is a host-side stand-in: the address kernels
// can use comes from hipGetSymbolAddress, once per device, with that device current (each GPU holds its own
// copy of the array at its own address).  Every call on a GPU shares that GPU's array: calls that overlap on one
// GPU race.  A launch writes every word it later reads, so nothing has to be cleared between calls.
constexpr uint32_t STATIC_DOT_GRID = 512;                    // workgroups of the launch
constexpr uint64_t STATIC_DOT_MAX_LEN = (uint64_t)1 << 26;   // EXT8s per table: 2 GiB each
constexpr size_t STATIC_DOT_RESULT_AT = 4096;                // word of the pinned buffer the result lands at
static __device__ __align__(256) uint32_t scratch[STATIC_DOT_GRID * 24];  // 48 KiB per GPU until the process ends
constexpr int STATIC_MAX_DEVICES = 64;
static uint32_t *g_scratch_ptr[STATIC_MAX_DEVICES];

// the sums of the partial rows, written where `sums` points (mapped host memory here)
__global__ __launch_bounds__(BLOCK) void sum_columns_to_host_kernel(const uint32_t *partials, uint32_t nblocks,
                                                                    uint32_t width, uint32_t *sums) {
  __shared__ uint32_t lds[BLOCK / 64];
  uint32_t o = blockIdx.x, v = 0;
  for (uint32_t b = threadIdx.x; b < nblocks; b += BLOCK) v = fadd(v, partials[(uint64_t)b * width + o]);
  v = wave_sum(v);
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < BLOCK / 64; w++) v = fadd(v, lds[w]);
    __hip_atomic_store(sums + o, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

int dot_pairs_static_setup(int device) {
  if (device < 0 || device >= STATIC_MAX_DEVICES) {
    set_error("invalid-parameter: device index beyond the static scratch table");
    return E_PARAM;
  }
  if (g_scratch_ptr[device]) return OK;
  uint32_t *ptr = nullptr;
  EXH_HIP(hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)));
  g_scratch_ptr[device] = ptr;
  return OK;
}

int dot_pairs_static_device(const uint32_t *d_e, const uint32_t *d_v, uint64_t len, uint32_t *out) {
  Context &c = ctx();
  int status = c.require();
  if (status) return status;
  if (len > STATIC_DOT_MAX_LEN) {
    set_error("invalid-parameter: dot-pairs without allocation takes tables of at most 2^26 EXT8s");
    return E_PARAM;
  }
  uint32_t *partials = c.device >= 0 && c.device < STATIC_MAX_DEVICES ? g_scratch_ptr[c.device] : nullptr;
  if (!partials) {
    set_error("device-error: the static scratch array was not set up on this device");
    return E_DEVICE;
  }
  const uint64_t n_pairs = len / 2;
  const uint32_t grid = (uint32_t)std::min<uint64_t>((n_pairs + BLOCK - 1) / BLOCK, STATIC_DOT_GRID);
  hipLaunchKernelGGL(dot_pairs_kernel, dim3(grid), dim3(BLOCK), 0, c.stream, d_e, d_v, n_pairs, partials);
  hipLaunchKernelGGL(sum_columns_to_host_kernel, dim3(24), dim3(BLOCK), 0, c.stream, partials, grid, 24u,
                     c.host_pinned_dev + STATIC_DOT_RESULT_AT);
  EXH_HIP(hipGetLastError());
  EXH_HIP(hipStreamSynchronize(c.stream));
  memcpy(out, c.host_pinned + STATIC_DOT_RESULT_AT, 96);
  return OK;
}

// FOLD-TABLE (src/field.lisp:365-370) of extension tables
template <int D>
__global__ __launch_bounds__(BLOCK) void fold_table_kernel(const uint32_t *in, uint32_t *out, uint64_t n_out,
                                                           RoundArgs<D> args) {
  uint64_t i = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
  if (i >= n_out) return;
  Ext<D> r;
#pragma unroll
  for (int c = 0; c < D; c++) r.c[c] = args.r_mont[c];
  store_ext<D>(out + i * D, fold_ext<D>(load_ext<D>(in + 2 * i * D), load_ext<D>(in + (2 * i + 1) * D), r));
}
template <int D>
static void fold_table_launch(const uint32_t *in, uint32_t *out, uint64_t n_out, const uint32_t *r) {
  RoundArgs<D> a;
  memset(&a, 0, sizeof(a));
  for (int k = 0; k < D; k++) a.r_mont[k] = to_mont(r[k] % P);
  uint32_t grid = (uint32_t)((n_out + BLOCK - 1) / BLOCK);
  hipLaunchKernelGGL(fold_table_kernel<D>, dim3(grid), dim3(BLOCK), 0, ctx().stream, in, out, n_out, a);
}
int fold_table_device(int D, const uint32_t *d_in, uint64_t len, const uint32_t *r, uint32_t *d_out) {
  int status = ctx().require();
  if (status) return status;
  if (D == 4)
    fold_table_launch<4>(d_in, d_out, len / 2, r);
  else
    fold_table_launch<8>(d_in, d_out, len / 2, r);
  EXH_HIP(hipGetLastError());
  return OK;
}

// EXT8 table (entries x 8) <-> 8 coordinate columns, for ENCODE-EXT (src/pcs.lisp:569-575)
__global__ __launch_bounds__(BLOCK) void split_coords_kernel(const uint32_t *table, uint32_t *cols, uint64_t len) {
  uint64_t i = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
  if (i >= len) return;
  Ext<8> e = load_ext<8>(table + i * 8);
#pragma unroll
  for (int d = 0; d < 8; d++) cols[(uint64_t)d * len + i] = e.c[d];
}
__global__ __launch_bounds__(BLOCK) void join_coords_kernel(const uint32_t *cols, uint32_t *table, uint64_t len) {
  uint64_t i = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
  if (i >= len) return;
  Ext<8> e;
#pragma unroll
  for (int d = 0; d < 8; d++) e.c[d] = cols[(uint64_t)d * len + i];
  store_ext<8>(table + i * 8, e);
}

// eq(rr, x) for all x of nv bits as one table (weights of the BaseFold sumcheck)
struct EqOne {
  int bits;
};
__global__ __launch_bounds__(BLOCK) void eq8_kernel(const uint32_t *factors, int bits, uint32_t *out, uint64_t total) {
  uint64_t x = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
  if (x >= total) return;
  Ext<8> e = ext_lift<8>(1);
  for (int b = 0; b < bits; b++)
    e = ext_mul_mont<8>(e, load_ext<8>(factors + ((size_t)b * 2 + (((x >> b) & 1) ? 0 : 1)) * 8));
  store_ext<8>(out + x * 8, e);
}

// copy `count` segments of `words` words each from src + offsets[i] to out
__global__ void gather_kernel(const uint32_t *src, const uint64_t *offsets, uint32_t words, uint32_t count,
                              uint32_t *out) {
  uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= (uint64_t)words * count) return;
  uint32_t seg = (uint32_t)(gid / words), w = (uint32_t)(gid % words);
  out[gid] = src[offsets[seg] + w];
}

namespace {
struct Owned {
  std::vector<void *> ptrs;
  ~Owned() {
    for (void *p : ptrs) ctx().pool.release(p);
  }
  uint32_t *alloc(uint64_t words) {
    void *p = ctx().pool.alloc(words * 4);
    if (!p) {
      set_error("device-out-of-memory: BaseFold buffers");
      return nullptr;
    }
    ptrs.push_back(p);
    return (uint32_t *)p;
  }
};
struct OracleTree {
  int level;
  uint32_t *cw, *levels;
  uint64_t cw_len, nleaves;
  int lc;
};
}  // namespace

static int gather_to_host(const uint32_t *src, const std::vector<uint64_t> &offsets, uint32_t words,
                          std::vector<uint32_t> *out) {
  Context &c = ctx();
  out->assign((size_t)offsets.size() * words, 0);
  if (offsets.empty()) return OK;
  uint64_t *d_off = nullptr;
  uint32_t *d_out = nullptr;
  EXH_HIP(hipMalloc((void **)&d_off, offsets.size() * 8));
  EXH_HIP(hipMalloc((void **)&d_out, out->size() * 4));
  EXH_HIP(hipMemcpy(d_off, offsets.data(), offsets.size() * 8, hipMemcpyHostToDevice));
  uint64_t total = out->size();
  hipLaunchKernelGGL(gather_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, c.stream, src, d_off, words,
                     (uint32_t)offsets.size(), d_out);
  EXH_HIP(hipStreamSynchronize(c.stream));
  EXH_HIP(hipMemcpy(out->data(), d_out, total * 4, hipMemcpyDeviceToHost));
  EXH_HIP(hipFree(d_off));
  EXH_HIP(hipFree(d_out));
  return OK;
}

// OPEN-QUERIES' two gathers for one (unit, class) (src/pcs.lisp:721-734).  Leaves: out[(q * ncols + k) * 4 + s] =
// symbol 4 * leaf_q + s of column k (LEAF-ROWS, src/pcs.lisp:275-277, as the (Q, rows, 4) array of
// FIELD-ARRAY-OF-LEAVES, :659-665): one thread per (q, k), one 16-byte load.
__global__ __launch_bounds__(BLOCK) void open_leaves_kernel(const uint32_t *cw, uint64_t cw_len, uint32_t ncols,
                                                            const uint64_t *leaf, uint32_t count, uint32_t *out) {
  uint64_t gid = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
  if (gid >= (uint64_t)count * ncols) return;
  uint32_t q = (uint32_t)(gid / ncols), k = (uint32_t)(gid % ncols);
  const uint4 v = *(const uint4 *)(cw + (uint64_t)k * cw_len + 4 * leaf[q]);
  *(uint4 *)(out + gid * 4) = v;
}

// Paths: out[(q * depth + d) * 8 ..] = the sibling of leaf_q's ancestor on level d (PATH, src/pcs.lisp:79-84); the
// levels lie leaves first, level d at digest 2 * nleaves - 2 * (nleaves >> d).  One thread per digest word.
__global__ __launch_bounds__(BLOCK) void open_paths_kernel(const uint32_t *levels, uint64_t nleaves, uint32_t depth,
                                                           const uint64_t *leaf, uint32_t count, uint32_t *out) {
  uint64_t gid = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
  if (gid >= (uint64_t)count * depth * 8) return;
  uint32_t w = (uint32_t)(gid % 8), d = (uint32_t)((gid / 8) % depth), q = (uint32_t)(gid / 8 / depth);
  uint64_t start = 2 * nleaves - 2 * (nleaves >> d);
  out[gid] = levels[(start + ((leaf[q] >> d) ^ 1)) * 8 + w];
}

int open_queries_device(const uint32_t *d_codewords, int ncols, int c, const uint32_t *d_levels, const uint64_t *leaves,
                        int count, uint32_t *out_leaves, uint8_t *out_paths, int *out_depth) {
  Context &cx = ctx();
  int status = cx.require();
  if (status) return status;
  const uint64_t nleaves = (uint64_t)1 << (c - 1), cw_len = (uint64_t)1 << (c + 1);
  const uint32_t depth = d_levels ? (uint32_t)cap_level_of(nleaves) : 0;
  if (out_depth) *out_depth = (int)depth;
  if (count == 0) return OK;
  const uint64_t leaf_words = (uint64_t)count * ncols * 4, path_words = (uint64_t)count * depth * 8;
  // one pooled buffer: the indices (padded to 16 bytes: the leaves are stored as uint4), the leaves, the paths
  const size_t idx_slots = ((size_t)count + 1) & ~(size_t)1;
  uint64_t *d_idx = (uint64_t *)cx.pool.alloc(idx_slots * 8 + (leaf_words + path_words) * 4);
  if (!d_idx) {
    set_error("device-out-of-memory: query openings");
    return E_NOMEM;
  }
  uint32_t *d_leaf_out = (uint32_t *)(d_idx + idx_slots), *d_path_out = d_leaf_out + leaf_words;
  hipError_t e = hipMemcpyAsync(d_idx, leaves, (size_t)count * 8, hipMemcpyHostToDevice, cx.stream);
  if (e == hipSuccess) {
    hipLaunchKernelGGL(open_leaves_kernel, dim3((uint32_t)(((uint64_t)count * ncols + BLOCK - 1) / BLOCK)), dim3(BLOCK),
                       0, cx.stream, d_codewords, cw_len, (uint32_t)ncols, d_idx, (uint32_t)count, d_leaf_out);
    if (path_words)
      hipLaunchKernelGGL(open_paths_kernel, dim3((uint32_t)((path_words + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0,
                         cx.stream, d_levels, nleaves, depth, d_idx, (uint32_t)count, d_path_out);
    e = hipGetLastError();
  }
  if (e == hipSuccess) e = hipMemcpyAsync(out_leaves, d_leaf_out, leaf_words * 4, hipMemcpyDeviceToHost, cx.stream);
  if (e == hipSuccess && path_words)
    e = hipMemcpyAsync(out_paths, d_path_out, path_words * 4, hipMemcpyDeviceToHost, cx.stream);
  hipError_t e2 = hipStreamSynchronize(cx.stream);  // the indices (pageable) and the pooled buffer are free after this
  cx.pool.release(d_idx);
  EXH_HIP(e);
  EXH_HIP(e2);
  return OK;
}

// ------------------------------------------------------------------ BASEFOLD's rounds
// The sumcheck of eq(rr, x) Phi(x) never needs the eq table or its folds.  After i rounds the folded eq table is
// prf_i eq(rr[i..], .) with prf_i = prod_{j<i} eq1(r_j, x_j), so with E = eq(rr[i+1..], .) over the pairs k,
//   DOT-PAIRS(tt, et, 0) = prf_i (1 - r_i) h0,  h0 = sum_k E[k] tt[2k]
//   DOT-PAIRS(tt, et, 1) = prf_i r_i h1,        h1 = sum_k E[k] tt[2k+1]
//   DOT-PAIRS(tt, et, 2) = prf_i (2 r_i - (1 - r_i)) (2 h1 - h0)
// (src/pcs.lisp:473-483, 607-612): the same field elements, from two weighted sums of the message table with split
// weights E[k] = LOW[k mod |LOW|] HIGH[k div |LOW|] as in the sumcheck prover (src/sumcheck.lisp:37-49).
//
// One launch per round does both of the round's passes over memory: its first workgroups fold the message table
// by the last challenge (FOLD-TABLE, src/field.lisp:365-370) and take h0, h1 of the folded table in the same
// pass; the others fold the codeword (RS:FOLD, src/rs.lisp:93-101).  The sums meet in counted totals (RoundTotals)
// and the last summing workgroup to arrive writes them into pinned host memory and raises a flag there, so the
// host neither copies nor waits on the stream: it polls the flag while the codeword's workgroups still run.
struct BfStepArgs {
  // the message table's part: workgroups [0, tt_blocks)
  const uint32_t *tt_in;  // 4 entries per pair when folding, else 2
  uint32_t *tt_out;       // the folded table (fold)
  const uint32_t *low, *high;
  uint64_t n_pairs;  // pairs after the fold
  uint32_t low_bits, pairs_per_thread, fold, do_sums, tt_blocks;
  uint32_t r_mont[8];
  RoundTotals totals;
  // 17 64-bit words in pinned host memory, each (host_seq << 32 | value): h0, h1, then 1 when the totals never
  // completed.  Every word says itself that it has arrived, so no fence orders them: a release at system scope
  // writes back the whole L2 of the elected workgroup's XCD, which the fold's stores of the other workgroups keep
  // dirty (measured: 90 us per round)
  unsigned long long *host_out;
  uint32_t host_seq;
  // the codeword's part: workgroups [tt_blocks, gridDim.x)
  const uint32_t *cw_in, *tw_inv2;
  uint32_t *cw_out;
  uint64_t cw_m;  // elements after the fold
};

template <bool FOLD>
__global__ __launch_bounds__(BLOCK) void bf_step_kernel(BfStepArgs a) {
  const uint32_t tid = threadIdx.x;
  Ext<8> r;
#pragma unroll
  for (int c = 0; c < 8; c++) r.c[c] = a.r_mont[c];
  if (blockIdx.x >= a.tt_blocks) {  // pair (a, b) at twiddle x: f0 = (a + b)/2, f1 = (a - b)/(2x), f0 + r (f1 - f0)
    const uint64_t s = (uint64_t)(blockIdx.x - a.tt_blocks) * BLOCK + tid;
    if (s >= a.cw_m) return;
    const Ext<8> x = load_ext<8>(a.cw_in + 2 * s * 8), y = load_ext<8>(a.cw_in + (2 * s + 1) * 8);
    const Ext<8> f0 = ext_scale_mont<8>(ext_add<8>(x, y), mont_mul(INV2, R2));
    const Ext<8> f1 = ext_scale_mont<8>(ext_sub<8>(x, y), a.tw_inv2[s]);
    store_ext<8>(a.cw_out + s * 8, ext_add<8>(f0, ext_mul_mont<8>(r, ext_sub<8>(f1, f0))));
    return;
  }
  const uint64_t tile = (uint64_t)BLOCK * a.pairs_per_thread, tile_start = (uint64_t)blockIdx.x * tile;
  const uint64_t low_mask = ((uint64_t)1 << a.low_bits) - 1;
  Acc96 acc[2][8];
#pragma unroll
  for (int q = 0; q < 2; q++)
#pragma unroll
    for (int c = 0; c < 8; c++) acc_zero(acc[q][c]);
  // a pair's words are requested one pair ahead of its arithmetic (Q quads per pair: 8 when folding, else 4)
  constexpr int Q = FOLD ? 8 : 4;
  uint4 raw[Q], ahead[Q];
  Ext<8> w = ext_zero<8>(), w_ahead = ext_zero<8>();
  auto fetch = [&](uint64_t i, uint4 *q, Ext<8> &wq) {
    const uint4 *p = reinterpret_cast<const uint4 *>(a.tt_in) + (uint64_t)Q * i;
#pragma unroll
    for (int j = 0; j < Q; j++) q[j] = p[j];
    if (a.do_sums) wq = load_ext<8>(a.low + (i & low_mask) * 8);
  };
  if (tile_start + tid < a.n_pairs) fetch(tile_start + tid, raw, w);
  for (uint32_t k = 0; k < a.pairs_per_thread; k++) {
    const uint64_t i = tile_start + (uint64_t)k * BLOCK + tid;
    if (i >= a.n_pairs) break;
    const bool more = k + 1 < a.pairs_per_thread && i + BLOCK < a.n_pairs;
    if (more) fetch(i + BLOCK, ahead, w_ahead);
    Ext<8> lo, hi;
    if constexpr (FOLD) {
      lo = fold_ext<8>(ext_from_quads<8>(raw), ext_from_quads<8>(raw + 2), r);
      hi = fold_ext<8>(ext_from_quads<8>(raw + 4), ext_from_quads<8>(raw + 6), r);
      store_ext<8>(a.tt_out + 2 * i * 8, lo);
      store_ext<8>(a.tt_out + (2 * i + 1) * 8, hi);
    } else {
      lo = ext_from_quads<8>(raw), hi = ext_from_quads<8>(raw + 2);
    }
    if (a.do_sums) {
      ext_mul_acc<8>(acc[0], lo, w);  // (the weight second: its tripled wrap coefficients serve both products)
      ext_mul_acc<8>(acc[1], hi, w);
    }
    if (more) {
#pragma unroll
      for (int j = 0; j < Q; j++) raw[j] = ahead[j];
      w = w_ahead;
    }
  }
  if (!a.do_sums) return;
  __shared__ uint32_t lds[BLOCK / 64][16];
  __shared__ uint32_t mine[16], sums[16];
  __shared__ uint32_t scratch[TOTALS_POLLS * BLOCK];
#pragma unroll
  for (int q = 0; q < 2; q++)
#pragma unroll
    for (int c = 0; c < 8; c++) {
      const uint32_t v = wave_sum(acc_reduce(acc[q][c]));
      if ((tid & 63) == 0) lds[tid >> 6][q * 8 + c] = v;
    }
  __syncthreads();
  if (tid < 2) {  // a workgroup's pairs share one HIGH weight (the tile is |LOW| pairs)
    Ext<8> t;
#pragma unroll
    for (int c = 0; c < 8; c++) {
      uint32_t v = lds[0][tid * 8 + c];
#pragma unroll
      for (int w = 1; w < BLOCK / 64; w++) v = fadd(v, lds[w][tid * 8 + c]);
      t.c[c] = v;
    }
    // times HIGH / R, then times R: the plain product
    t = ext_mul_mont<8>(t, load_ext<8>(a.high + (tile_start >> a.low_bits) * 8));
#pragma unroll
    for (int c = 0; c < 8; c++) mine[tid * 8 + c] = mont_mul(t.c[c], R2);
  }
  __syncthreads();
  bool ok;
  if (!add_and_elect(a.totals, mine, 16, scratch, sums, &ok, 0, 16, a.tt_blocks - 1, a.tt_blocks)) return;
  if (tid < 17) {
    const uint32_t value = tid < 16 ? (ok ? sums[tid] : 0u) : (ok ? 0u : 1u);
    __hip_atomic_store(a.host_out + tid, ((unsigned long long)a.host_seq << 32) | value, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

// `words` words from device memory into pinned host memory as 64-bit words (seq << 32 | value), each its own flag
__global__ __launch_bounds__(BLOCK) void deliver_kernel(const uint32_t *src, uint32_t words, unsigned long long *host_dst,
                                                        uint32_t seq) {
  for (uint32_t u = threadIdx.x; u < words; u += BLOCK)
    __hip_atomic_store(host_dst + u, ((unsigned long long)seq << 32) | src[u], __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_SYSTEM);
}

// segments of 8 words from anywhere in device memory, side by side into out
__global__ __launch_bounds__(BLOCK) void gather8_kernel(const uint32_t *const *src, uint32_t count, uint32_t *out) {
  const uint64_t gid = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
  if (gid >= (uint64_t)count * 8) return;
  out[gid] = src[gid / 8][gid % 8];
}

__global__ __launch_bounds__(BLOCK) void zero_words_kernel(uint32_t *p, uint64_t words) {
  const uint64_t gid = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
  if (gid < words) p[gid] = 0;
}

// the host's side of such words in pinned memory: true once all n carry seq (their low halves then go to out);
// false when the stream ran dry without them
static bool await_words(Context &c, const volatile unsigned long long *w, size_t n, uint32_t seq, uint32_t *out) {
  auto all_there = [&]() {
    for (size_t u = n; u-- > 0;)
      if ((uint32_t)(w[u] >> 32) != seq) return false;
    return true;
  };
  uint32_t spins = 0;
  bool there = false;
  while (!(there = all_there())) {
    if ((++spins & 1023) == 0 && hipStreamQuery(c.stream) != hipErrorNotReady) break;
  }
  if (!there) {
    (void)hipStreamSynchronize(c.stream);
    if (!all_there()) return false;
  }
  std::atomic_thread_fence(std::memory_order_acquire);
  for (size_t u = 0; u < n; u++) out[u] = (uint32_t)w[u];
  return true;
}

// regions of the context's pinned host buffer BaseFold's rounds use (in 32-bit words): a slot of 17 64-bit words
// per round, then a slot of 128 * 8 64-bit words per oracle cap
constexpr size_t BF_PIN = 32768, BF_ROUND_SLOT = 40, BF_MAX_ROUNDS = 40, BF_CAP_SLOT = 2048, BF_MAX_ORACLES = 14;
static_assert(CAP_PIN == BF_PIN + BF_MAX_ROUNDS * BF_ROUND_SLOT, "a commitment's cap lands in the first cap slot");
static_assert(BF_PIN + BF_MAX_ROUNDS * BF_ROUND_SLOT + BF_MAX_ORACLES * BF_CAP_SLOT <= 65536, "the pinned buffer");
constexpr uint32_t BF_GROUPS = 32;  // rows of totals of a round's sums (16 words each)

// BASEFOLD (src/pcs.lisp:581-657) over ncls size classes, ascending, the last one nv: class c's table d_h[k]
// (2^c EXT8s) joins the message table and the codeword at level nv - c (:590-600, :635-639).  d_cws (optional, and
// optional per class): the class's codeword ENCODE-EXT(H_c) (2^(c+1) EXT8s) when the caller has it already --
// encoding is linear, so the codeword of a combination of committed columns is the same combination of their
// committed codewords (COMBINE-COLUMNS over the codewords) -- else it is encoded here, coordinate by coordinate.
int basefold_prove_classes(Transcript &tr, int nv, int ncls, const int *cls, const uint32_t *const *d_hs,
                           const uint32_t *rr, const uint32_t *v, int grind_bits, int queries, uint64_t *out_qs,
                           uint32_t *out_chal, uint32_t *out_final, const uint32_t *const *d_cws) {
  Context &c = ctx();
  int status = c.require();
  if (status) return status;
  if (ncls < 1 || cls[ncls - 1] != nv || queries < 1 || nv > 30) {
    set_error("invalid-parameter: basefold takes its classes in ascending order, the largest being nv <= 30");
    return E_PARAM;
  }
  for (int k = 0; k < ncls; k++)
    if (cls[k] < 1 || (k && cls[k] <= cls[k - 1])) {
      set_error("invalid-parameter: basefold classes must ascend");
      return E_PARAM;
    }
  const uint32_t *d_h = d_hs[ncls - 1];
  const int fl = nv - 5 > 0 ? nv - 5 : 0;
  const uint64_t len = (uint64_t)1 << nv;
  Owned mem;
  // the folded message tables ping-pong between two buffers (the class's own table is read in round 0 and never
  // written); so do the folded codewords, except that a level with an oracle tree keeps a buffer of its own
  uint32_t *tt_a = mem.alloc(len * 4 + 8), *tt_b = mem.alloc(len * 2 + 8);
  uint32_t *cw_b = mem.alloc(len * 8), *cw_c = mem.alloc(len * 4 + 8);
  uint32_t *cw0 = nullptr, *cols = nullptr, *cwcols = nullptr;
  const bool given = d_cws && d_cws[ncls - 1];
  if (!given) {
    cw0 = mem.alloc(2 * len * 8), cols = mem.alloc(len * 8), cwcols = mem.alloc(2 * len * 8);
    if (!cw0 || !cols || !cwcols) return E_NOMEM;
  } else if (ncls > 1) {  // the joining classes add their codewords into the working one
    cols = mem.alloc(len * 4), cwcols = mem.alloc(len * 8);
    if (!cols || !cwcols) return E_NOMEM;
  }
  const uint32_t max_grid = 1024;
  uint32_t *partials = mem.alloc((uint64_t)max_grid * 24 + 24), *factors = mem.alloc((uint64_t)nv * 16 + 16);
  if (!tt_a || !tt_b || !cw_b || !cw_c || !partials || !factors) return E_NOMEM;
  uint32_t *sums = partials + (uint64_t)max_grid * 24;
  const uint32_t grid_len = (uint32_t)((len + BLOCK - 1) / BLOCK);
  // cw = ENCODE-EXT(H) unless given
  const uint32_t *cw = given ? d_cws[ncls - 1] : cw0;
  if (!given) {
    hipLaunchKernelGGL(split_coords_kernel, dim3(grid_len), dim3(BLOCK), 0, c.stream, d_h, cols, len);
    if ((status = rs_encode_columns(cols, 8, nv, cwcols))) return status;
    hipLaunchKernelGGL(join_coords_kernel, dim3(2 * grid_len), dim3(BLOCK), 0, c.stream, cwcols, cw0, 2 * len);
  }
  // ---- the rounds' split weights: round i sums over the pairs k of variables i+1 .. nv-1; LOW covers a workgroup's
  // tile, HIGH the rest
  std::vector<int> low_bits(std::max(fl, 1), 0);
  std::vector<uint64_t> low_off(std::max(fl, 1), 0), high_off(std::max(fl, 1), 0);
  uint32_t *weights = nullptr;
  {
    std::vector<uint32_t> f((size_t)nv * 16);
    for (int b = 0; b < nv; b++)
      for (int k = 0; k < 8; k++) {
        uint32_t r = rr[(size_t)b * 8 + k] % P;
        f[((size_t)b * 2) * 8 + k] = to_mont(r);
        f[((size_t)b * 2 + 1) * 8 + k] = to_mont(fsub(k == 0 ? 1u : 0u, r));
      }
    EXH_HIP(hipMemcpyAsync(factors, f.data(), f.size() * 4, hipMemcpyHostToDevice, c.stream));
    EXH_HIP(hipStreamSynchronize(c.stream));  // `f` is pageable
    if (fl > BF_MAX_ROUNDS || 2 * fl > 64) {
      set_error("invalid-parameter: basefold rounds beyond the buffers");
      return E_PARAM;
    }
    std::vector<int> first, bits;
    std::vector<uint64_t> off;
    uint64_t pos = 0;
    for (int i = 0; i < fl; i++) {
      const int rest = nv - 1 - i;  // variables of the pairs
      // (tiles of 2^10 to 2^12 pairs, at least a thousand of them while the table is that large: long tiles in few
      // workgroups trail their loads one after another, short ones pay the reduction and the atomics per tile)
      low_bits[i] = std::min(rest, std::min(std::max(rest - 10, 10), 12));
      low_off[i] = pos, first.push_back(i + 1), bits.push_back(low_bits[i]), off.push_back(pos);
      pos += (uint64_t)1 << low_bits[i];
      high_off[i] = pos, first.push_back(i + 1 + low_bits[i]), bits.push_back(rest - low_bits[i]), off.push_back(pos);
      pos += (uint64_t)1 << (rest - low_bits[i]);
    }
    if (fl > 0) {
      weights = mem.alloc(pos * 8);
      if (!weights) return E_NOMEM;
      if ((status = eq_tables_launch(8, (int)first.size(), first.data(), bits.data(), off.data(), factors, nv, weights)))
        return status;
    }
  }
  EXH_HIP(hipGetLastError());
  Domain *dom;
  if ((status = get_domain(nv + 1, &dom))) return status;

  hf::E prf = hf::lift(1, 8), claim = hf::from(v, 8);
  // y_c = H_c at the point's last c coordinates, for the classes still to join; ysum their sum (:593-595)
  const uint32_t one8[8] = {1, 0, 0, 0, 0, 0, 0, 0};
  std::vector<hf::E> yc(ncls, hf::zero(8));
  hf::E ysum = hf::zero(8);
  for (int k = 0; k + 1 < ncls; k++) {
    const uint64_t clen = (uint64_t)1 << cls[k], n_pairs = clen / 2;
    uint32_t *eqc = tt_a;  // the eq table of the point's tail (at most half of the buffer's room)
    hipLaunchKernelGGL(eq8_kernel, dim3((uint32_t)((clen + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, c.stream,
                       factors + (size_t)(nv - cls[k]) * 16, cls[k], eqc, clen);
    uint32_t grid = (uint32_t)std::min<uint64_t>((n_pairs + BLOCK - 1) / BLOCK, max_grid);
    hipLaunchKernelGGL(dot_pairs_kernel, dim3(grid), dim3(BLOCK), 0, c.stream, d_hs[k], eqc, n_pairs, partials);
    hipLaunchKernelGGL(sum_columns_kernel, dim3(24), dim3(BLOCK), 0, c.stream, partials, grid, 24u, sums);
    uint32_t dots[24];
    EXH_HIP(hipMemcpyAsync(dots, sums, 96, hipMemcpyDeviceToHost, c.stream));
    EXH_HIP(hipStreamSynchronize(c.stream));
    yc[k] = hf::add(hf::from(dots, 8), hf::from(dots + 8, 8));  // even entries' products + odd entries' products
    ysum = hf::add(ysum, yc[k]);
  }
  // ---- the rounds' totals (cleared by a kernel: callers may record this path) and the pinned slots
  const uint64_t total_words = (uint64_t)std::max(fl, 1) * BF_GROUPS * 16 * 2 + std::max(fl, 1) + 1;
  uint32_t *totals_mem = mem.alloc(total_words + (total_words & 1));
  if (!totals_mem) return E_NOMEM;
  hipLaunchKernelGGL(zero_words_kernel, dim3((uint32_t)((total_words + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, c.stream,
                     totals_mem, total_words);
  uint32_t *arrivals = totals_mem + (uint64_t)std::max(fl, 1) * BF_GROUPS * 16 * 2;
  volatile uint32_t *pin = c.host_pinned + BF_PIN;
  uint32_t *pin_dev = c.host_pinned_dev + BF_PIN;
  if (++c.log_seq == 0) ++c.log_seq;  // (a word of an earlier proof carries an earlier number)
  const uint32_t seq = c.log_seq;

  std::vector<OracleTree> oracles;
  const uint32_t *tt = d_h;  // the table the next step reads
  uint32_t x[8] = {0};
  // the launch of round i: fold the table by x (the challenge of round i - 1) when i > 0, sum round i's h0, h1;
  // with_cw: fold the codeword of level i - 1 as well, into cw_out
  auto launch_step = [&](int i, bool fold, bool do_sums, uint32_t *cw_out) -> int {
    BfStepArgs a;
    memset(&a, 0, sizeof(a));
    const uint64_t entries = fold ? len >> i : len >> i;  // entries of the table summed (after the fold)
    (void)entries;
    const uint64_t n_pairs = (len >> i) / 2;
    a.tt_in = tt, a.fold = fold ? 1 : 0, a.do_sums = do_sums ? 1 : 0, a.n_pairs = n_pairs;
    if (fold) a.tt_out = (tt == tt_a) ? tt_b : tt_a;
    uint32_t tile = 1;
    if (do_sums) {
      a.low = weights + low_off[i] * 8, a.high = weights + high_off[i] * 8, a.low_bits = (uint32_t)low_bits[i];
      tile = (uint32_t)1 << low_bits[i];  // |LOW| pairs: one HIGH weight per workgroup
    } else {
      tile = (uint32_t)std::min<uint64_t>(std::max<uint64_t>(n_pairs, 1), 4 * BLOCK);
    }
    a.pairs_per_thread = std::max<uint32_t>(1, tile / BLOCK);
    a.tt_blocks = n_pairs ? (uint32_t)((n_pairs + tile - 1) / tile) : 0;
    for (int k = 0; k < 8; k++) a.r_mont[k] = to_mont(x[k]);
    if (do_sums) {
      uint32_t groups = 1;
      while (groups * 2 <= BF_GROUPS && groups * 2 <= a.tt_blocks) groups *= 2;
      a.totals.totals = reinterpret_cast<unsigned long long *>(totals_mem) + (uint64_t)i * BF_GROUPS * 16;
      a.totals.arrivals = arrivals + i;
      a.totals.groups = groups, a.totals.pstride = 16, a.totals.spin_limit = 200000;
      a.host_out = reinterpret_cast<unsigned long long *>(pin_dev + (size_t)i * BF_ROUND_SLOT), a.host_seq = seq;
    }
    uint32_t cw_blocks = 0;
    if (cw_out) {
      const uint64_t m = (len >> (i - 1));  // elements of the folded codeword: half of level i - 1's 2^(nv + 2 - i)
      a.cw_in = cw, a.cw_out = cw_out, a.cw_m = m, a.tw_inv2 = dom->tw_inv2 + dom->off[i - 1];
      cw_blocks = (uint32_t)((m + BLOCK - 1) / BLOCK);
    }
    if (a.tt_blocks + cw_blocks == 0) return OK;
    c.prof_begin("basefold_step", i, (fold ? 3 : 2) * n_pairs * 32 * (do_sums || fold ? 1 : 0) + (cw_out ? 3 * a.cw_m * 32 : 0));
    if (fold)
      hipLaunchKernelGGL(bf_step_kernel<true>, dim3(a.tt_blocks + cw_blocks), dim3(BLOCK), 0, c.stream, a);
    else
      hipLaunchKernelGGL(bf_step_kernel<false>, dim3(a.tt_blocks + cw_blocks), dim3(BLOCK), 0, c.stream, a);
    c.prof_end();
    EXH_HIP(hipGetLastError());
    if (fold) tt = a.tt_out;
    if (cw_out) cw = cw_out;
    return OK;
  };
  if (fl > 0 && (status = launch_step(0, false, true, nullptr))) return status;
  size_t cap_slots = 0;
  for (int i = 0; i < fl; i++) {
    // ---- the round's message from h0, h1
    uint32_t hh[17];
    if (!await_words(c, reinterpret_cast<const volatile unsigned long long *>(pin + (size_t)i * BF_ROUND_SLOT), 17, seq,
                     hh) ||
        hh[16]) {
      set_error("device-error: a basefold round's sums did not arrive");
      return E_DEVICE;
    }
    const hf::E h0 = hf::from(hh, 8), h1 = hf::from(hh + 8, 8);
    const hf::E ri = hf::from(rr + 8 * (size_t)i, 8), one_r = hf::sub(hf::lift(1, 8), ri);
    const hf::E eqx[3] = {one_r, ri, hf::sub(hf::scale(ri, 2), one_r)};
    const hf::E hx[3] = {h0, h1, hf::sub(hf::scale(h1, 2), h0)};
    uint32_t ev[24];
    const hf::E a_term = ncls > 1 ? hf::mul(prf, ysum) : hf::zero(8);  // the classes still to join, :607-612
    for (int parity = 0; parity < 3; parity++) {
      hf::E t = hf::mul(hf::mul(prf, eqx[parity]), hx[parity]);
      if (ncls > 1) t = hf::add(t, hf::mul(a_term, eqx[parity]));
      memcpy(ev + 8 * parity, t.data(), 32);
    }
    uint64_t dims[2] = {3, 8};
    if ((status = tr.send(ev, 2, dims, nullptr))) return status;
    if (hf::add(hf::from(ev, 8), hf::from(ev + 8, 8)) != claim) {
      set_error("verification-failure: pcs: basefold sumcheck round " + std::to_string(i) + " failed");
      return E_REJECT;
    }
    tr.challenge(8, x);
    if (out_chal) memcpy(out_chal + 8 * i, x, 32);
    claim = hf::lagrange({hf::from(ev, 8), hf::from(ev + 8, 8), hf::from(ev + 16, 8)}, hf::from(x, 8));
    prf = hf::mul(prf, hf::eq1(hf::from(rr + 8 * i, 8), hf::from(x, 8)));
    // ---- level l: fold the table and the codeword by x; an oracle tree over the folded codeword; the joins
    const int l = i + 1;
    const uint64_t cur = len >> i;  // elements of the folded codeword
    const bool oracle = l >= 2 && l < fl && l % 2 == 0;
    bool joins = false;
    for (int k = 0; k + 1 < ncls; k++) joins = joins || nv - cls[k] == l;
    uint32_t *cw_out = nullptr;
    if (l < fl) {  // (the last level's codeword is never looked at)
      if (oracle) {
        if (oracles.size() >= BF_MAX_ORACLES) {
          set_error("invalid-parameter: basefold oracle levels beyond the buffers");
          return E_PARAM;
        }
        cw_out = mem.alloc(cur * 8);
        if (!cw_out) return E_NOMEM;
      } else {
        cw_out = (cw == cw_b) ? cw_c : cw_b;
        if (cur * 8 > (cw_out == cw_b ? len * 8 : len * 4)) cw_out = cw_b;  // (only level 1 needs the larger one)
      }
    }
    // the next round's sums ride on the fold unless a class joins in between
    const bool more = l < fl;
    if ((status = launch_step(l, true, more && !joins, cw_out))) return status;
    if (oracle) {  // an oracle tree over the folded codeword, its cap to the host behind a flag
      OracleTree o;
      o.level = l;
      o.cw_len = cur;
      o.nleaves = cur / 4;
      o.lc = cap_level_of(o.nleaves);
      o.cw = cw_out;
      o.levels = mem.alloc((2 * o.nleaves) * 8);
      if (!o.levels) return E_NOMEM;
      uint64_t rows = 0, cap_off = 0;
      if ((status = merkle_tree_launch(o.levels, o.nleaves, 2, o.cw, 1, o.cw_len, &rows, &cap_off))) return status;
      const size_t cap_at = BF_MAX_ROUNDS * BF_ROUND_SLOT + cap_slots * BF_CAP_SLOT;
      hipLaunchKernelGGL(deliver_kernel, dim3(1), dim3(BLOCK), 0, c.stream, o.levels + cap_off, (uint32_t)(8 * rows),
                         reinterpret_cast<unsigned long long *>(pin_dev + cap_at), seq);
      EXH_HIP(hipGetLastError());
      cap_slots++;
      std::vector<uint32_t> cap_words(8 * rows);
      if (!await_words(c, reinterpret_cast<const volatile unsigned long long *>(pin + cap_at), 8 * rows, seq,
                       cap_words.data())) {
        set_error("device-error: a basefold oracle's cap did not arrive");
        return E_DEVICE;
      }
      std::vector<uint8_t> cap(32 * rows);
      memcpy(cap.data(), cap_words.data(), 32 * rows);
      if ((status = tr.send_bytes(cap.data(), (int64_t)(32 * rows), nullptr))) return status;
      oracles.push_back(o);
    }
    if (joins) {
      for (int k = 0; k + 1 < ncls; k++)  // the classes that join at this level, :635-639
        if (nv - cls[k] == l) {
          const uint64_t clen = (uint64_t)1 << cls[k];
          const uint32_t gl = (uint32_t)((clen + BLOCK - 1) / BLOCK);
          uint32_t *tt_w = const_cast<uint32_t *>(tt), *cw_w = const_cast<uint32_t *>(cw);  // folded: ours to write
          scale_add_launch<8>(tt_w, d_hs[k], tt_w, clen, one8);
          if (l < fl) {
            const uint32_t *cwk = d_cws ? d_cws[k] : nullptr;
            if (!cwk) {  // ENCODE-EXT of the class's table, into a buffer of its own
              uint32_t *joined = mem.alloc(2 * clen * 8);
              if (!joined) return E_NOMEM;
              hipLaunchKernelGGL(split_coords_kernel, dim3(gl), dim3(BLOCK), 0, c.stream, d_hs[k], cols, clen);
              if ((status = rs_encode_columns(cols, 8, cls[k], cwcols))) return status;
              hipLaunchKernelGGL(join_coords_kernel, dim3(2 * gl), dim3(BLOCK), 0, c.stream, cwcols, joined, 2 * clen);
              cwk = joined;
            }
            if (oracle) {  // the oracle keeps the codeword it hashed: the sum goes to a buffer of its own
              uint32_t *sum = mem.alloc(2 * clen * 8);
              if (!sum) return E_NOMEM;
              scale_add_launch<8>(cw, cwk, sum, 2 * clen, one8);
              cw = sum;
            } else {
              scale_add_launch<8>(cw_w, cwk, cw_w, 2 * clen, one8);
            }
          }
          ysum = hf::sub(ysum, yc[k]);
        }
      EXH_HIP(hipGetLastError());
      if (more && (status = launch_step(l, false, true, nullptr))) return status;
    }
  }
  // the final table in the clear, the final claim, grinding, the query positions
  uint64_t mlen = len >> fl;
  std::vector<uint32_t> m(mlen * 8);
  EXH_HIP(hipMemcpyAsync(m.data(), tt, mlen * 32, hipMemcpyDeviceToHost, c.stream));
  EXH_HIP(hipStreamSynchronize(c.stream));
  uint64_t dims[2] = {mlen, 8};
  if ((status = tr.send(m.data(), 2, dims, nullptr))) return status;
  if (out_final) memcpy(out_final, m.data(), mlen * 32);
  hf::E mval = fl < nv ? hf::mle_eval(m.data(), nv - fl, rr + 8 * fl, 8) : hf::from(m.data(), 8);
  if (hf::mul(prf, mval) != claim) {
    set_error("verification-failure: pcs: basefold final claim");
    return E_REJECT;
  }
  tr.grind(grind_bits);
  std::vector<uint64_t> qs(queries);
  tr.challenge_bits(nv - 1, queries, qs.data());
  if (out_qs) memcpy(out_qs, qs.data(), 8 * (size_t)queries);
  // ---- the oracle openings, recorded (src/pcs.lisp:651-655): every queried leaf's four symbols and every path's
  // siblings of every oracle in one gather of 8-word segments and one copy back
  if (!oracles.empty()) {
    std::vector<const uint32_t *> segs;
    for (const OracleTree &o : oracles)
      for (int q = 0; q < queries; q++) {
        const uint64_t li = qs[q] >> o.level;
        for (int s = 0; s < 4; s++) segs.push_back(o.cw + (4 * li + s) * 8);
        uint64_t level_start = 0, n = o.nleaves, idx = li;
        for (int d = 0; d < o.lc; d++) {
          segs.push_back(o.levels + (level_start + (idx ^ 1)) * 8);
          level_start += n;
          n /= 2;
          idx >>= 1;
        }
      }
    const size_t nseg = segs.size();
    uint32_t *d_ptrs = mem.alloc(nseg * 2 + 2), *d_out = mem.alloc(nseg * 8);
    if (!d_ptrs || !d_out) return E_NOMEM;
    std::vector<uint32_t> got(nseg * 8);
    EXH_HIP(hipMemcpyAsync(d_ptrs, segs.data(), nseg * 8, hipMemcpyHostToDevice, c.stream));
    hipLaunchKernelGGL(gather8_kernel, dim3((uint32_t)((nseg * 8 + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, c.stream,
                       reinterpret_cast<const uint32_t *const *>(d_ptrs), (uint32_t)nseg, d_out);
    EXH_HIP(hipGetLastError());
    EXH_HIP(hipMemcpyAsync(got.data(), d_out, nseg * 32, hipMemcpyDeviceToHost, c.stream));
    EXH_HIP(hipStreamSynchronize(c.stream));
    size_t at = 0;
    for (const OracleTree &o : oracles) {
      std::vector<uint32_t> leaves((size_t)queries * 32);  // (Q, 8 rows, 4 symbols): row d holds coordinate d
      std::vector<uint32_t> path;
      for (int q = 0; q < queries; q++) {
        for (int s = 0; s < 4; s++, at++)
          for (int d = 0; d < 8; d++) leaves[((size_t)q * 8 + d) * 4 + s] = got[at * 8 + d];
        for (int d = 0; d < o.lc; d++, at++) path.insert(path.end(), got.begin() + at * 8, got.begin() + at * 8 + 8);
      }
      uint64_t d3[3] = {(uint64_t)queries, 8, 4};
      if ((status = tr.send(leaves.data(), 3, d3, nullptr, false))) return status;
      if ((status = tr.send_bytes((const uint8_t *)path.data(), (int64_t)path.size() * 4, nullptr, false))) return status;
    }
  }
  return OK;
}

int basefold_prove(Transcript &tr, int nv, const uint32_t *rr, const uint32_t *v, const uint32_t *d_h, int grind_bits,
                   int queries, uint64_t *out_qs, uint32_t *out_chal, uint32_t *out_final, const uint32_t *d_cw) {
  return basefold_prove_classes(tr, nv, 1, &nv, &d_h, rr, v, grind_bits, queries, out_qs, out_chal, out_final,
                                d_cw ? &d_cw : nullptr);
}

// The final opening over several size classes, one key per class, each a unit of its own with its own tree:
// the class's combined column H_c = COMBINE-COLUMNS of its columns with the caller's coefficients
// (src/pcs.lisp:434-441, 709-716), BASEFOLD over the classes, then OPEN-QUERIES (:721-734): per key the queried
// leaves (Q, ncols, 4), recorded, and its tree's paths up to the cap level, recorded.
int pcs_open(Transcript &tr, int nv, int nkeys, const OpenClass *keys, const uint32_t *rr, const uint32_t *v,
             int grind_bits, int queries, uint64_t *out_qs) {
  Context &c = ctx();
  int status = c.require();
  if (status) return status;
  if (nkeys < 1 || nkeys > 32) {
    set_error("invalid-parameter: opening keys");
    return E_PARAM;
  }
  Owned mem;
  std::vector<int> cls(nkeys);
  std::vector<const uint32_t *> hs(nkeys), cws(nkeys, nullptr);
  for (int k = 0; k < nkeys; k++) {
    cls[k] = keys[k].c;
    if (keys[k].c < 1 || keys[k].c > 30 || keys[k].ncols < 1) {
      set_error("invalid-parameter: opening key");
      return E_PARAM;
    }
    uint32_t *h = mem.alloc(((uint64_t)8) << keys[k].c);
    if (!h) return E_NOMEM;
    if ((status = combine_columns_device(8, keys[k].d_columns, keys[k].ncols, (uint64_t)1 << keys[k].c, keys[k].coef, h)))
      return status;
    hs[k] = h;
    // ENCODE-EXT of the combined column by the encoder's linearity: the same combination of the committed
    // codewords (2^(c+1) symbols per column), no transform
    if (keys[k].d_codewords) {
      uint32_t *cwk = mem.alloc(((uint64_t)16) << keys[k].c);
      if (!cwk) return E_NOMEM;
      if ((status = combine_columns_device(8, keys[k].d_codewords, keys[k].ncols, (uint64_t)2 << keys[k].c,
                                           keys[k].coef, cwk)))
        return status;
      cws[k] = cwk;
    }
  }
  std::vector<uint64_t> qs(queries > 0 ? queries : 1);
  if ((status = basefold_prove_classes(tr, nv, nkeys, cls.data(), hs.data(), rr, v, grind_bits, queries, qs.data(),
                                       nullptr, nullptr, cws.data())))
    return status;
  if (out_qs) memcpy(out_qs, qs.data(), 8 * (size_t)queries);
  for (int k = 0; k < nkeys; k++) {
    const OpenClass &key = keys[k];
    std::vector<uint64_t> leaves(queries);
    for (int q = 0; q < queries; q++) leaves[q] = qs[q] >> (nv - key.c);
    const int max_depth = cap_level_of((uint64_t)1 << (key.c - 1));
    std::vector<uint32_t> rows((size_t)queries * key.ncols * 4);
    std::vector<uint8_t> paths((size_t)queries * max_depth * 32 + 1);
    int depth = 0;
    if ((status = open_queries_device(key.d_codewords, key.ncols, key.c, key.d_levels, leaves.data(), queries,
                                      rows.data(), paths.data(), &depth)))
      return status;
    uint64_t d3[3] = {(uint64_t)queries, (uint64_t)key.ncols, 4};
    if ((status = tr.send(rows.data(), 3, d3, nullptr, false))) return status;
    if ((status = tr.send_bytes(paths.data(), (int64_t)queries * depth * 32, nullptr, false))) return status;
  }
  return OK;
}

// ---- the verifier's side of that opening, on the host (src/pcs.lisp:39-95, 581-657, 752-843)
namespace {
using Digest = std::array<uint8_t, 32>;
// LEAF-DIGEST (:44-52): rows of 4 values hashed 64 at a time, chained h = BLAKE3(h || d_i)
Digest host_leaf_digest(const uint32_t *rows, uint64_t nrows) {
  Digest h{}, d{};
  bool have = false;
  std::vector<uint8_t> buf;
  for (uint64_t start = 0; start < nrows; start += 64) {
    const uint64_t cnt = std::min<uint64_t>(64, nrows - start);
    buf.resize(16 * cnt);
    for (uint64_t k = 0; k < 4 * cnt; k++)
      for (int b = 0; b < 4; b++) buf[4 * k + b] = (uint8_t)(rows[4 * start + k] >> (8 * b));
    blake3_hash(buf.data(), buf.size(), d.data(), 32);
    if (have) {
      uint8_t hd[64];
      memcpy(hd, h.data(), 32), memcpy(hd + 32, d.data(), 32);
      blake3_hash(hd, 64, h.data(), 32);
    } else {
      h = d, have = true;
    }
  }
  return h;
}
Digest host_node(const uint8_t *left, const uint8_t *right) {  // :54-55
  uint8_t lr[64];
  Digest out;
  memcpy(lr, left, 32), memcpy(lr + 32, right, 32);
  blake3_hash(lr, 64, out.data(), 32);
  return out;
}
// the twiddle of fold level l at index s in a domain of 2^n points: level 0 holds the powers of the root in
// bit-reversed order, level l + 1 [s] = level l [2 s]^2 (src/rs.lisp:39-55)
uint32_t host_twiddle(int n, int l, uint64_t s) {
  const uint32_t w = fpow(3, (uint64_t)(P - 1) >> n);
  uint64_t i = s << l, rev = 0;
  for (int b = 0; b < n - 1; b++) rev |= ((i >> b) & 1) << (n - 2 - b);
  return fpow(fpow(w, rev), (uint64_t)1 << l);
}
// ENCODE (src/rs.lisp:60-85) of 2^(n-1) base values to 2^n symbols, for the final table's few entries
std::vector<uint32_t> host_encode(const std::vector<uint32_t> &message, int n) {
  const uint64_t len = (uint64_t)1 << n;
  std::vector<uint32_t> x(len);
  for (uint64_t i = 0; i < len; i++) x[i] = message[i % (len / 2)] % P;
  for (int b = n - 2; b >= 0; b--) {
    const uint64_t half = (uint64_t)1 << b;
    for (uint64_t k = 0; k < len / (2 * half); k++) {
      const uint32_t t = host_twiddle(n, b, k);
      for (uint64_t j = 0; j < half; j++) {
        uint32_t &a = x[2 * half * k + j], &cc = x[2 * half * k + half + j];
        const uint32_t tc = fmul(t, cc), lo = fadd(a, tc), hi = fsub(a, tc);
        a = lo, cc = hi;
      }
    }
  }
  return x;
}
}  // namespace

// CHECK-PATH with INJECTED-AT (src/pcs.lisp:86-95)
bool check_path_host(const uint8_t *h_in, const uint8_t *path, int depth, uint64_t i, const uint8_t *cap, int ninj,
                     const int *inj_level, const uint8_t *inj_digests) {
  Digest h;
  memcpy(h.data(), h_in, 32);
  for (int l = 1; l <= depth; l++) {
    const uint8_t *sib = path + 32 * (size_t)(l - 1);
    h = (i & 1) ? host_node(sib, h.data()) : host_node(h.data(), sib);
    i >>= 1;
    for (int k = 0; k < ninj; k++)
      if (inj_level[k] == l) h = host_node(h.data(), inj_digests + 32 * (size_t)k);
  }
  return memcmp(h.data(), cap + 32 * i, 32) == 0;
}

static int reject(const std::string &what) {
  set_error("verification-failure: pcs: " + what);
  return E_REJECT;
}

int pcs_verify_opening(Transcript &tr, int nv, int nkeys, const OpenClass *keys, const uint32_t *rr, const uint32_t *v,
                       int grind_bits, int queries) {
  if (nkeys < 1 || nkeys > 32 || keys[nkeys - 1].c != nv || queries < 1) {
    set_error("invalid-parameter: opening keys");
    return E_PARAM;
  }
  const int fl = nv - 5 > 0 ? nv - 5 : 0, Q = queries;
  int status;
  hf::E prf = hf::lift(1, 8), claim = hf::from(v, 8);
  std::vector<hf::E> chal;
  std::vector<int> olv;
  std::vector<std::vector<uint8_t>> caps;
  for (int i = 0; i < fl; i++) {  // BASEFOLD, the verifier's side
    uint32_t ev[24], x[8];
    uint64_t dims[2] = {3, 8};
    if ((status = tr.send(nullptr, 2, dims, ev))) return status;
    if (hf::add(hf::from(ev, 8), hf::from(ev + 8, 8)) != claim) return reject("basefold sumcheck round " + std::to_string(i) + " failed");
    tr.challenge(8, x);
    chal.push_back(hf::from(x, 8));
    claim = hf::lagrange({hf::from(ev, 8), hf::from(ev + 8, 8), hf::from(ev + 16, 8)}, hf::from(x, 8));
    prf = hf::mul(prf, hf::eq1(hf::from(rr + 8 * (size_t)i, 8), hf::from(x, 8)));
    const int l = i + 1;
    if (l >= 2 && l < fl && l % 2 == 0) {
      std::vector<uint8_t> cap;
      if ((status = tr.send_bytes(nullptr, -1, &cap))) return status;
      olv.push_back(l);
      caps.push_back(cap);
    }
  }
  const uint64_t mlen = (uint64_t)1 << (nv - fl);
  std::vector<uint32_t> m(mlen * 8);
  {
    uint64_t dims[2] = {mlen, 8};
    if ((status = tr.send(nullptr, 2, dims, m.data()))) return status;
    hf::E mval = fl < nv ? hf::mle_eval(m.data(), nv - fl, rr + 8 * (size_t)fl, 8) : hf::from(m.data(), 8);
    if (hf::mul(prf, mval) != claim) return reject("basefold final claim");
  }
  uint64_t nonce;
  if ((status = tr.verify_grind(grind_bits, &nonce))) return status;
  std::vector<uint64_t> qs(Q);
  tr.challenge_bits(nv - 1, Q, qs.data());
  // ---- VERIFY-QUERIES: the oracles' leaves and paths (:763-774)
  std::vector<std::vector<uint32_t>> oleaves(olv.size());
  for (size_t o = 0; o < olv.size(); o++) {
    const int l = olv[o];
    const uint64_t nleaves = (uint64_t)1 << (nv - 1 - l);
    const int depth = cap_level_of(nleaves);
    uint64_t d3[3] = {(uint64_t)Q, 8, 4};
    oleaves[o].assign((size_t)Q * 32, 0);
    std::vector<uint8_t> paths;
    if ((status = tr.send(nullptr, 3, d3, oleaves[o].data(), false))) return status;
    if ((status = tr.send_bytes(nullptr, -1, &paths, false))) return status;
    if (paths.size() != (size_t)Q * depth * 32) return reject("merkle path length");
    if (caps[o].size() != 32 * (nleaves >> depth)) return reject("oracle opening shape");
    for (int q = 0; q < Q; q++) {
      const Digest h = host_leaf_digest(oleaves[o].data() + 32 * (size_t)q, 8);
      if (!check_path_host(h.data(), paths.data() + 32 * (size_t)q * depth, depth, qs[q] >> l, caps[o].data(), 0, nullptr,
                           nullptr))
        return reject("oracle merkle path");
    }
  }
  // every key's leaves and its tree's paths; inj_c += sum_k coef_k leaf_k (:776-808)
  std::vector<std::vector<hf::E>> inj(nkeys, std::vector<hf::E>((size_t)Q * 4, hf::zero(8)));
  for (int k = 0; k < nkeys; k++) {
    const OpenClass &key = keys[k];
    if (key.c < 1 || key.c > nv || (k && key.c <= keys[k - 1].c)) {
      set_error("invalid-parameter: opening keys must ascend in class");
      return E_PARAM;
    }
    const uint64_t nleaves = (uint64_t)1 << (key.c - 1);
    const int depth = cap_level_of(nleaves), nc = key.ncols;
    uint64_t d3[3] = {(uint64_t)Q, (uint64_t)nc, 4};
    std::vector<uint32_t> leaves((size_t)Q * nc * 4);
    std::vector<uint8_t> paths;
    if ((status = tr.send(nullptr, 3, d3, leaves.data(), false))) return status;
    if ((status = tr.send_bytes(nullptr, -1, &paths, false))) return status;
    if (paths.size() != (size_t)Q * depth * 32) return reject("merkle path length");
    for (int q = 0; q < Q; q++) {
      const Digest h = host_leaf_digest(leaves.data() + (size_t)q * nc * 4, nc);
      if (!check_path_host(h.data(), paths.data() + 32 * (size_t)q * depth, depth, qs[q] >> (nv - key.c), key.cap, 0,
                           nullptr, nullptr))
        return reject("merkle path of class " + std::to_string(key.c));
      for (int sy = 0; sy < 4; sy++) {
        hf::E &held = inj[k][(size_t)q * 4 + sy];
        for (int col = 0; col < nc; col++)
          held = hf::add(held, hf::scale(hf::from(key.coef + 8 * (size_t)col, 8), leaves[((size_t)q * nc + col) * 4 + sy]));
      }
    }
  }
  // fold each query's symbols down to the final table's codeword (:810-843)
  std::vector<std::vector<uint32_t>> menc(8);
  for (int d = 0; d < 8; d++) {  // ENCODE-EXT of the final table, coordinate by coordinate
    std::vector<uint32_t> col(mlen);
    for (uint64_t i = 0; i < mlen; i++) col[i] = m[i * 8 + d];
    menc[d] = host_encode(col, nv - fl + 1);
  }
  const uint32_t inv2 = finv(2);
  for (int q = 0; q < Q; q++) {
    uint64_t base = 4 * qs[q];
    std::vector<hf::E> held(4, hf::zero(8));
    for (int level = 0; level <= fl; level++) {
      if (level > 0) {
        const int l = level - 1;
        std::vector<hf::E> next;
        for (size_t t2 = 0; t2 + 1 < held.size(); t2 += 2) {  // RS:FOLD (src/rs.lisp:93-101)
          const uint64_t sidx = base / 2 + t2 / 2;
          const hf::E &a = held[t2], &b = held[t2 + 1];
          const hf::E f0 = hf::scale(hf::add(a, b), inv2);
          const hf::E f1 = hf::scale(hf::sub(a, b), finv(fmul(2, host_twiddle(nv + 1, l, sidx))));
          next.push_back(hf::add(f0, hf::mul(chal[l], hf::sub(f1, f0))));
        }
        held = next;
        base /= 2;
        for (size_t o = 0; o < olv.size(); o++)
          if (olv[o] == level) {
            const uint32_t *leaf = oleaves[o].data() + 32 * (size_t)q;
            const uint64_t ob = 4 * (qs[q] >> level);
            std::vector<hf::E> sym(4, hf::zero(8));
            for (int sy = 0; sy < 4; sy++)
              for (int d = 0; d < 8; d++) sym[sy][d] = leaf[4 * d + sy];
            if (sym[base - ob] != held[0]) return reject("fold consistency");
            held = sym;
            base = ob;
          }
      }
      for (int k = 0; k < nkeys; k++)  // INJECT
        if (nv - keys[k].c == level) {
          const uint64_t cb = 4 * (qs[q] >> level);
          for (size_t sy = 0; sy < held.size(); sy++)
            held[sy] = hf::add(held[sy], inj[k][(size_t)q * 4 + (base - cb) + sy]);
        }
    }
    for (size_t sy = 0; sy < held.size(); sy++)
      for (int d = 0; d < 8; d++)
        if (held[sy][d] != menc[d][base + sy]) return reject("final codeword consistency");
  }
  return OK;
}

int basefold_verify(Transcript &tr, int nv, const uint32_t *rr, const uint32_t *v, int grind_bits, int queries,
                    uint64_t *out_qs) {
  const int fl = nv - 5 > 0 ? nv - 5 : 0;
  int status;
  hf::E prf = hf::lift(1, 8), claim = hf::from(v, 8);
  for (int i = 0; i < fl; i++) {
    uint32_t ev[24], x[8];
    uint64_t dims[2] = {3, 8};
    if ((status = tr.send(nullptr, 2, dims, ev))) return status;
    if (hf::add(hf::from(ev, 8), hf::from(ev + 8, 8)) != claim) {
      set_error("verification-failure: pcs: basefold sumcheck round " + std::to_string(i) + " failed");
      return E_REJECT;
    }
    tr.challenge(8, x);
    claim = hf::lagrange({hf::from(ev, 8), hf::from(ev + 8, 8), hf::from(ev + 16, 8)}, hf::from(x, 8));
    prf = hf::mul(prf, hf::eq1(hf::from(rr + 8 * i, 8), hf::from(x, 8)));
    int l = i + 1;
    if (l >= 2 && l < fl && l % 2 == 0) {
      uint64_t nleaves = ((uint64_t)1 << (nv + 1 - l)) / 4;
      uint64_t rows = nleaves >> cap_level_of(nleaves);
      if ((status = tr.send_bytes(nullptr, (int64_t)(32 * rows), nullptr))) return status;
    }
  }
  uint64_t mlen = (uint64_t)1 << (nv - fl);
  std::vector<uint32_t> m(mlen * 8);
  uint64_t dims[2] = {mlen, 8};
  if ((status = tr.send(nullptr, 2, dims, m.data()))) return status;
  hf::E mval = fl < nv ? hf::mle_eval(m.data(), nv - fl, rr + 8 * fl, 8) : hf::from(m.data(), 8);
  if (hf::mul(prf, mval) != claim) {
    set_error("verification-failure: pcs: basefold final claim");
    return E_REJECT;
  }
  uint64_t nonce;
  if ((status = tr.verify_grind(grind_bits, &nonce))) return status;
  std::vector<uint64_t> qs(queries);
  tr.challenge_bits(nv - 1, queries, qs.data());
  if (out_qs) memcpy(out_qs, qs.data(), 8 * (size_t)queries);
  return OK;
}

}  // namespace exh
