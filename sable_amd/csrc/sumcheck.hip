// sumcheck.hip -- sumcheck session: weight tables, round launches, partial-sum reduction, folds.
#include "sumcheck.hpp"

#include <mutex>
#include "rtc.hpp"
#include <atomic>

#include <string.h>

#include <map>

#include "context.hpp"
#include "hostfield.hpp"
#include "interp.hpp"

namespace exh {

// ------------------------------------------------------------------ small kernels

// eq weights for every round in one launch.  Table k covers the eq point's variables
// [first, first + bits): entry x = prod_b (x_b ? r_b : 1 - r_b) (src/field.lisp:354-363: bit b of the
// index pairs with the b-th variable).  factors[v] = (r_v R, (1 - r_v) R): each product is exact.
struct EqTables {
  int count;
  uint64_t off[64];  // in EXTs
  int first[64], bits[64];
};

// (both set-up kernels also clear the totals of the grid launch of LDS-resident slices: the first launch of a
// session is the one place that comes before every use)
// `staged` (null: none): the session's constants as the host staged them in pinned memory, `staged_words` of them,
// factors first; the launch brings them to `staged_dst` for the launches behind it (in place of a copy on the
// stream before it) and takes the factors from there itself.
template <int D>
__global__ __launch_bounds__(BLOCK) void eq_tables_kernel(EqTables tabs, const uint32_t *factors,
                                                          uint32_t n_factor_words, uint32_t *out, uint64_t total,
                                                          uint32_t *zero, uint64_t zero_words,
                                                          const uint32_t *staged = nullptr, uint32_t staged_words = 0,
                                                          uint32_t *staged_dst = nullptr) {
  uint64_t gid = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
  for (uint64_t z = gid; z < zero_words; z += (uint64_t)gridDim.x * BLOCK) zero[z] = 0;
  if (staged) {
    for (uint64_t z = gid; z < staged_words; z += (uint64_t)gridDim.x * BLOCK) staged_dst[z] = staged[z];
    factors = staged;
  }
  // every variable's two factors into LDS first: an entry is a chain of up to `bits` products, and a load from
  // memory inside each link is most of the kernel's time
  __shared__ uint32_t lds_factors[2 * MAXROUNDS * 8];
  for (uint32_t u = threadIdx.x; u < n_factor_words; u += BLOCK) lds_factors[u] = factors[u];
  __syncthreads();
  if (gid >= total) return;
  int k = 0;
  uint64_t start = 0;
  while (k + 1 < tabs.count && gid >= start + ((uint64_t)1 << tabs.bits[k])) {
    start += (uint64_t)1 << tabs.bits[k];
    k++;
  }
  uint64_t x = gid - start;
  Ext<D> e = ext_lift<D>(1);
  for (int b = 0; b < tabs.bits[k]; b++) {
    const uint32_t *f = lds_factors + ((size_t)(tabs.first[k] + b) * 2 + (((x >> b) & 1) ? 0 : 1)) * D;
    Ext<D> fe;
#pragma unroll
    for (int c = 0; c < D; c++) fe.c[c] = f[c];
    e = ext_mul_mont<D>(e, fe);
  }
  store_ext<D>(out + (tabs.off[k] + x) * D, e);
}

template <int D>
__global__ __launch_bounds__(BLOCK) void fill_ones_kernel(uint32_t *out, uint64_t n, uint32_t *zero, uint64_t zero_words,
                                                          const uint32_t *staged = nullptr, uint32_t staged_words = 0,
                                                          uint32_t *staged_dst = nullptr) {
  uint64_t gid = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
  for (uint64_t z = gid; z < zero_words; z += (uint64_t)gridDim.x * BLOCK) zero[z] = 0;
  if (staged)
    for (uint64_t z = gid; z < staged_words; z += (uint64_t)gridDim.x * BLOCK) staged_dst[z] = staged[z];
  if (gid < n) store_ext<D>(out + gid * D, ext_lift<D>(1));
}

// base values lifted to (v, 0, ..., 0) (src/sumcheck.lisp:75-82)
template <int D>
__global__ __launch_bounds__(BLOCK) void lift_kernel(const uint32_t *in, uint32_t *out, uint64_t n) {
  uint64_t gid = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
  if (gid < n) store_ext<D>(out + gid * D, ext_lift<D>(in[gid]));
}

// one fold without sums (the last round): thread per folded entry
template <int D, bool IN_BASE>
__global__ __launch_bounds__(BLOCK) void fold_kernel(const uint32_t *in, uint32_t *out, uint64_t n_out,
                                                     RoundArgs<D> args) {
  uint64_t gid = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
  if (gid >= n_out) return;
  Ext<D> r;
#pragma unroll
  for (int c = 0; c < D; c++) r.c[c] = args.r_mont[c];
  Ext<D> o;
  if constexpr (IN_BASE) {
    uint2 e = *reinterpret_cast<const uint2 *>(in + 2 * gid);
    o = fold_base<D>(e.x, e.y, r);
  } else {
    o = fold_ext<D>(load_ext<D>(in + 2 * gid * D), load_ext<D>(in + (2 * gid + 1) * D), r);
  }
  store_ext<D>(out + gid * D, o);
}

// sums[o] = sum over the workgroups' partials: one workgroup per output word
__global__ __launch_bounds__(BLOCK) void reduce_partials_kernel(const uint32_t *partials, uint32_t nblocks,
                                                                uint32_t stride, uint32_t *sums) {
  __shared__ uint32_t lds[BLOCK / 64];
  uint32_t o = blockIdx.x, v = 0;
  for (uint32_t b = threadIdx.x; b < nblocks; b += BLOCK) v = fadd(v, partials[(uint64_t)b * stride + o]);
  v = wave_sum(v);
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < BLOCK / 64; w++) v = fadd(v, lds[w]);
    sums[o] = v;
  }
}

// the interpreter's launchers live in interp.hip (one translation unit per degree and kind: they are the
// slowest kernels of the library to compile)
// ------------------------------------------------------------------ registry of generated kernels
static std::map<std::pair<std::string, int>, KernelSet> &registry() {
  static std::map<std::pair<std::string, int>, KernelSet> r;
  return r;
}
static std::mutex g_registry_mutex;  // (proofs may run on two host threads: see side_context)
void register_kernels(const std::string &key, int D, KernelSet set) {
  std::lock_guard<std::mutex> lock(g_registry_mutex);
  registry()[{key, D}] = set;
}
const KernelSet *find_kernels(const std::string &key, int D) {
  std::lock_guard<std::mutex> lock(g_registry_mutex);
  auto it = registry().find({key, D});
  return it == registry().end() ? nullptr : &it->second;
}

// ------------------------------------------------------------------ the session
// regions of the context's pinned host buffer (in words): per-round results | the session's eq point
// and block weights | the device loop's constants | the device loop's logs and final tables
constexpr uint32_t SLICE_GROUPS = 16;  // rows of totals per round of a grid launch of LDS-resident slices
constexpr uint32_t ROUND_GROUPS = 32;  // rows of totals of a streaming round (its workgroups' atomics spread over them)
constexpr size_t PIN_BEGIN = 16384, PIN_BEGIN_WORDS = 4096;
constexpr size_t PIN_LOOP = PIN_BEGIN + PIN_BEGIN_WORDS, PIN_LOOP_WORDS = 12288;
constexpr size_t PIN_DOWN = PIN_LOOP + PIN_LOOP_WORDS, PIN_DOWN_WORDS = 32768;
static inline uint32_t next_pow2(uint64_t v) {
  uint32_t p = 1;
  while (p < v) p <<= 1;
  return p;
}

static uint32_t tile_pairs_per_thread(uint64_t n_pairs, uint64_t max_grid, uint64_t low_span);

int SumcheckSession::begin(const Statement &statement, int D_, int n_, const uint32_t *const *tables,
                           const int *strides, const uint32_t *eq, const uint32_t *bw, int K_, const uint32_t *consts,
                           int degree, bool claim_mode_, bool defer_setup) {
  Context &c = ctx();
  int status = c.require();
  if (status) return status;
  D = D_, n = n_, K = K_;
  epoch = ++c.session_epoch;
  if ((D != 4 && D != 8) || n < 0 || n > 40 || K < 1) {
    set_error("invalid-parameter: sumcheck shape");
    return E_PARAM;
  }
  st = statement;
  if (degree < 0) degree = st.degree;
  points = degree > 1 ? degree : 1;
  claim_mode = claim_mode_;
  if (claim_mode)
    st.plan_claim();
  else
    st.plan(points);
  eq0.clear();
  if (eq && n > 0) eq0.assign(eq, eq + D);
  int T = st.T();
  if (T > MAXT || points > 16 || !make_desc(st, &desc)) {
    set_error("invalid-parameter: statement beyond the kernels' limits");
    beyond_limits = true;
    return E_PARAM;
  }
  (void)rtc_collect();
  kernels = find_kernels(st.key(), D);
  generated = kernels != nullptr;
  if (st.direct) {
    // a statement in direct form has no interpreter to fall back on: without its kernels the caller takes another
    // way (beyond_limits: the statement in parts).  Like any unseen statement it is compiled in the background
    // when the tables are large enough for the difference to matter, for the next proof; exh_stmt_generate asks
    // for the kernels ahead of time and can wait for them.
    if (claim_mode || st.nacc != points) {
      set_error("invalid-parameter: a statement in direct form is proved at the wire points it was made for");
      return E_PARAM;
    }
    if (!generated) {
      static const int min_n = getenv("EXACTA_HIP_RTC_MIN_N") ? atoi(getenv("EXACTA_HIP_RTC_MIN_N")) : 20;
      if (rtc_enabled() && n >= min_n) rtc_request(st.key(), desc, D, direct_source(st, desc, "RtStmt"));
      set_error("invalid-parameter: the kernels of the statement in direct form are not compiled (yet)");
      beyond_limits = true;
      return E_PARAM;
    }
  }
  if (!generated && !claim_mode && rtc_enabled()) {
    // no kernel yet for this statement: the interpreter serves this proof; for tables large enough for the
    // difference to matter, kernels are compiled in the background for the next one
    static const int min_n = getenv("EXACTA_HIP_RTC_MIN_N") ? atoi(getenv("EXACTA_HIP_RTC_MIN_N")) : 20;
    if (n >= min_n) rtc_request(st.key(), desc, D);
  }
  has_eq = eq != nullptr;
  has_bw = bw != nullptr;
  size = (uint64_t)K << n;
  round = 0;
  pending_fold = false;
  generation = 0;
  group_coef.assign(st.groups.size() * D, 0);
  group_coefficients(st, D, consts, group_coef.data());
  bw_sum.assign(D, 0);
  if (has_bw) {
    for (int b = 0; b < K; b++)
      for (int k = 0; k < D; k++) bw_sum[k] = fadd(bw_sum[k], bw[(size_t)b * D + k] % P);
  }

  // ---- layout of the misc arena: eq factors | weight tables | bw | ones | partials | sums | lifted
  low_off.assign(n, 0), high_off.assign(n, 0), low_bits.assign(n, 0), n_high.assign(n, 0);
  EqTables eqt;
  memset(&eqt, 0, sizeof(eqt));
  uint64_t pos = (uint64_t)2 * n;  // in EXTs: the eq factors come first
  uint64_t bw_off = 0, ones_off = 0, ones_len = 0, total_eq = 0;
  if (has_bw) {
    bw_off = pos;
    pos += K;
  }
  // the device-driven loop's constants follow at once, so that one copy can bring the eq point, the
  // block weights, the message map, the constant-group terms and the control block's head
  const uint64_t mt_words = (uint64_t)points * std::max(st.nacc, 1) * D, c0_words = (uint64_t)std::max(n, 1) * points * D;
  const uint64_t mt_off = pos * D, c0_off = mt_off + mt_words, ctrl_off = c0_off + c0_words;
  pos += (mt_words + c0_words + (sizeof(Ctrl) + 3) / 4 + D - 1) / D;
  for (int j = 0; j < n; j++) {
    // LOW takes the lower half of the remaining variables as in SPLIT-WEIGHTS, but at least as many as a
    // workgroup's tile of pairs spans (2^13), so that one HIGH weight covers the tile and is applied
    // once per workgroup; the weights are the same products either way
    int from = j + 1, rest = n - from;
    int middle = has_bw ? n : from + std::max(rest / 2, std::min(rest, 13));
    low_bits[j] = middle - from;
    n_high[j] = has_bw ? (uint64_t)K : (uint64_t)1 << (n - middle);
    if (has_eq) {
      if (eqt.count + 2 > 64) {
        set_error("invalid-parameter: too many rounds");
        return E_PARAM;
      }
      low_off[j] = pos;
      eqt.off[eqt.count] = pos, eqt.first[eqt.count] = from, eqt.bits[eqt.count] = middle - from;
      eqt.count++;
      pos += (uint64_t)1 << (middle - from);
      total_eq += (uint64_t)1 << (middle - from);
      if (!has_bw) {
        high_off[j] = pos;
        eqt.off[eqt.count] = pos, eqt.first[eqt.count] = middle, eqt.bits[eqt.count] = n - middle;
        eqt.count++;
        pos += (uint64_t)1 << (n - middle);
        total_eq += (uint64_t)1 << (n - middle);
      }
    } else {
      ones_len = std::max(ones_len, std::max((uint64_t)1 << low_bits[j], n_high[j]));
    }
    if (has_bw) high_off[j] = bw_off;
  }
  if (!has_eq && n > 0) {
    ones_off = pos;
    pos += ones_len;
    for (int j = 0; j < n; j++) {
      low_off[j] = ones_off;
      if (!has_bw) high_off[j] = ones_off;
    }
  }
  uint64_t pairs0 = size / 2;
  max_grid = pairs0 ? (pairs0 + BLOCK - 1) / BLOCK : 1;
  // two workgroups per compute unit: the round kernels' registers let three be resident, so a grid of four per
  // unit ran a third of its workgroups in a second, thin wave (measured: 512 workgroups beat 1024 by 3 % of the
  // prove, 256 lose 15 %)
  const uint64_t grid_cap = std::min<uint64_t>(1024, 2 * (uint64_t)std::max(c.compute_units, 1));
  if (max_grid > grid_cap) max_grid = grid_cap;
  node_slots_n = node_slots(desc);  // grid sums of the sweep that serves rounds 0 and 1 from the base tables
  pstride = next_pow2((uint64_t)std::max(std::max(st.nacc, 1), node_slots_n <= MAXACC ? node_slots_n : 0) * D);
  uint64_t partial_off = pos * D;  // from here in words
  // (a workgroup's partial row per workgroup of the largest grid a round can take: tiles stop growing at the span
  // of a HIGH weight, see tile_pairs_per_thread)
  uint64_t partial_rows = max_grid;
  for (int j = 0; j < n; j++) {
    const uint64_t pairs = (size >> j) / 2, tile = (uint64_t)BLOCK * tile_pairs_per_thread(pairs, max_grid, (uint64_t)1 << low_bits[j]);
    partial_rows = std::max(partial_rows, (pairs + tile - 1) / tile);
  }
  uint64_t words = partial_off + (partial_rows + 1) * (uint64_t)pstride + 64;
  words += 64;
  words += words & 1;  // the 64-bit totals of the grid launch of slices: [MAXTAIL][SLICE_GROUPS][pstride]
  const uint64_t slice_totals_off = words;
  words += (uint64_t)2 * MAXTAIL * SLICE_GROUPS * pstride;
  // the streaming rounds' own totals ([round][ROUND_GROUPS][pstride] 64-bit words) and arrival counters follow, so
  // that the set-up kernel clears them all in one go
  const uint64_t round_totals_off = words;
  words += (uint64_t)2 * std::max(n, 1) * ROUND_GROUPS * pstride;
  const uint64_t arrivals_off = words;
  words += (uint64_t)std::max(n, 1) + 1;
  words += words & 1;
  zeroed_words = words - slice_totals_off;
  // mixed base / extension inputs: lift the base ones
  bool any_base = false, all_base = true;
  for (int t = 0; t < T; t++) {
    if (strides[t] == 1)
      any_base = true;
    else if (strides[t] == D)
      all_base = false;
    else {
      set_error("invalid-parameter: table stride must be 1 or D");
      return E_PARAM;
    }
  }
  uint64_t lifted_off = words;
  if (any_base && !all_base)
    for (int t = 0; t < T; t++)
      if (strides[t] == 1) words += size * D;
  const uint64_t direct_off = words;  // a direct statement's constant slots
  if (st.direct) words += (uint64_t)std::max(st.direct_slots, 1) * D;
  if ((status = arena_misc().reserve(words * 4))) return status;
  uint32_t *base = (uint32_t *)arena_misc().ptr;
  d_weights = base;
  d_partials = base + partial_off;
  d_sums = d_partials + partial_rows * (uint64_t)pstride;
  d_slice_totals = reinterpret_cast<unsigned long long *>(base + slice_totals_off);
  d_round_totals = reinterpret_cast<unsigned long long *>(base + round_totals_off);
  d_arrivals = base + arrivals_off;
  d_ctrl = reinterpret_cast<Ctrl *>(base + ctrl_off);
  d_mtilde = base + mt_off;
  d_c0 = base + c0_off;
  d_direct = nullptr;
  if (st.direct) {
    d_direct = base + direct_off;
    direct_host.assign((size_t)std::max(st.direct_slots, 1) * D, 0u);
    if (st.direct_slots) direct_slot_values(st, D, consts, direct_host.data());
    for (uint32_t &w : direct_host) w = to_mont(w);
    EXH_HIP(hipMemcpyAsync(d_direct, direct_host.data(), direct_host.size() * 4, hipMemcpyHostToDevice, c.stream));
  }

  cur.assign(T, nullptr);
  cur_base = all_base;
  for (int t = 0; t < T; t++) cur[t] = tables[t];
  if (any_base && !all_base) {
    uint32_t *dst = base + lifted_off;
    for (int t = 0; t < T; t++)
      if (strides[t] == 1) {
        uint32_t grid = (uint32_t)((size + BLOCK - 1) / BLOCK);
        if (D == 4)
          hipLaunchKernelGGL(lift_kernel<4>, dim3(grid), dim3(BLOCK), 0, c.stream, tables[t], dst, size);
        else
          hipLaunchKernelGGL(lift_kernel<8>, dim3(grid), dim3(BLOCK), 0, c.stream, tables[t], dst, size);
        cur[t] = dst;
        dst += size * D;
      }
  }

  // ---- upload the eq factors and block weights, build the weight tables
  // staged in pinned memory when it fits (no wait: the region is not written again before this
  // session's next wait), else in a vector that must outlive the copy
  const size_t host_words = (size_t)(2 * n + (has_bw ? K : 0)) * D;
  // (a session with buffers of its own may be one of several begun back to back: each waits for its copy)
  const bool staged = host_words <= PIN_BEGIN_WORDS && !private_buffers;
  std::vector<uint32_t> spill(staged ? 0 : host_words, 0);
  uint32_t *host = staged ? c.host_pinned + PIN_BEGIN : spill.data();
  if (staged) memset(host, 0, host_words * 4);
  if (has_eq)
    for (int v = 0; v < n; v++)
      for (int k = 0; k < D; k++) {
        uint32_t r = eq[(size_t)v * D + k] % P, one_minus = fsub(k == 0 ? 1u : 0u, r);
        host[((size_t)v * 2) * D + k] = to_mont(r);
        host[((size_t)v * 2 + 1) * D + k] = to_mont(one_minus);
      }
  if (has_bw)
    for (size_t i = 0; i < (size_t)K * D; i++) host[(size_t)2 * n * D + i] = bw[i] % P;
  static_assert(sizeof(EqTables) <= sizeof(setup.eqt), "EqTables outgrew its stash");
  memcpy(setup.eqt, &eqt, sizeof(eqt));
  setup.total_eq = has_eq ? total_eq : 0;
  setup.ones_off = ones_off, setup.ones_len = has_eq ? 0 : ones_len;
  setup_words = host_words;
  setup_deferred = defer_setup && staged;
  if (!setup_deferred) {
    if (host_words) EXH_HIP(hipMemcpyAsync(base, host, host_words * 4, hipMemcpyHostToDevice, c.stream));
    if (!staged) EXH_HIP(hipStreamSynchronize(c.stream));
    if ((status = launch_setup())) return status;
  }
  // the folded generations: the first holds half the input, the second a quarter
  if (n > 0) {
    if ((status = arena_a().reserve((size_t)T * (size / 2) * D * 4))) return status;
    if (n > 1 && (status = arena_b().reserve((size_t)T * (size / 4) * D * 4))) return status;
  }
  EXH_HIP(hipGetLastError());
  return OK;
}

// the weight tables of every round from the eq point's factors (or all-ones tables without one)
// EQ-TABLE (src/field.lisp:354-363) of a point of k coordinates, left on the device: entry x is the product over
// b of (x_b ? r_b : 1 - r_b).  The same kernel as the sessions' weight tables, over one table.
int eq_table_device(int D, int k, const uint32_t *r, uint32_t *d_out) {
  Context &c = ctx();
  int status = c.require();
  if (status) return status;
  if (k == 0) {
    uint32_t one[8] = {1, 0, 0, 0, 0, 0, 0, 0};
    EXH_HIP(hipMemcpyAsync(d_out, one, (size_t)D * 4, hipMemcpyHostToDevice, c.stream));
    EXH_HIP(hipStreamSynchronize(c.stream));
    return OK;
  }
  std::vector<uint32_t> factors((size_t)2 * k * D);
  for (int v = 0; v < k; v++)
    for (int cc = 0; cc < D; cc++) {
      uint32_t rv = r[(size_t)v * D + cc] % P;
      factors[((size_t)v * 2) * D + cc] = to_mont(rv);
      factors[((size_t)v * 2 + 1) * D + cc] = to_mont(fsub(cc == 0 ? 1u : 0u, rv));
    }
  uint32_t *d_factors = (uint32_t *)c.pool.alloc(factors.size() * 4);
  if (!d_factors) {
    set_error("device-out-of-memory: eq factors");
    return E_NOMEM;
  }
  struct Release {  // the pooled buffer goes back on every way out
    Pool &pool;
    void *ptr;
    ~Release() { pool.release(ptr); }
  } release{c.pool, d_factors};
  EXH_HIP(hipMemcpyAsync(d_factors, factors.data(), factors.size() * 4, hipMemcpyHostToDevice, c.stream));
  EqTables eqt;
  memset(&eqt, 0, sizeof(eqt));
  eqt.count = 1, eqt.off[0] = 0, eqt.first[0] = 0, eqt.bits[0] = k;
  const uint64_t total = (uint64_t)1 << k;
  uint32_t grid = (uint32_t)((total + BLOCK - 1) / BLOCK);
  if (D == 4)
    hipLaunchKernelGGL(eq_tables_kernel<4>, dim3(grid), dim3(BLOCK), 0, c.stream, eqt, d_factors,
                       (uint32_t)factors.size(), d_out, total, nullptr, (uint64_t)0);
  else
    hipLaunchKernelGGL(eq_tables_kernel<8>, dim3(grid), dim3(BLOCK), 0, c.stream, eqt, d_factors,
                       (uint32_t)factors.size(), d_out, total, nullptr, (uint64_t)0);
  EXH_HIP(hipGetLastError());
  EXH_HIP(hipStreamSynchronize(c.stream));  // `factors` (pageable) and the pooled buffer are free to go after this
  return OK;
}

// Eq tables over ranges of a point's variables, one launch: table k covers the variables [first[k], first[k] +
// bits[k]) and lands at d_out + off[k] * D (2^bits[k] elements); d_factors holds (r_v R, (1 - r_v) R) per variable,
// 2 n_vars D words.  At most 64 tables.  Enqueued on the context's stream; nothing is waited for.
int eq_tables_launch(int D, int count, const int *first, const int *bits, const uint64_t *off,
                     const uint32_t *d_factors, int n_vars, uint32_t *d_out) {
  Context &c = ctx();
  if (count < 1 || count > 64 || n_vars > MAXROUNDS || (D != 4 && D != 8)) {
    set_error("invalid-parameter: eq tables (at most 64 tables over at most 48 variables)");
    return E_PARAM;
  }
  EqTables eqt;
  memset(&eqt, 0, sizeof(eqt));
  eqt.count = count;
  uint64_t total = 0;
  for (int k = 0; k < count; k++) {
    eqt.off[k] = off[k], eqt.first[k] = first[k], eqt.bits[k] = bits[k];
    total += (uint64_t)1 << bits[k];
  }
  const uint32_t grid = (uint32_t)((total + BLOCK - 1) / BLOCK);
  if (D == 4)
    hipLaunchKernelGGL(eq_tables_kernel<4>, dim3(grid), dim3(BLOCK), 0, c.stream, eqt, d_factors,
                       (uint32_t)(2 * n_vars * D), d_out, total, nullptr, (uint64_t)0);
  else
    hipLaunchKernelGGL(eq_tables_kernel<8>, dim3(grid), dim3(BLOCK), 0, c.stream, eqt, d_factors,
                       (uint32_t)(2 * n_vars * D), d_out, total, nullptr, (uint64_t)0);
  EXH_HIP(hipGetLastError());
  return OK;
}

static uint64_t tail_pairs(int T, int D);

int SumcheckSession::launch_setup(const uint32_t *staged, size_t staged_words) {
  Context &c = ctx();
  uint32_t *base = d_weights;
  EqTables eqt;
  memcpy(&eqt, setup.eqt, sizeof(eqt));
  // a session whose first round fits the one-workgroup launch never takes the grid launch
  uint32_t *zero = reinterpret_cast<uint32_t *>(d_slice_totals);
  uint64_t zero_words = size / 2 > tail_pairs(st.T(), D) ? zeroed_words : 0;
  const uint32_t zero_grid = (uint32_t)((zero_words + 4 * BLOCK - 1) / (4 * BLOCK));  // four words a thread
  bool cleared = false;
  c.prof_begin("weights", 0, 0);
  if (setup.total_eq) {
    uint32_t grid = std::max((uint32_t)((setup.total_eq + BLOCK - 1) / BLOCK), zero_grid);
    // tables are laid out in launch order, so thread gid maps to table k by running sums; the
    // offsets themselves may skip other regions, so they are taken from eqt.off
    if (D == 4)
      hipLaunchKernelGGL(eq_tables_kernel<4>, dim3(grid), dim3(BLOCK), 0, c.stream, eqt, base, (uint32_t)(2 * n * D), base,
                         setup.total_eq, zero, zero_words, staged, (uint32_t)staged_words, base);
    else
      hipLaunchKernelGGL(eq_tables_kernel<8>, dim3(grid), dim3(BLOCK), 0, c.stream, eqt, base, (uint32_t)(2 * n * D), base,
                         setup.total_eq, zero, zero_words, staged, (uint32_t)staged_words, base);
    cleared = zero_words > 0;
    zero_words = 0;
    staged = nullptr;
  }
  if (setup.ones_len) {
    uint32_t grid = std::max((uint32_t)((setup.ones_len + BLOCK - 1) / BLOCK), zero_words ? zero_grid : 0u);
    if (D == 4)
      hipLaunchKernelGGL(fill_ones_kernel<4>, dim3(grid), dim3(BLOCK), 0, c.stream, base + setup.ones_off * D,
                         setup.ones_len, zero, zero_words, staged, (uint32_t)staged_words, base);
    else
      hipLaunchKernelGGL(fill_ones_kernel<8>, dim3(grid), dim3(BLOCK), 0, c.stream, base + setup.ones_off * D,
                         setup.ones_len, zero, zero_words, staged, (uint32_t)staged_words, base);
    staged = nullptr;
    cleared = cleared || zero_words > 0;
    zero_words = 0;
  }
  c.prof_end();
  slice_totals_clear = cleared;  // else (no set-up kernel ran) the grid launch clears them itself
  EXH_HIP(hipGetLastError());
  if (staged) {  // (no set-up kernel ran)
    set_error("device-error: the session's staged constants were left behind");
    return E_DEVICE;
  }
  return OK;
}

// Pairs per thread of a streaming launch over n_pairs pairs: a tile (BLOCK * pairs per thread) grows to fit the
// grid's cap, but not beyond the span of one HIGH weight when it can stay within it -- the weight is then applied
// once per workgroup, where a larger tile would pay an extension product per pair; the grid is larger instead, and
// its workgroups follow one another.  low_span: 2^low_bits of the round, 0 when the launch does not sum.
static uint32_t tile_pairs_per_thread(uint64_t n_pairs, uint64_t max_grid, uint64_t low_span) {
  uint32_t ppt = 1;
  while ((n_pairs + (uint64_t)BLOCK * ppt - 1) / ((uint64_t)BLOCK * ppt) > max_grid &&
         !(low_span >= BLOCK && (uint64_t)BLOCK * ppt * 2 > low_span && (uint64_t)BLOCK * ppt <= low_span))
    ppt *= 2;
  return ppt;
}

template <int D>
static int launch_round(SumcheckSession &s, bool fold, bool do_sums, const std::vector<uint32_t *> &outs,
                        uint64_t n_pairs, int j, bool double_fold = false) {
  Context &c = ctx();
  RoundArgs<D> a;
  memset(&a, 0, sizeof(a));
  int T = s.st.T();
  for (int t = 0; t < T; t++) {
    a.in[t] = s.cur[t];
    a.out[t] = fold ? outs[t] : nullptr;
  }
  a.n_pairs = n_pairs;
  a.do_sums = do_sums ? 1 : 0;
  uint32_t ppt = 1;
  if (do_sums) {
    a.low = s.d_weights + s.low_off[j] * D;
    a.high = s.d_weights + s.high_off[j] * D;
    a.low_bits = (uint32_t)s.low_bits[j];
  }
  ppt = tile_pairs_per_thread(n_pairs, s.max_grid, do_sums ? (uint64_t)1 << a.low_bits : 0);
  a.pairs_per_thread = ppt;
  a.deferred = do_sums && ((uint64_t)BLOCK * ppt <= ((uint64_t)1 << a.low_bits)) ? 1 : 0;
  a.partials = s.d_partials;
  a.pstride = s.pstride;
  a.double_fold = double_fold ? 1 : 0;
  if (s.device_loop) a.ctrl = s.d_ctrl;
  a.consts = s.d_direct;
  uint32_t grid = (uint32_t)((n_pairs + (uint64_t)BLOCK * ppt - 1) / ((uint64_t)BLOCK * ppt));
  const bool own_epilogue = do_sums && s.device_loop && s.st.nacc > 0;
  if (own_epilogue) {
    // as many rows of totals as the elected workgroup's polls and scratch cover
    const uint32_t width = (uint32_t)s.st.nacc * D;
    uint32_t groups = 1;
    while (groups * 2 <= ROUND_GROUPS && groups * 2 <= grid && groups * 2 * width <= MAXPTS * MAXACC * 8 &&
           groups * 2 * width <= (uint32_t)TOTALS_POLLS * BLOCK)
      groups *= 2;
    a.totals = s.d_round_totals + (size_t)j * ROUND_GROUPS * s.pstride;
    a.arrivals = s.d_arrivals + j;
    a.groups = groups, a.points = (uint32_t)s.points, a.spin_limit = 200000;
    a.mtilde = s.d_mtilde, a.c0 = s.d_c0 + (size_t)j * s.points * D;
    if (!s.slice_totals_clear) {  // no set-up kernel cleared them
      EXH_HIP(hipMemsetAsync(a.totals, 0, (size_t)ROUND_GROUPS * s.pstride * 8, c.stream));
      EXH_HIP(hipMemsetAsync(a.arrivals, 0, 4, c.stream));
    }
  }
  if (fold && !s.device_loop)
    for (int k = 0; k < D; k++) a.r_mont[k] = to_mont(s.pending_r[k]);
  {
    // bytes this launch must move: every table read once, the folded tables written once
    uint64_t in_words = (double_fold ? 8 : fold ? 4 : 2) * n_pairs * (s.cur_base ? 1 : D),
             out_words = fold ? 2 * n_pairs * D : 0;
    const char *name = double_fold ? "round_fold2_base"
                       : fold      ? (s.cur_base ? "round_fold_base" : "round_fold_ext")
                                   : (s.cur_base ? "round_base" : "round_ext");
    c.prof_begin(name, j, (uint64_t)T * 4 * (in_words + out_words));
  }
  if (double_fold)
    s.kernels->launch_fold2(&a, grid, c.stream);
  else if (s.generated)
    s.kernels->launch(&a, s.cur_base, fold, grid, c.stream);
  else
    launch_interp<D>(a, s.desc, s.cur_base, fold, grid, c.stream);
  c.prof_end();
  if (do_sums && s.device_loop && !own_epilogue) {
    EpilogueArgs e;
    e.partials = s.d_partials, e.nblocks = grid, e.pstride = s.pstride, e.nacc = (uint32_t)s.st.nacc;
    e.points = (uint32_t)s.points, e.mtilde = s.d_mtilde, e.c0 = s.d_c0 + (size_t)j * s.points * D, e.ctrl = s.d_ctrl;
    c.prof_begin("epilogue", j, 0);
    if (D == 4)
      hipLaunchKernelGGL(epilogue_kernel<4>, dim3(1), dim3(EPI_BLOCK), 0, c.stream, e);
    else
      hipLaunchKernelGGL(epilogue_kernel<8>, dim3(1), dim3(EPI_BLOCK), 0, c.stream, e);
    c.prof_end();
  }
  if (do_sums && !s.device_loop) {
    uint32_t width = (uint32_t)s.st.nacc * D;
    hipLaunchKernelGGL(reduce_partials_kernel, dim3(width), dim3(BLOCK), 0, c.stream, s.d_partials, grid, s.pstride,
                       s.d_sums);
  }
  EXH_HIP(hipGetLastError());
  return OK;
}

// [deg][m] = 1 / prod_{q != m, q <= deg} (m - q), in Montgomery form: the denominators of the Lagrange basis
// over the nodes 0..deg
static void fill_inv_den(uint32_t *out) {
  // computed once: forty-nine field inversions on the host are ten microseconds between two launches of a prove
  static const std::vector<uint32_t> table = [] {
    std::vector<uint32_t> t((MAXDEG + 1) * (MAXDEG + 1), 0);
    for (int deg = 1; deg <= MAXDEG; deg++)
      for (int m = 0; m <= deg; m++) {
        uint32_t den = 1;
        for (int q = 0; q <= deg; q++)
          if (q != m) den = fmul(den, m > q ? (uint32_t)(m - q) : P - (uint32_t)(q - m));
        t[deg * (MAXDEG + 1) + m] = to_mont(finv(den));
      }
    return t;
  }();
  memcpy(out, table.data(), table.size() * 4);
}

// Rounds 0 and 1 from one sweep of the base tables (nothing folded): the slot sums in as many launches as the
// generated kernels need, then the epilogue that sends both rounds' messages.
template <int D>
static int launch_nodes_round(SumcheckSession &s, uint64_t n_pairs) {
  Context &c = ctx();
  NodesArgs<D> a;
  memset(&a, 0, sizeof(a));
  int T = s.st.T();
  for (int t = 0; t < T; t++) a.in[t] = s.cur[t];
  a.low = s.d_weights + s.low_off[1] * D;  // round 1's weights; round 0's extra factor goes in by the epilogue
  a.high = s.d_weights + s.high_off[1] * D;
  a.low_bits = (uint32_t)s.low_bits[1];
  a.n_pairs = n_pairs;
  // (two workgroups fit a compute unit beside the accumulators: the session's grid cap has them all resident
  // at once, which spreads each workgroup's fixed work -- first loads, the reduction over lanes -- over the most pairs)
  uint32_t ppt = 1;
  ppt = tile_pairs_per_thread(n_pairs, s.max_grid, (uint64_t)1 << a.low_bits);
  a.pairs_per_thread = ppt;
  a.deferred = (uint64_t)BLOCK * ppt <= ((uint64_t)1 << a.low_bits) ? 1 : 0;
  uint32_t grid = (uint32_t)((n_pairs + (uint64_t)BLOCK * ppt - 1) / ((uint64_t)BLOCK * ppt));
  // the two rounds' epilogue, run by the last workgroup of the last pass (see RoundTotals)
  NodesEpilogueArgs &e = a.epi;
  e.e.partials = nullptr, e.e.nblocks = grid, e.e.pstride = s.pstride, e.e.nacc = (uint32_t)s.st.nacc;
  e.e.points = (uint32_t)s.points, e.e.mtilde = s.d_mtilde, e.e.c0 = s.d_c0;
  e.e.ctrl = s.d_ctrl;
  e.eq1 = s.has_eq ? s.d_weights + (size_t)2 * D : nullptr;  // the eq factors lead the arena: (w_v, 1 - w_v) per variable
  e.groups = (uint32_t)s.desc.G, e.slots = (uint32_t)s.node_slots_n;
  for (int g = 0; g < s.desc.G; g++) {
    e.deg[g] = (uint32_t)s.desc.deg[g], e.nev[g] = (uint32_t)s.desc.nev[g];
    for (int k = 0; k < s.desc.nev[g]; k++) e.ev[g][k] = (uint8_t)s.desc.ev[g][k];
  }
  fill_inv_den(e.inv_den);
  {
    const uint32_t width = (uint32_t)s.node_slots_n * D;
    uint32_t groups = 1;
    while (groups * 2 <= ROUND_GROUPS && groups * 2 <= grid && groups * 2 * width <= MAXPTS * MAXACC * 8 &&
           groups * 2 * width <= (uint32_t)TOTALS_POLLS * BLOCK)
      groups *= 2;
    a.totals.totals = s.d_round_totals;  // round 0's region
    a.totals.arrivals = s.d_arrivals;
    a.totals.groups = groups, a.totals.pstride = s.pstride, a.totals.spin_limit = 200000;
    a.passes = (uint32_t)s.kernels->nodes_passes;
    if (!s.slice_totals_clear) {  // no set-up kernel cleared them
      EXH_HIP(hipMemsetAsync(a.totals.totals, 0, (size_t)ROUND_GROUPS * s.pstride * 8, c.stream));
      EXH_HIP(hipMemsetAsync(a.totals.arrivals, 0, 4, c.stream));
    }
  }
  // (the bytes the sweep is credited with when launches are timed: the two reads of the base tables it stands for,
  // round 0's sums and the fold that would have produced round 1's tables, shared among its passes; a pass moves
  // one read of them)
  for (int pass = 0; pass < s.kernels->nodes_passes; pass++) {
    c.prof_begin("round_nodes_base", 0, (uint64_t)T * 32 * n_pairs / (uint64_t)s.kernels->nodes_passes);
    s.kernels->launch_nodes(&a, pass, grid, c.stream);
    c.prof_end();
  }
  EXH_HIP(hipGetLastError());
  return OK;
}

// the total weight of round j's pairs, sum_h HIGH[h] sum_l LOW[l]: what a constant term is multiplied by
static hf::E weight_sum(const SumcheckSession &s, int j) {
  hf::E wsum = hf::lift(1, s.D);
  uint64_t nl = (uint64_t)1 << s.low_bits[j];
  if (!s.has_eq) wsum = hf::lift((uint32_t)(nl % P), s.D);
  if (s.has_bw)
    wsum = hf::mul(wsum, s.bw_sum);
  else if (!s.has_eq)
    wsum = hf::scale(wsum, (uint32_t)(s.n_high[j] % P));
  return wsum;
}

Arena &SumcheckSession::arena_a() { return private_buffers ? own_a : ctx().fold_a; }
Arena &SumcheckSession::arena_b() { return private_buffers ? own_b : ctx().fold_b; }
Arena &SumcheckSession::arena_misc() { return private_buffers ? own_misc : ctx().misc; }
SumcheckSession::~SumcheckSession() {
  if (private_buffers) {  // everything queued on them has to have run before they go back to the driver
    if (own_a.ptr || own_b.ptr || own_misc.ptr) (void)hipStreamSynchronize(ctx().stream);
    own_a.release(), own_b.release(), own_misc.release();
  }
}

int SumcheckSession::owns_arenas() const {
  if (private_buffers || epoch == ctx().session_epoch) return OK;
  set_error("invalid-parameter: another sumcheck session was begun since; one session is open at a time");
  return E_PARAM;
}

int SumcheckSession::round_sums(uint32_t *out) {
  Context &c = ctx();
  if (int owned = owns_arenas()) return owned;
  if (setup_deferred) {
    set_error("invalid-parameter: the session was set up for the device-driven loop");
    return E_PARAM;
  }
  if (round >= n) {
    set_error("invalid-parameter: no rounds left");
    return E_PARAM;
  }
  if (round > 0 && !pending_fold) {
    set_error("invalid-parameter: fold the previous round's challenge first");
    return E_PARAM;
  }
  int T = st.T(), j = round, status;
  uint64_t n_pairs;
  if (pending_fold) {  // fused: fold round j-1's variable, then sum round j
    uint64_t out_size = size / 2;
    Arena &dst = (generation % 2 == 0) ? arena_a() : arena_b();
    out_buf.assign(T, nullptr);
    for (int t = 0; t < T; t++) out_buf[t] = (uint32_t *)dst.ptr + (uint64_t)t * out_size * D;
    n_pairs = out_size / 2;
    status = D == 4 ? launch_round<4>(*this, true, true, out_buf, n_pairs, j)
                    : launch_round<8>(*this, true, true, out_buf, n_pairs, j);
    if (status) return status;
    for (int t = 0; t < T; t++) cur[t] = out_buf[t];
    cur_base = false;
    size = out_size;
    generation++;
    pending_fold = false;
  } else {
    n_pairs = size / 2;
    status = D == 4 ? launch_round<4>(*this, false, true, out_buf, n_pairs, j)
                    : launch_round<8>(*this, false, true, out_buf, n_pairs, j);
    if (status) return status;
  }
  size_t words = (size_t)st.nacc * D;
  if (words) EXH_HIP(hipMemcpyAsync(c.host_pinned, d_sums, words * 4, hipMemcpyDeviceToHost, c.stream));
  EXH_HIP(hipStreamSynchronize(c.stream));

  // ---- the message rows from the groups' sums
  // total weight of the pairs, for the constant group
  hf::E wsum = weight_sum(*this, j);
  if (claim_mode) {  // sum_g coef_g ((1 - r_0) G(0) + r_0 G(1)), or G(0) + G(1) without eq
    hf::E total = hf::zero(D), one = hf::lift(1, D);
    for (size_t g = 0; g < st.groups.size(); g++) {
      const Group &grp = st.groups[g];
      hf::E coef(group_coef.begin() + g * D, group_coef.begin() + (g + 1) * D);
      if (grp.tabs.empty()) {
        total = hf::add(total, hf::mul(coef, has_eq ? wsum : hf::scale(wsum, 2)));
        continue;
      }
      uint32_t fix = fpow(R1, grp.tabs.size());
      hf::E g0(c.host_pinned + (size_t)grp.acc_base * D, c.host_pinned + (size_t)(grp.acc_base + 1) * D);
      hf::E g1(c.host_pinned + (size_t)(grp.acc_base + 1) * D, c.host_pinned + (size_t)(grp.acc_base + 2) * D);
      g0 = hf::scale(g0, fix), g1 = hf::scale(g1, fix);
      hf::E v = has_eq ? hf::add(hf::mul(hf::sub(one, eq0), g0), hf::mul(eq0, g1)) : hf::add(g0, g1);
      total = hf::add(total, hf::mul(coef, v));
    }
    memcpy(out, total.data(), 4 * D);
    return OK;
  }
  std::vector<int> wire(points);
  for (int k = 0; k < points; k++) wire[k] = k == 0 ? 0 : k + 1;
  std::vector<hf::E> rows(points, hf::zero(D));
  for (size_t g = 0; g < st.groups.size(); g++) {
    const Group &grp = st.groups[g];
    hf::E coef(group_coef.begin() + g * D, group_coef.begin() + (g + 1) * D);
    if (grp.tabs.empty()) {
      hf::E v = hf::mul(coef, wsum);
      for (int k = 0; k < points; k++) rows[k] = hf::add(rows[k], v);
      continue;
    }
    // the kernel's sums carry R^-degree (none for a statement in direct form)
    uint32_t fix = st.direct ? 1u : fpow(R1, grp.tabs.size());
    std::vector<hf::E> vals;
    for (size_t k = 0; k < grp.evalx.size(); k++) {
      hf::E v(c.host_pinned + (size_t)(grp.acc_base + k) * D, c.host_pinned + (size_t)(grp.acc_base + k + 1) * D);
      vals.push_back(hf::scale(v, fix));
    }
    bool at_wire = st.direct || (int)grp.tabs.size() >= points;  // evaluated at the wire points themselves
    for (int k = 0; k < points; k++) {
      hf::E gv = at_wire ? vals[k] : hf::interpolate(grp.evalx, vals, hf::lift((uint32_t)wire[k], D));
      rows[k] = hf::add(rows[k], hf::mul(coef, gv));
    }
  }
  for (int k = 0; k < points; k++) memcpy(out + (size_t)k * D, rows[k].data(), 4 * D);
  return OK;
}

int SumcheckSession::fold(const uint32_t *r) {
  if (int owned = owns_arenas()) return owned;
  if (round >= n || pending_fold) {
    set_error("invalid-parameter: nothing to fold");
    return E_PARAM;
  }
  for (int k = 0; k < D; k++) pending_r[k] = r[k] % P;
  pending_fold = true;
  round++;
  return OK;
}

int SumcheckSession::flush() {
  Context &c = ctx();
  if (!pending_fold) return OK;
  int T = st.T();
  uint64_t out_size = size / 2;
  Arena &dst = (generation % 2 == 0) ? arena_a() : arena_b();
  RoundArgs<4> a4;
  RoundArgs<8> a8;
  memset(&a4, 0, sizeof(a4));
  memset(&a8, 0, sizeof(a8));
  for (int k = 0; k < D; k++) a4.r_mont[k % 4] = a8.r_mont[k] = to_mont(pending_r[k]);
  uint32_t grid = (uint32_t)((out_size + BLOCK - 1) / BLOCK);
  for (int t = 0; t < T; t++) {
    uint32_t *o = (uint32_t *)dst.ptr + (uint64_t)t * out_size * D;
    if (D == 4 && cur_base)
      hipLaunchKernelGGL((fold_kernel<4, true>), dim3(grid), dim3(BLOCK), 0, c.stream, cur[t], o, out_size, a4);
    else if (D == 4)
      hipLaunchKernelGGL((fold_kernel<4, false>), dim3(grid), dim3(BLOCK), 0, c.stream, cur[t], o, out_size, a4);
    else if (cur_base)
      hipLaunchKernelGGL((fold_kernel<8, true>), dim3(grid), dim3(BLOCK), 0, c.stream, cur[t], o, out_size, a8);
    else
      hipLaunchKernelGGL((fold_kernel<8, false>), dim3(grid), dim3(BLOCK), 0, c.stream, cur[t], o, out_size, a8);
    cur[t] = o;
  }
  EXH_HIP(hipGetLastError());
  cur_base = false;
  size = out_size;
  generation++;
  pending_fold = false;
  return OK;
}

// table t's entries (stride 1 or D) as `padded` extension elements at out + t * padded * D: lifted, then zeros
struct PadArgs {
  const uint32_t *in[MAXT];
  uint32_t *out;
  uint64_t size, padded;
  uint32_t in_stride, D;
};
__global__ __launch_bounds__(BLOCK) void pad_tables_kernel(PadArgs a) {
  const uint64_t u = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;  // word of table blockIdx.y's output
  if (u >= a.padded * a.D) return;
  const uint64_t x = u / a.D;
  const uint32_t k = (uint32_t)(u % a.D);
  uint32_t v = 0;
  if (x < a.size) v = a.in_stride == 1 ? (k == 0 ? a.in[blockIdx.y][x] : 0u) : a.in[blockIdx.y][x * a.D + k];
  a.out[((uint64_t)blockIdx.y * a.padded) * a.D + u] = v;
}

int SumcheckSession::finish_device(uint32_t *d_out, uint64_t padded) {
  Context &c = ctx();
  if (int owned = owns_arenas()) return owned;
  int status = flush();
  if (status) return status;
  const int T = st.T();
  if (padded < size || T < 1) {
    set_error("invalid-parameter: the padded length of the folded tables");
    return E_PARAM;
  }
  PadArgs a;
  memset(&a, 0, sizeof(a));
  for (int t = 0; t < T; t++) a.in[t] = cur[t];
  a.out = d_out, a.size = size, a.padded = padded, a.in_stride = cur_base ? 1u : (uint32_t)D, a.D = (uint32_t)D;
  const uint32_t grid = (uint32_t)((padded * D + BLOCK - 1) / BLOCK);
  hipLaunchKernelGGL(pad_tables_kernel, dim3(grid, T), dim3(BLOCK), 0, c.stream, a);
  EXH_HIP(hipGetLastError());
  return OK;
}

int SumcheckSession::finish(uint32_t *finals, uint32_t *const *folded) {
  Context &c = ctx();
  if (int owned = owns_arenas()) return owned;
  int status = flush();
  if (status) return status;
  int T = st.T();
  if (!finals && !folded) return OK;
  // each table's current entries (K of them after n rounds), lifted if still base
  const uint64_t words = size * (cur_base ? 1 : D);
  const bool cached = !cur_base && final_cache.size() == (size_t)T * words;
  std::vector<uint32_t> all(cached ? 0 : (size_t)T * words);
  if (!cached) {
    for (int t = 0; t < T; t++)
      EXH_HIP(hipMemcpyAsync(all.data() + (size_t)t * words, cur[t], words * 4, hipMemcpyDeviceToHost, c.stream));
    EXH_HIP(hipStreamSynchronize(c.stream));
  }
  for (int t = 0; t < T; t++) {
    const uint32_t *tmp = (cached ? final_cache.data() : all.data()) + (size_t)t * words;
    for (uint64_t x = 0; x < size; x++) {
      uint32_t e[8] = {0};
      if (cur_base)
        e[0] = tmp[x];
      else
        memcpy(e, &tmp[x * D], 4 * D);
      if (x == 0 && finals) memcpy(finals + (size_t)t * D, e, 4 * D);
      if (folded && folded[t]) memcpy(folded[t] + x * D, e, 4 * D);
    }
  }
  return OK;
}

// ------------------------------------------------------------------ the device-driven loop
// rounds with at most this many pairs run in the one-workgroup tail: one pair per thread, and the
// tables (two entries per pair) must fit the tail's LDS
static uint64_t tail_pairs(int T, int D) {
  uint64_t p = BLOCK;
  while (p > 1 && (uint64_t)T * 2 * p * D * 4 > TAIL_LDS_BYTES) p /= 2;
  return p;
}

// the Lagrange basis of the group's node e over its nodes at wire point k (0, 2, 3, ...), times the power of R the
// group's sums carry (R^-degree)
static uint32_t map_scalar(const Group &grp, size_t e, int k, int points, bool direct) {
  // (a direct statement's accumulators hold w times the form's value in Montgomery form, reduced once: no power of R)
  const uint32_t fix = direct ? 1u : fpow(R1, grp.tabs.size());
  if ((int)grp.tabs.size() >= points) return (int)e == k ? fix : 0u;  // evaluated at the wire points themselves
  const int wire = k == 0 ? 0 : k + 1;
  uint32_t num = 1, den = 1;
  for (size_t o = 0; o < grp.evalx.size(); o++) {
    if (o == e) continue;
    int64_t a = wire - grp.evalx[o], b = grp.evalx[e] - grp.evalx[o];
    num = fmul(num, (uint32_t)(((a % (int64_t)P) + P) % P));
    den = fmul(den, (uint32_t)(((b % (int64_t)P) + P) % P));
  }
  return fmul(fmul(num, finv(den)), fix);
}

void SumcheckSession::message_map_scalars(std::vector<uint32_t> *lagfix, std::vector<int> *acc_group) const {
  const int nacc = std::max(st.nacc, 1);
  lagfix->assign((size_t)points * nacc, 0u);
  acc_group->assign((size_t)nacc, -1);
  for (size_t g = 0; g < st.groups.size(); g++) {
    const Group &grp = st.groups[g];
    if (grp.tabs.empty()) continue;
    for (size_t e = 0; e < grp.evalx.size(); e++) {
      (*acc_group)[grp.acc_base + e] = (int)g;
      for (int k = 0; k < points; k++) (*lagfix)[(size_t)k * nacc + grp.acc_base + e] = map_scalar(grp, e, k, points, st.direct);
    }
  }
}

bool SumcheckSession::device_capable() const {
  if (points > MAXPTS || n > MAXROUNDS) return false;
  // the session's staged eq point and block weights, then the loop's message map, constant terms and the head
  // of the control block share one pinned staging area (many block weights overflow it: the host-driven rounds
  // take such a session)
  const size_t up_words = (size_t)points * std::max(st.nacc, 1) * D + (size_t)n * points * D + offsetof(Ctrl, msg) / 4;
  return setup_words + up_words <= PIN_BEGIN_WORDS + PIN_LOOP_WORDS;
}

int SumcheckSession::run_device(const DevB3S &state, uint32_t *messages, uint32_t *challenges, DevB3S *final_state) {
  Context &c = ctx();
  if (int owned = owns_arenas()) return owned;
  if (round != 0 || pending_fold || claim_mode || !device_capable()) {
    set_error("invalid-parameter: the device loop starts a fresh session of at most 7 wire points whose constants "
              "fit its staging buffer");
    return E_PARAM;
  }
  if (n == 0) return OK;
  const int T = st.T(), nacc = st.nacc;
  // ---- constants: control block, message map (times R), per-round constant terms
  // (staged in pinned memory: message map | constant terms | head of the control block)
  const size_t mt_words = (size_t)points * std::max(nacc, 1) * D, c0_words = (size_t)n * points * D;
  const size_t head_words = offsetof(Ctrl, msg) / 4, up_words = mt_words + c0_words + head_words;
  // (right behind the session's staged eq point and block weights: the device keeps the same order)
  uint32_t *up = c.host_pinned + PIN_BEGIN + setup_words;
  memset(up, 0, up_words * 4);
  uint32_t *mt = up, *c0 = mt + mt_words;
  Ctrl *hc = reinterpret_cast<Ctrl *>(c0 + c0_words);  // only its head is staged
  hc->tr = state;
  for (size_t g = 0; g < st.groups.size(); g++) {
    const Group &grp = st.groups[g];
    hf::E coef(group_coef.begin() + g * D, group_coef.begin() + (g + 1) * D);
    if (grp.tabs.empty()) {
      for (int j = 0; j < n; j++) {
        hf::E v = hf::mul(coef, weight_sum(*this, j));
        for (int k = 0; k < points; k++)
          for (int cc = 0; cc < D; cc++)
            c0[((size_t)j * points + k) * D + cc] = fadd(c0[((size_t)j * points + k) * D + cc], v[cc]);
      }
      continue;
    }
    for (size_t e = 0; e < grp.evalx.size(); e++) {
      for (int k = 0; k < points; k++) {
        hf::E m = hf::scale(coef, map_scalar(grp, e, k, points, st.direct));
        uint32_t *dst = mt + ((size_t)k * nacc + grp.acc_base + e) * D;
        for (int cc = 0; cc < D; cc++) dst[cc] = to_mont(m[cc]);
      }
    }
  }
  // A session whose every round runs in the one-workgroup launch needs no set-up launch: that launch builds the
  // weight tables itself from the eq point's factors, which lead the session's constants (EXACTA_HIP_NO_OWN_WEIGHTS=1:
  // never)
  {
    const char *no_own = getenv("EXACTA_HIP_NO_OWN_WEIGHTS");
    own_weights = setup_deferred && has_eq && !has_bw && setup.total_eq > 0 && !setup.ones_len &&
                  size / 2 <= tail_pairs(T, D) && n <= MAXTAIL && !(no_own && no_own[0] == '1');
  }
  if (chain_hook) {  // the chain's launch writes what the copy below would bring
    if (!setup_deferred) {
      set_error("invalid-parameter: a chained session defers its set-up");
      return E_PARAM;
    }
    int st_hook = chain_hook();
    if (st_hook) return st_hook;
    setup_deferred = false;
    if (!own_weights && (st_hook = launch_setup())) return st_hook;
  } else if (setup_deferred) {
    // the session's constants and the loop's, staged in pinned memory, reach the device with the set-up launch,
    // which reads them where they lie; with one copy on the stream when there is no such launch
    // (EXACTA_HIP_COPY_CONSTANTS=1: always by that copy, the set-up launch behind it)
    const char *copy_constants = getenv("EXACTA_HIP_COPY_CONSTANTS");
    const bool by_launch = !own_weights && (setup.total_eq || setup.ones_len) && c.host_pinned_dev &&
                           !(copy_constants && copy_constants[0] == '1');
    if (!by_launch)
      EXH_HIP(hipMemcpyAsync(d_weights, c.host_pinned + PIN_BEGIN, (setup_words + up_words) * 4, hipMemcpyHostToDevice,
                             c.stream));
    setup_deferred = false;
    int st_setup = own_weights ? OK
                   : by_launch ? launch_setup(c.host_pinned_dev + PIN_BEGIN, setup_words + up_words)
                               : launch_setup();
    if (st_setup) return st_setup;
  } else {
    EXH_HIP(hipMemcpyAsync(d_mtilde, up, up_words * 4, hipMemcpyHostToDevice, c.stream));
  }

  device_loop = true;
  bool tail_done = false;
  int status = OK, j = 0;
  int folds_due = 0;  // folds by the last challenges drawn that the tables still await (2 after the base-field sweep for rounds 0 and 1)
  const char *no_nodes = getenv("EXACTA_HIP_NO_BASE_ROUND1");
  for (; j < n && status == OK; j++) {
    const bool fold_due = folds_due > 0;
    uint64_t n_pairs = (size >> folds_due) / 2;  // pairs summed in round j (after the pending folds)
    if (folds_due == 2) {  // round 2 after the base-field sweep: both folds at once, then the sums
      round = j;
      uint64_t out_size = size / 4;
      Arena &dst = ((generation + 1) % 2 == 0) ? arena_a() : arena_b();
      out_buf.assign(T, nullptr);
      for (int t = 0; t < T; t++) out_buf[t] = (uint32_t *)dst.ptr + (uint64_t)t * out_size * D;
      status = D == 4 ? launch_round<4>(*this, true, true, out_buf, n_pairs, j, true)
                      : launch_round<8>(*this, true, true, out_buf, n_pairs, j, true);
      for (int t = 0; t < T; t++) cur[t] = out_buf[t];
      cur_base = false;
      size = out_size;
      generation += 2;
      folds_due = 1;
      tail_done = false;
      continue;
    }
    if (n_pairs <= tail_pairs(T, D) && n - j <= MAXTAIL) break;
    round = j;
    // once every workgroup of a resident grid can hold its slice of the tables in LDS, the rounds down
    // to where one workgroup suffices run in one launch
    const bool pow2 = (size & (size - 1)) == 0;
    // (several blocks: the pairs are an odd multiple of a power of two, and the grid that multiple of one, so that
    // every workgroup's slice is a power of two of pairs and halves with the rounds; a fold pairs neighbours, so a
    // slice need not lie in one block)
    uint64_t odd = n_pairs;
    while (odd > 1 && odd % 2 == 0) odd /= 2;
    uint64_t slice_max = SLICE_LDS_BYTES / ((uint64_t)T * 2 * D * 4);
    if (const char *cap = getenv("EXACTA_HIP_MAX_SLICE_PAIRS"))  // tests: keep more rounds on the streaming kernels
      slice_max = std::min<uint64_t>(slice_max, strtoull(cap, nullptr, 10));
    // (proofs running side by side share the device: each one's grid takes its part, a power of two)
    const uint64_t grid_max =
        std::min<uint64_t>(256, c.compute_units > 0 ? c.compute_units : 1) / (c.share > 1 ? 2 : 1);
    if (odd > 1) {  // (EXACTA_HIP_NO_BLOCK_SLICES=1: tables of several blocks stay on the streaming kernels)
      const char *no_block_slices = getenv("EXACTA_HIP_NO_BLOCK_SLICES");
      if (no_block_slices && no_block_slices[0] == '1') odd = 17;
    }
    if (odd <= 16 && odd <= grid_max && n_pairs > tail_pairs(T, D) && n_pairs <= slice_max * grid_max) {
      int count = 0;
      while ((n_pairs >> count) > tail_pairs(T, D) && count < MAXTAIL && j + count < n) count++;
      const uint64_t left = 2 * (n_pairs >> count);  // entries per table after these rounds
      uint64_t grid = odd;
      while (grid * 2 <= grid_max && grid * 2 <= left && (n_pairs / (grid * 2)) >= BLOCK) grid *= 2;
      while (n_pairs / grid > slice_max && grid * 2 <= grid_max && grid * 2 <= left) grid *= 2;
      // (fewer pairs than two workgroups have threads, yet more than the one-workgroup launch holds -- statements
      // of many tables: two workgroups' rounds still cost a fraction of a streaming launch per round)
      if (grid == 1 && grid_max >= 2 && left >= 2) grid = 2;
      // the grid's workgroups wait for one another: all of them must be resident at once.  The runtime says how
      // many of this kernel a compute unit holds with the slices' LDS; a grid beyond that stays on the streaming
      // kernels (asked once per kernel and size)
      bool resident = true;
      if (count > 0 && grid > 1 && n_pairs / grid <= slice_max) {
        const uint32_t lds_bytes = (uint32_t)((uint64_t)T * (2 * n_pairs / grid) * D * 4);
        static std::map<std::pair<const void *, uint32_t>, int> asked;
        static std::mutex asked_mutex;
        std::lock_guard<std::mutex> asked_lock(asked_mutex);
        auto key = std::make_pair(generated ? (const void *)kernels : (const void *)(uintptr_t)D, lds_bytes);
        auto it = asked.find(key);
        if (it == asked.end()) {
          int blocks = generated ? (kernels->tail_blocks_per_cu ? kernels->tail_blocks_per_cu(lds_bytes) : -1)
                                 : (D == 4 ? tail_interp_blocks_per_cu<4>(lds_bytes) : tail_interp_blocks_per_cu<8>(lds_bytes));
          it = asked.emplace(key, blocks).first;
        }
        resident = it->second < 0 ||
                   (uint64_t)it->second * (uint64_t)std::max(c.compute_units, 1) / (uint64_t)std::max(c.share, 1) >= grid;
      }
      if (count > 0 && grid > 1 && n_pairs / grid <= slice_max && resident) {
        status = launch_tail(j, count, (uint32_t)grid, fold_due);
        folds_due = 0;
        tail_done = status == OK;  // the tables are contiguous in one arena, nothing pending
        j += count - 1;
        continue;
      }
    }
    // rounds 0 and 1 from one sweep of the base tables, when round 2 is a streaming round as well: their sums
    // come from base-field products on a grid of (X0, X1) and the tables are not folded until round 2
    const bool nodes_rounds = j == 0 && cur_base && folds_due == 0 && n >= 3 && generated && kernels->nodes_passes > 0 &&
                              node_slots_n <= MAXACC && pow2 && (n_pairs / 4) > slice_max * grid_max &&
                              !(no_nodes && no_nodes[0] == '1');
    if (nodes_rounds) {
      status = D == 4 ? launch_nodes_round<4>(*this, n_pairs / 2) : launch_nodes_round<8>(*this, n_pairs / 2);
      folds_due = 2;
      tail_done = false;
      j++;  // two rounds done
      continue;
    }
    if (!fold_due) {
      status = D == 4 ? launch_round<4>(*this, false, true, out_buf, n_pairs, j)
                      : launch_round<8>(*this, false, true, out_buf, n_pairs, j);
    } else {
      uint64_t out_size = size / 2;
      Arena &dst = (generation % 2 == 0) ? arena_a() : arena_b();
      out_buf.assign(T, nullptr);
      for (int t = 0; t < T; t++) out_buf[t] = (uint32_t *)dst.ptr + (uint64_t)t * out_size * D;
      status = D == 4 ? launch_round<4>(*this, true, true, out_buf, n_pairs, j)
                      : launch_round<8>(*this, true, true, out_buf, n_pairs, j);
      for (int t = 0; t < T; t++) cur[t] = out_buf[t];
      cur_base = false;
      size = out_size;
      generation++;
    }
    folds_due = 1;
    tail_done = false;
  }
  uint32_t *down = c.host_pinned + PIN_DOWN;
  const size_t ctrl_words = (sizeof(Ctrl) + 3) / 4;
  bool logged_to_host = false;
  if (status == OK && j < n) {  // the tail: rounds j .. n-1 and the last fold, in one workgroup
    // when a single entry per table is left at the end (the finals travel in the control block), the launch
    // itself delivers the control block to pinned host memory
    const bool deliver =
        !c.profiling && !chain_hook && ((size >> ((folds_due > 0 ? 1 : 0) + (n - j))) == 1 || finals_stay);
    if (deliver) {
      if (++c.log_seq == 0) ++c.log_seq;  // 0 is what the flag is reset to
      host_log = c.host_pinned_dev + PIN_DOWN, host_flag_at = (uint32_t)ctrl_words, host_seq = c.log_seq;
      reinterpret_cast<volatile uint32_t *>(down)[ctrl_words] = 0;
      reinterpret_cast<volatile uint32_t *>(down)[ctrl_words + 1] = 0;
    }
    status = launch_tail(j, n - j, 1, folds_due > 0);
    host_log = nullptr;
    folds_due = 0;
    tail_done = status == OK;
    logged_to_host = deliver && tail_done;
  }
  device_loop = false;
  if (status) return status;
  if (chain_hook) {  // nothing comes back here: the chain reads the control block on the device
    if (!tail_done || size != 1) {
      set_error("device-error: a chained sumcheck did not end in the one-workgroup launch");
      return E_DEVICE;
    }
    round = n;
    return OK;
  }
  // ---- read the logs back, and with them what the tail left of the tables: one wait for both
  const size_t final_words = (size_t)T * size * D;
  final_cache.clear();
  const bool in_ctrl = tail_done && size == 1;  // the tail left the finals in the control block
  const bool with_finals = tail_done && !in_ctrl && !finals_stay && ctrl_words + final_words <= PIN_DOWN_WORDS;
  if (logged_to_host) {
    // the flag follows the block through the same path, so seeing it means the block is there; a stream that
    // ends without raising it (a launch gave up) is caught by the query
    volatile uint32_t *flag = reinterpret_cast<volatile uint32_t *>(down) + ctrl_words;
    uint32_t spins = 0;
    while (*flag != c.log_seq) {
      // (any answer but "not ready" ends the polling: a stream in an error state never raises the flag, and the
      // wait below reports what happened)
      if ((++spins & 1023) == 0 && hipStreamQuery(c.stream) != hipErrorNotReady) break;
    }
    if (*flag != c.log_seq) {
      EXH_HIP(hipStreamSynchronize(c.stream));
      if (*flag != c.log_seq) {
        set_error("device-error: the device loop ended without delivering its logs");
        return E_DEVICE;
      }
    }
    std::atomic_thread_fence(std::memory_order_acquire);
  } else {
    EXH_HIP(hipMemcpyAsync(down, d_ctrl, sizeof(Ctrl), hipMemcpyDeviceToHost, c.stream));
    if (with_finals)  // the tail wrote table t at t * size * D of one arena
      EXH_HIP(hipMemcpyAsync(down + ctrl_words, cur[0], final_words * 4, hipMemcpyDeviceToHost, c.stream));
    EXH_HIP(hipStreamSynchronize(c.stream));
  }
  const Ctrl *rc = reinterpret_cast<const Ctrl *>(down);
  if (with_finals) final_cache.assign(down + ctrl_words, down + ctrl_words + final_words);
  if (in_ctrl) final_cache.assign(rc->finals, rc->finals + final_words);
  if (rc->gave_up) {
    set_error("device-error: a workgroup of the grid launch gave up waiting for the others");
    return E_DEVICE;
  }
  if ((int)rc->round != n) {
    set_error("device-error: the device loop completed " + std::to_string(rc->round) + " of " + std::to_string(n) +
              " rounds");
    return E_DEVICE;
  }
  for (int r = 0; r < n; r++) {
    memcpy(messages + (size_t)r * points * D, rc->msg[r], (size_t)points * D * 4);
    memcpy(challenges + (size_t)r * D, rc->chal[r], (size_t)D * 4);
  }
  if (final_state) *final_state = rc->tr;
  round = n;
  pending_fold = folds_due > 0;  // after a round kernel the last challenge's fold is still to do
  if (pending_fold) memcpy(pending_r, rc->chal[n - 1], (size_t)D * 4);
  return OK;
}

int SumcheckSession::launch_tail(int j, int rounds, uint32_t grid, bool first_fold) {
  Context &c = ctx();
  const int T = st.T();
  // it folds (first_fold ? 1 : 0) + rounds times; the result goes where alternating arenas would put it
  int folds = (first_fold ? 1 : 0) + rounds;
  uint64_t final_size = size >> folds;
  int last_gen = generation + folds - 1;
  Arena &dst = (last_gen % 2 == 0) ? arena_a() : arena_b();
  int status = dst.reserve((size_t)T * final_size * D * 4);
  if (status) return status;
  const uint64_t slice_entries = (first_fold ? size / 2 : size) / grid;
  // groups of workgroups share a row of totals: few enough that a workgroup polls all the rows' words at
  // once, one per thread (a second pass of polls is a second trip to memory in every round)
  uint32_t groups = 1;
  while (groups * 2 <= SLICE_GROUPS && grid % (groups * 2) == 0 && groups * 2 * (uint32_t)st.nacc * D <= BLOCK) groups *= 2;
  auto fill = [&](auto &a) {
    memset(&a, 0, sizeof(a));
    for (int t = 0; t < T; t++) a.in[t] = cur[t];
    a.out = (uint32_t *)dst.ptr;
    a.weights = d_weights;
    a.entries = (uint32_t)size;
    a.in_base = cur_base ? 1 : 0;
    a.first_fold = first_fold ? 1 : 0;
    a.rounds = (uint32_t)rounds;
    a.first_round = (uint32_t)j;
    a.capacity = (uint32_t)(grid > 1 ? slice_entries : 2 * tail_pairs(T, D));
    a.lds_bytes = (uint32_t)(T * a.capacity * D * 4);
    a.points = (uint32_t)points;
    a.ctrl = d_ctrl;
    a.mtilde = d_mtilde;
    a.c0 = d_c0 + (size_t)j * points * D;
    a.totals = d_slice_totals;
    a.pstride = pstride;
    a.groups = groups;
    a.spin_limit = 200000;
    a.host_log = host_log, a.host_flag_at = host_flag_at, a.host_seq = host_seq;
    a.consts = d_direct;
    for (int jj = 0; jj < rounds; jj++) {
      a.low_off[jj] = low_off[j + jj];
      a.high_off[jj] = high_off[j + jj];
      a.low_bits[jj] = (uint32_t)low_bits[j + jj];
    }
    if (own_weights && grid == 1 && j == 0 && rounds == n) {  // the launch builds the weight tables behind its tables
      uint64_t own_entries = (uint64_t)2 * n;
      for (int jj = 0; jj < n; jj++) own_entries += ((uint64_t)1 << low_bits[jj]) + n_high[jj];
      a.factors = d_weights, a.n_vars = (uint32_t)n;
      a.lds_bytes += (uint32_t)(own_entries * D * 4);
    }
  };
  if (grid > 1 && !slice_totals_clear)  // the rounds' totals start at zero (64-bit words)
    EXH_HIP(hipMemsetAsync(d_slice_totals, 0, (size_t)rounds * groups * pstride * 8, c.stream));
  if (grid > 1) slice_totals_clear = false;
  const bool hold = held_tail && grid == 1 && generated && kernels->launch_tail_glue && j + rounds == n;
  if (hold) {  // the caller launches it, with its own next step behind the rounds
    if (D == 4) {
      TailArgs<4> a;
      fill(a);
      held_tail->assign(reinterpret_cast<uint8_t *>(&a), reinterpret_cast<uint8_t *>(&a) + sizeof(a));
    } else {
      TailArgs<8> a;
      fill(a);
      held_tail->assign(reinterpret_cast<uint8_t *>(&a), reinterpret_cast<uint8_t *>(&a) + sizeof(a));
    }
    cur_base = false;
    for (int t = 0; t < T; t++) cur[t] = (uint32_t *)dst.ptr + (uint64_t)t * final_size * D;
    size = final_size;
    generation += folds;
    return OK;
  }
  c.prof_begin(grid > 1 ? "slices" : "tail", j,
               (uint64_t)T * size * (cur_base ? 1 : D) * 4 + (uint64_t)T * final_size * D * 4);
  if (D == 4) {
    TailArgs<4> a;
    fill(a);
    if (generated)
      kernels->launch_tail(&a, grid, c.stream);
    else
      launch_tail_interp<4>(a, desc, grid, c.stream);
  } else {
    TailArgs<8> a;
    fill(a);
    if (generated)
      kernels->launch_tail(&a, grid, c.stream);
    else
      launch_tail_interp<8>(a, desc, grid, c.stream);
  }
  c.prof_end();
  EXH_HIP(hipGetLastError());
  cur_base = false;
  for (int t = 0; t < T; t++) cur[t] = (uint32_t *)dst.ptr + (uint64_t)t * final_size * D;
  size = final_size;
  generation += folds;
  return OK;
}

}  // namespace exh
