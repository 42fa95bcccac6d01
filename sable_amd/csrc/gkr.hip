// gkr.hip -- see gkr.hpp.
#include "gkr.hpp"

#include <string.h>

#include <vector>

#include "context.hpp"
#include "forms.hpp"
#include "hostfield.hpp"
#include "prover.hpp"
#include "gkr_glue.hpp"
#include "sumcheck_kernels.hpp"

namespace exh {

// parent (b, x) of children (b, x) and (b, x + 2^m): p = p0 q1 + p1 q0, q = q0 q1
template <int D>
__global__ __launch_bounds__(BLOCK) void gkr_reduce_kernel(const uint32_t *p, const uint32_t *q, uint32_t *pp,
                                                           uint32_t *qq, uint32_t m, uint64_t n_out) {
  uint64_t o = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
  if (o >= n_out) return;
  uint64_t half = (uint64_t)1 << m, b = o >> m, x = o & (half - 1);
  uint64_t c0 = (b << (m + 1)) + x, c1 = c0 + half;
  Ext<D> p0 = load_ext<D>(p + c0 * D), p1 = load_ext<D>(p + c1 * D);
  Ext<D> q0 = load_ext<D>(q + c0 * D), q1 = load_ext<D>(q + c1 * D);
  // products carry 1/R; multiplying one factor of each product by R^2 first makes them exact
  Ext<D> q1r, q0r;
#pragma unroll
  for (int c = 0; c < D; c++) q1r.c[c] = mont_mul(q1.c[c], R2), q0r.c[c] = mont_mul(q0.c[c], R2);
  store_ext<D>(pp + o * D, ext_add<D>(ext_mul_mont<D>(p0, q1r), ext_mul_mont<D>(p1, q0r)));
  store_ext<D>(qq + o * D, ext_mul_mont<D>(q0, q1r));
}

// The layers m_top .. 0 of one lookup's tree with one block, in one workgroup: layer m has 2^m <= BLOCK parents,
// a thread takes one, and the workgroup's barrier stands between a layer's writes and the next one's reads.  (A
// launch per layer is 4 us each for a few hundred products.)
constexpr int REDUCE_TOP_LAYERS = 9;  // m_top <= 8: 256 parents
struct ReduceTopArgs {
  const uint32_t *p, *q;  // layer m_top + 1
  uint32_t *pp[REDUCE_TOP_LAYERS], *qq[REDUCE_TOP_LAYERS];
  int m_top;
};
template <int D>
__global__ __launch_bounds__(BLOCK) void gkr_reduce_top_kernel(ReduceTopArgs a) {
  static_assert((1 << (REDUCE_TOP_LAYERS - 1)) <= BLOCK, "a thread per parent");
  const uint32_t *p = a.p, *q = a.q;
  for (int m = a.m_top; m >= 0; m--) {
    const uint32_t o = threadIdx.x, half = 1u << m;
    if (o < half) {
      Ext<D> p0 = load_ext<D>(p + o * D), p1 = load_ext<D>(p + (o + half) * D);
      Ext<D> q0 = load_ext<D>(q + o * D), q1 = load_ext<D>(q + (o + half) * D);
      Ext<D> q1r, q0r;
#pragma unroll
      for (int c = 0; c < D; c++) q1r.c[c] = mont_mul(q1.c[c], R2), q0r.c[c] = mont_mul(q0.c[c], R2);
      store_ext<D>(a.pp[m] + o * D, ext_add<D>(ext_mul_mont<D>(p0, q1r), ext_mul_mont<D>(p1, q0r)));
      store_ext<D>(a.qq[m] + o * D, ext_mul_mont<D>(q0, q1r));
    }
    __threadfence();
    __syncthreads();
    p = a.pp[m], q = a.qq[m];
  }
}

int gkr_reduce_layer(int D, int K, int m, const uint32_t *p, const uint32_t *q, uint32_t *pp, uint32_t *qq) {
  Context &c = ctx();
  int status = c.require();
  if (status) return status;
  uint64_t n_out = (uint64_t)K << m;
  uint32_t grid = (uint32_t)((n_out + BLOCK - 1) / BLOCK);
  if (D == 4)
    hipLaunchKernelGGL(gkr_reduce_kernel<4>, dim3(grid), dim3(BLOCK), 0, c.stream, p, q, pp, qq, (uint32_t)m, n_out);
  else
    hipLaunchKernelGGL(gkr_reduce_kernel<8>, dim3(grid), dim3(BLOCK), 0, c.stream, p, q, pp, qq, (uint32_t)m, n_out);
  EXH_HIP(hipGetLastError());
  return OK;
}

// the lower and upper halves of each block, as K contiguous blocks each (HALVES-PER-BLOCK,
// src/gkr.lisp:190-197); only needed when K > 1: with one block the halves are views
// (every vector of a layer in one launch: blockIdx.y picks the vector; the halves of vector i go to
// out + (2 i) n_out D and out + (2 i + 1) n_out D)
struct HalvesArgs {
  const uint32_t *v[MAXT];
  uint32_t *out;
  uint32_t size_bits;
  uint64_t n_out;
};
template <int D>
__global__ __launch_bounds__(BLOCK) void halves_kernel(HalvesArgs a) {
  uint64_t o = (uint64_t)blockIdx.x * BLOCK + threadIdx.x;
  if (o >= a.n_out) return;
  const uint32_t *v = a.v[blockIdx.y];
  uint32_t *lower = a.out + (uint64_t)(2 * blockIdx.y) * a.n_out * D, *upper = lower + a.n_out * D;
  uint64_t size = (uint64_t)1 << a.size_bits, b = o >> a.size_bits, x = o & (size - 1);
  store_ext<D>(lower + o * D, load_ext<D>(v + (b * 2 * size + x) * D));
  store_ext<D>(upper + o * D, load_ext<D>(v + (b * 2 * size + size + x) * D));
}


namespace {

int block_bits(int k) {  // src/gkr.lisp:23-25
  int b = 0;
  for (int v = k - 1; v > 0; v >>= 1) b++;
  return b;
}

// LAYER-STATEMENT (src/gkr.lisp:30-41) as a form; with_bw: (* bw statement)
Statement layer_statement(int lookups, bool with_bw) {
  std::string form = "(+";
  std::vector<std::string> tables, constants;
  if (with_bw) tables.push_back("BW");
  for (int l = 0; l < lookups; l++) {
    std::string s = std::to_string(l);
    form += " (* A" + s + " P0-" + s + " Q1-" + s + ") (* A" + s + " P1-" + s + " Q0-" + s + ") (* AL" + s + " Q0-" + s +
            " Q1-" + s + ")";
    for (const char *name : {"P0-", "P1-", "Q0-", "Q1-"}) tables.push_back(name + s);
    constants.push_back("A" + s);
    constants.push_back("AL" + s);
  }
  form += ")";
  if (with_bw) form = "(* BW " + form + ")";
  Statement st;
  compile_statement(form, tables, constants, &st);
  return st;
}

// a_l for each lookup from one challenge stream, then lambda; constants a_l, a_l lambda (:43-51)
void layer_challenges(Transcript &tr, int D, int L, std::vector<uint32_t> &consts, std::vector<hf::E> &as,
                      hf::E &lam) {
  std::vector<uint32_t> raw((size_t)L * D);
  tr.challenges(L, D, raw.data());
  lam.assign(D, 0);
  tr.challenge(D, lam.data());
  consts.assign((size_t)2 * L * D, 0);
  as.clear();
  for (int l = 0; l < L; l++) {
    hf::E a(raw.begin() + (size_t)l * D, raw.begin() + (size_t)(l + 1) * D);
    hf::E al = hf::mul(a, lam);
    memcpy(&consts[(size_t)(2 * l) * D], a.data(), 4 * D);
    memcpy(&consts[(size_t)(2 * l + 1) * D], al.data(), 4 * D);
    as.push_back(a);
  }
}

hf::E layer_claim(int D, const std::vector<hf::E> &as, const hf::E &lam, const std::vector<hf::E> &cp,
                  const std::vector<hf::E> &cq) {  // :53-55
  hf::E acc = hf::zero(D);
  for (size_t l = 0; l < as.size(); l++) acc = hf::add(acc, hf::mul(as[l], hf::add(cp[l], hf::mul(lam, cq[l]))));
  return acc;
}

hf::E fold_pair(const hf::E &lo, const hf::E &hi, const hf::E &r) { return hf::add(lo, hf::mul(r, hf::sub(hi, lo))); }

void next_claims(int D, int L, const uint32_t *finals, const hf::E &tt, std::vector<hf::E> &cp,
                 std::vector<hf::E> &cq) {  // :57-63
  for (int l = 0; l < L; l++) {
    const uint32_t *f = finals + (size_t)(4 * l) * D;
    cp[l] = fold_pair(hf::from(f, D), hf::from(f + D, D), tt);
    cq[l] = fold_pair(hf::from(f + 2 * D, D), hf::from(f + 3 * D, D), tt);
  }
}

hf::E padded_mass(int D, int lk, int K, const std::vector<uint32_t> &rb) {  // :68-71
  std::vector<uint32_t> e = hf::eq_table(rb.data(), lk, D);
  hf::E mass = hf::zero(D);
  for (size_t b = K; b < ((size_t)1 << lk); b++) mass = hf::add(mass, hf::from(&e[b * D], D));
  return mass;
}

std::vector<uint32_t> block_weights(int D, int K, const std::vector<uint32_t> &rb) {  // :73-77
  if (rb.empty()) {
    std::vector<uint32_t> one((size_t)D, 0);
    one[0] = 1;
    return one;
  }
  std::vector<uint32_t> e = hf::eq_table(rb.data(), (int)(rb.size() / D), D);
  e.resize((size_t)K * D);
  return e;
}

int send_finals(Transcript &tr, int D, int ntables, const uint32_t *finals, hf::E &tt) {  // :208-213
  uint64_t dims[2] = {1, (uint64_t)D};
  for (int t = 0; t < ntables; t++) {
    int status = tr.send(finals + (size_t)t * D, 2, dims, nullptr);
    if (status) return status;
  }
  tt.assign(D, 0);
  tr.challenge(D, tt.data());
  return OK;
}

struct DeviceBuffers {  // frees what it allocated when the proof ends
  std::vector<void *> owned;
  ~DeviceBuffers() {
    for (void *p : owned) ctx().pool.release(p);
  }
  uint32_t *alloc(uint64_t words) {
    void *p = ctx().pool.alloc(words * 4);
    if (!p) return nullptr;
    owned.push_back(p);
    return (uint32_t *)p;
  }
};


constexpr size_t GKR_BW_PIN = 8192, GKR_BW_PIN_WORDS = 1024;  // words of the context's pinned buffer (see below)

// what the chain's sticky word means for the proof (host side)
int chain_outcome(uint32_t failed) {
  if (!failed) return OK;
  set_error("device-error: a chained layer's sumcheck did not complete (a workgroup gave up waiting, or rounds are "
            "missing); the proof is void");
  return E_DEVICE;
}

// PROVE-UPPER's in-block layers with one block, chained on the device (see gkr_glue_kernel): every launch of every
// layer's sumcheck is enqueued at once, the host waits once and reads the log.
// `held`: the finished layer's last launch (its rounds in one workgroup), not enqueued yet: the step rides on it
// (tail_glue_kernel); empty: the step is a launch of its own.
template <int D>
static int launch_glue(const GlueArgs<D> &a, std::vector<uint8_t> *held = nullptr, const KernelSet *kernels = nullptr) {
  Context &c = ctx();
  if (held && !held->empty() && kernels && kernels->launch_tail_glue) {
    c.prof_begin("tail", a.prev_rounds, 0);
    kernels->launch_tail_glue(held->data(), &a, c.stream);
    c.prof_end();
    held->clear();
    EXH_HIP(hipGetLastError());
    return OK;
  }
  c.prof_begin("gkr_glue", a.n, 0);
  hipLaunchKernelGGL(gkr_glue_kernel<D>, dim3(1), dim3(64), 0, c.stream, a);
  c.prof_end();
  EXH_HIP(hipGetLastError());
  return OK;
}

template <int D>
static int prove_upper_chained(Transcript &tr, int n, int L, const std::vector<std::vector<const uint32_t *>> &layers,
                               const std::string &label, uint32_t *out_ri, uint32_t *out_cp, uint32_t *out_cq) {
  Context &c = ctx();
  const int NT = 4 * L;
  Statement st = layer_statement(L, false);
  // the log: the roots, then per layer its round messages, challenges, finals and fresh point
  std::vector<size_t> log_off(n - 1);
  size_t words = (size_t)2 * L * D;
  for (int layer = 0; layer < n - 1; layer++) {
    const int points = layer > 0 ? 2 : 1;
    log_off[layer] = words;
    words += (size_t)layer * points * D + (size_t)layer * D + (size_t)NT * D + D;
  }
  DeviceBuffers bufs;
  GkrChainState *chain = reinterpret_cast<GkrChainState *>(bufs.alloc((sizeof(GkrChainState) + 3) / 4));
  uint32_t *d_log = bufs.alloc(words);
  if (!chain || !d_log) {
    set_error("device-out-of-memory: the GKR chain's log");
    return E_NOMEM;
  }
  const DevB3S first = device_state(tr);
  EXH_HIP(hipMemcpyAsync(&chain->tr, &first, sizeof(first), hipMemcpyHostToDevice, c.stream));
  // (a fill kernel would do as well; the chain is never captured into a graph)
  EXH_HIP(hipMemsetAsync(&chain->failed, 0, sizeof(chain->failed), c.stream));
  const std::vector<int> strides(NT, D);
  const std::vector<uint32_t> no_point((size_t)n * D, 0), no_consts((size_t)2 * L * D, 0);
  auto layer_tables = [&](int layer) {  // with one block the halves are views (LAYER-TABLES, src/gkr.lisp:199-206)
    std::vector<const uint32_t *> tabs(NT);
    const uint64_t size = (uint64_t)1 << layer;
    for (int l = 0; l < L; l++)
      for (int w = 0; w < 2; w++) {
        const uint32_t *v = layers[layer + 1][2 * l + w];
        tabs[4 * l + 2 * w] = v;
        tabs[4 * l + 2 * w + 1] = v + size * D;
      }
    return tabs;
  };
  int status;
  {  // the largest layer first, for its buffers alone: the arenas then never grow (and never wait) mid-chain
    SumcheckSession widest;
    std::vector<const uint32_t *> tabs = layer_tables(n - 2);
    if ((status = widest.begin(st, D, n - 2, tabs.data(), strides.data(), no_point.data(), nullptr, 1, no_consts.data(),
                               n - 2 > 0 ? 2 : 0, false, true)))
      return status;
  }
  const Ctrl *prev_ctrl = nullptr;
  std::vector<const uint32_t *> prev_tabs;
  const DevB3S unused_state = first;
  // a layer's last launch waits here for the next step, which rides on it (EXACTA_HIP_NO_GKR_FUSE=1: never)
  std::vector<uint8_t> held;
  const KernelSet *held_kernels = nullptr;
  const char *no_fuse = getenv("EXACTA_HIP_NO_GKR_FUSE");
  const bool fuse = !(no_fuse && no_fuse[0] == '1');
  for (int layer = 0; layer <= n - 1; layer++) {  // launch `layer` closes layer - 1 and opens `layer`; the last only closes
    GlueArgs<D> a;
    memset(&a, 0, sizeof(a));
    a.chain = chain, a.L = L, a.NT = NT;
    if (layer == 0) {
      a.close_kind = 1, a.log = d_log;
      for (int i = 0; i < 2 * L; i++) a.tabs[i] = layers[0][i];
    } else if (layer == 1) {  // layer 0 has no rounds: its finals are its tables' single entries
      a.close_kind = 3, a.prev_rounds = 0, a.prev_points = 1, a.log = d_log + log_off[0];
      for (int t = 0; t < NT; t++) a.tabs[t] = prev_tabs[t];
    } else {
      a.close_kind = 2, a.prev_ctrl = prev_ctrl, a.prev_rounds = layer - 1, a.prev_points = 2;
      a.log = d_log + log_off[layer - 1];
    }
    if (layer == n - 1) {
      if ((status = launch_glue<D>(a, &held, held_kernels))) return status;
      break;
    }
    const int degree = layer > 0 ? 2 : 0;
    const std::string header = header_bytes(label, layer, degree, 1);
    if (header.size() > 64) {
      set_error("invalid-parameter: label too long for the chained layers");
      return E_PARAM;
    }
    a.open = 1, a.n = layer, a.header_len = (int)header.size();
    for (size_t i = 0; i < header.size(); i++) a.header[i / 4] |= (uint32_t)(uint8_t)header[i] << (8 * (i % 4));
    std::vector<const uint32_t *> tabs = layer_tables(layer);
    if (layer == 0) {
      if ((status = launch_glue<D>(a))) return status;
    } else {
      SumcheckSession s;
      if ((status = s.begin(st, D, layer, tabs.data(), strides.data(), no_point.data(), nullptr, 1, no_consts.data(),
                            degree, false, true)))
        return status;
      std::vector<uint32_t> lagfix;
      std::vector<int> acc_group;
      s.message_map_scalars(&lagfix, &acc_group);
      a.points = s.points, a.nacc = std::max(s.st.nacc, 1), a.c0_words = layer * s.points * D;
      if ((int)lagfix.size() > MAXPTS * MAXACC || !s.setup_deferred) {
        set_error("invalid-parameter: layer statement beyond the chained layers' limits");
        return E_PARAM;
      }
      memcpy(a.lagfix, lagfix.data(), lagfix.size() * 4);
      for (int e = 0; e < a.nacc; e++) {
        const Group *g = acc_group[e] >= 0 ? &s.st.groups[acc_group[e]] : nullptr;
        if (!g || g->parts.size() != 1 || g->parts[0].coeff != 1 || g->parts[0].consts.size() != 1 ||
            g->parts[0].consts[0] >= GLUE_MAXCONST) {
          set_error("invalid-parameter: layer statement beyond the chained layers' limits");
          return E_PARAM;
        }
        a.acc_const[e] = (uint8_t)g->parts[0].consts[0];
      }
      a.factors = s.d_weights, a.mtilde = s.d_mtilde, a.c0 = s.d_c0, a.ctrl = s.d_ctrl;
      // (the step of this layer rides on the last launch of the layer before, when that was held back)
      std::vector<uint8_t> held_now;
      s.chain_hook = [&]() { return launch_glue<D>(a, &held, held_kernels); };
      if (fuse) s.held_tail = &held_now;
      if ((status = s.run_device(unused_state, nullptr, nullptr, nullptr))) return status;
      held.swap(held_now);
      held_kernels = s.kernels;
      prev_ctrl = s.d_ctrl;
    }
    prev_tabs = tabs;
  }
  // ---- one wait, then the log
  std::vector<uint32_t> log(words);
  DevB3S last;
  uint32_t failed = 0;
  EXH_HIP(hipMemcpyAsync(log.data(), d_log, words * 4, hipMemcpyDeviceToHost, c.stream));
  EXH_HIP(hipMemcpyAsync(&last, &chain->tr, sizeof(last), hipMemcpyDeviceToHost, c.stream));
  EXH_HIP(hipMemcpyAsync(&failed, &chain->failed, sizeof(failed), hipMemcpyDeviceToHost, c.stream));
  EXH_HIP(hipStreamSynchronize(c.stream));
  if ((status = chain_outcome(failed))) return status;
  // the messages as they were sent, recorded without hashing them again; the transcript takes the device's state
  uint64_t dims[2] = {2, (uint64_t)D};
  for (int l = 0; l < L; l++)
    if ((status = tr.send(&log[(size_t)l * 2 * D], 2, dims, nullptr, false))) return status;
  const uint32_t *fin = nullptr, *tt = nullptr, *rho = nullptr;
  for (int layer = 0; layer < n - 1; layer++) {
    const int points = layer > 0 ? 2 : 1;
    const uint32_t *msg = &log[log_off[layer]];
    rho = msg + (size_t)layer * points * D;
    fin = rho + (size_t)layer * D;
    tt = fin + (size_t)NT * D;
    dims[0] = (uint64_t)points;
    for (int j = 0; j < layer; j++)
      if ((status = tr.send(msg + (size_t)j * points * D, 2, dims, nullptr, false))) return status;
    dims[0] = 1;
    for (int t = 0; t < NT; t++)
      if ((status = tr.send(fin + (size_t)t * D, 2, dims, nullptr, false))) return status;
  }
  if ((status = adopt_device_state(tr, last))) return status;
  if (out_ri) {
    memcpy(out_ri, rho, (size_t)(n - 2) * D * 4);
    memcpy(out_ri + (size_t)(n - 2) * D, tt, (size_t)D * 4);
  }
  std::vector<hf::E> cp(L), cq(L);
  next_claims(D, L, fin, hf::from(tt, D), cp, cq);
  for (int l = 0; l < L; l++) {
    if (out_cp) memcpy(out_cp + (size_t)l * D, cp[l].data(), 4 * D);
    if (out_cq) memcpy(out_cq + (size_t)l * D, cq[l].data(), 4 * D);
  }
  return OK;
}

}  // namespace

int gkr_prove_upper(Transcript &tr, int n, int K, int L, const uint32_t *const *leaves, const std::string &label,
                    uint32_t *out_ri, uint32_t *out_rb, uint32_t *out_cp, uint32_t *out_cq) {
  Context &c = ctx();
  int status = c.require();
  if (status) return status;
  int D = tr.D, lk = block_bits(K), NT = 4 * L;
  if (L < 1 || NT + 1 > MAXT || n < 0 || n > 30 || K < 1) {
    set_error("invalid-parameter: GKR shape");
    return E_PARAM;
  }
  uint64_t Kp = (uint64_t)1 << lk;
  DeviceBuffers bufs;
  // FRACTION-TREES: every in-block layer, bottom up, kept on the device
  std::vector<std::vector<const uint32_t *>> layers(n + 1, std::vector<const uint32_t *>(2 * L));
  for (int i = 0; i < 2 * L; i++) layers[n][i] = leaves[i];
  // one allocation holds every layer above the leaves: 2 L K (2^n - 1) entries
  if ((status = c.tree.reserve(((((uint64_t)K << n) - K) * 2 * L * D + 64) * 4))) return status;
  uint32_t *next = (uint32_t *)c.tree.ptr;
  const int m_top = K == 1 ? std::min(n - 1, REDUCE_TOP_LAYERS - 1) : -1;  // these layers in one launch per lookup
  for (int m = n - 1; m >= 0; m--)
    for (int l = 0; l < L; l++) {
      uint64_t words = ((uint64_t)K << m) * D;
      uint32_t *pp = next, *qq = next + words;
      next += 2 * words;
      if (m > m_top &&
          (status = gkr_reduce_layer(D, K, m, layers[m + 1][2 * l], layers[m + 1][2 * l + 1], pp, qq)))
        return status;
      layers[m][2 * l] = pp;
      layers[m][2 * l + 1] = qq;
    }
  for (int l = 0; l < L && m_top >= 0; l++) {
    ReduceTopArgs a;
    memset(&a, 0, sizeof(a));
    a.p = layers[m_top + 1][2 * l], a.q = layers[m_top + 1][2 * l + 1], a.m_top = m_top;
    for (int m = m_top; m >= 0; m--)
      a.pp[m] = const_cast<uint32_t *>(layers[m][2 * l]), a.qq[m] = const_cast<uint32_t *>(layers[m][2 * l + 1]);
    if (D == 4)
      hipLaunchKernelGGL(gkr_reduce_top_kernel<4>, dim3(1), dim3(BLOCK), 0, c.stream, a);
    else
      hipLaunchKernelGGL(gkr_reduce_top_kernel<8>, dim3(1), dim3(BLOCK), 0, c.stream, a);
    EXH_HIP(hipGetLastError());
  }
  {  // one block: the layers chained on the device, one wait for the whole proof
    const char *host_rounds = getenv("EXACTA_HIP_HOST_ROUNDS"), *no_chain = getenv("EXACTA_HIP_NO_GKR_CHAIN");
    const bool off = (host_rounds && host_rounds[0] == '1') || (no_chain && no_chain[0] == '1');
    if (K == 1 && n >= 2 && n - 2 <= MAXROUNDS && L * D <= 12 && 2 * L <= GLUE_MAXCONST && !off) {
      status = D == 4 ? prove_upper_chained<4>(tr, n, L, layers, label, out_ri, out_cp, out_cq)
                      : prove_upper_chained<8>(tr, n, L, layers, label, out_ri, out_cp, out_cq);
      if (status) return status;
      EXH_HIP(hipStreamSynchronize(c.stream));
      return OK;
    }
  }
  // the per-block roots, and the top tree over the block index on the host (2^lk entries)
  std::vector<std::vector<std::vector<uint32_t>>> top(lk + 1, std::vector<std::vector<uint32_t>>(2 * L));
  EXH_HIP(hipStreamSynchronize(c.stream));
  for (int l = 0; l < L; l++) {
    std::vector<uint32_t> p(Kp * D, 0), q(Kp * D, 0);
    EXH_HIP(hipMemcpy(p.data(), layers[0][2 * l], (size_t)K * D * 4, hipMemcpyDeviceToHost));
    EXH_HIP(hipMemcpy(q.data(), layers[0][2 * l + 1], (size_t)K * D * 4, hipMemcpyDeviceToHost));
    for (uint64_t b = K; b < Kp; b++) q[b * D] = 1;  // padded with 0/1
    top[lk][2 * l] = p;
    top[lk][2 * l + 1] = q;
  }
  for (int j = lk - 1; j >= 0; j--)
    for (int l = 0; l < L; l++) {
      uint64_t len = (uint64_t)1 << j;
      const std::vector<uint32_t> &p = top[j + 1][2 * l], &q = top[j + 1][2 * l + 1];
      std::vector<uint32_t> pp(len * D), qq(len * D);
      for (uint64_t b = 0; b < len; b++) {
        hf::E p0 = hf::from(&p[b * D], D), p1 = hf::from(&p[(b + len) * D], D);
        hf::E q0 = hf::from(&q[b * D], D), q1 = hf::from(&q[(b + len) * D], D);
        hf::E np = hf::add(hf::mul(p0, q1), hf::mul(p1, q0)), nq = hf::mul(q0, q1);
        memcpy(&pp[b * D], np.data(), 4 * D);
        memcpy(&qq[b * D], nq.data(), 4 * D);
      }
      top[j][2 * l] = pp;
      top[j][2 * l + 1] = qq;
    }

  Statement st = layer_statement(L, false), st_blk = layer_statement(L, true);
  std::vector<hf::E> cp(L), cq(L), as;
  hf::E lam, tt;
  std::vector<uint32_t> consts, finals((size_t)(NT + 1) * D), rho((size_t)(n + lk + 1) * D);
  std::vector<uint32_t> r, ri;
  uint64_t dims2[2] = {2, (uint64_t)D};
  std::vector<int> strides(NT + 1, D);
  // The top tree is a tree of one block over the block index: its roots and layers are PROVE-UPPER's with one
  // block under the label's "-top", so the chain above serves it as well (one wait instead of one per layer).
  bool top_chained = false;
  {
    const char *host_rounds = getenv("EXACTA_HIP_HOST_ROUNDS"), *no_chain = getenv("EXACTA_HIP_NO_GKR_CHAIN");
    const bool off = (host_rounds && host_rounds[0] == '1') || (no_chain && no_chain[0] == '1');
    if (lk >= 1 && lk - 1 <= MAXROUNDS && L * D <= 12 && 2 * L <= GLUE_MAXCONST && !off) {
      // every level of every lookup's top tree in one buffer, one copy
      std::vector<std::vector<const uint32_t *>> top_layers(lk + 1, std::vector<const uint32_t *>(2 * L));
      std::vector<uint32_t> all;
      std::vector<std::vector<size_t>> at(lk + 1, std::vector<size_t>(2 * L));
      for (int j = 0; j <= lk; j++)
        for (int i = 0; i < 2 * L; i++) {
          at[j][i] = all.size();
          all.insert(all.end(), top[j][i].begin(), top[j][i].end());
        }
      uint32_t *d_top = bufs.alloc(all.size());
      if (!d_top) return E_NOMEM;
      EXH_HIP(hipMemcpyAsync(d_top, all.data(), all.size() * 4, hipMemcpyHostToDevice, c.stream));
      for (int j = 0; j <= lk; j++)
        for (int i = 0; i < 2 * L; i++) top_layers[j][i] = d_top + at[j][i];
      r.assign((size_t)lk * D, 0);
      std::vector<uint32_t> ocp((size_t)L * D), ocq((size_t)L * D);
      status = D == 4 ? prove_upper_chained<4>(tr, lk + 1, L, top_layers, label + "-top", r.data(), ocp.data(), ocq.data())
                      : prove_upper_chained<8>(tr, lk + 1, L, top_layers, label + "-top", r.data(), ocp.data(), ocq.data());
      if (status) return status;
      for (int l = 0; l < L; l++) {
        cp[l] = hf::from(&ocp[(size_t)l * D], D);
        cq[l] = hf::from(&ocq[(size_t)l * D], D);
      }
      top_chained = true;
    }
  }
  if (!top_chained) {
    for (int l = 0; l < L; l++) {  // the roots
      uint32_t root[16];
      memcpy(root, top[0][2 * l].data(), 4 * D);
      memcpy(root + D, top[0][2 * l + 1].data(), 4 * D);
      if ((status = tr.send(root, 2, dims2, nullptr))) return status;
      cp[l] = hf::from(root, D);
      cq[l] = hf::from(root + D, D);
    }
  }
  for (int j = 0; j < lk && !top_chained; j++) {  // the top tree, layer by layer
    layer_challenges(tr, D, L, consts, as, lam);
    uint64_t size = (uint64_t)1 << j;
    std::vector<const uint32_t *> tabs(NT);
    for (int l = 0; l < L; l++)
      for (int w = 0; w < 2; w++) {
        uint32_t *d = bufs.alloc(2 * size * D);
        if (!d) return E_NOMEM;
        EXH_HIP(hipMemcpy(d, top[j + 1][2 * l + w].data(), 2 * size * D * 4, hipMemcpyHostToDevice));
        tabs[4 * l + 2 * w] = d;                 // lower half: children b
        tabs[4 * l + 2 * w + 1] = d + size * D;  // upper half: children b + 2^j
      }
    status = sumcheck_prove(tr, j, st, tabs.data(), strides.data(), j > 0 ? r.data() : nullptr, consts.data(),
                            label + "-top", nullptr, 1, j > 0 ? 2 : 0, rho.data(), finals.data(), nullptr);
    if (status) return status;
    if ((status = send_finals(tr, D, NT, finals.data(), tt))) return status;
    next_claims(D, L, finals.data(), tt, cp, cq);
    r.assign(rho.begin(), rho.begin() + (size_t)j * D);
    r.insert(r.end(), tt.begin(), tt.end());
  }
  std::vector<uint32_t> rb = r;
  if (Kp != (uint64_t)K) {
    hf::E mass = padded_mass(D, lk, K, rb);
    for (int l = 0; l < L; l++) cq[l] = hf::sub(cq[l], mass);
  }
  for (int layer = 0; layer < n - 1; layer++) {  // the in-block layers
    layer_challenges(tr, D, L, consts, as, lam);
    std::vector<uint32_t> bw = block_weights(D, K, rb);
    uint64_t size = (uint64_t)1 << layer;
    std::vector<const uint32_t *> tabs(NT);
    if (K == 1) {  // the halves are views
      for (int l = 0; l < L; l++)
        for (int w = 0; w < 2; w++) {
          const uint32_t *v = layers[layer + 1][2 * l + w];
          tabs[4 * l + 2 * w] = v;
          tabs[4 * l + 2 * w + 1] = v + size * D;
        }
    } else {  // one launch splits the layer's 2 L vectors
      const uint64_t n_out = K * size;
      HalvesArgs h;
      memset(&h, 0, sizeof(h));
      if (!(h.out = bufs.alloc((uint64_t)NT * n_out * D))) return E_NOMEM;
      h.size_bits = (uint32_t)layer, h.n_out = n_out;
      for (int i = 0; i < 2 * L; i++) {
        h.v[i] = layers[layer + 1][i];
        tabs[2 * i] = h.out + (uint64_t)(2 * i) * n_out * D;
        tabs[2 * i + 1] = h.out + (uint64_t)(2 * i + 1) * n_out * D;
      }
      const dim3 grid((uint32_t)((n_out + BLOCK - 1) / BLOCK), (uint32_t)(2 * L));
      if (D == 4)
        hipLaunchKernelGGL(halves_kernel<4>, grid, dim3(BLOCK), 0, c.stream, h);
      else
        hipLaunchKernelGGL(halves_kernel<8>, grid, dim3(BLOCK), 0, c.stream, h);
      EXH_HIP(hipGetLastError());
    }
    // With several blocks the folded tables (one entry per block) stay on the device, zero padded to 2^lk, as the
    // tables of the sumcheck over the block index; the weights, padded alike, go before them in one copy.
    uint32_t *d_blk = nullptr;
    if (lk > 0) {
      if (!(d_blk = bufs.alloc((uint64_t)(NT + 1) * Kp * D))) return E_NOMEM;
    }
    status = sumcheck_prove(tr, layer, st, tabs.data(), strides.data(), layer > 0 ? ri.data() : nullptr,
                            consts.data(), label, bw.data(), K, layer > 0 ? 2 : 0, rho.data(),
                            lk > 0 ? nullptr : finals.data(), nullptr, lk > 0 ? d_blk + Kp * D : nullptr, Kp);
    if (status) return status;
    std::vector<uint32_t> rbn;
    if (lk > 0) {  // bind the block index: the blocks' values and weights, padded with zeros
      std::vector<const uint32_t *> btabs(NT + 1);
      std::vector<uint32_t> bwp(Kp * D, 0);
      memcpy(bwp.data(), bw.data(), (size_t)K * D * 4);
      for (int t = 0; t <= NT; t++) btabs[t] = d_blk + (uint64_t)t * Kp * D;
      // the weights' table: read by the sumcheck's first launch from pinned memory where the host puts it (a part
      // of the context's buffer nothing else uses; the host waits for this sumcheck before it writes there again),
      // or copied beside the blocks' values when it is longer than that part
      if (Kp * D <= GKR_BW_PIN_WORDS && c.host_pinned_dev) {
        memcpy(c.host_pinned + GKR_BW_PIN, bwp.data(), Kp * D * 4);
        btabs[0] = c.host_pinned_dev + GKR_BW_PIN;
      } else {
        EXH_HIP(hipMemcpy(d_blk, bwp.data(), Kp * D * 4, hipMemcpyHostToDevice));
      }
      std::vector<uint32_t> f2((size_t)(NT + 1) * D);
      rbn.assign((size_t)lk * D, 0);
      status = sumcheck_prove(tr, lk, st_blk, btabs.data(), strides.data(), nullptr, consts.data(), label + "-blk",
                              nullptr, 1, -1, rbn.data(), f2.data(), nullptr);
      if (status) return status;
      memcpy(finals.data(), f2.data() + D, (size_t)NT * D * 4);  // bw's final comes first
    }
    if ((status = send_finals(tr, D, NT, finals.data(), tt))) return status;
    next_claims(D, L, finals.data(), tt, cp, cq);
    ri.assign(rho.begin(), rho.begin() + (size_t)layer * D);
    ri.insert(ri.end(), tt.begin(), tt.end());
    rb = rbn;
  }
  if (out_ri && !ri.empty()) memcpy(out_ri, ri.data(), ri.size() * 4);
  if (out_rb && !rb.empty()) memcpy(out_rb, rb.data(), rb.size() * 4);
  for (int l = 0; l < L; l++) {
    if (out_cp) memcpy(out_cp + (size_t)l * D, cp[l].data(), 4 * D);
    if (out_cq) memcpy(out_cq + (size_t)l * D, cq[l].data(), 4 * D);
  }
  EXH_HIP(hipStreamSynchronize(c.stream));
  return OK;
}

int gkr_verify_upper(Transcript &tr, int n, int K, int L, const std::string &label, uint32_t *out_roots,
                     uint32_t *out_ri, uint32_t *out_rb, uint32_t *out_cp, uint32_t *out_cq) {
  int D = tr.D, lk = block_bits(K), NT = 4 * L, status;
  if (L < 1 || NT + 1 > MAXT || n < 0 || K < 1) {
    set_error("invalid-parameter: GKR shape");
    return E_PARAM;
  }
  uint64_t Kp = (uint64_t)1 << lk;
  std::vector<hf::E> cp(L), cq(L), as;
  hf::E lam, tt;
  uint64_t dims2[2] = {2, (uint64_t)D}, dims1[2] = {1, (uint64_t)D};
  for (int l = 0; l < L; l++) {
    uint32_t root[16];
    if ((status = tr.send(nullptr, 2, dims2, root))) return status;
    if (out_roots) memcpy(out_roots + (size_t)l * 2 * D, root, 8 * D);
    cp[l] = hf::from(root, D);
    cq[l] = hf::from(root + D, D);
  }
  Statement st = layer_statement(L, false), st_blk = layer_statement(L, true);
  std::vector<uint32_t> consts, finals((size_t)NT * D), rho((size_t)(n + lk + 1) * D), r, ri, rb;
  uint32_t reduced[8], expected[8];
  auto receive_finals = [&]() -> int {  // :84-89
    for (int t = 0; t < NT; t++) {
      int s = tr.send(nullptr, 2, dims1, &finals[(size_t)t * D]);
      if (s) return s;
    }
    tt.assign(D, 0);
    tr.challenge(D, tt.data());
    return OK;
  };
  for (int j = 0; j < lk; j++) {  // the top tree
    layer_challenges(tr, D, L, consts, as, lam);
    hf::E claim = layer_claim(D, as, lam, cp, cq);
    if ((status = sumcheck_verify(tr, j, st, claim.data(), j > 0 ? r.data() : nullptr, consts.data(), 1,
                                  label + "-top", j > 0 ? 2 : 0, rho.data(), reduced)))
      return status;
    if ((status = receive_finals())) return status;
    evaluate_statement(st, D, finals.data(), consts.data(), expected);
    if (memcmp(reduced, expected, 4 * D)) {
      set_error("verification-failure: gkr-top: layer " + std::to_string(j) + " of the top tree");
      return E_REJECT;
    }
    next_claims(D, L, finals.data(), tt, cp, cq);
    r.assign(rho.begin(), rho.begin() + (size_t)j * D);
    r.insert(r.end(), tt.begin(), tt.end());
  }
  rb = r;
  if (Kp != (uint64_t)K) {
    hf::E mass = padded_mass(D, lk, K, rb);
    for (int l = 0; l < L; l++) cq[l] = hf::sub(cq[l], mass);
  }
  for (int layer = 0; layer < n - 1; layer++) {  // the in-block layers
    layer_challenges(tr, D, L, consts, as, lam);
    std::vector<uint32_t> bw = block_weights(D, K, rb);
    hf::E claim = layer_claim(D, as, lam, cp, cq);
    if ((status = sumcheck_verify(tr, layer, st, claim.data(), layer > 0 ? ri.data() : nullptr, consts.data(), K,
                                  label, layer > 0 ? 2 : 0, rho.data(), reduced)))
      return status;
    std::vector<uint32_t> rbn;
    if (lk > 0) {
      rbn.assign((size_t)lk * D, 0);
      uint32_t red2[8];
      if ((status = sumcheck_verify(tr, lk, st_blk, reduced, nullptr, consts.data(), 1, label + "-blk", -1,
                                    rbn.data(), red2)))
        return status;
      memcpy(reduced, red2, 4 * D);
    }
    if ((status = receive_finals())) return status;
    hf::E weight = hf::zero(D);
    if (K > 1) {  // sum_b bw_b eq(rbn, b)
      std::vector<uint32_t> e = hf::eq_table(rbn.data(), lk, D);
      for (int b = 0; b < K; b++)
        weight = hf::add(weight, hf::mul(hf::from(&bw[(size_t)b * D], D), hf::from(&e[(size_t)b * D], D)));
    } else {
      weight = hf::from(bw.data(), D);
    }
    evaluate_statement(st, D, finals.data(), consts.data(), expected);
    hf::E want = hf::mul(weight, hf::from(expected, D));
    if (memcmp(reduced, want.data(), 4 * D)) {
      set_error("verification-failure: gkr-layer: in-block layer " + std::to_string(layer));
      return E_REJECT;
    }
    next_claims(D, L, finals.data(), tt, cp, cq);
    ri.assign(rho.begin(), rho.begin() + (size_t)layer * D);
    ri.insert(ri.end(), tt.begin(), tt.end());
    rb = rbn;
  }
  if (out_ri && !ri.empty()) memcpy(out_ri, ri.data(), ri.size() * 4);
  if (out_rb && !rb.empty()) memcpy(out_rb, rb.data(), rb.size() * 4);
  for (int l = 0; l < L; l++) {
    if (out_cp) memcpy(out_cp + (size_t)l * D, cp[l].data(), 4 * D);
    if (out_cq) memcpy(out_cq + (size_t)l * D, cq[l].data(), 4 * D);
  }
  return OK;
}

}  // namespace exh
