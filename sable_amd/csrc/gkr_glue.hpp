// gkr_glue.hpp -- the step between two layers' sumchecks of LogUp-GKR on the device (device code; see gkr.hip for
// the chain it belongs to), as a launch of its own and as the end of the launch that finishes a layer's rounds.
#pragma once
#include "sumcheck_kernels.hpp"

namespace exh {

// ------------------------------------------------------------------ the layers chained on the device
// With one block, the layers' sumchecks run back to back without the host: between two of them one small launch
// (one wavefront) does what PROVE-UPPER does on the host there (src/gkr.lisp:248-271) -- it sends the finished
// layer's finals and draws the fresh point (SEND-FINALS), forms the next layer's point, draws the layer's
// challenges (LAYER-CHALLENGES), absorbs the next sumcheck's header and writes that sumcheck's constants where its
// launches expect them: the eq point's factors, the message map, the head of the control block with the
// transcript's state.  Everything the host needs afterwards goes to a log it reads once at the end.
struct GkrChainState {
  DevB3S tr;                       // the transcript between launches
  uint32_t point[MAXROUNDS + 1][8];  // the next layer's eq point (canonical)
  // sticky: a chained layer's sumcheck did not complete (a workgroup of a grid launch gave up, or the control
  // block does not count the layer's rounds); the host reads it after its one wait and voids the proof
  uint32_t failed;
};

constexpr int GLUE_MAXCONST = 8;  // constants of a layer statement the launch can form: a_l and a_l lambda, l < 4

template <int D>
struct GlueArgs {
  GkrChainState *chain;
  int close_kind;  // 0: nothing to close, 1: send the roots, 2: a layer's finals from its control block, 3: from tables
  const Ctrl *prev_ctrl;
  int prev_rounds, prev_points;
  const uint32_t *tabs[MAXT];  // kind 1: the root of p and of q per lookup; kind 3: the layer's tables (one entry each)
  int NT, L;
  uint32_t *log;  // kind 1: the roots (2 L D words); kinds 2, 3: the layer's messages, challenges, finals, fresh point
  int open;       // open the next layer's sumcheck
  int n;          // its rounds
  uint32_t header[16];  // its header's bytes (src/sumcheck.lisp:24-27), as little-endian words
  int header_len;
  uint32_t *factors, *mtilde, *c0;
  Ctrl *ctrl;
  int points, nacc, c0_words;
  uint32_t lagfix[MAXPTS * MAXACC];
  uint8_t acc_const[MAXACC];  // the constant (a_l: 2 l, a_l lambda: 2 l + 1) that is the accumulator's group coefficient
};

// absorb(bytes) for LEN bytes held as little-endian words in LDS: the length as u64 LE, then the bytes
__device__ inline void dev_absorb_bytes(RunB3S &s, const uint32_t *words, uint32_t len) {
  const uint32_t lane = threadIdx.x & 63, total = 8 + len;
  for (uint32_t base = 0; base < total; base += 64) {
    const uint32_t g = base + lane;
    uint32_t word = g < 4 ? len : (g < 8 || g >= total) ? 0 : words[(g - 8) >> 2];
    rb3s_append_bytes(s, (word >> (8 * (g & 3))) & 0xff, total - base < 64 ? total - base : 64);
  }
}

// a word of a control block that this workgroup, or a launch before it, wrote: through the L2 (the first-level
// cache may still hold the line as it was when the launch began)
__device__ __forceinline__ uint32_t fresh_word(const uint32_t *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// One wavefront (the first of its workgroup) runs it, every lane the same steps.
template <int D>
__device__ __forceinline__ void gkr_glue_body(const GlueArgs<D> &a) {
  __shared__ uint32_t ring[RING_WORDS];
  __shared__ uint32_t buf[64];
  __shared__ uint32_t chal[16];
  __shared__ uint32_t fin[MAXT * 8];
  __shared__ uint32_t consts[GLUE_MAXCONST][8];
  __shared__ uint32_t point[MAXROUNDS + 1][8];
  const uint32_t lane = threadIdx.x;
  RunB3S tr;
  {  // the transcript's state where the last launch (or this one's rounds) left it
    const uint32_t *g = reinterpret_cast<const uint32_t *>(a.close_kind == 2 ? &a.prev_ctrl->tr : &a.chain->tr);
    if (lane < sizeof(DevB3S) / 4) buf[lane] = fresh_word(g + lane);
    __builtin_amdgcn_wave_barrier();
    rb3s_load(tr, ring, reinterpret_cast<const DevB3S *>(buf));
  }
  __builtin_amdgcn_wave_barrier();
  if (a.close_kind == 1) {  // the roots: one message (2, D) per lookup
    for (int l = 0; l < a.L; l++) {
      if (lane < 2 * D) buf[lane] = a.tabs[2 * l + lane / D][lane % D];
      __builtin_amdgcn_wave_barrier();
      dev_absorb_words(tr, buf, 2 * D);
      if (lane < 2 * D) a.log[l * 2 * D + lane] = buf[lane];
      __builtin_amdgcn_wave_barrier();
    }
  } else if (a.close_kind != 0) {
    const int R = a.prev_rounds, mw = a.prev_points * D;
    uint32_t *log_msg = a.log, *log_chal = log_msg + R * mw, *log_fin = log_chal + R * D, *log_tt = log_fin + a.NT * D;
    if (a.close_kind == 2) {
      if (lane == 0 && (fresh_word(&a.prev_ctrl->gave_up) != 0 || fresh_word(&a.prev_ctrl->round) != (uint32_t)R))
        a.chain->failed = 1;
      for (int u = lane; u < R * mw; u += 64) log_msg[u] = fresh_word(&a.prev_ctrl->msg[u / mw][u % mw]);
      for (int u = lane; u < R * D; u += 64) {
        const uint32_t v = fresh_word(&a.prev_ctrl->chal[u / D][u % D]);
        log_chal[u] = v;
        point[u / D][u % D] = v;  // the layer's challenges open the next layer's point
      }
    }
    // SEND-FINALS: one message (1, D) per table, then the fresh point (the finals fetched in one trip)
    for (int u = lane; u < a.NT * D; u += 64) {
      const uint32_t v = a.close_kind == 2 ? fresh_word(&a.prev_ctrl->finals[u]) : a.tabs[u / D][u % D];
      fin[u] = v;
      log_fin[u] = v;
    }
    __builtin_amdgcn_wave_barrier();
    for (int t = 0; t < a.NT; t++) dev_absorb_words(tr, fin + t * D, D);
    dev_challenge(tr, D, chal);
    __builtin_amdgcn_wave_barrier();
    if (lane < D) {
      log_tt[lane] = chal[lane];
      point[R][lane] = chal[lane];
    }
    __builtin_amdgcn_wave_barrier();
    for (int u = lane; u < (R + 1) * D; u += 64) a.chain->point[u / D][u % D] = point[u / D][u % D];
  }
  if (a.open) {
    if (a.close_kind == 0 || a.close_kind == 1)
      for (int u = lane; u < a.n * D; u += 64) point[u / D][u % D] = a.chain->point[u / D][u % D];
    // LAYER-CHALLENGES: a_l from one stream of L D base challenges, then lambda
    dev_challenge(tr, a.L * D, chal);
    __builtin_amdgcn_wave_barrier();
    if (lane < (uint32_t)(a.L * D)) consts[2 * (lane / D)][lane % D] = chal[lane];
    __builtin_amdgcn_wave_barrier();
    dev_challenge(tr, D, chal);
    __builtin_amdgcn_wave_barrier();
    if (lane < (uint32_t)a.L) {  // a_l lambda, exact: one factor carries R
      Ext<D> x, y;
#pragma unroll
      for (int c = 0; c < D; c++) x.c[c] = consts[2 * lane][c], y.c[c] = to_mont(chal[c]);
      const Ext<D> z = ext_mul_mont<D>(x, y);
#pragma unroll
      for (int c = 0; c < D; c++) consts[2 * lane + 1][c] = z.c[c];
    }
    __builtin_amdgcn_wave_barrier();
    if (lane < 16) buf[lane] = a.header[lane];
    __builtin_amdgcn_wave_barrier();
    dev_absorb_bytes(tr, buf, (uint32_t)a.header_len);
    if (a.n > 0) {
      // the eq point's factors r_v R and (1 - r_v) R, variable by variable
      for (int u = lane; u < a.n * D; u += 64) {
        const uint32_t v = u / D, k = u % D, r = point[v][k];
        a.factors[(2 * v) * D + k] = to_mont(r);
        a.factors[(2 * v + 1) * D + k] = to_mont(fsub(k == 0 ? 1u : 0u, r));
      }
      // the message map: the accumulator's group coefficient times its scalar, in Montgomery form
      for (int u = lane; u < a.points * a.nacc * D; u += 64) {
        const int e = u / D, c = u % D;
        a.mtilde[u] = to_mont(fmul(consts[a.acc_const[e % a.nacc]][c], a.lagfix[e]));
      }
      for (int u = lane; u < a.c0_words; u += 64) a.c0[u] = 0;
      uint32_t *head = reinterpret_cast<uint32_t *>(a.ctrl);
      for (uint32_t u = sizeof(DevB3S) / 4 + lane; u < offsetof(Ctrl, msg) / 4; u += 64) head[u] = 0;
      __builtin_amdgcn_wave_barrier();
      rb3s_store(tr, &a.ctrl->tr);
    }
  }
  rb3s_store(tr, &a.chain->tr);
}

template <int D>
__global__ __launch_bounds__(64) void gkr_glue_kernel(GlueArgs<D> a) {
  gkr_glue_body<D>(a);
}

// The launch that finishes a layer's rounds (one workgroup, the tables in LDS) going straight on to the step
// above: the layer's finals are in the control block this workgroup has just written, and its first wavefront
// closes the layer and opens the next one without a launch in between.
template <int D, class S>
__global__ __launch_bounds__(BLOCK) __attribute__((amdgpu_waves_per_eu(1, 1))) void tail_glue_kernel(TailArgs<D> t,
                                                                                                    GlueArgs<D> g) {
  tail_body<D>(S::d, t);
  __syncthreads();
  if (threadIdx.x < 64) gkr_glue_body<D>(g);
}

}  // namespace exh
