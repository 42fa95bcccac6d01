// prover.cpp -- see prover.hpp.
#include "prover.hpp"

#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <memory>
#include <vector>

#include "hostfield.hpp"

namespace exh {

// label | n u16 | degree u16 | blocks u32, little-endian (src/sumcheck.lisp:24-27)
std::string header_bytes(const std::string &label, int n, int degree, int blocks) {
  std::string h = label + "|";
  h.push_back((char)(n & 0xff)), h.push_back((char)((n >> 8) & 0xff));
  h.push_back((char)(degree & 0xff)), h.push_back((char)((degree >> 8) & 0xff));
  for (int i = 0; i < 4; i++) h.push_back((char)(((uint32_t)blocks >> (8 * i)) & 0xff));
  return h;
}
void absorb_header(Transcript &tr, const std::string &label, int n, int degree, int blocks) {
  std::string h = header_bytes(label, n, degree, blocks);
  tr.absorb((const uint8_t *)h.data(), h.size());
}

DevB3S device_state(const Transcript &tr) {
  DevB3S state;
  memcpy(state.cv, tr.state.cv, 32);
  for (int i = 0; i < 16; i++)
    state.block[i] = (uint32_t)tr.state.block[4 * i] | (uint32_t)tr.state.block[4 * i + 1] << 8 |
                     (uint32_t)tr.state.block[4 * i + 2] << 16 | (uint32_t)tr.state.block[4 * i + 3] << 24;
  state.used = tr.state.used;
  state.counter_lo = (uint32_t)tr.state.counter, state.counter_hi = (uint32_t)(tr.state.counter >> 32);
  return state;
}
int adopt_device_state(Transcript &tr, const DevB3S &state) {
  if (state.used > 64) {
    set_error("device-error: the device transcript's final state is malformed");
    return E_DEVICE;
  }
  memcpy(tr.state.cv, state.cv, 32);
  for (int i = 0; i < 64; i++) tr.state.block[i] = (uint8_t)(state.block[i / 4] >> (8 * (i % 4)));
  tr.state.used = state.used;
  tr.state.counter = ((uint64_t)state.counter_hi << 32) | state.counter_lo;
  return OK;
}

// A statement with more table monomials or accumulators than one kernel holds (the leaf-layer and zerocheck
// statement of a domain with many lookups and constraints, src/domain.lisp:95-114) is a sum of statements that
// fit: the monomials are dealt into parts, every part is a session of its own over the same tables, the parts'
// rounds run in step and a round's message is the sum of theirs.  Host-driven rounds: the reference's
// GENERIC-ROUND-SUMS role (src/sumcheck.lisp:282-317), the way that always works, not the fast one.
static bool fits_one_kernel(const Statement &st, int points) {  // points < 0: planned for the honest claim
  Statement planned = st;
  if (points < 0)
    planned.plan_claim();
  else
    planned.plan(points);
  StmtDesc d;
  return planned.T() <= MAXT && make_desc(planned, &d);
}

// the parts: as many of the expanded form's groups each as still fit one kernel
static int deal_parts(const Statement &st, int points, std::vector<Statement> *parts) {
  if (st.T() > MAXT || points > 16) {
    set_error("invalid-parameter: statement beyond the kernels' limits");
    return E_PARAM;
  }
  Statement part = st;
  part.factored_groups.clear(), part.factored_linear.clear(), part.expanded_groups.clear();
  auto with = [&](Statement base, const Group &g) {
    base.expanded_groups.push_back(g);
    base.groups = base.expanded_groups, base.planned_points = -1;
    return base;
  };
  for (const Group &g : st.expanded_groups) {
    Statement grown = with(part, g);
    if (fits_one_kernel(grown, points)) {
      part = grown;
      continue;
    }
    if (!part.expanded_groups.empty()) parts->push_back(part);
    part.expanded_groups.clear();
    part = with(part, g);
    if (!fits_one_kernel(part, points)) {
      set_error("invalid-parameter: a monomial of the statement is beyond the kernels' limits");
      return E_PARAM;
    }
  }
  if (!part.expanded_groups.empty()) parts->push_back(part);
  return OK;
}

// HYPERCUBE-SUM of a statement that one kernel does not hold: the sum of its parts' claims
int hypercube_sum_wide(const Statement &st, int D, int n, const uint32_t *const *d_tables, const int *strides,
                       const uint32_t *eq, const uint32_t *consts, uint32_t *out) {
  std::vector<Statement> parts;
  int status = deal_parts(st, -1, &parts);
  if (status) return status;
  std::vector<uint32_t> total((size_t)D, 0u);
  for (Statement &p : parts) {
    SumcheckSession s;
    s.private_buffers = true;
    if ((status = s.begin(p, D, n, d_tables, strides, eq, nullptr, 1, consts, -1, true))) return status;
    uint32_t sums[16 * 8];
    if ((status = s.round_sums(sums))) return status;
    for (int k = 0; k < D; k++) total[(size_t)k] = fadd(total[(size_t)k], sums[k]);
  }
  memcpy(out, total.data(), 4 * (size_t)D);
  return OK;
}

static int sumcheck_prove_wide(Transcript &tr, int n, const Statement &st, const uint32_t *const *d_tables,
                               const int *strides, const uint32_t *eq, const uint32_t *consts, const std::string &label,
                               const uint32_t *bw, int K, int degree, int points, uint32_t *out_chal,
                               uint32_t *out_finals, uint32_t *const *out_folded, uint32_t *d_folded,
                               uint64_t d_folded_len) {
  const int D = tr.D;
  std::vector<Statement> parts;
  if (int dealt = deal_parts(st, points, &parts)) return dealt;
  std::vector<std::unique_ptr<SumcheckSession>> sessions;
  int status;
  for (Statement &p : parts) {
    sessions.emplace_back(new SumcheckSession());
    sessions.back()->private_buffers = true;
    if ((status = sessions.back()->begin(p, D, n, d_tables, strides, eq, bw, K, consts, degree, false, false)))
      return status;
  }
  absorb_header(tr, label, n, degree, bw ? K : 1);
  std::vector<uint32_t> sums((size_t)points * D), total((size_t)points * D);
  for (int j = 0; j < n; j++) {
    std::fill(total.begin(), total.end(), 0u);
    for (auto &s : sessions) {
      if ((status = s->round_sums(sums.data()))) return status;
      for (size_t o = 0; o < total.size(); o++) total[o] = fadd(total[o], sums[o]);
    }
    uint64_t dims[2] = {(uint64_t)points, (uint64_t)D};
    if ((status = tr.send(total.data(), 2, dims, nullptr))) return status;
    uint32_t *r = out_chal + (size_t)j * D;
    tr.challenge(D, r);
    for (auto &s : sessions)
      if ((status = s->fold(r))) return status;
  }
  // every part folded the same tables
  if (d_folded && (status = sessions[0]->finish_device(d_folded, d_folded_len))) return status;
  return sessions[0]->finish(out_finals, out_folded);
}

int sumcheck_prove(Transcript &tr, int n, const Statement &st, const uint32_t *const *d_tables, const int *strides,
                   const uint32_t *eq, const uint32_t *consts, const std::string &label, const uint32_t *bw, int K,
                   int degree, uint32_t *out_chal, uint32_t *out_finals, uint32_t *const *out_folded,
                   uint32_t *d_folded, uint64_t d_folded_len) {
  int D = tr.D;
  if (degree < 0) degree = st.degree;
  int points = degree > 1 ? degree : 1;
  SumcheckSession first, second;
  const char *host_rounds = getenv("EXACTA_HIP_HOST_ROUNDS");
  // the device drives the rounds when it can: the session then sends all its constants in one copy
  const bool device_rounds = n > 0 && n <= MAXROUNDS && points <= MAXPTS && !(host_rounds && host_rounds[0] == '1');
  int status = first.begin(st, D, n, d_tables, strides, eq, bw, K, consts, degree, false, device_rounds);
  bool direct = false;
  if (status == E_PARAM && first.beyond_limits) {
    // Too wide for accumulators per table group.  The fast way: the statement in direct form, one session whose
    // kernels evaluate the written form at every wire point (compiled at run time, once per form and degree);
    // the way that always works: its monomials dealt into parts proved in step.
    const char *no_direct = getenv("EXACTA_HIP_NO_DIRECT");
    Statement direct_st;
    if (!(no_direct && no_direct[0] == '1') && n > 0 && make_direct(st, points, &direct_st)) {
      status = second.begin(direct_st, D, n, d_tables, strides, eq, bw, K, consts, degree, false, device_rounds);
      direct = status == OK;
    }
    if (!direct)
      return sumcheck_prove_wide(tr, n, st, d_tables, strides, eq, consts, label, bw, K, degree, points, out_chal,
                                 out_finals, out_folded, d_folded, d_folded_len);
  }
  if (status) return status;
  SumcheckSession &s = direct ? second : first;
  absorb_header(tr, label, n, degree, bw ? K : 1);
  if (device_rounds && s.device_capable()) {
    // the rounds run back to back on the device, transcript included.  This transcript then takes the messages
    // as they were sent and the hash state the device's transcript ended in; with EXACTA_HIP_REPLAY=1 it absorbs
    // the messages itself instead and checks that it draws the same challenges (a diagnostic: the two
    // transcripts are the same function, and the tests hold the device's to the oracle's bytes)
    DevB3S state = device_state(tr), final_state;
    std::vector<uint32_t> messages((size_t)n * points * D), challenges((size_t)n * D);
    {  // (EXACTA_HIP_FETCH_FINALS=1: fetch the folded tables with the logs all the same)
      const char *fetch = getenv("EXACTA_HIP_FETCH_FINALS");
      s.finals_stay = d_folded && !out_finals && !out_folded && !(fetch && fetch[0] == '1');
    }
    if ((status = s.run_device(state, messages.data(), challenges.data(), &final_state))) return status;
    const char *replay = getenv("EXACTA_HIP_REPLAY");
    const bool replaying = replay && replay[0] == '1';
    for (int j = 0; j < n; j++) {
      uint64_t dims[2] = {(uint64_t)points, (uint64_t)D};
      int st_send = tr.send(&messages[(size_t)j * points * D], 2, dims, nullptr, replaying);
      if (st_send) return st_send;
      uint32_t *r = out_chal + (size_t)j * D;
      if (replaying) {
        tr.challenge(D, r);
        if (memcmp(r, &challenges[(size_t)j * D], 4 * D) != 0) {
          set_error("device-error: the device transcript drew a different challenge in round " + std::to_string(j));
          return E_DEVICE;
        }
      } else {
        memcpy(r, &challenges[(size_t)j * D], 4 * D);
      }
    }
    if (!replaying && (status = adopt_device_state(tr, final_state))) return status;
    if (d_folded && (status = s.finish_device(d_folded, d_folded_len))) return status;
    return s.finish(out_finals, out_folded);
  }
  uint32_t sums[16 * 8];
  for (int j = 0; j < n; j++) {
    if ((status = s.round_sums(sums))) return status;
    uint64_t dims[2] = {(uint64_t)points, (uint64_t)D};
    if ((status = tr.send(sums, 2, dims, nullptr))) return status;
    uint32_t *r = out_chal + (size_t)j * D;
    tr.challenge(D, r);
    if ((status = s.fold(r))) return status;
  }
  if (d_folded && (status = s.finish_device(d_folded, d_folded_len))) return status;
  return s.finish(out_finals, out_folded);
}

// g(X) at x from the message (g at 0, 2, 3, ...) and the claim, which gives g(1)
// (NEXT-CLAIM, src/sumcheck.lisp:137-145)
static int next_claim(int D, int points, hf::E &claim, const uint32_t *message, const uint32_t *eq_rj,
                      const uint32_t *x) {
  std::vector<hf::E> vals;
  hf::E g0 = hf::from(message, D), g1;
  if (eq_rj) {  // claim = (1 - r) g(0) + r g(1)
    hf::E r = hf::from(eq_rj, D);
    if (hf::is_zero(r)) {
      set_error("field-division-by-zero: ext-inv of the eq point's coordinate");
      return E_DIVZERO;
    }
    g1 = hf::mul(hf::sub(claim, hf::mul(hf::sub(hf::lift(1, D), r), g0)), hf::inv(r));
  } else {
    g1 = hf::sub(claim, g0);
  }
  vals.push_back(g0);
  vals.push_back(g1);
  for (int k = 1; k < points; k++) vals.push_back(hf::from(message + (size_t)k * D, D));
  claim = hf::lagrange(vals, hf::from(x, D));
  return OK;
}

int sumcheck_verify(Transcript &tr, int n, const Statement &st, const uint32_t *claim_in, const uint32_t *eq,
                    const uint32_t *consts, int blocks, const std::string &label, int degree, uint32_t *out_chal,
                    uint32_t *out_reduced) {
  (void)consts;
  int D = tr.D;
  if (degree < 0) degree = st.degree;
  int points = degree > 1 ? degree : 1;
  if (points > 16) {
    set_error("invalid-parameter: degree");
    return E_PARAM;
  }
  hf::E claim(D);
  for (int k = 0; k < D; k++) claim[k] = claim_in[k] % P;
  absorb_header(tr, label, n, degree, blocks);
  for (int j = 0; j < n; j++) {
    uint32_t message[16 * 8];
    uint64_t dims[2] = {(uint64_t)points, (uint64_t)D};
    int status = tr.send(nullptr, 2, dims, message);
    if (status) {
      set_error(status == E_EXHAUSTED ? "transcript-exhausted: round message" : "message-shape-error: round message");
      return status;
    }
    uint32_t *r = out_chal + (size_t)j * D;
    tr.challenge(D, r);
    if ((status = next_claim(D, points, claim, message, eq ? eq + (size_t)j * D : nullptr, r))) return status;
  }
  memcpy(out_reduced, claim.data(), 4 * D);
  return OK;
}

int check_final(const Statement &st, int D, const uint32_t *reduced, const uint32_t *finals, const uint32_t *consts) {
  uint32_t expected[8];
  evaluate_statement(st, D, finals, consts, expected);
  if (memcmp(expected, reduced, 4 * D) != 0) {
    set_error("verification-failure: sumcheck-final: reduced claim differs from the statement at the final values");
    return E_REJECT;
  }
  return OK;
}

}  // namespace exh
