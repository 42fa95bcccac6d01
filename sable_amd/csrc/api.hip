// api.hip -- the C ABI (include/exacta_hip.h, include/exacta_host.h) over the C++ internals.
#include <string.h>

#include <map>
#include <memory>
#include <mutex>
#include <thread>

#include "../../include/exacta_host.h"
#include "commit.hpp"
#include "context.hpp"
#include "domain.hpp"
#include "gkr.hpp"
#include "hostfield.hpp"
#include "prover.hpp"
#include "rtc.hpp"
#include "sumcheck.hpp"
#include "transcript.hpp"

using namespace exh;

namespace {
// Every entry point runs under one lock: the context, its handle maps, pool, arenas and pinned staging area are
// one per process, and a host with several threads (ctypes releases Python's lock during a call) would otherwise
// interleave inside them.  Calls from several threads are therefore safe and take turns; they do not overlap.
std::recursive_mutex g_api_mutex;
struct ApiLock {
  std::lock_guard<std::recursive_mutex> guard{g_api_mutex};
};
std::map<uint64_t, std::unique_ptr<Statement>> g_stmts;
std::map<uint64_t, std::unique_ptr<SumcheckSession>> g_sessions;
std::map<uint64_t, std::unique_ptr<Transcript>> g_transcripts;
uint64_t g_next = 1;

Statement *stmt_of(exh_stmt h) {
  auto it = g_stmts.find(h);
  if (it == g_stmts.end()) {
    set_error("invalid-parameter: unknown statement handle");
    return nullptr;
  }
  return it->second.get();
}
Transcript *tr_of(exh_transcript h) {
  auto it = g_transcripts.find(h);
  if (it == g_transcripts.end()) {
    set_error("invalid-parameter: unknown transcript handle");
    return nullptr;
  }
  return it->second.get();
}
DeviceTable *table_of(exh_table h) {
  auto it = ctx().tables.find(h);
  if (it == ctx().tables.end()) {
    set_error("invalid-parameter: unknown table handle");
    return nullptr;
  }
  return &it->second;
}
exh_table add_table(uint32_t *ptr, uint64_t n_u32, int stride, bool owned) {
  Context &c = ctx();
  uint64_t h = c.next_handle++;
  c.tables[h] = DeviceTable{ptr, n_u32, stride, owned};
  return h;
}
// device pointers and strides of a list of table handles, each checked against `entries`
int gather_tables(const exh_table *tables, int n, int D, uint64_t entries, std::vector<const uint32_t *> *ptrs,
                  std::vector<int> *strides) {
  ptrs->clear();
  strides->clear();
  for (int t = 0; t < n; t++) {
    DeviceTable *dt = table_of(tables[t]);
    if (!dt) return E_PARAM;
    if (dt->stride != 1 && dt->stride != D) {
      set_error("invalid-parameter: table stride must be 1 or the transcript's degree");
      return E_PARAM;
    }
    if (dt->n_u32 != entries * (uint64_t)dt->stride) {
      set_error("invalid-parameter: table size: expected " + std::to_string(entries) + " entries");
      return E_PARAM;
    }
    ptrs->push_back(dt->ptr);
    strides->push_back(dt->stride);
  }
  return OK;
}
}  // namespace

extern "C" {

// ------------------------------------------------------------------ context
int exh_init(int device) {
  ApiLock api_lock;
  return ctx_init(device);
}
void exh_shutdown(void) {
  ApiLock api_lock;
  // a compilation still running is waited for here, so that a host that shuts the library down before it exits
  // keeps its own exit handlers (the hard exit of rtc.cpp is for a process that ends without this call)
  (void)rtc_idle(true);
  g_sessions.clear();
  ctx_shutdown();
}
const char *exh_last_error(void) { return last_error(); }
int exh_synchronize(void) {
  ApiLock api_lock;
  int status = ctx().require();
  if (status) return status;
  EXH_HIP(hipDeviceSynchronize());
  return OK;
}

// ---- issue-rate measurement (issue_rate.hip)
int exh_issue_rate_ops(void) { return issue_rate_ops(); }
int exh_issue_rate(int op, int chains, int workgroups, int iterations, char *name, int name_cap, float *ms,
                   double *instructions_per_wave, int *clock_khz, int *compute_units) {
  ApiLock api_lock;
  const char *op_name = nullptr;
  float t = 0;
  int status = issue_rate(op, chains, workgroups, iterations, &op_name, &t, instructions_per_wave, clock_khz,
                          compute_units);
  if (status) return status;
  if (ms) *ms = t;
  if (name && name_cap > 0 && op_name) {
    strncpy(name, op_name, name_cap - 1);
    name[name_cap - 1] = 0;
  }
  return OK;
}

int exh_profile_enable(int on) {
  ApiLock api_lock;
  Context &c = ctx();
  int status = c.require();
  if (status) return status;
  (void)hipStreamSynchronize(c.stream);
  c.prof_clear();
  c.profiling = on != 0;
  return OK;
}
int exh_profile_count(void) {
  ApiLock api_lock;
  return (int)ctx().profile.size();
}
int exh_profile_entry(int index, char *name, int name_cap, int *round, float *ms, uint64_t *alg_bytes) {
  ApiLock api_lock;
  Context &c = ctx();
  if (index < 0 || index >= (int)c.profile.size()) {
    set_error("invalid-parameter: profile index");
    return E_PARAM;
  }
  ProfileEntry &e = c.profile[index];
  if (e.ms < 0) {
    EXH_HIP(hipEventSynchronize(e.stop));
    EXH_HIP(hipEventElapsedTime(&e.ms, e.start, e.stop));
  }
  if (name && name_cap > 0) {
    strncpy(name, e.name.c_str(), name_cap - 1);
    name[name_cap - 1] = 0;
  }
  if (round) *round = e.round;
  if (ms) *ms = e.ms;
  if (alg_bytes) *alg_bytes = e.alg_bytes;
  return OK;
}

// ------------------------------------------------------------------ tables
int exh_table_alloc(uint64_t n_u32, int stride, exh_table *out) {
  ApiLock api_lock;
  int status = ctx().require();
  if (status) return status;
  if (stride < 1 || stride > 8 || n_u32 % stride) {
    set_error("invalid-parameter: table stride");
    return E_PARAM;
  }
  void *ptr = ctx().pool.alloc(n_u32 * 4);
  if (!ptr) {
    set_error("device-out-of-memory: table of " + std::to_string(n_u32 * 4) + " bytes");
    return E_NOMEM;
  }
  *out = add_table((uint32_t *)ptr, n_u32, stride, true);
  return OK;
}

int exh_table_upload(const uint32_t *host, uint64_t n_u32, int stride, exh_table *out) {
  ApiLock api_lock;
  for (uint64_t i = 0; i < n_u32; i++)
    if (host[i] >= P) {
      set_error("invalid-parameter: table values must be canonical (below p)");
      return E_PARAM;
    }
  int status = exh_table_alloc(n_u32, stride, out);
  if (status) return status;
  DeviceTable *dt = table_of(*out);
  EXH_HIP(hipMemcpy(dt->ptr, host, n_u32 * 4, hipMemcpyHostToDevice));
  return OK;
}

int exh_table_wrap(void *device_ptr, uint64_t n_u32, int stride, exh_table *out) {
  ApiLock api_lock;
  int status = ctx().require();
  if (status) return status;
  if (!device_ptr || stride < 1 || stride > 8 || ((uintptr_t)device_ptr & 15)) {
    set_error("invalid-parameter: wrapped table must be a 16-byte aligned device pointer");
    return E_PARAM;
  }
  *out = add_table((uint32_t *)device_ptr, n_u32, stride, false);
  return OK;
}

int exh_table_download(exh_table table, uint64_t offset_u32, uint32_t *host, uint64_t n_u32) {
  ApiLock api_lock;
  DeviceTable *dt = table_of(table);
  if (!dt) return E_PARAM;
  if (offset_u32 + n_u32 > dt->n_u32) {
    set_error("invalid-parameter: download beyond the table");
    return E_PARAM;
  }
  EXH_HIP(hipStreamSynchronize(ctx().stream));
  EXH_HIP(hipMemcpy(host, dt->ptr + offset_u32, n_u32 * 4, hipMemcpyDeviceToHost));
  return OK;
}

int exh_table_free(exh_table table) {
  ApiLock api_lock;
  DeviceTable *dt = table_of(table);
  if (!dt) return E_PARAM;
  if (dt->owned && dt->ptr) ctx().pool.release(dt->ptr);  // stream-ordered reuse: no wait
  ctx().tables.erase(table);
  return OK;
}

void *exh_table_device_ptr(exh_table table) {
  ApiLock api_lock;
  DeviceTable *dt = table_of(table);
  return dt ? dt->ptr : nullptr;
}

int exh_table_random(uint64_t seed, uint64_t n_u32, int stride, exh_table *out) {
  ApiLock api_lock;
  std::vector<uint32_t> host(n_u32);
  uint64_t x = seed;
  for (uint64_t i = 0; i < n_u32;) {
    x += 0x9E3779B97F4A7C15ull;  // SplitMix64
    uint64_t z = x;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    uint32_t w = (uint32_t)(z >> 33);
    if (w < P) host[i++] = w;
  }
  int status = exh_table_alloc(n_u32, stride, out);
  if (status) return status;
  EXH_HIP(hipMemcpy(table_of(*out)->ptr, host.data(), n_u32 * 4, hipMemcpyHostToDevice));
  return OK;
}

// ------------------------------------------------------------------ statements
int exh_stmt_compile(const char *form, const char *const *tables, int n_tables, const char *const *constants,
                     int n_constants, exh_stmt *out) {
  ApiLock api_lock;
  auto st = std::make_unique<Statement>();
  std::vector<std::string> tn, cn;
  for (int i = 0; i < n_tables; i++) tn.push_back(tables[i]);
  for (int i = 0; i < n_constants; i++) cn.push_back(constants[i]);
  int status = compile_statement(form, tn, cn, st.get());
  if (status) return status;
  *out = g_next++;
  g_stmts[*out] = std::move(st);
  return OK;
}
int exh_stmt_degree(exh_stmt stmt) {
  ApiLock api_lock;
  Statement *st = stmt_of(stmt);
  return st ? st->degree : E_PARAM;
}
int exh_stmt_free(exh_stmt stmt) {
  ApiLock api_lock;
  if (!stmt_of(stmt)) return E_PARAM;
  g_stmts.erase(stmt);
  return OK;
}
int exh_stmt_has_generated_kernel(exh_stmt stmt, int D) {
  ApiLock api_lock;
  Statement *st = stmt_of(stmt);
  if (!st) return E_PARAM;
  Statement copy = *st;
  copy.plan(copy.degree > 1 ? copy.degree : 1);
  if (ctx().ready) (void)rtc_collect();
  if (find_kernels(copy.key(), D)) return 1;
  StmtDesc desc;
  Statement direct;  // a statement too wide for the table groups' kernels: those of its direct form
  if ((copy.T() > MAXT || !make_desc(copy, &desc)) && make_direct(*st, copy.degree > 1 ? copy.degree : 1, &direct))
    return find_kernels(direct.key(), D) ? 1 : 0;
  return 0;
}
int exh_stmt_generate_idle(int wait) {
  ApiLock api_lock;
  return rtc_idle(wait != 0);
}
int exh_stmt_generate(exh_stmt stmt, int D, int degree, int wait) {
  ApiLock api_lock;
  Statement *st = stmt_of(stmt);
  if (!st) return E_PARAM;
  int status = ctx().require();
  if (status) return status;
  if (D != 4 && D != 8) {
    set_error("invalid-parameter: degree");
    return E_PARAM;
  }
  Statement copy = *st;
  if (degree < 0) degree = copy.degree;
  copy.plan(degree > 1 ? degree : 1);
  if (find_kernels(copy.key(), D)) return 1;
  StmtDesc desc;
  if (copy.T() > MAXT || !make_desc(copy, &desc)) {
    // too wide for accumulators per table group: the kernels of its direct form, which evaluate the written
    // form itself at every wire point
    Statement direct;
    if (!make_direct(*st, degree > 1 ? degree : 1, &direct) || !make_desc(direct, &desc)) {
      set_error("invalid-parameter: statement beyond the kernels' limits");
      return E_PARAM;
    }
    if (find_kernels(direct.key(), D)) return 1;
    rtc_request(direct.key(), desc, D, direct_source(direct, desc, "RtStmt"));
    return rtc_status(direct.key(), D, wait != 0);
  }
  rtc_request(copy.key(), desc, D);
  return rtc_status(copy.key(), D, wait != 0);
}

// ------------------------------------------------------------------ sumcheck sessions
int exh_sumcheck_begin(exh_stmt stmt, int D, int n, const exh_table *tables, int n_tables, const uint32_t *eq,
                       const uint32_t *bw, int K, const uint32_t *constants, int degree, exh_session *out) {
  ApiLock api_lock;
  Statement *st = stmt_of(stmt);
  if (!st) return E_PARAM;
  if (n_tables != st->T() || (!bw && K != 1) || K < 1 || n < 0 || n > 40) {
    set_error("invalid-parameter: sumcheck arguments");
    return E_PARAM;
  }
  std::vector<const uint32_t *> ptrs;
  std::vector<int> strides;
  int status = gather_tables(tables, n_tables, D, (uint64_t)K << n, &ptrs, &strides);
  if (status) return status;
  auto s = std::make_unique<SumcheckSession>();
  if ((status = s->begin(*st, D, n, ptrs.data(), strides.data(), eq, bw, K, constants, degree))) return status;
  *out = g_next++;
  g_sessions[*out] = std::move(s);
  return OK;
}
static SumcheckSession *session_of(exh_session h) {
  auto it = g_sessions.find(h);
  if (it == g_sessions.end()) {
    set_error("invalid-parameter: unknown session handle");
    return nullptr;
  }
  return it->second.get();
}
int exh_sumcheck_round(exh_session session, uint32_t *out_sums) {
  ApiLock api_lock;
  SumcheckSession *s = session_of(session);
  return s ? s->round_sums(out_sums) : E_PARAM;
}
int exh_sumcheck_fold(exh_session session, const uint32_t *r) {
  ApiLock api_lock;
  SumcheckSession *s = session_of(session);
  return s ? s->fold(r) : E_PARAM;
}
int exh_sumcheck_run(exh_session session, const uint32_t *cv, const uint8_t *block, uint32_t used, uint64_t counter,
                     uint32_t *out_messages, uint32_t *out_challenges) {
  ApiLock api_lock;
  SumcheckSession *s = session_of(session);
  if (!s || !cv || !block || used > 64 || !out_messages || !out_challenges) {
    set_error("invalid-parameter: exh_sumcheck_run arguments");
    return E_PARAM;
  }
  DevB3S state;
  memcpy(state.cv, cv, 32);
  for (int i = 0; i < 16; i++)
    state.block[i] = (uint32_t)block[4 * i] | (uint32_t)block[4 * i + 1] << 8 | (uint32_t)block[4 * i + 2] << 16 |
                     (uint32_t)block[4 * i + 3] << 24;
  state.used = used;
  state.counter_lo = (uint32_t)counter, state.counter_hi = (uint32_t)(counter >> 32);
  return s->run_device(state, out_messages, out_challenges);
}
int exh_sumcheck_finish(exh_session session, uint32_t *finals, uint32_t *const *folded) {
  ApiLock api_lock;
  SumcheckSession *s = session_of(session);
  if (!s) return E_PARAM;
  int status = s->finish(finals, folded);
  g_sessions.erase(session);
  return status;
}

// ------------------------------------------------------------------ host field helpers
int exh_ext_mul(int D, const uint32_t *a, const uint32_t *b, uint32_t *out) {
  ApiLock api_lock;
  if (D != 4 && D != 8) return E_PARAM;
  hf::mul_raw(D, a, b, out);
  return OK;
}
int exh_ext_inv(int D, const uint32_t *a, uint32_t *out) {
  ApiLock api_lock;
  if (D != 4 && D != 8) return E_PARAM;
  hf::E x = hf::from(a, D);
  if (hf::is_zero(x)) {
    memset(out, 0, 4 * D);
    set_error("field-division-by-zero: ext-inv");
    return E_DIVZERO;
  }
  hf::E r = hf::inv(x);
  memcpy(out, r.data(), 4 * D);
  return OK;
}
int exh_eq_table(int D, int k, const uint32_t *r, uint32_t *out) {
  ApiLock api_lock;
  if ((D != 4 && D != 8) || k < 0 || k > 24) return E_PARAM;
  std::vector<uint32_t> t = hf::eq_table(r, k, D);
  memcpy(out, t.data(), t.size() * 4);
  return OK;
}

int exh_eq_table_device(int D, int k, const uint32_t *r, exh_table *out) {
  ApiLock api_lock;
  if ((D != 4 && D != 8) || k < 0 || k > 26 || (k > 0 && !r) || !out) {
    set_error("invalid-parameter: eq table of k <= 26 coordinates of degree 4 or 8");
    return E_PARAM;
  }
  int status = exh_table_alloc(((uint64_t)D) << k, D, out);
  if (status) return status;
  status = eq_table_device(D, k, r, table_of(*out)->ptr);
  if (status) exh_table_free(*out);
  return status;
}

// ------------------------------------------------------------------ transcript
int exh_blake3(const uint8_t *in, uint64_t len, uint8_t *out, uint64_t out_len) {
  ApiLock api_lock;
  blake3_hash(in, len, out, out_len);
  return OK;
}
int exh_transcript_new(const uint8_t *label, uint64_t label_len, int D, const uint8_t *proof, uint64_t proof_len,
                       exh_transcript *out) {
  ApiLock api_lock;
  if (D != 4 && D != 8) {
    set_error("invalid-parameter: degree: expected 4 or 8");
    return E_PARAM;
  }
  auto tr = std::make_unique<Transcript>(label, label_len, D);
  if (proof) {
    int status = tr->load_proof(proof, proof_len);
    if (status) {
      static const char *reasons[] = {"", "magic", "truncated", "trailing-bytes", "unknown-tag", "value-range", "rank",
                                      "dimension"};
      set_error(std::string("malformed-proof: ") + reasons[tr->malformed_reason]);
      return status;
    }
  }
  *out = g_next++;
  g_transcripts[*out] = std::move(tr);
  return OK;
}
int exh_transcript_free(exh_transcript h) {
  ApiLock api_lock;
  if (!tr_of(h)) return E_PARAM;
  g_transcripts.erase(h);
  return OK;
}
int exh_transcript_absorb(exh_transcript h, const uint8_t *data, uint64_t len) {
  ApiLock api_lock;
  Transcript *tr = tr_of(h);
  if (!tr) return E_PARAM;
  tr->absorb(data, len);
  return OK;
}
int exh_transcript_send(exh_transcript h, const uint32_t *vals, int rank, const uint64_t *dims, uint32_t *out,
                        int absorb) {
  ApiLock api_lock;
  Transcript *tr = tr_of(h);
  if (!tr) return E_PARAM;
  int status = tr->send(vals, rank, dims, out, absorb != 0);
  if (status == E_SHAPE) set_error("message-shape-error");
  if (status == E_EXHAUSTED) set_error("transcript-exhausted");
  return status;
}
int exh_transcript_send_bytes(exh_transcript h, const uint8_t *bytes, int64_t len, uint8_t *out, uint64_t cap,
                              uint64_t *out_len, int absorb) {
  ApiLock api_lock;
  Transcript *tr = tr_of(h);
  if (!tr) return E_PARAM;
  std::vector<uint8_t> got;
  int status = tr->send_bytes(bytes, len, &got, absorb != 0);
  if (status == E_SHAPE) set_error("message-shape-error");
  if (status == E_EXHAUSTED) set_error("transcript-exhausted");
  if (status) return status;
  if (out_len) *out_len = got.size();
  if (out) memcpy(out, got.data(), got.size() < cap ? got.size() : cap);
  return OK;
}
int exh_transcript_challenge_base(exh_transcript h, int k, uint32_t *out) {
  ApiLock api_lock;
  Transcript *tr = tr_of(h);
  if (!tr) return E_PARAM;
  tr->challenge_base(k, out);
  return OK;
}
int exh_transcript_challenge_bits(exh_transcript h, int nbits, int k, uint64_t *out) {
  ApiLock api_lock;
  Transcript *tr = tr_of(h);
  if (!tr) return E_PARAM;
  tr->challenge_bits(nbits, k, out);
  return OK;
}
int exh_transcript_grind(exh_transcript h, int bits, uint64_t *nonce) {
  ApiLock api_lock;
  Transcript *tr = tr_of(h);
  if (!tr) return E_PARAM;
  *nonce = tr->grind(bits);
  return OK;
}
int exh_transcript_verify_grind(exh_transcript h, int bits, uint64_t *nonce) {
  ApiLock api_lock;
  Transcript *tr = tr_of(h);
  if (!tr) return E_PARAM;
  int status = tr->verify_grind(bits, nonce);
  if (status == E_REJECT) set_error("verification-failure: proof-of-work");
  return status;
}
int exh_transcript_digest(exh_transcript h, uint8_t out[32]) {
  ApiLock api_lock;
  Transcript *tr = tr_of(h);
  if (!tr) return E_PARAM;
  tr->state.digest(out, 32);
  return OK;
}
int exh_transcript_state(exh_transcript h, uint32_t cv[8], uint8_t block[64], uint32_t *used, uint64_t *counter) {
  ApiLock api_lock;
  Transcript *tr = tr_of(h);
  if (!tr || !cv || !block || !used || !counter) return E_PARAM;
  memcpy(cv, tr->state.cv, 32);
  memset(block, 0, 64);
  memcpy(block, tr->state.block, tr->state.used);
  *used = tr->state.used;
  *counter = tr->state.counter;
  return OK;
}
int exh_transcript_finished(exh_transcript h) {
  ApiLock api_lock;
  Transcript *tr = tr_of(h);
  return tr ? (tr->finished() ? 1 : 0) : E_PARAM;
}
int exh_transcript_message_count(exh_transcript h, uint64_t *count) {
  ApiLock api_lock;
  Transcript *tr = tr_of(h);
  if (!tr) return E_PARAM;
  *count = tr->messages.size();
  return OK;
}
int exh_transcript_proof(exh_transcript h, uint8_t *out, uint64_t cap, uint64_t *out_len) {
  ApiLock api_lock;
  Transcript *tr = tr_of(h);
  if (!tr) return E_PARAM;
  std::vector<uint8_t> bytes = tr->encode_proof();
  *out_len = bytes.size();
  if (out && cap >= bytes.size()) memcpy(out, bytes.data(), bytes.size());
  return OK;
}

// ------------------------------------------------------------------ sumcheck protocol
int exh_hypercube_sum(exh_stmt stmt, int D, int n, const exh_table *tables, int n_tables, const uint32_t *eq,
                      const uint32_t *constants, uint32_t *out) {
  ApiLock api_lock;
  Statement *st = stmt_of(stmt);
  if (!st) return E_PARAM;
  if (n_tables != st->T()) {
    set_error("invalid-parameter: table count");
    return E_PARAM;
  }
  std::vector<const uint32_t *> ptrs;
  std::vector<int> strides;
  int status = gather_tables(tables, n_tables, D, (uint64_t)1 << n, &ptrs, &strides);
  if (status) return status;
  if (n == 0) {  // one row: the statement at the tables' only entries
    std::vector<uint32_t> tv((size_t)n_tables * D, 0);
    for (int t = 0; t < n_tables; t++)
      EXH_HIP(hipMemcpy(&tv[(size_t)t * D], ptrs[t], 4 * strides[t], hipMemcpyDeviceToHost));
    evaluate_statement(*st, D, tv.data(), constants, out);
    return OK;
  }
  SumcheckSession s;
  status = s.begin(*st, D, n, ptrs.data(), strides.data(), eq, nullptr, 1, constants, -1, true);
  if (status == E_PARAM && s.beyond_limits)
    return hypercube_sum_wide(*st, D, n, ptrs.data(), strides.data(), eq, constants, out);
  if (status) return status;
  uint32_t sums[16 * 8];
  if ((status = s.round_sums(sums))) return status;
  memcpy(out, sums, 4 * D);
  return OK;
}

int exh_prove(exh_transcript h, int n, exh_stmt stmt, const exh_table *tables, int n_tables, const uint32_t *eq,
              const uint32_t *constants, const uint8_t *label, uint64_t label_len, const uint32_t *bw, int K,
              int degree, uint32_t *out_chal, uint32_t *out_finals, uint32_t *const *out_folded) {
  ApiLock api_lock;
  Transcript *tr = tr_of(h);
  Statement *st = stmt_of(stmt);
  if (!tr || !st) return E_PARAM;
  if (n_tables != st->T() || (!bw && K != 1) || K < 1) {
    set_error("invalid-parameter: prove arguments");
    return E_PARAM;
  }
  std::vector<const uint32_t *> ptrs;
  std::vector<int> strides;
  int status = gather_tables(tables, n_tables, tr->D, (uint64_t)K << n, &ptrs, &strides);
  if (status) return status;
  return sumcheck_prove(*tr, n, *st, ptrs.data(), strides.data(), eq, constants,
                        std::string((const char *)label, label_len), bw, K, degree, out_chal, out_finals, out_folded);
}

int exh_verify(exh_transcript h, int n, exh_stmt stmt, const uint32_t *claim, const uint32_t *eq,
               const uint32_t *constants, int blocks, const uint8_t *label, uint64_t label_len, int degree,
               uint32_t *out_chal, uint32_t *out_reduced) {
  ApiLock api_lock;
  Transcript *tr = tr_of(h);
  Statement *st = stmt_of(stmt);
  if (!tr || !st) return E_PARAM;
  return sumcheck_verify(*tr, n, *st, claim, eq, constants, blocks, std::string((const char *)label, label_len),
                         degree, out_chal, out_reduced);
}

int exh_check_final(exh_stmt stmt, int D, const uint32_t *reduced, const uint32_t *finals, const uint32_t *constants) {
  ApiLock api_lock;
  Statement *st = stmt_of(stmt);
  if (!st) return E_PARAM;
  return check_final(*st, D, reduced, finals, constants);
}

int exh_stmt_evaluate(exh_stmt stmt, int D, const uint32_t *table_values, const uint32_t *constants, uint32_t *out) {
  ApiLock api_lock;
  Statement *st = stmt_of(stmt);
  if (!st) return E_PARAM;
  if (D != 4 && D != 8) {
    set_error("invalid-parameter: degree");
    return E_PARAM;
  }
  evaluate_statement(*st, D, table_values, constants, out);
  return OK;
}

// ------------------------------------------------------------------ domains
namespace {
int domain_column_of(const exh_domain_column *in, int n, int K, DomainColumn *out) {
  DeviceTable *dt = table_of(in->data);
  if (!dt) return E_PARAM;
  if (!in->name || dt->stride != 1) {
    set_error("invalid-parameter: a domain column is a named table of base values");
    return E_PARAM;
  }
  out->name = in->name;
  for (char &ch : out->name) ch = (char)toupper((unsigned char)ch);
  out->kind = in->kind, out->c = in->kind == COL_FULL ? 0 : in->c, out->shared = in->shared != 0;
  out->ptr = dt->ptr, out->entries = dt->n_u32;
  (void)n, (void)K;
  return OK;
}
}  // namespace

int exh_domain_table(const exh_domain_column *column, int half, int n, int K, exh_table *out) {
  ApiLock api_lock;
  DomainColumn col;
  int status = domain_column_of(column, n, K, &col);
  if (status) return status;
  if (n < 2 || n > 40 || K < 1) {
    set_error("invalid-parameter: domain table arguments");
    return E_PARAM;
  }
  if ((status = exh_table_alloc((uint64_t)K << (n - 1), 1, out))) return status;
  if ((status = domain_table(col, half, n, K, table_of(*out)->ptr))) {
    exh_table_free(*out);
    *out = 0;
  }
  return status;
}

int exh_domain_leaves(int D, int n, int K, const exh_domain_column *columns, int n_columns, const char *tag,
                      const char *const *values, int n_values, const char *num, const uint32_t *z,
                      const uint32_t *betas, exh_table *out_p, exh_table *out_q) {
  ApiLock api_lock;
  if ((D != 4 && D != 8) || n < 2 || n > 40 || K < 1 || n_columns < 0 || n_values < 0 || !tag) {
    set_error("invalid-parameter: domain leaves arguments");
    return E_PARAM;
  }
  std::vector<DomainColumn> cols((size_t)n_columns);
  int status;
  for (int k = 0; k < n_columns; k++)
    if ((status = domain_column_of(columns + k, n, K, &cols[(size_t)k]))) return status;
  std::vector<std::string> vs;
  for (int k = 0; k < n_values; k++) vs.push_back(values[k]);
  uint64_t words = ((uint64_t)K << n) * D;
  if ((status = exh_table_alloc(words, D, out_p))) return status;
  if ((status = exh_table_alloc(words, D, out_q))) {
    exh_table_free(*out_p);
    return status;
  }
  if ((status = domain_leaves(D, n, K, cols, tag, vs, num, z, betas, table_of(*out_p)->ptr, table_of(*out_q)->ptr))) {
    exh_table_free(*out_p);
    exh_table_free(*out_q);
    *out_p = *out_q = 0;
  }
  return status;
}

// ------------------------------------------------------------------ GKR
int exh_gkr_reduce_layer(exh_table p, exh_table q, int D, int K, int m, exh_table *out_p, exh_table *out_q) {
  ApiLock api_lock;
  DeviceTable *dp = table_of(p), *dq = table_of(q);
  if (!dp || !dq) return E_PARAM;
  uint64_t in_entries = (uint64_t)K << (m + 1);
  if ((D != 4 && D != 8) || dp->stride != D || dq->stride != D || dp->n_u32 != in_entries * D ||
      dq->n_u32 != in_entries * D) {
    set_error("invalid-parameter: layer tables must hold K * 2^(m+1) extension elements");
    return E_PARAM;
  }
  int status;
  if ((status = exh_table_alloc((in_entries / 2) * D, D, out_p))) return status;
  if ((status = exh_table_alloc((in_entries / 2) * D, D, out_q))) return status;
  return gkr_reduce_layer(D, K, m, dp->ptr, dq->ptr, table_of(*out_p)->ptr, table_of(*out_q)->ptr);
}

int exh_gkr_prove_upper(exh_transcript h, int n, int K, int lookups, const exh_table *leaves, const uint8_t *label,
                        uint64_t label_len, uint32_t *out_ri, uint32_t *out_rb, uint32_t *out_cp, uint32_t *out_cq) {
  ApiLock api_lock;
  Transcript *tr = tr_of(h);
  if (!tr) return E_PARAM;
  std::vector<const uint32_t *> ptrs;
  std::vector<int> strides;
  int status = gather_tables(leaves, 2 * lookups, tr->D, (uint64_t)K << n, &ptrs, &strides);
  if (status) return status;
  for (int s : strides)
    if (s != tr->D) {
      set_error("invalid-parameter: GKR leaves are extension elements");
      return E_PARAM;
    }
  return gkr_prove_upper(*tr, n, K, lookups, ptrs.data(), std::string((const char *)label, label_len), out_ri, out_rb,
                         out_cp, out_cq);
}

namespace {
struct TreeCall {
  Transcript *tr = nullptr;
  std::vector<const uint32_t *> ptrs;
  std::string label;
};
int prepare_tree(const exh_gkr_tree &t, TreeCall *call) {
  call->tr = tr_of(t.tr);
  if (!call->tr) return E_PARAM;
  if (t.lookups < 1 || t.lookups > MAXT / 4 || t.n < 0 || t.n > 30 || t.K < 1 || !t.leaves) {
    set_error("invalid-parameter: GKR shape (lookups, n, K, leaves)");
    return E_PARAM;
  }
  std::vector<int> strides;
  int status = gather_tables(t.leaves, 2 * t.lookups, call->tr->D, (uint64_t)t.K << t.n, &call->ptrs, &strides);
  if (status) return status;
  for (int s : strides)
    if (s != call->tr->D) {
      set_error("invalid-parameter: GKR leaves are extension elements");
      return E_PARAM;
    }
  call->label.assign((const char *)t.label, t.label_len);
  return OK;
}
int run_tree(const exh_gkr_tree &t, TreeCall &call) {
  try {  // (nothing may leave a thread's body as an exception: a proof of 2^22 leaves holds large host vectors)
    return gkr_prove_upper(*call.tr, t.n, t.K, t.lookups, call.ptrs.data(), call.label, t.out_ri, t.out_rb, t.out_cp,
                           t.out_cq);
  } catch (const std::bad_alloc &) {
    set_error("device-out-of-memory: host memory ran out during prove-upper");
    return E_NOMEM;
  } catch (const std::exception &e) {
    set_error(std::string("device-error: prove-upper: ") + e.what());
    return E_DEVICE;
  }
}
}  // namespace

int exh_gkr_prove_upper_pair(exh_gkr_tree *first, exh_gkr_tree *second) {
  ApiLock api_lock;
  if (!first || !second || first->tr == second->tr) {
    set_error("invalid-parameter: two trees, each with a transcript of its own");
    return E_PARAM;
  }
  Context &main_context = ctx();
  TreeCall a, b;
  if ((first->status = prepare_tree(*first, &a))) return first->status;
  if ((second->status = prepare_tree(*second, &b))) return second->status;
  Context *side = nullptr;
  int status = side_context(&side);
  if (status) return status;
  if (main_context.profiling) {  // (the timed launches are the library's own stream's)
    first->status = run_tree(*first, a);
    second->status = first->status ? first->status : run_tree(*second, b);
    return first->status ? first->status : second->status;
  }
  {  // what the library's stream still has to do (the second tree's leaves, perhaps) comes first on the other too
    hipEvent_t queued;
    EXH_HIP(hipEventCreateWithFlags(&queued, hipEventDisableTiming));
    hipError_t recorded = hipEventRecord(queued, main_context.stream);
    if (recorded == hipSuccess) recorded = hipStreamWaitEvent(side->stream, queued, 0);
    (void)hipEventDestroy(queued);
    EXH_HIP(recorded);
  }
  std::string second_error;
  struct Shared {  // both proofs' grids take half the device while they run side by side; whole again on every way out
    Context &one, &other;
    Shared(Context &a, Context &b) : one(a), other(b) { one.share = other.share = 2; }
    ~Shared() { one.share = other.share = 1; }
  };
  {
    Shared shared(main_context, *side);
    second->status = E_DEVICE;
    std::thread worker;
    try {
      worker = std::thread([&] {
        use_context(side);
        second->status = hipSetDevice(side->device) == hipSuccess ? run_tree(*second, b) : E_DEVICE;
        if (second->status) second_error = last_error();
        use_context(nullptr);
      });
    } catch (const std::exception &e) {  // no second thread: one tree after the other
      first->status = run_tree(*first, a);
      second->status = first->status ? first->status : run_tree(*second, b);
      return first->status ? first->status : second->status;
    }
    first->status = run_tree(*first, a);
    worker.join();
  }
  if (first->status) return first->status;
  if (second->status) set_error(second_error);
  return second->status;
}

int exh_gkr_verify_upper(exh_transcript h, int n, int K, int lookups, const uint8_t *label, uint64_t label_len,
                         uint32_t *out_roots, uint32_t *out_ri, uint32_t *out_rb, uint32_t *out_cp,
                         uint32_t *out_cq) {
  ApiLock api_lock;
  Transcript *tr = tr_of(h);
  if (!tr) return E_PARAM;
  return gkr_verify_upper(*tr, n, K, lookups, std::string((const char *)label, label_len), out_roots, out_ri, out_rb,
                          out_cp, out_cq);
}

// ------------------------------------------------------------------ Reed-Solomon, Merkle, BaseFold
int exh_rs_encode(exh_table messages, int ncols, int c, exh_table *codewords) {
  ApiLock api_lock;
  DeviceTable *m = table_of(messages);
  if (!m) return E_PARAM;
  if (ncols < 1 || c < 0 || c > 23 || m->stride != 1 || m->n_u32 != ((uint64_t)ncols << c)) {
    set_error("invalid-parameter: messages must hold ncols * 2^c base values, c <= 23");
    return E_PARAM;
  }
  int status = exh_table_alloc((uint64_t)ncols << (c + 1), 1, codewords);
  if (status) return status;
  return rs_encode_columns(m->ptr, ncols, c, table_of(*codewords)->ptr);
}

int exh_merkle_commit(exh_table codewords, int ncols, int c, exh_table *levels, uint8_t *cap, uint64_t *cap_rows) {
  ApiLock api_lock;
  DeviceTable *cw = table_of(codewords);
  if (!cw) return E_PARAM;
  if (ncols < 1 || c < 1 || c > 23 || cw->n_u32 != ((uint64_t)ncols << (c + 1))) {
    set_error("invalid-parameter: codewords must hold ncols * 2^(c+1) symbols, 1 <= c <= 23");
    return E_PARAM;
  }
  uint64_t nleaves = (uint64_t)1 << (c - 1);
  exh_table lv;
  int status = exh_table_alloc((2 * nleaves - 1) * 8, 8, &lv);
  if (status) return status;
  status = merkle_commit_columns(cw->ptr, ncols, c, table_of(lv)->ptr, cap, cap_rows);
  if (status || !levels)
    exh_table_free(lv);
  else
    *levels = lv;
  return status;
}

int exh_open_queries(exh_table codewords, int ncols, int c, exh_table levels, const uint64_t *leaves, int count,
                     uint32_t *out_leaves, uint8_t *out_paths, int *out_depth) {
  ApiLock api_lock;
  DeviceTable *cw = table_of(codewords);
  if (!cw) return E_PARAM;
  if (ncols < 1 || c < 1 || c > 23 || cw->n_u32 != ((uint64_t)ncols << (c + 1))) {
    set_error("invalid-parameter: codewords must hold ncols * 2^(c+1) symbols, 1 <= c <= 23");
    return E_PARAM;
  }
  const uint64_t nleaves = (uint64_t)1 << (c - 1);
  const uint32_t *d_levels = nullptr;
  if (levels) {
    DeviceTable *lv = table_of(levels);
    if (!lv) return E_PARAM;
    if (lv->n_u32 != (2 * nleaves - 1) * 8 || !out_paths) {
      set_error("invalid-parameter: levels must hold 2 * 2^(c-1) - 1 digests, and the paths need a buffer");
      return E_PARAM;
    }
    d_levels = lv->ptr;
  }
  if (count < 0 || count > (1 << 20) || (count > 0 && (!leaves || !out_leaves))) {
    set_error("invalid-parameter: 0 <= count <= 2^20 leaf indices and a buffer for their rows");
    return E_PARAM;
  }
  for (int q = 0; q < count; q++)
    if (leaves[q] >= nleaves) {
      set_error("invalid-parameter: leaf index beyond the tree's 2^(c-1) leaves");
      return E_PARAM;
    }
  return open_queries_device(cw->ptr, ncols, c, d_levels, leaves, count, out_leaves, out_paths, out_depth);
}

int exh_rs_fold(exh_table codeword, int D, uint64_t m, int n_domain, int level, const uint32_t *r, exh_table *out) {
  ApiLock api_lock;
  DeviceTable *cw = table_of(codeword);
  if (!cw) return E_PARAM;
  if ((D != 4 && D != 8) || cw->n_u32 != 2 * m * D || n_domain < 1 || n_domain > 24 || level < 0 ||
      m != ((uint64_t)1 << (n_domain - 1 - level))) {
    set_error("invalid-parameter: codeword of 2m extension elements on level `level` of the 2^n_domain tables");
    return E_PARAM;
  }
  int status = exh_table_alloc(m * D, D, out);
  if (status) return status;
  if ((status = rs_fold_device(D, m, n_domain, level, cw->ptr, r, table_of(*out)->ptr))) {
    exh_table_free(*out);
    *out = 0;
  }
  return status;
}

int exh_table_scale_add(exh_table h, const uint32_t *scale, exh_table column, exh_table *out) {
  ApiLock api_lock;
  DeviceTable *tc = table_of(column), *th = h ? table_of(h) : nullptr;
  if (!tc || (h && !th)) return E_PARAM;
  const int D = tc->stride;
  if (!scale || !out || (D != 4 && D != 8) || tc->n_u32 < (uint64_t)D || (th && (th->stride != D || th->n_u32 != tc->n_u32))) {
    set_error("invalid-parameter: scale-add takes extension tables of one shape");
    return E_PARAM;
  }
  int status = exh_table_alloc(tc->n_u32, D, out);
  if (status) return status;
  status = scale_add_device(D, th ? th->ptr : nullptr, tc->ptr, tc->n_u32 / D, scale, table_of(*out)->ptr);
  if (status) exh_table_free(*out);
  return status;
}

int exh_dot_pairs(exh_table e, exh_table v, uint32_t *out) {
  ApiLock api_lock;
  DeviceTable *te = table_of(e), *tv = table_of(v);
  if (!te || !tv) return E_PARAM;
  if (!out || te->stride != 8 || tv->stride != 8 || te->n_u32 != tv->n_u32 || te->n_u32 < 16 || (te->n_u32 / 8) % 2) {
    set_error("invalid-parameter: dot-pairs takes two tables of the same even number of EXT8s");
    return E_PARAM;
  }
  return dot_pairs_device(te->ptr, tv->ptr, te->n_u32 / 8, out);
}

static int open_keys(const exh_open_key *keys, int n_keys, bool prover, std::vector<OpenClass> *out) {
  if (!keys || n_keys < 1 || n_keys > 32) {
    set_error("invalid-parameter: opening keys");
    return E_PARAM;
  }
  for (int k = 0; k < n_keys; k++) {
    OpenClass oc;
    oc.c = keys[k].c, oc.ncols = keys[k].ncols, oc.coef = keys[k].coefficients, oc.cap = keys[k].cap;
    if (oc.c < 1 || oc.c > 30 || oc.ncols < 1 || !oc.coef || (!prover && !oc.cap)) {
      set_error("invalid-parameter: opening key");
      return E_PARAM;
    }
    if (prover) {
      DeviceTable *cols = table_of(keys[k].columns), *cw = table_of(keys[k].codewords), *lv = table_of(keys[k].levels);
      const uint64_t nleaves = (uint64_t)1 << (oc.c - 1);
      if (!cols || !cw || !lv) return E_PARAM;
      if (cols->n_u32 != ((uint64_t)oc.ncols << oc.c) || cw->n_u32 != ((uint64_t)oc.ncols << (oc.c + 1)) ||
          lv->n_u32 != (2 * nleaves - 1) * 8) {
        set_error("invalid-parameter: opening key: columns, codewords or levels of another shape");
        return E_PARAM;
      }
      oc.d_columns = cols->ptr, oc.d_codewords = cw->ptr, oc.d_levels = lv->ptr;
    }
    out->push_back(oc);
  }
  return OK;
}

int exh_pcs_open(exh_transcript h, int nv, int n_keys, const exh_open_key *keys, const uint32_t *rr, const uint32_t *v,
                 int grind_bits, int queries, uint64_t *out_qs) {
  ApiLock api_lock;
  Transcript *tr = tr_of(h);
  if (!tr || !rr || !v) return E_PARAM;
  std::vector<OpenClass> oc;
  int status = open_keys(keys, n_keys, true, &oc);
  if (status) return status;
  return pcs_open(*tr, nv, n_keys, oc.data(), rr, v, grind_bits, queries, out_qs);
}

int exh_pcs_verify_opening(exh_transcript h, int nv, int n_keys, const exh_open_key *keys, const uint32_t *rr,
                           const uint32_t *v, int grind_bits, int queries) {
  ApiLock api_lock;
  Transcript *tr = tr_of(h);
  if (!tr || !rr || !v) return E_PARAM;
  std::vector<OpenClass> oc;
  int status = open_keys(keys, n_keys, false, &oc);
  if (status) return status;
  return pcs_verify_opening(*tr, nv, n_keys, oc.data(), rr, v, grind_bits, queries);
}

int exh_merkle_levels_injected(exh_table leaves, int n_injected, const int32_t *inject_level, const exh_table *injected,
                               exh_table *levels) {
  ApiLock api_lock;
  DeviceTable *lv = table_of(leaves);
  if (!lv || !levels || n_injected < 0 || n_injected > 16 || lv->n_u32 % 8) return E_PARAM;
  const uint64_t nleaves = lv->n_u32 / 8;
  std::vector<const uint32_t *> inj;
  std::vector<int> at;
  for (int k = 0; k < n_injected; k++) {
    DeviceTable *t = table_of(injected[k]);
    if (!t) return E_PARAM;
    if (inject_level[k] < 1 || inject_level[k] > 40 || t->n_u32 != (nleaves >> inject_level[k]) * 8) {
      set_error("invalid-parameter: an injected class has as many digests as its level has nodes");
      return E_PARAM;
    }
    inj.push_back(t->ptr), at.push_back(inject_level[k]);
  }
  int status = exh_table_alloc((2 * nleaves - 1) * 8, 8, levels);
  if (status) return status;
  status = merkle_levels_injected_device(lv->ptr, nleaves, n_injected, at.data(), inj.data(), table_of(*levels)->ptr);
  if (status) exh_table_free(*levels);
  return status;
}

int exh_check_path(const uint8_t h[32], const uint8_t *path, int depth, uint64_t i, const uint8_t *cap, int n_injected,
                   const int32_t *inject_level, const uint8_t *injected_digests) {
  ApiLock api_lock;
  if (!h || !cap || depth < 0 || (depth && !path)) return E_PARAM;
  std::vector<int> at(inject_level, inject_level + (n_injected > 0 ? n_injected : 0));
  return check_path_host(h, path, depth, i, cap, n_injected, at.data(), injected_digests) ? 1 : 0;
}

int exh_dot_pairs_static(exh_table e, exh_table v, uint32_t *out) {
  ApiLock api_lock;
  DeviceTable *te = table_of(e), *tv = table_of(v);
  if (!te || !tv) return E_PARAM;
  if (!out || te->stride != 8 || tv->stride != 8 || te->n_u32 != tv->n_u32 || te->n_u32 < 16 || (te->n_u32 / 8) % 2) {
    set_error("invalid-parameter: dot-pairs takes two tables of the same even number of EXT8s");
    return E_PARAM;
  }
  return dot_pairs_static_device(te->ptr, tv->ptr, te->n_u32 / 8, out);
}

int exh_fold_table(exh_table table, const uint32_t *r, exh_table *out) {
  ApiLock api_lock;
  DeviceTable *t = table_of(table);
  if (!t) return E_PARAM;
  const int D = t->stride;
  if (!r || !out || (D != 4 && D != 8) || t->n_u32 < (uint64_t)2 * D || (t->n_u32 / D) % 2) {
    set_error("invalid-parameter: fold-table takes an even number of extension elements");
    return E_PARAM;
  }
  const uint64_t len = t->n_u32 / D;
  int status = exh_table_alloc(len / 2 * D, D, out);
  if (status) return status;
  status = fold_table_device(D, t->ptr, len, r, table_of(*out)->ptr);
  if (status) exh_table_free(*out);
  return status;
}

int exh_combine_columns(exh_table columns, int ncols, uint64_t len, int D, const uint32_t *coefficients, exh_table *out) {
  ApiLock api_lock;
  DeviceTable *cols = table_of(columns);
  if (!cols) return E_PARAM;
  if ((D != 4 && D != 8) || ncols < 1 || len < 1 || !coefficients || !out || cols->stride != 1 ||
      cols->n_u32 != (uint64_t)ncols * len) {
    set_error("invalid-parameter: columns must hold ncols * len base values, coefficients ncols elements of degree 4 or 8");
    return E_PARAM;
  }
  int status = exh_table_alloc(len * D, D, out);
  if (status) return status;
  status = combine_columns_device(D, cols->ptr, ncols, len, coefficients, table_of(*out)->ptr);
  if (status) exh_table_free(*out);
  return status;
}

int exh_pcs_commit(exh_transcript h, exh_table columns, int ncols, int c, exh_table *codewords, exh_table *levels) {
  ApiLock api_lock;
  Transcript *tr = tr_of(h);
  if (!tr) return E_PARAM;
  exh_table cw;
  int status = exh_rs_encode(columns, ncols, c, &cw);
  if (status) return status;
  std::vector<uint8_t> cap(32 * ((size_t)1 << 7));
  uint64_t rows = 0;
  if ((status = exh_merkle_commit(cw, ncols, c, levels, cap.data(), &rows))) {
    exh_table_free(cw);
    return status;
  }
  status = tr->send_bytes(cap.data(), (int64_t)(32 * rows), nullptr);
  if (status) {  // nothing is handed back on failure
    exh_table_free(cw);
    if (levels) {
      exh_table_free(*levels);
      *levels = 0;
    }
    return status;
  }
  if (codewords)
    *codewords = cw;
  else
    exh_table_free(cw);
  return OK;
}

int exh_basefold_prove(exh_transcript h, int nv, const uint32_t *rr, const uint32_t *v, exh_table table, int grind_bits,
                       int queries, uint64_t *out_qs, uint32_t *out_chal, uint32_t *out_final) {
  ApiLock api_lock;
  Transcript *tr = tr_of(h);
  DeviceTable *dt = table_of(table);
  if (!tr || !dt) return E_PARAM;
  if (nv < 1 || nv > 23 || dt->stride != 8 || dt->n_u32 != ((uint64_t)8 << nv)) {
    set_error("invalid-parameter: BaseFold takes 2^nv EXT8s, 1 <= nv <= 23");
    return E_PARAM;
  }
  return basefold_prove(*tr, nv, rr, v, dt->ptr, grind_bits, queries, out_qs, out_chal, out_final);
}
int exh_basefold_prove_classes(exh_transcript h, int nv, int n_classes, const int *classes, const exh_table *hs,
                               const uint32_t *rr, const uint32_t *v, int grind_bits, int queries, uint64_t *out_qs) {
  ApiLock api_lock;
  Transcript *tr = tr_of(h);
  if (!tr || n_classes < 1 || n_classes > 32 || !classes || !hs || nv < 1 || nv > 23) {
    set_error("invalid-parameter: BaseFold over 1 to 32 classes, 1 <= nv <= 23");
    return E_PARAM;
  }
  std::vector<const uint32_t *> tables(n_classes);
  for (int k = 0; k < n_classes; k++) {
    DeviceTable *dt = table_of(hs[k]);
    if (!dt || classes[k] < 1 || classes[k] > nv || dt->stride != 8 || dt->n_u32 != ((uint64_t)8 << classes[k])) {
      set_error("invalid-parameter: a class's combined column is 2^c EXT8s");
      return E_PARAM;
    }
    tables[k] = dt->ptr;
  }
  return basefold_prove_classes(*tr, nv, n_classes, classes, tables.data(), rr, v, grind_bits, queries, out_qs, nullptr,
                                nullptr, nullptr);
}
int exh_basefold_prove_encoded(exh_transcript h, int nv, const uint32_t *rr, const uint32_t *v, exh_table table,
                               exh_table codeword, int grind_bits, int queries, uint64_t *out_qs, uint32_t *out_chal,
                               uint32_t *out_final) {
  ApiLock api_lock;
  Transcript *tr = tr_of(h);
  DeviceTable *dt = table_of(table), *dc = table_of(codeword);
  if (!tr || !dt || !dc) return E_PARAM;
  if (nv < 1 || nv > 23 || dt->stride != 8 || dt->n_u32 != ((uint64_t)8 << nv) || dc->stride != 8 ||
      dc->n_u32 != ((uint64_t)16 << nv)) {
    set_error("invalid-parameter: BaseFold takes 2^nv EXT8s and their codeword of 2^(nv+1) EXT8s, 1 <= nv <= 23");
    return E_PARAM;
  }
  return basefold_prove(*tr, nv, rr, v, dt->ptr, grind_bits, queries, out_qs, out_chal, out_final, dc->ptr);
}

int exh_basefold_verify(exh_transcript h, int nv, const uint32_t *rr, const uint32_t *v, int grind_bits, int queries,
                        uint64_t *out_qs) {
  ApiLock api_lock;
  Transcript *tr = tr_of(h);
  if (!tr) return E_PARAM;
  return basefold_verify(*tr, nv, rr, v, grind_bits, queries, out_qs);
}

}  // extern "C"
