// sumcheck.hpp -- the device side of the sumcheck prover as a session: the tables stay in HBM, each
// round returns its message rows, each fold takes the round's challenge.  It replaces the bodies of
// the reference's round kernel call and FOLD-FLAT-TABLE inside PROVE (src/sumcheck.lisp:547-563).
#pragma once
#include <stdint.h>

#include <string>
#include <functional>
#include <vector>

#include "context.hpp"
#include "forms.hpp"
#include "sumcheck_kernels.hpp"

namespace exh {

struct KernelSet {  // the launchers generated for one statement and one degree D, at build time or at run time
  std::function<void(const void *args, bool in_base, bool fold, uint32_t grid, hipStream_t stream)> launch;
  std::function<void(const void *args, uint32_t grid, hipStream_t stream)> launch_tail;
  // base tables folded twice at once (round 2 after the base-field sweep), and that sweep's slot sums
  std::function<void(const void *args, uint32_t grid, hipStream_t stream)> launch_fold2;
  std::function<void(const void *args, int pass, uint32_t grid, hipStream_t stream)> launch_nodes;
  int nodes_passes = 0;  // launches of launch_nodes per round (0: not available)
  // workgroups of the tail kernel a compute unit holds at once with that much dynamic LDS (-1: unknown)
  std::function<int(uint32_t lds_bytes)> tail_blocks_per_cu;
  // LogUp-GKR's layer statement only: the one-workgroup launch of the last rounds followed, in the same launch, by
  // the step between two layers (TailArgs<D>, GlueArgs<D>)
  std::function<void(const void *tail_args, const void *step_args, hipStream_t stream)> launch_tail_glue;
};
// EQ-TABLE of k coordinates (canonical, host) into 2^k elements of device memory
int eq_table_device(int D, int k, const uint32_t *r, uint32_t *d_out);
// eq tables over ranges of a point's variables in one launch (see sumcheck.hip)
int eq_tables_launch(int D, int count, const int *first, const int *bits, const uint64_t *off,
                     const uint32_t *d_factors, int n_vars, uint32_t *d_out);
void register_kernels(const std::string &key, int D, KernelSet set);
const KernelSet *find_kernels(const std::string &key, int D);

struct SumcheckSession {
  int D = 4, n = 0, K = 1, points = 1;
  Statement st;
  bool generated = false;  // a kernel generated for the statement is in use (else the interpreter)
  const KernelSet *kernels = nullptr;
  StmtDesc desc;
  std::vector<const uint32_t *> cur;  // current tables (device)
  bool cur_base = false;
  uint64_t size = 0;  // entries per table now
  int round = 0;
  bool has_eq = false, has_bw = false;
  std::vector<uint32_t> group_coef;  // G * D
  std::vector<uint32_t> bw_sum;      // sum of the block weights (D), for the constant group
  // per-round weight tables on the device
  uint32_t *d_weights = nullptr;
  std::vector<uint64_t> low_off, high_off;
  std::vector<int> low_bits;
  std::vector<uint64_t> n_high;
  uint32_t *d_partials = nullptr, *d_sums = nullptr, *d_lifted = nullptr;
  unsigned long long *d_slice_totals = nullptr;  // the totals of the grid launch of slices
  bool slice_totals_clear = false;               // cleared by the session's set-up kernel and not used since
  unsigned long long *d_round_totals = nullptr;  // the streaming rounds' totals, a region per round
  uint32_t *d_arrivals = nullptr;                // and their arrival counters
  uint64_t zeroed_words = 0;                     // what the set-up kernel clears: all three
  uint32_t *host_log = nullptr;                  // set around the loop's last launch: where it delivers the logs
  uint32_t host_flag_at = 0, host_seq = 0;
  uint64_t max_grid = 0;
  uint32_t pstride = 0;  // words per workgroup partial
  int node_slots_n = 0;  // slot sums of the base-field sweep that serves rounds 0 and 1
  bool device_loop = false;
  Ctrl *d_ctrl = nullptr;
  std::vector<uint32_t> final_cache;  // the tables as the device loop's tail left them, when read back with its logs
  uint32_t *d_mtilde = nullptr, *d_c0 = nullptr;
  // a statement in direct form: its constant slots at this proof's constants (Montgomery form), host and device
  uint32_t *d_direct = nullptr;
  std::vector<uint32_t> direct_host;
  bool pending_fold = false;
  uint32_t pending_r[8];
  int generation = 0;
  std::vector<uint32_t *> out_buf;  // scratch for the launch

  // tables[t]: K * 2^n entries of stride strides[t] (1 or D), block-major, on the device.
  // eq: n * D host words or null; bw: K * D host words or null; consts: C * D host words.
  int begin(const Statement &statement, int D, int n, const uint32_t *const *tables, const int *strides,
            const uint32_t *eq, const uint32_t *bw, int K, const uint32_t *consts, int degree,
            bool claim_mode = false, bool defer_setup = false);
  // With defer_setup the eq point and block weights stay staged on the host and the weight-table
  // kernels are not launched: run_device sends them with its own constants in one copy and launches then.
  // Set before begin: the session keeps its folded generations and weights in buffers of its own instead of the
  // context's, so that several sessions can be open side by side (the parts of a statement too wide for one
  // kernel, proved in step).  Such a session runs host-driven rounds.
  bool private_buffers = false;
  // The caller takes what the rounds leave of the tables on the device (finish_device) and never asks for them on
  // the host: the device-driven loop then need not fetch them with its logs, and its last launch can deliver the
  // logs to pinned memory itself whatever the tables' final length.
  bool finals_stay = false;
  // Set before run_device by a caller that chains several sumchecks on the device (the layers of LogUp-GKR): the
  // loop's constants (eq factors, message map, constant terms, the head of the control block with the transcript's
  // state) are then written in device memory by the launch this hook enqueues, instead of being staged and copied
  // from the host; run_device enqueues its launches and returns without waiting or reading anything back, and the
  // control block (logs, finals) stays in device memory for the chain's next launch.
  std::function<int()> chain_hook;
  // Set with chain_hook by a caller whose next step can ride on this session's last launch: that launch (one
  // workgroup, the last rounds) is then not enqueued; its arguments are left here (a TailArgs<D>) for the caller to
  // launch, after this session has returned and even after the next one has begun (they are plain addresses).
  std::vector<uint8_t> *held_tail = nullptr;
  // the scalar (Lagrange basis times the power of R the sums carry) that maps accumulator `acc` to wire point k in
  // the message map: lagfix[k * nacc + acc], and the group each accumulator belongs to
  void message_map_scalars(std::vector<uint32_t> *lagfix, std::vector<int> *acc_group) const;
  bool beyond_limits = false;  // begin refused the statement for its size alone: its parts may still fit
  Arena own_a, own_b, own_misc;
  Arena &arena_a();
  Arena &arena_b();
  Arena &arena_misc();
  ~SumcheckSession();
  uint64_t epoch = 0;  // Context::session_epoch at begin
  // OK while this is the latest session begun (its arenas have not been handed to another one)
  int owns_arenas() const;
  bool setup_deferred = false;
  bool own_weights = false;  // the one launch that runs every round builds the weight tables itself
  size_t setup_words = 0;
  struct {
    uint64_t total_eq = 0, ones_off = 0, ones_len = 0;
    unsigned char eqt[1536];  // the EqTables argument of eq_tables_kernel
  } setup;
  int launch_setup(const uint32_t *staged = nullptr, size_t staged_words = 0);
  // claim mode: round_sums returns the honest claim sum_x w(x) F(tables(x)) in out[0..D) (n >= 1)
  bool claim_mode = false;
  std::vector<uint32_t> eq0;  // the eq point's first coordinate, for the claim
  int round_sums(uint32_t *out /* points * D */);
  // All rounds on the device without a host round trip: the transcript runs on the device from the
  // given B3S state; afterwards messages[j] (points * D words) and challenges[j] (D words) hold what
  // was sent and drawn, final_state (optional) the transcript's hash state after the last challenge, and the
  // session is ready for finish().  Needs points <= MAXPTS.
  int run_device(const DevB3S &state, uint32_t *messages, uint32_t *challenges, DevB3S *final_state = nullptr);
  // rounds first_round .. first_round + rounds - 1 with the tables in LDS, over `grid` workgroups
  int launch_tail(int first_round, int rounds, uint32_t grid, bool first_fold);
  // the device-driven loop fits this session: rounds, wire points, and its constants in the pinned staging area
  bool device_capable() const;
  int fold(const uint32_t *r /* D */);
  // finals: T * D; folded[t] (optional): K * D each
  int finish(uint32_t *finals, uint32_t *const *folded);
  // the same tables left on the device instead: table t's entries at d_out + t * padded * D, lifted if still base,
  // zeros from its last entry up to `padded` (what a sumcheck over the block index takes as its tables).  Enqueued
  // on the session's stream; nothing is copied to the host.
  int finish_device(uint32_t *d_out, uint64_t padded);
  // device pointers of the current (fully or partly folded) tables, after any pending fold
  int flush();
};

}  // namespace exh
