// context.hpp -- the library's one device context: the HIP device and stream, device tables behind
// opaque handles, and a grow-only workspace so the proving loop does not allocate per round.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <map>
#include <string>
#include <vector>

#include "transcript.hpp"

namespace exh {

#define EXH_HIP(call)                                                                              \
  do {                                                                                             \
    hipError_t exh_err__ = (call);                                                                 \
    if (exh_err__ != hipSuccess) {                                                                 \
      ::exh::set_error(std::string("device-error: ") + #call + ": " + hipGetErrorString(exh_err__)); \
      return ::exh::E_DEVICE;                                                                      \
    }                                                                                              \
  } while (0)

struct DeviceTable {
  uint32_t *ptr = nullptr;
  uint64_t n_u32 = 0;
  int stride = 1;     // 1: base values, D: extension elements
  bool owned = true;  // allocated by the library (freed by exh_table_free)
};

// A device buffer that only grows; contents are scratch between calls.
struct Arena {
  void *ptr = nullptr;
  size_t bytes = 0;
  int reserve(size_t need);
  void release();
};

// Device buffers that are reused instead of returned to the driver: tables and per-proof buffers are
// allocated and freed around every call, and hipMalloc / hipFree cost more than the kernels between
// them.  Everything a context does runs on its one stream and every context has a pool of its own, so a
// buffer given out again is safe to write as soon as the earlier work queued on it has run: no wait on release.
struct Pool {
  std::multimap<size_t, void *> idle;  // by size
  std::map<void *, size_t> sizes;      // every buffer the pool owns, live or idle
  size_t idle_bytes = 0;
  void *alloc(size_t bytes);  // nullptr when the device is out of memory (idle buffers are returned first)
  void release(void *ptr);
  void trim();                // hipFree of everything idle
};

// One timed kernel launch (HIP events on the library's stream), kept while profiling is on.
struct ProfileEntry {
  std::string name;
  int round = 0;
  uint64_t alg_bytes = 0;  // bytes the launch must move: tables read + tables written
  hipEvent_t start = nullptr, stop = nullptr;
  float ms = -1.0f;
};

struct Context {
  bool ready = false;
  bool profiling = false;
  std::vector<ProfileEntry> profile;
  // bracket a launch: prof_begin records the start event, prof_end the stop event (no-ops unless
  // profiling is on)
  void prof_begin(const char *name, int round, uint64_t alg_bytes);
  void prof_end();
  void prof_clear();
  int device = -1;
  int compute_units = 0;
  hipStream_t stream = nullptr;
  std::map<uint64_t, DeviceTable> tables;
  uint64_t next_handle = 1;
  Arena fold_a, fold_b;  // the two generations of folded tables
  uint64_t session_epoch = 0;  // bumped by every session begin: the arenas belong to the latest session
  Pool pool;
  Arena misc;            // weights, partial sums, small results
  Arena tree;            // the layers of a fraction tree above its leaves, for the length of one proof
  uint32_t *host_pinned = nullptr;  // small pinned buffer for per-round results
  size_t host_pinned_words = 0;
  uint32_t *host_pinned_dev = nullptr;  // the same buffer as kernels address it
  uint32_t log_seq = 0;  // counts the control blocks that launches delivered to host_pinned themselves
  // how many proofs are running side by side (see side_context): a grid whose workgroups wait for one another
  // may take 1 / share of the device, so that the grids of all of them are resident together
  int share = 1;
  int require();  // OK, or E_DEVICE with the reason when the library is not initialised
};

// The context of the calling thread: the library's own, unless the thread has been given another with
// use_context.  The side context has a stream, workspace and pinned buffer of its own (no tables: handles belong to
// the library's context), so that a second host thread can run a proof on it while the first runs one on the
// library's; it is made on first use.
Context &ctx();
void use_context(Context *c);  // nullptr: back to the library's own
int side_context(Context **out);
int ctx_init(int device);
void ctx_shutdown();

// issue_rate.hip: one timed launch of independent (or dependent) chains of one VALU instruction
int issue_rate(int op, int chains, int workgroups, int iterations, const char **name, float *ms,
               double *instructions_per_wave, int *clock_khz, int *compute_units);
int issue_rate_ops();

}  // namespace exh
