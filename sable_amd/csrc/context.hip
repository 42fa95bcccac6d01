// context.hip -- see context.hpp.
#include "context.hpp"

#include "commit.hpp"

namespace exh {

static Context g_ctx, g_side;
static thread_local Context *t_ctx = nullptr;
Context &ctx() { return t_ctx ? *t_ctx : g_ctx; }
void use_context(Context *c) { t_ctx = c; }

static int pinned_buffer(Context &c) {
  c.host_pinned_words = 1 << 16;
  // coherent and mapped: a kernel writes a sumcheck's logs into it directly and the host polls for them
  EXH_HIP(hipHostMalloc((void **)&c.host_pinned, c.host_pinned_words * 4, hipHostMallocMapped | hipHostMallocCoherent));
  EXH_HIP(hipHostGetDevicePointer((void **)&c.host_pinned_dev, c.host_pinned, 0));
  return OK;
}

int side_context(Context **out) {
  int status = g_ctx.require();
  if (status) return status;
  Context &c = g_side;
  if (!c.ready) {
    EXH_HIP(hipStreamCreate(&c.stream));
    if ((status = pinned_buffer(c))) return status;
    c.device = g_ctx.device;
    c.compute_units = g_ctx.compute_units;
    c.ready = true;
  }
  *out = &c;
  return OK;
}

int Arena::reserve(size_t need) {
  if (need <= bytes) return OK;
  if (ptr) {
    hipError_t e = hipFree(ptr);
    ptr = nullptr;
    bytes = 0;
    if (e != hipSuccess) {
      set_error(std::string("device-error: hipFree: ") + hipGetErrorString(e));
      return E_DEVICE;
    }
  }
  size_t rounded = (need + ((size_t)1 << 20) - 1) & ~(((size_t)1 << 20) - 1);
  hipError_t e = hipMalloc(&ptr, rounded);
  if (e != hipSuccess) {
    ptr = nullptr;
    set_error(std::string("device-out-of-memory: ") + std::to_string(rounded) + " bytes: " + hipGetErrorString(e));
    return E_NOMEM;
  }
  bytes = rounded;
  return OK;
}

void Arena::release() {
  if (ptr) (void)hipFree(ptr);
  ptr = nullptr;
  bytes = 0;
}

static size_t pool_round(size_t bytes) {
  size_t unit = bytes < ((size_t)1 << 20) ? 4096 : (size_t)1 << 20;
  return bytes ? (bytes + unit - 1) / unit * unit : unit;
}

void *Pool::alloc(size_t bytes) {
  size_t want = pool_round(bytes);
  auto it = idle.find(want);
  if (it != idle.end()) {
    void *p = it->second;
    idle.erase(it);
    idle_bytes -= want;
    return p;
  }
  void *p = nullptr;
  if (hipMalloc(&p, want) != hipSuccess) {
    (void)hipGetLastError();
    trim();
    if (hipMalloc(&p, want) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
  }
  sizes[p] = want;
  return p;
}

void Pool::release(void *ptr) {
  auto it = sizes.find(ptr);
  if (it == sizes.end()) return;
  constexpr size_t IDLE_LIMIT = (size_t)64 << 30;  // of the 288 GB
  if (idle_bytes + it->second > IDLE_LIMIT) {
    (void)hipFree(ptr);
    sizes.erase(it);
    return;
  }
  idle.emplace(it->second, ptr);
  idle_bytes += it->second;
}

void Pool::trim() {
  for (auto &kv : idle) {
    (void)hipFree(kv.second);
    sizes.erase(kv.second);
  }
  idle.clear();
  idle_bytes = 0;
}

int Context::require() {
  if (!ready) {
    set_error("device-error: the library is not initialised (exh_init), or no MI355X is visible");
    return E_DEVICE;
  }
  return OK;
}

void Context::prof_begin(const char *name, int round, uint64_t alg_bytes) {
  if (!profiling) return;
  ProfileEntry e;
  e.name = name, e.round = round, e.alg_bytes = alg_bytes;
  if (hipEventCreate(&e.start) != hipSuccess || hipEventCreate(&e.stop) != hipSuccess) return;
  (void)hipEventRecord(e.start, stream);
  profile.push_back(e);
}
void Context::prof_end() {
  if (!profiling || profile.empty()) return;
  (void)hipEventRecord(profile.back().stop, stream);
}
void Context::prof_clear() {
  for (ProfileEntry &e : profile) {
    if (e.start) (void)hipEventDestroy(e.start);
    if (e.stop) (void)hipEventDestroy(e.stop);
  }
  profile.clear();
}

int ctx_init(int device) {
  Context &c = g_ctx;
  if (c.ready) return OK;
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count <= 0) {
    set_error(std::string("device-error: no HIP device: ") + (e == hipSuccess ? "count 0" : hipGetErrorString(e)));
    return E_DEVICE;
  }
  if (device < 0 || device >= count) {
    set_error("invalid-parameter: device index");
    return E_PARAM;
  }
  EXH_HIP(hipSetDevice(device));
  hipDeviceProp_t prop;
  EXH_HIP(hipGetDeviceProperties(&prop, device));
  if (std::string(prop.gcnArchName).rfind("gfx950", 0) != 0) {
    set_error(std::string("device-error: kernels are built for gfx950, found ") + prop.gcnArchName);
    return E_DEVICE;
  }
  EXH_HIP(hipStreamCreate(&c.stream));
  {
    int pinned_status = pinned_buffer(c);
    if (pinned_status) return pinned_status;
  }
  {  // the device address of the static scratch array, with this device current
    int scratch_status = dot_pairs_static_setup(device);
    if (scratch_status) return scratch_status;
  }
  c.device = device;
  c.compute_units = prop.multiProcessorCount;
  c.ready = true;
  return OK;
}

static void release_context(Context &c) {
  if (!c.ready) return;
  (void)hipStreamSynchronize(c.stream);
  c.prof_clear();
  for (auto &kv : c.tables)
    if (kv.second.owned && kv.second.ptr) c.pool.release(kv.second.ptr);
  c.tables.clear();
  c.pool.trim();
  c.fold_a.release();
  c.fold_b.release();
  c.misc.release();
  c.tree.release();
  if (c.host_pinned) (void)hipHostFree(c.host_pinned);
  c.host_pinned = nullptr;
  (void)hipStreamDestroy(c.stream);
  c.stream = nullptr;
  c.ready = false;
}

void ctx_shutdown() {
  release_context(g_side);
  release_context(g_ctx);
}

}  // namespace exh
