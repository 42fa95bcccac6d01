// rtc.cpp -- see rtc.hpp.
#include "rtc.hpp"

#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>
#include <stdlib.h>
#include <unistd.h>

#include <stdio.h>

#include <atomic>
#include <chrono>
#include <map>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

#include "context.hpp"
#include "forms.hpp"
#include "sumcheck.hpp"

namespace exh {

namespace {

// the device headers the kernels are written in, embedded at build time: {file name, text}
struct EmbeddedSource {
  const char *name, *text;
};
const EmbeddedSource kSources[] = {
#include "gen/kernel_sources.inc"
};
constexpr int kNSources = sizeof(kSources) / sizeof(kSources[0]);

// one hiprtc program
struct Part {
  std::vector<std::string> exprs;    // name expressions, e.g. exh::tail_kernel<4, exh::RtStmt>
  std::vector<std::string> lowered;  // their symbols in the code object
  std::vector<char> code;
  std::string log;
  bool ok = false;
};

struct Job {
  std::string key;
  int D = 4;
  StmtDesc desc;
  std::string source;  // the text of struct RtStmt when it is not the plain descriptor's
  std::vector<Part> parts;
  std::vector<std::thread> threads;
  std::atomic<int> running{0};
  enum { COMPILING, LOADED, FAILED } state = COMPILING;
  std::string error;
  std::vector<hipModule_t> modules;
};

std::mutex g_mutex;
// one compilation at a time in the process: the compiler's options are process-wide state
std::mutex g_compiler;
std::atomic<bool> g_stop{false};
std::map<std::pair<std::string, int>, std::unique_ptr<Job>> g_jobs;

void compile_part(Job *job, Part *part) {
  std::lock_guard<std::mutex> one_at_a_time(g_compiler);
  if (g_stop.load()) {  // the process is ending: a compilation that has not begun is dropped
    part->log = "the process ended before the compilation began";
    job->running--;
    return;
  }
  // the descriptor sits in an unnamed namespace, as in the sources generated at build time: with external linkage
  // its fields do not fold to constants before the loops over them are unrolled, and the compilation does not end
  std::string source = "#include \"sumcheck_kernels.hpp\"\nnamespace exh {\nnamespace {\n" +
                       (job->source.empty() ? desc_source(job->desc, "RtStmt") : job->source) + "}\n}\n";
  const char *names[kNSources], *texts[kNSources];
  for (int i = 0; i < kNSources; i++) names[i] = kSources[i].name, texts[i] = kSources[i].text;
  hiprtcProgram prog = nullptr;
  if (hiprtcCreateProgram(&prog, source.c_str(), "statement.hip", kNSources, texts, names) != HIPRTC_SUCCESS) {
    part->log = "hiprtcCreateProgram failed";
    job->running--;
    return;
  }
  for (const std::string &e : part->exprs) hiprtcAddNameExpression(prog, e.c_str());
  // the build's flags for the generated kernels: complete unrolling (the descriptor folds to the statement's own
  // operations) and no packed-fp32 code generation
  const char *options[] = {"--offload-arch=gfx950", "-O3", "-std=c++17", "-mllvm", "-pragma-unroll-threshold=1000000",
                           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
  static const bool verbose = getenv("EXACTA_HIP_RTC_LOG") != nullptr;
  auto started = std::chrono::steady_clock::now();
  if (verbose) fprintf(stderr, "exacta-hip: compiling %s\n", part->exprs[0].c_str());
  hiprtcResult r = hiprtcCompileProgram(prog, (int)(sizeof(options) / sizeof(options[0])), options);
  if (verbose)
    fprintf(stderr, "exacta-hip: %s: %s after %.1f s\n", part->exprs[0].c_str(), hiprtcGetErrorString(r),
            std::chrono::duration<double>(std::chrono::steady_clock::now() - started).count());
  size_t log_size = 0;
  if (hiprtcGetProgramLogSize(prog, &log_size) == HIPRTC_SUCCESS && log_size > 1) {
    part->log.resize(log_size);
    hiprtcGetProgramLog(prog, &part->log[0]);
  }
  if (r == HIPRTC_SUCCESS) {
    size_t code_size = 0;
    bool ok = hiprtcGetCodeSize(prog, &code_size) == HIPRTC_SUCCESS && code_size > 0;
    if (ok) {
      part->code.resize(code_size);
      ok = hiprtcGetCode(prog, part->code.data()) == HIPRTC_SUCCESS;
    }
    for (const std::string &e : part->exprs) {
      const char *low = nullptr;
      if (hiprtcGetLoweredName(prog, e.c_str(), &low) != HIPRTC_SUCCESS || !low) ok = false;
      part->lowered.push_back(low ? low : "");
    }
    part->ok = ok;
  } else if (part->log.empty()) {
    part->log = hiprtcGetErrorString(r);
  }
  hiprtcDestroyProgram(&prog);
  job->running--;
}

// the one-workgroup kernel of a statement: with half the registers for a statement in direct form at F_p^8 (see
// tail_kernel_narrow)
std::string tail_expression(int D, bool direct) {
  return std::string(direct && D == 8 ? "exh::tail_kernel_narrow<" : "exh::tail_kernel<") + std::to_string(D) + ", exh::RtStmt>";
}

// the kernel behind launcher arguments passed by value as one struct
void launch_module(hipFunction_t f, const void *args, uint32_t grid, uint32_t lds_bytes, hipStream_t s) {
  void *params[] = {const_cast<void *>(args)};
  (void)hipModuleLaunchKernel(f, grid, 1, 1, BLOCK, 1, 1, lds_bytes, s, params, nullptr);
}

template <int D>
uint32_t tail_lds(const void *args) {
  return static_cast<const TailArgs<D> *>(args)->lds_bytes;
}

int load_job(Job *job) {
  for (std::thread &t : job->threads)
    if (t.joinable()) t.join();
  job->threads.clear();
  for (Part &p : job->parts)
    if (!p.ok) {
      job->state = Job::FAILED;
      job->error = "run-time compilation of the statement's kernels failed: " + p.log;
      return OK;  // the interpreter goes on serving the statement
    }
  std::map<std::string, hipFunction_t> fn;
  for (Part &p : job->parts) {
    hipModule_t mod = nullptr;
    hipError_t e = hipModuleLoadData(&mod, p.code.data());
    if (e != hipSuccess) {
      job->state = Job::FAILED;
      job->error = std::string("device-error: hipModuleLoadData: ") + hipGetErrorString(e);
      set_error(job->error);
      return E_DEVICE;
    }
    job->modules.push_back(mod);
    for (size_t k = 0; k < p.exprs.size(); k++) {
      hipFunction_t f = nullptr;
      e = hipModuleGetFunction(&f, mod, p.lowered[k].c_str());
      if (e != hipSuccess) {
        job->state = Job::FAILED;
        job->error = std::string("device-error: hipModuleGetFunction ") + p.lowered[k] + ": " + hipGetErrorString(e);
        set_error(job->error);
        return E_DEVICE;
      }
      fn[p.exprs[k]] = f;
    }
    p.code.clear();
    p.code.shrink_to_fit();
  }
  const std::string d = std::to_string(job->D), st = "exh::RtStmt";
  hipFunction_t round[2][2];
  for (int base = 0; base < 2; base++)
    for (int fold = 0; fold < 2; fold++)
      round[base][fold] = fn["exh::round_kernel<" + d + ", " + (base ? "true" : "false") + ", " + (fold ? "true" : "false") +
                             ", " + st + ">"];
  hipFunction_t fold2 = fn["exh::round_kernel_fold2<" + d + ", " + st + ">"];
  hipFunction_t tail = fn[tail_expression(job->D, !job->source.empty())];
  int passes = node_slots(job->desc) <= MAXACC ? nodes_launches(job->desc, job->D) : 0;
  std::vector<hipFunction_t> nodes;
  for (int p = 0; p < passes; p++)
    nodes.push_back(fn["exh::nodes_kernel<" + d + ", " + st + ", " + std::to_string(p) + ", " +
                       std::to_string(nodes_slots_per_pass(job->desc, job->D)) + ">"]);
  const int D = job->D;
  KernelSet set;
  set.launch = [=](const void *args, bool in_base, bool fold, uint32_t grid, hipStream_t s) {
    launch_module(round[in_base ? 1 : 0][fold ? 1 : 0], args, grid, 0, s);
  };
  set.launch_fold2 = [=](const void *args, uint32_t grid, hipStream_t s) { launch_module(fold2, args, grid, 0, s); };
  set.launch_nodes = [=](const void *args, int pass, uint32_t grid, hipStream_t s) {
    launch_module(nodes[(size_t)pass], args, grid, 0, s);
  };
  set.launch_tail = [=](const void *args, uint32_t grid, hipStream_t s) {
    launch_module(tail, args, grid, D == 4 ? tail_lds<4>(args) : tail_lds<8>(args), s);
  };
  set.tail_blocks_per_cu = [=](uint32_t lds_bytes) {
    int blocks = 0;
    if (hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, tail, BLOCK, lds_bytes) != hipSuccess) return -1;
    return blocks;
  };
  set.nodes_passes = passes;
  register_kernels(job->key, job->D, set);
  job->state = Job::LOADED;
  return OK;
}

}  // namespace

bool rtc_enabled() {
  static const bool on = getenv("EXACTA_HIP_NO_RTC") == nullptr;
  return on;
}

namespace {
// A process that ends while a statement compiles cannot wait for the compiler (a compilation has been seen never
// to end once the process is in exit()) and must not run the compiler's own clean-up under it.  So the process
// ends at once then, with the status it was given: open C streams are flushed and later clean-ups are skipped.
// The compiler's library is loaded when it is first used and registers its clean-up then; clean-ups run
// last-registered first, so this one is registered after a first, trivial compilation.
void end_of_process(int status, void *) {
  g_stop = true;
  bool compiling = false;
  {
    std::lock_guard<std::mutex> lock(g_mutex);
    for (auto &kv : g_jobs)
      if (kv.second->running.load() > 0) compiling = true;
    if (!compiling)
      for (auto &kv : g_jobs)
        for (std::thread &t : kv.second->threads)
          if (t.joinable()) t.join();
  }
  if (compiling) {
    // a short grace for a compilation about to end (the ordinary exit then goes on); beyond it the hard exit
    for (int waited_ms = 0; waited_ms < 2000 && compiling; waited_ms += 50) {
      std::this_thread::sleep_for(std::chrono::milliseconds(50));
      compiling = false;
      std::lock_guard<std::mutex> lock(g_mutex);
      for (auto &kv : g_jobs)
        if (kv.second->running.load() > 0) compiling = true;
    }
    if (!compiling) {
      std::lock_guard<std::mutex> lock(g_mutex);
      for (auto &kv : g_jobs)
        for (std::thread &t : kv.second->threads)
          if (t.joinable()) t.join();
      return;
    }
    fflush(nullptr);
    _exit(status);
  }
}

void prepare_compiler() {
  static std::once_flag once;
  std::call_once(once, [] {
    {
      std::lock_guard<std::mutex> one_at_a_time(g_compiler);
      hiprtcProgram prog = nullptr;
      if (hiprtcCreateProgram(&prog, "extern \"C\" __global__ void exh_probe() {}\n", "probe.hip", 0, nullptr, nullptr) ==
          HIPRTC_SUCCESS) {
        const char *options[] = {"--offload-arch=gfx950"};
        (void)hiprtcCompileProgram(prog, 1, options);
        hiprtcDestroyProgram(&prog);
      }
    }
    on_exit(end_of_process, nullptr);
  });
}
}  // namespace

void rtc_request(const std::string &key, const StmtDesc &desc, int D, const std::string &source) {
  prepare_compiler();
  std::lock_guard<std::mutex> lock(g_mutex);
  auto at = std::make_pair(key, D);
  if (g_jobs.count(at)) return;
  auto job = std::make_unique<Job>();
  job->key = key, job->D = D, job->desc = desc, job->source = source;
  const std::string d = std::to_string(D), st = "exh::RtStmt";
  // one program with the set's kernels, compiled on one background thread
  job->parts.resize(1);
  std::vector<std::string> &exprs = job->parts[0].exprs;
  for (const char *base : {"true", "false"})
    for (const char *fold : {"true", "false"})
      exprs.push_back("exh::round_kernel<" + d + ", " + base + ", " + fold + ", " + st + ">");
  // (the double fold follows the base-field sweep, which a statement in direct form does not take)
  if (source.empty()) exprs.push_back("exh::round_kernel_fold2<" + d + ", " + st + ">");
  exprs.push_back(tail_expression(D, !source.empty()));
  int passes = node_slots(desc) <= MAXACC ? nodes_launches(desc, D) : 0;
  for (int p = 0; p < passes; p++)
    exprs.push_back("exh::nodes_kernel<" + d + ", " + st + ", " + std::to_string(p) + ", " +
                    std::to_string(nodes_slots_per_pass(desc, D)) + ">");
  job->running = (int)job->parts.size();
  Job *raw = job.get();
  raw->threads.emplace_back([raw] {
    for (Part &p : raw->parts) compile_part(raw, &p);
  });
  g_jobs[at] = std::move(job);
}

int rtc_collect() {
  std::lock_guard<std::mutex> lock(g_mutex);
  int status = OK;
  for (auto &kv : g_jobs) {
    Job *job = kv.second.get();
    if (job->state == Job::COMPILING && job->running.load() == 0) {
      int s = load_job(job);
      if (s) status = s;
    }
  }
  return status;
}

int rtc_idle(bool wait) {
  {
    std::lock_guard<std::mutex> lock(g_mutex);
    for (auto &kv : g_jobs) {
      if (kv.second->running.load() == 0) continue;
      if (!wait) return 0;
      for (std::thread &t : kv.second->threads)
        if (t.joinable()) t.join();
    }
  }
  int status = rtc_collect();
  return status ? status : 1;
}

int rtc_status(const std::string &key, int D, bool wait) {
  {
    std::lock_guard<std::mutex> lock(g_mutex);
    auto it = g_jobs.find({key, D});
    if (it == g_jobs.end()) return find_kernels(key, D) ? 1 : 0;
    if (wait)
      for (std::thread &t : it->second->threads)
        if (t.joinable()) t.join();
  }
  int status = rtc_collect();
  if (status) return status;
  std::lock_guard<std::mutex> lock(g_mutex);
  Job *job = g_jobs[{key, D}].get();
  if (job->state == Job::FAILED) {
    set_error("device-error: " + job->error);
    return E_DEVICE;
  }
  return job->state == Job::LOADED ? 1 : 0;
}


}  // namespace exh
