// runtime_hip: device runtime for the HIP backend -- device/stream set-up,
// memory, copies, hiprtc compilation for gfx950 with an in-process and an
// on-disk code-object cache, and kernel launches on one HIP stream.
//
// Takes the place of the reference's CUDA runtime (src/runtime_cuda.c:192-435)
// with the same call surface (init / alloc / free / copy / memset / compile /
// launch / sync / program_destroy) but none of its mechanism: it links
// libamdhip64 and libhiprtc directly, never synchronises after a launch, and
// shares one module between all runners whose source text is identical.
#include "runtime_hip.h"

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <hip/hiprtc.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdlib>
#include <cstring>
#include <unordered_map>
#include <fstream>
#include <map>
#include <memory>

namespace polyhip {

namespace {

struct Module {
  hipModule_t mod = nullptr;
  std::vector<char> code;
  ~Module() { if (mod) (void)hipModuleUnload(mod); }
};

struct Runtime {
  bool tried = false;
  bool ok = false;
  int device = 0;
  hipStream_t stream = nullptr;
  hipStream_t side[3] = {nullptr, nullptr, nullptr};   // further streams of a plan's captured graphs, made on first use
  GraphLaunches *record = nullptr, *update = nullptr;   // see runtime_graph_record / runtime_graph_update
  LaunchTimes *times = nullptr;                         // see runtime_time_launches
  hipStream_t launch_on = nullptr;     // where program_launch puts kernels when not the main stream
  std::map<uint64_t, std::weak_ptr<Module>> modules;   // keyed by source hash
  std::map<uint64_t, std::vector<char>> code_cache;    // compiled, not yet loaded
};

Runtime &rt() {
  static Runtime r;
  return r;
}

bool check(hipError_t e, const char *what) {
  if (e == hipSuccess) return true;
  log_err("runtime_hip", "%s failed: %s", what, hipGetErrorString(e));
  return false;
}

std::string cache_dir() {
  const char *off = getenv("POLY_CACHE");
  if (off && strcmp(off, "0") == 0) return "";
  std::string base;
  if (const char *d = getenv("POLY_HIP_CACHE_DIR")) base = d;
  else if (const char *x = getenv("XDG_CACHE_HOME")) base = std::string(x) + "/polygrad_hip";
  else if (const char *h = getenv("HOME")) base = std::string(h) + "/.cache/polygrad_hip";
  else return "";
  mkdir(base.substr(0, base.find_last_of('/')).c_str(), 0755);
  mkdir(base.c_str(), 0755);
  return base;
}

}  // namespace

std::string runtime_cache_dir() { return cache_dir(); }

// hiprtc needs no device, so this also serves compile-only checks.
bool compile_to_code_object(const std::string &source, std::vector<char> *code, std::string *log) {
  // Compiler options; they are part of the cache key.  Contraction to FMA is off so
  // that a*b+c rounds twice, as in the reference's CPU backend (x86-64 baseline, no FMA).
  // Packed FP32 instructions are kept out of generated code on purpose.
  static const char *opts[] = {"--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off", "-Xclang",
                               "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-value"};
  const int n_opts = (int)(sizeof(opts) / sizeof(opts[0]));
  uint64_t h = fnv1a(source.data(), source.size());
  for (int i = 0; i < n_opts; i++) h = h * 1099511628211ULL ^ fnv1a(opts[i], strlen(opts[i]));
  // a code object on disk belongs to the compiler that made it
  int rtc_major = 0, rtc_minor = 0;
  if (hiprtcVersion(&rtc_major, &rtc_minor) == HIPRTC_SUCCESS) h = h * 1099511628211ULL ^ (uint64_t)(rtc_major * 100000 + rtc_minor);
  Runtime &r = rt();
  auto it = r.code_cache.find(h);
  if (it != r.code_cache.end()) { *code = it->second; return true; }
  std::string dir = cache_dir();
  std::string path = dir.empty() ? "" : strf("%s/%016llx_%zu.hsaco", dir.c_str(), (unsigned long long)h, source.size());
  if (!path.empty()) {
    std::ifstream f(path, std::ios::binary);
    if (f) {
      code->assign(std::istreambuf_iterator<char>(f), std::istreambuf_iterator<char>());
      if (!code->empty()) { r.code_cache[h] = *code; return true; }
    }
  }
  hiprtcProgram prog;
  if (hiprtcCreateProgram(&prog, source.c_str(), "poly_kernel.hip", 0, nullptr, nullptr) != HIPRTC_SUCCESS) {
    *log = "hiprtcCreateProgram failed";
    return false;
  }
  hiprtcResult res = hiprtcCompileProgram(prog, n_opts, opts);
  size_t ls = 0;
  hiprtcGetProgramLogSize(prog, &ls);
  if (ls > 1) { log->resize(ls); hiprtcGetProgramLog(prog, &(*log)[0]); }
  if (res != HIPRTC_SUCCESS) { hiprtcDestroyProgram(&prog); return false; }
  size_t cs = 0;
  hiprtcGetCodeSize(prog, &cs);
  code->resize(cs);
  hiprtcGetCode(prog, code->data());
  hiprtcDestroyProgram(&prog);
  r.code_cache[h] = *code;
  if (!path.empty()) {
    std::string tmp = path + strf(".%d.tmp", (int)getpid());
    std::ofstream f(tmp, std::ios::binary);
    if (f) {
      f.write(code->data(), (std::streamsize)code->size());
      f.close();
      rename(tmp.c_str(), path.c_str());
    }
  }
  return true;
}

int runtime_init() {
  Runtime &r = rt();
  if (r.tried) return r.ok ? 0 : -1;
  r.tried = true;
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || n < 1) {
    log_err("runtime_hip", "no HIP device available");
    return -1;
  }
  int dev = 0;
  if (const char *d = getenv("POLY_HIP_DEVICE")) dev = atoi(d);
  if (dev < 0 || dev >= n) dev = 0;
  if (!check(hipSetDevice(dev), "hipSetDevice")) return -1;
  r.device = dev;
  if (!check(hipStreamCreateWithFlags(&r.stream, hipStreamNonBlocking), "hipStreamCreate")) return -1;
  r.ok = true;
  return 0;
}

void *runtime_stream() { return runtime_init() == 0 ? (void *)rt().stream : nullptr; }

void *runtime_side_stream(int k) {
  if (runtime_init() != 0 || k < 0 || k >= kSideStreams) return nullptr;
  Runtime &r = rt();
  if (!r.side[k] && !check(hipStreamCreateWithFlags(&r.side[k], hipStreamNonBlocking), "hipStreamCreate")) r.side[k] = nullptr;
  return (void *)r.side[k];
}

void runtime_launch_on(void *stream) { rt().launch_on = (hipStream_t)stream; }

void *runtime_alloc(size_t nbytes) {
  if (runtime_init() != 0) return nullptr;
  void *p = nullptr;
  if (nbytes == 0) nbytes = 4;
  if (!check(hipMalloc(&p, nbytes), "hipMalloc")) return nullptr;
  // Fresh memory reads as zero, like the reference's host allocator (calloc,
  // src/exec_plan.c:228-231); ordered on the stream every kernel runs on.
  if (!check(hipMemsetAsync(p, 0, nbytes, rt().stream), "hipMemsetAsync")) { (void)hipFree(p); return nullptr; }
  return p;
}

void runtime_free(void *p) {
  if (!p || runtime_init() != 0) return;
  // The stream may still be using the memory.
  (void)hipStreamSynchronize(rt().stream);
  (void)hipFree(p);
}

int runtime_copy(void *dst, const void *src, size_t n, int kind) {
  if (runtime_init() != 0) return -1;
  hipMemcpyKind k = kind == 0 ? hipMemcpyHostToDevice : kind == 1 ? hipMemcpyDeviceToHost : hipMemcpyDeviceToDevice;
  if (n == 0) return 0;
  if (!check(hipMemcpyAsync(dst, src, n, k, rt().stream), "hipMemcpyAsync")) return -1;
  return check(hipStreamSynchronize(rt().stream), "hipStreamSynchronize") ? 0 : -1;
}

int runtime_memset(void *p, int value, size_t n) {
  if (runtime_init() != 0) return -1;
  if (n == 0) return 0;
  return check(hipMemsetAsync(p, value, n, rt().stream), "hipMemsetAsync") ? 0 : -1;
}

bool runtime_device_can_read(const void *p) {
  if (!p || runtime_init() != 0) return false;
  hipPointerAttribute_t a;
  memset(&a, 0, sizeof(a));
  if (hipPointerGetAttributes(&a, p) != hipSuccess) {
    (void)hipGetLastError();      // an address HIP knows nothing about; the error must not stick
    return false;
  }
  // device memory, managed memory, or host memory that HIP pinned (hipHostMalloc)
  return a.type == hipMemoryTypeDevice || a.type == hipMemoryTypeManaged || a.type == hipMemoryTypeHost ||
         a.type == hipMemoryTypeArray;
}

int runtime_sync() {
  if (runtime_init() != 0) return -1;
  return check(hipStreamSynchronize(rt().stream), "hipStreamSynchronize") ? 0 : -1;
}

struct Program {
  std::shared_ptr<Module> module;
  hipFunction_t fn = nullptr;
  std::string entry;
};

Program *program_create(const std::string &source, const std::string &entry) {
  if (runtime_init() != 0) return nullptr;
  if (getenv("POLY_DUMP_KERNELS"))
    fprintf(stderr, "=== HIP KERNEL %s ===\n%s\n=== END ===\n", entry.c_str(), source.c_str());
  Runtime &r = rt();
  uint64_t h = fnv1a(source.data(), source.size());
  std::shared_ptr<Module> m;
  auto it = r.modules.find(h);
  if (it != r.modules.end()) m = it->second.lock();
  if (!m) {
    std::vector<char> code;
    std::string log;
    if (!compile_to_code_object(source, &code, &log)) {
      log_err("runtime_hip", "hiprtc failed for %s:\n%s", entry.c_str(), log.c_str());
      fprintf(stderr, "=== FAILED HIP KERNEL %s ===\n%s\n=== END ===\n", entry.c_str(), source.c_str());
      return nullptr;
    }
    m = std::make_shared<Module>();
    m->code = std::move(code);
    if (!check(hipModuleLoadData(&m->mod, m->code.data()), "hipModuleLoadData")) return nullptr;
    r.modules[h] = m;
  }
  Program *p = new Program();
  p->module = m;
  p->entry = entry;
  if (!check(hipModuleGetFunction(&p->fn, m->mod, entry.c_str()), "hipModuleGetFunction")) {
    delete p;
    return nullptr;
  }
  return p;
}

void program_destroy(Program *p) { delete p; }

std::shared_ptr<void> runtime_table(const std::string &source, const std::string &entry, size_t bytes, const LaunchSpec &ls) {
  if (runtime_init() != 0) return nullptr;
  static std::unordered_map<uint64_t, std::weak_ptr<void>> cache;
  const uint64_t h = fnv1a(source.data(), source.size()) ^ (uint64_t)bytes;
  auto it = cache.find(h);
  if (it != cache.end()) if (std::shared_ptr<void> live = it->second.lock()) return live;
  void *buf = runtime_alloc(bytes);
  if (!buf) return nullptr;
  std::shared_ptr<void> owner(buf, [](void *p) { runtime_free(p); });
  Program *prog = program_create(source, entry);
  if (!prog) return nullptr;
  void *arg = buf;
  void *args[1] = {&arg};
  int rc = program_launch(prog, args, ls);
  if (rc == 0) rc = runtime_sync();
  program_destroy(prog);
  if (rc != 0) return nullptr;
  cache[h] = owner;
  return owner;
}

void runtime_time_launches(LaunchTimes *t) { rt().times = t; }
void runtime_graph_record(GraphLaunches *g) { rt().record = g; rt().update = nullptr; }
void runtime_graph_update(GraphLaunches *g) { rt().update = g; rt().record = nullptr; }

int program_launch(Program *p, void **kernel_args, const LaunchSpec &ls) {
  if (!p || runtime_init() != 0) return -1;
  Runtime &r = rt();
  if (GraphLaunches *u = r.update) {
    // the same launch as when the graph was captured, with other argument values: only the
    // node's arguments change
    if (u->failed || u->next >= u->nodes.size()) { u->failed = true; return -1; }
    hipGraphNode_t node = (hipGraphNode_t)u->nodes[u->next++];
    hipKernelNodeParams kp;
    memset(&kp, 0, sizeof kp);
    if (hipGraphKernelNodeGetParams(node, &kp) != hipSuccess) { (void)hipGetLastError(); u->failed = true; return -1; }
    if (kp.func != (void *)p->fn || kp.blockDim.x != ls.block[0] || kp.sharedMemBytes != ls.lds_bytes) { u->failed = true; return -1; }
    kp.gridDim = dim3(ls.grid[0], ls.grid[1], ls.grid[2]);     // (a grid may follow a variable's value)
    kp.kernelParams = kernel_args;
    kp.extra = nullptr;
    if (hipGraphExecKernelNodeSetParams((hipGraphExec_t)u->exec, node, &kp) != hipSuccess) { (void)hipGetLastError(); u->failed = true; return -1; }
    return 0;
  }
  hipStream_t stream = r.launch_on ? r.launch_on : r.stream;
  if (LaunchTimes *t = r.times) {
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) { t->failed = true; return -1; }
    t->events.push_back((void *)e0);
    t->events.push_back((void *)e1);
    // (this entry point takes the grid in threads, not in workgroups; a grid whose thread
    // count does not fit its 32 bits is launched the usual way between the two events)
    const unsigned long long tx = (unsigned long long)ls.grid[0] * ls.block[0], ty = (unsigned long long)ls.grid[1] * ls.block[1],
                             tz = (unsigned long long)ls.grid[2] * ls.block[2];
    hipError_t e;
    if (tx <= 0xffffffffull && ty <= 0xffffffffull && tz <= 0xffffffffull) {
      e = hipExtModuleLaunchKernel(p->fn, (uint32_t)tx, (uint32_t)ty, (uint32_t)tz, ls.block[0], ls.block[1], ls.block[2], ls.lds_bytes, stream,
                                   kernel_args, nullptr, e0, e1, 0);
    } else {
      (void)hipEventRecord(e0, stream);
      e = hipModuleLaunchKernel(p->fn, ls.grid[0], ls.grid[1], ls.grid[2], ls.block[0], ls.block[1], ls.block[2], ls.lds_bytes, stream, kernel_args, nullptr);
      (void)hipEventRecord(e1, stream);
    }
    if (!check(e, "hipExtModuleLaunchKernel")) { t->failed = true; return -1; }
    return 0;
  }
  hipError_t e = hipModuleLaunchKernel(p->fn, ls.grid[0], ls.grid[1], ls.grid[2], ls.block[0], ls.block[1],
                                       ls.block[2], ls.lds_bytes, stream, kernel_args, nullptr);
  if (!check(e, "hipModuleLaunchKernel")) return -1;
  if (GraphLaunches *g = r.record) {
    // which node of the graph under capture the launch became: the one the stream now depends on
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    const hipGraphNode_t *deps = nullptr;
    size_t n_deps = 0;
    if (hipStreamGetCaptureInfo_v2(stream, &status, nullptr, nullptr, &deps, &n_deps) != hipSuccess || status != hipStreamCaptureStatusActive ||
        n_deps != 1) {
      (void)hipGetLastError();
      g->failed = true;
    } else {
      g->nodes.push_back((void *)deps[0]);
    }
  }
  return 0;
}

}  // namespace polyhip
