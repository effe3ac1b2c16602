// backend_hip: the C ABI of the backend -- the PolyBackendDesc row (lower_item /
// execute / free_runner / get_allocator), the allocator, the runtime wrappers
// and the render-only entry points.  Declarations and the reference interfaces
// they replace are in include/polygrad_hip.h.
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <cstring>

#include "polygrad_hip.h"
#include "runtime_hip.h"
#include "templates.h"

// Scratch memory of poly_hip_execute_static: stage-one results of a two-stage kernel go
// here instead of into memory the runner allocates.  Every GPU the library runs on holds
// its own copy of the array, at its own address, until the process ends.  In host code
// the name below only stands for the symbol; the device address comes from
// hipGetSymbolAddress (static_scratch()).
static __device__ __align__(256) unsigned char poly_static_scratch[POLY_HIP_STATIC_SCRATCH_BYTES];

namespace polyhip {

static RenderOptions options_from_flags(int flags) {
  RenderOptions o;
  if (flags & 1) o.allow_templates = false;
  if (flags & 2) o.allow_vectorize = false;
  if (flags & 4) o.allow_coop_reduce = false;
  if (const char *e = getenv("POLY_HIP_NO_TEMPLATES")) if (*e == '1') o.allow_templates = false;
  return o;
}

// Kernel symbols name what the kernel is (class, and a hash of its source), so
// identical kernels share one module and a profiler can tell the others apart.
static void name_kernel(RenderedKernel *rk) {
  static const char *const tag[] = {"ew", "rowred", "thrred", "mm", "gather", "copy", "attn"};
  auto rename = [](std::string &src, const std::string &from, const std::string &to) {
    for (size_t pos = 0; (pos = src.find(from, pos)) != std::string::npos; pos += to.size()) src.replace(pos, from.size(), to);
  };
  uint64_t h = fnv1a(rk->source.data(), rk->source.size());
  std::string name = strf("poly_%s_%08x", tag[(int)rk->klass], (unsigned)(h ^ (h >> 32)));
  if (rk->klass == KernelClass::MATMUL_MFMA) {
    // strategy: "mfma 32x32x16 bf16 M=.. N=.. K=.. Z=.. tile .. A:k-major B:n-major"
    long long M = 0, N = 0, K = 0, Z = 0;
    const char *p = strstr(rk->strategy.c_str(), "M=");
    if (p && sscanf(p, "M=%lld N=%lld K=%lld Z=%lld", &M, &N, &K, &Z) == 4)
      name = strf("poly_mm_%lldx%lldx%lld_z%lld_%s%s_%08x", M, N, K, Z, strstr(p, "A:k-major") ? "k" : "m",
                  strstr(p, "B:k-major") ? "k" : "n", (unsigned)(h ^ (h >> 32)));
  }
  rename(rk->source, " poly_k(", " " + name + "(");
  rk->entry = name;
  if (!rk->fallback_source.empty()) {
    rename(rk->fallback_source, " poly_k(", " " + name + "_slow(");
    rk->fallback_entry = name + "_slow";
  }
  for (size_t i = 0; i < rk->pres.size(); i++) {
    const std::string pn = name + (i == 0 ? "_pre" : strf("_pre%zu", i + 1));
    rename(rk->pres[i].source, " poly_k(", " " + pn + "(");
    rk->pres[i].entry = pn;
  }
}

static bool render_root(const PolyUOp *root, const char *fn_name, int flags, RenderedKernel *rk) {
  KernelGraph g;
  if (!g.build(root)) { log_err("render_hip", "%s: %s", fn_name, g.error.c_str()); return false; }
  std::string err;
  if (!render_kernel(g, "poly_k", options_from_flags(flags), rk, &err)) {
    log_err("render_hip", "%s: %s", fn_name, err.c_str());
    return false;
  }
  name_kernel(rk);
  return true;
}

HipRunner *runner_create(const PolyUOp *root, const char *fn_name, int flags) {
  if (runtime_init() != 0) return nullptr;
  RenderedKernel rk;
  if (!render_root(root, fn_name ? fn_name : "kernel", flags, &rk)) return nullptr;
  return runner_from_rendered(rk, fn_name, true);
}

// A kernel that only streams through its buffers and moves more bytes than the caches hold
// (the 4 MiB L2 of each XCD aside, the memory-side cache is 256 MiB) reads with the
// nontemporal hint: what it reads once then leaves the caches to what is read again, and
// the memory system serves the reads at a higher rate (three 256 MiB inputs and one output
// of that size: 5.3 -> 6.3 TB/s; read-only rows: 6.1 -> 6.9 TB/s).  Its stores get the hint
// too where the output alone exceeds that cache, so none of it could be found there by a
// later kernel anyway (the AdamW update: 6.1 -> 6.4 TB/s).  A kernel that reads its input
// a second time keeps plain accesses.  Matmul, attention, gather and
// copy kernels reuse what they read and are left alone.
static void streaming_hints(RenderedKernel *rk) {
  if (rk->klass != KernelClass::ELEMENTWISE && rk->klass != KernelClass::ROW_REDUCE && rk->klass != KernelClass::THREAD_REDUCE) return;
  const double cache = 256.0 * 1048576.0;
  // (a row chain over rows too long for its registers reads them once per phase, the second
  // time from the L2 that the first pass filled: 0.38 -> 0.45 ms with the hint on the
  // derivative of the loss over 4096 rows of 50 257 logits)
  bool loads = rk->bytes >= cache && !rk->rereads_inputs, stores = loads && rk->bytes_written > cache;
  const bool off = getenv("POLY_HIP_NO_STREAMING_HINTS") != nullptr;
  if (off) loads = stores = false;
  bool forced = false;
  if (const char *mode = measurement_env("POLY_HIP_STREAM")) {
    const char *mb = measurement_env("POLY_HIP_STREAM_MB");
    const bool big = rk->bytes >= (mb ? atof(mb) : 256.0) * 1048576.0;
    loads = big && strchr(mode, 'L');
    stores = big && strchr(mode, 'S');
    forced = true;
  }
  struct Form { bool loads, stores; const char *label, *defs, *text; };
  static const Form forms[] = {{false, false, "nt_none", "", ""},
                               {true, false, "nt_loads", "#define POLY_NT_LOADS 1\n", ", streaming loads"},
                               {true, true, "nt_all", "#define POLY_NT_LOADS 1\n#define POLY_NT_STORES 1\n", ", streaming loads and stores"},
                               {false, true, "nt_stores", "#define POLY_NT_STORES 1\n", ", streaming stores"}};
  const Form *rule = &forms[0];
  for (const Form &f : forms) if (f.loads == loads && f.stores == stores) rule = &f;
  // With the search on, a kernel of a quarter of the cache's size and more also comes in the
  // other forms (not the stores alone): which one is fastest depends on what the kernels
  // around it leave in the caches and look for there, and that the timing on the plan's
  // own buffers sees.  The hint changes no value.
  std::vector<RenderedKernel::Variant> others;
  // (a kernel that already carries its final symbol name has no candidates: they are named when chosen)
  const bool unnamed = rk->source.find(" poly_k(") != std::string::npos;
  if (matmul_tuning_enabled() && !off && !forced && unnamed && rk->bytes >= cache / 4 && !rk->rereads_inputs) {
    if (rk->variants.empty()) rk->variants.push_back({"default", rk->source, rk->strategy, rk->launch});
    for (int fi = 0; fi < 3; fi++) {
      const Form &f = forms[fi];
      if (&f == rule) continue;
      for (const RenderedKernel::Variant &v : rk->variants)
        others.push_back({v.label == "default" ? std::string(f.label) : v.label + "+" + f.label, f.defs + v.source, v.strategy + f.text, v.launch});
    }
  }
  if (rule != &forms[0]) {
    rk->source = rule->defs + rk->source;
    for (RenderedKernel::Variant &v : rk->variants) { v.source = rule->defs + v.source; v.strategy += rule->text; }
    rk->strategy += rule->text;
  }
  for (RenderedKernel::Variant &v : others) rk->variants.push_back(std::move(v));
}

HipRunner *runner_from_rendered(const RenderedKernel &rk, const char *fn_name, bool named) {
  if (runtime_init() != 0) return nullptr;
  HipRunner *r = new HipRunner();
  r->name = fn_name ? fn_name : "kernel";
  r->rk = rk;
  streaming_hints(&r->rk);
  if (!named) name_kernel(&r->rk);
  r->main = program_create(r->rk.source, r->rk.entry);
  if (!r->main) { runner_destroy(r); return nullptr; }
  if (!r->rk.guards.empty()) {
    r->flag = runtime_alloc(sizeof(int));
    if (!r->flag) { runner_destroy(r); return nullptr; }
    for (const RenderedKernel::Guard &gd : r->rk.guards) {
      Program *p = program_create(gd.source, gd.entry);
      if (!p) { runner_destroy(r); return nullptr; }
      r->guards.push_back(p);
    }
    r->fallback = program_create(r->rk.fallback_source, r->rk.fallback_entry);
    if (!r->fallback) { runner_destroy(r); return nullptr; }
  }
  if (!r->rk.pres.empty()) {
    if (!r->rk.guards.empty()) { log_err("lower", "%s: a two-stage kernel cannot also be guarded", r->name.c_str()); runner_destroy(r); return nullptr; }
    for (const RenderedKernel::Pre &pk : r->rk.pres) {
      Program *p = program_create(pk.source, pk.entry);
      if (!p) { runner_destroy(r); return nullptr; }
      r->pres.push_back(p);
    }
    // the scratch memory itself is allocated by the first ordinary launch
    // (runner_ensure_scratch): a runner that only ever runs on scratch memory handed in
    // from outside never holds any of its own
  }
  for (const RenderedKernel::Table &t : r->rk.tables) {
    std::shared_ptr<void> tab = runtime_table(t.source, t.entry, t.bytes, t.launch);
    if (!tab) { runner_destroy(r); return nullptr; }
    r->tables.push_back(tab);
  }
  size_t n = (size_t)r->rk.n_params + (size_t)r->rk.n_vars + r->rk.tables.size() + 2;
  r->vetted.assign((size_t)r->rk.n_params, nullptr);
  r->ptr_store.resize(n);
  r->var_store.resize(n);
  r->arg_ptrs.resize(n);
  return r;
}

int runner_use_variant(HipRunner *r, int idx) {
  if (!r || idx < 0 || idx >= (int)r->rk.variants.size()) return -1;
  const RenderedKernel::Variant &v = r->rk.variants[(size_t)idx];
  RenderedKernel named;
  named.klass = r->rk.klass;
  named.source = v.source;
  named.strategy = v.strategy;
  name_kernel(&named);
  Program *p = program_create(named.source, named.entry);
  if (!p) return -1;
  program_destroy(r->main);
  r->main = p;
  r->rk.source = named.source;
  r->rk.entry = named.entry;
  r->rk.strategy = v.strategy;
  r->rk.launch = v.launch;
  return 0;
}

int runner_ensure_scratch(HipRunner *r) {
  if (!r || (r->pres.empty() && r->rk.scratch_bytes == 0) || r->scratch) return 0;
  r->scratch = runtime_alloc(r->rk.scratch_bytes);
  r->owns_scratch = true;
  return r->scratch ? 0 : -1;
}

void runner_share_scratch(HipRunner *r, void *pool) {
  if (!r || !pool || r->rk.scratch_bytes == 0) return;
  if (r->scratch && r->owns_scratch) runtime_free(r->scratch);
  r->scratch = pool;
  r->owns_scratch = false;
}

void runner_destroy(HipRunner *r) {
  if (!r) return;
  if (r->main) program_destroy(r->main);
  for (Program *p : r->guards) program_destroy(p);
  if (r->fallback) program_destroy(r->fallback);
  for (Program *p : r->pres) program_destroy(p);
  if (r->scratch && r->owns_scratch) runtime_free(r->scratch);
  if (r->flag) runtime_free(r->flag);
  delete r;
}

int runner_launch(HipRunner *r, void **args, int n_args, void *scratch_from_caller) {
  const int np = r->rk.n_params, nv = r->rk.n_vars;
  if (n_args < np + nv) {
    log_err("execute", "%s: expected %d args, got %d", r->name.c_str(), np + nv, n_args);
    return -1;
  }
  for (int i = 0; i < np; i++) {
    if (!args[i]) { log_err("execute", "%s: null buffer for param %d", r->name.c_str(), i); return -1; }
    // The reference's callers hand some slots over as host addresses whatever the device
    // (constants of the frontend's registry, src/frontend.c:2231-2232; the loss and the
    // bias corrections of a training step, src/instance.c:1299-1311).  A kernel would
    // fault on them: refuse, once per new pointer.
    if (args[i] != r->vetted[(size_t)i]) {
      if (!runtime_device_can_read(args[i])) {
        log_err("execute", "%s: param %d (%p) is not device memory; upload it with the allocator's copy_in first",
                r->name.c_str(), i, args[i]);
        return -1;
      }
      r->vetted[(size_t)i] = args[i];
    }
    r->ptr_store[(size_t)i] = args[i];
    r->arg_ptrs[(size_t)i] = &r->ptr_store[(size_t)i];
  }
  // DEFINE_VAR values arrive as pointers to host ints; kernels take them by value.
  for (int v = 0; v < nv; v++) {
    if (!args[np + v]) { log_err("execute", "%s: null var %d", r->name.c_str(), v); return -1; }
    r->var_store[(size_t)v] = *(const int *)args[np + v];
    r->arg_ptrs[(size_t)(np + v)] = &r->var_store[(size_t)v];
  }
  const int nt = (int)r->tables.size();
  for (int t = 0; t < nt; t++) {
    r->ptr_store[(size_t)(np + nv + t)] = r->tables[(size_t)t].get();
    r->arg_ptrs[(size_t)(np + nv + t)] = &r->ptr_store[(size_t)(np + nv + t)];
  }
  if (!r->pres.empty() || r->rk.scratch_bytes > 0) {      // (scratch memory without a first stage: a product that leaves block maxima there)
    void *scratch = scratch_from_caller;
    if (!scratch) {
      if (runner_ensure_scratch(r) != 0) { log_err("execute", "%s: no scratch memory", r->name.c_str()); return -1; }
      scratch = r->scratch;
    }
    r->ptr_store[(size_t)(np + nv + nt)] = scratch;
    r->arg_ptrs[(size_t)(np + nv + nt)] = &r->ptr_store[(size_t)(np + nv + nt)];
    for (size_t i = 0; i < r->pres.size() && !r->skip_pres; i++)
      if (program_launch(r->pres[i], r->arg_ptrs.data(), r->rk.pres[i].launch) != 0) return -1;
    return program_launch(r->main, r->arg_ptrs.data(), r->rk.launch);
  }
  if (r->guards.empty()) return program_launch(r->main, r->arg_ptrs.data(), r->rk.launch);
  // The guard writes *flag (1 = fast path valid, 0 = not); the fast kernel and
  // its generic twin both launch and exactly one of them does the work.
  r->ptr_store[(size_t)(np + nv + nt)] = r->flag;
  r->arg_ptrs[(size_t)(np + nv + nt)] = &r->ptr_store[(size_t)(np + nv + nt)];
  for (size_t gi = 0; gi < r->guards.size(); gi++) {
    const RenderedKernel::Guard &gd = r->rk.guards[gi];
    enum { kMaxGuardArgs = 8 };     // a guard reads one or two buffers; no heap use per launch
    if (gd.arg_params.size() > kMaxGuardArgs) { log_err("execute", "%s: guard with %zu arguments", r->name.c_str(), gd.arg_params.size()); return -1; }
    void *vals[kMaxGuardArgs + 1];
    void *gargs[kMaxGuardArgs + 1];
    vals[0] = r->flag;
    gargs[0] = &vals[0];
    for (size_t i = 0; i < gd.arg_params.size(); i++) { vals[i + 1] = args[gd.arg_params[i]]; gargs[i + 1] = &vals[i + 1]; }
    if (program_launch(r->guards[gi], gargs, gd.launch) != 0) return -1;
  }
  if (program_launch(r->main, r->arg_ptrs.data(), r->rk.launch) != 0) return -1;
  return program_launch(r->fallback, r->arg_ptrs.data(), r->rk.fallback_launch);
}

}  // namespace polyhip

using namespace polyhip;

// Device address of poly_static_scratch on the current device, looked up once per device
// (with that device current) and kept; NULL after an error message when the lookup fails.
static void *static_scratch() {
  enum { kMaxDevices = 64 };
  static void *ptr_of[kMaxDevices];
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    log_err("execute_static", "no current HIP device");
    return nullptr;
  }
  if (!ptr_of[dev]) {
    void *p = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(poly_static_scratch));
    if (e != hipSuccess || !p) {
      log_err("execute_static", "hipGetSymbolAddress failed: %s", hipGetErrorString(e));
      return nullptr;
    }
    ptr_of[dev] = p;
  }
  return ptr_of[dev];
}

extern "C" {

int poly_hip_init(void) {
  if (runtime_init() != 0) return -1;
  return static_scratch() ? 0 : -1;
}
int poly_hip_available(void) { return runtime_init() == 0 ? 1 : 0; }
void *poly_hip_alloc(size_t nbytes) { return runtime_alloc(nbytes); }
void poly_hip_free(void *p) { runtime_free(p); }
int poly_hip_copy_htod(void *dst, const void *src, size_t n) { return runtime_copy(dst, src, n, 0); }
int poly_hip_copy_dtoh(void *dst, const void *src, size_t n) { return runtime_copy(dst, src, n, 1); }
int poly_hip_copy_dtod(void *dst, const void *src, size_t n) { return runtime_copy(dst, src, n, 2); }
int poly_hip_memset(void *p, int value, size_t n) { return runtime_memset(p, value, n); }
int poly_hip_sync(void) { return runtime_sync(); }
void *poly_hip_stream(void) { return runtime_stream(); }

struct PolyHipProgram { Program *p; };

PolyHipProgram *poly_hip_compile(const char *source, const char *entry) {
  if (!source || !entry) return nullptr;
  Program *p = program_create(source, entry);
  if (!p) return nullptr;
  PolyHipProgram *h = new PolyHipProgram();
  h->p = p;
  return h;
}

int poly_hip_launch(PolyHipProgram *prog, void **kernel_args, int n_args, unsigned gx, unsigned gy,
                    unsigned gz, unsigned bx, unsigned by, unsigned bz, unsigned lds_bytes) {
  (void)n_args;
  if (!prog) return -1;
  LaunchSpec ls;
  ls.grid[0] = gx; ls.grid[1] = gy; ls.grid[2] = gz;
  ls.block[0] = bx; ls.block[1] = by; ls.block[2] = bz;
  ls.lds_bytes = lds_bytes;
  return program_launch(prog->p, kernel_args, ls);
}

void poly_hip_program_destroy(PolyHipProgram *prog) {
  if (!prog) return;
  program_destroy(prog->p);
  delete prog;
}

// ── vtable ────────────────────────────────────────────────────────────────

int poly_hip_lower_item(PolyCtx *ctx, PolyUOp *scheduled_root, const char *fn_name, PolyRunner *out) {
  (void)ctx;  // the lowering only reads the graph; it creates no UOps
  if (!scheduled_root || !out) return -1;
  HipRunner *r = runner_create(scheduled_root, fn_name, 0);
  if (!r) return -1;
  out->kind = POLY_RUNNER_COMPILED;
  out->handle = r;
  out->handle_size = 0;
  for (int i = 0; i < 3; i++) { out->grid[i] = (int)r->rk.launch.grid[i]; out->block[i] = (int)r->rk.launch.block[i]; }
  return 0;
}

int poly_hip_execute(PolyRunner *runner, void **args, int n_args) {
  if (!runner || !runner->handle) { log_err("execute", "runner has no handle"); return -1; }
  return runner_launch((HipRunner *)runner->handle, args, n_args);
}

int poly_hip_execute_static(PolyRunner *runner, void **args, int n_args) {
  if (!runner || !runner->handle) { log_err("execute_static", "runner has no handle"); return -1; }
  HipRunner *r = (HipRunner *)runner->handle;
  if (r->rk.scratch_bytes > (size_t)POLY_HIP_STATIC_SCRATCH_BYTES) {
    log_err("execute_static", "%s needs %zu bytes of scratch memory, the static array holds %u", r->name.c_str(),
            r->rk.scratch_bytes, (unsigned)POLY_HIP_STATIC_SCRATCH_BYTES);
    return -1;
  }
  void *scratch = static_scratch();
  if (!scratch) return -1;
  // Stage one writes every scratch element stage two reads, so what an earlier call left
  // in the array needs no clearing.
  return runner_launch(r, args, n_args, scratch);
}

void poly_hip_free_runner(PolyRunner *runner) {
  if (!runner || !runner->handle) return;
  runner_destroy((HipRunner *)runner->handle);
  runner->handle = nullptr;
}

static void *alloc_fn(size_t nbytes, void *dev_ctx) { (void)dev_ctx; return runtime_alloc(nbytes); }
static void free_fn(void *h, void *dev_ctx) { (void)dev_ctx; runtime_free(h); }
static int copy_in_fn(void *dst, const void *src, size_t n, void *dev_ctx) { (void)dev_ctx; return runtime_copy(dst, src, n, 0); }
static int copy_out_fn(void *dst, const void *src, size_t n, void *dev_ctx) { (void)dev_ctx; return runtime_copy(dst, src, n, 1); }
static int copy_between_fn(void *dst, const void *src, size_t n, void *dev_ctx) { (void)dev_ctx; return runtime_copy(dst, src, n, 2); }

static const PolyAllocator kHipAllocator = {alloc_fn, free_fn, copy_in_fn, copy_out_fn, copy_between_fn, nullptr};
const PolyAllocator *poly_hip_get_allocator(void) { return &kHipAllocator; }

static const PolyBackendDesc kHipBackend = {"hip", POLY_DEVICE_HIP, false, poly_hip_lower_item,
                                            poly_hip_execute, poly_hip_free_runner, poly_hip_get_allocator};
const PolyBackendDesc *poly_hip_backend_desc(void) { return &kHipBackend; }

// ── render-only entry points ──────────────────────────────────────────────

static char *dup_string(const std::string &s) {
  char *p = (char *)malloc(s.size() + 1);
  if (p) memcpy(p, s.c_str(), s.size() + 1);
  return p;
}

char *poly_hip_render(PolyUOp *scheduled_root, const char *fn_name, int flags, int *launch_out) {
  RenderedKernel rk;
  if (!scheduled_root || !render_root(scheduled_root, fn_name ? fn_name : "kernel", flags, &rk)) return nullptr;
  if (launch_out) {
    for (int i = 0; i < 3; i++) { launch_out[i] = (int)rk.launch.grid[i]; launch_out[3 + i] = (int)rk.launch.block[i]; }
    launch_out[6] = (int)rk.launch.lds_bytes;
  }
  std::string all = rk.source;
  for (const RenderedKernel::Guard &g : rk.guards) all += "\n// ---- guard ----\n" + g.source;
  if (!rk.fallback_source.empty()) all += "\n// ---- fallback ----\n" + rk.fallback_source;
  for (const RenderedKernel::Pre &pk : rk.pres)
    all += strf("\n// ---- first stage ---- grid=%u,%u block=%u scratch=%zu\n", pk.launch.grid[0], pk.launch.grid[1], pk.launch.block[0], rk.scratch_bytes) + pk.source;
  for (size_t i = 1; i < rk.variants.size(); i++) all += "\n// ---- variant " + rk.variants[i].label + "\n" + rk.variants[i].source;
  return dup_string(all);
}

char *poly_hip_describe(PolyUOp *scheduled_root, int flags) {
  RenderedKernel rk;
  if (!scheduled_root || !render_root(scheduled_root, "kernel", flags, &rk)) return nullptr;
  return dup_string(strf("%s: %s bytes=%.0f flops=%.0f grid=%u,%u,%u block=%u", kernel_class_name(rk.klass),
                         rk.strategy.c_str(), rk.bytes, rk.flops, rk.launch.grid[0], rk.launch.grid[1],
                         rk.launch.grid[2], rk.launch.block[0]));
}

int poly_hip_compile_check(const char *source) {
  if (!source) return -1;
  // A rendered bundle may hold several translation units (guard, fallback).
  std::string all(source);
  size_t pos = 0;
  while (pos < all.size()) {
    size_t next = all.find("\n// ---- ", pos);
    std::string unit = all.substr(pos, next == std::string::npos ? std::string::npos : next - pos);
    std::vector<char> code;
    std::string log;
    if (!compile_to_code_object(unit, &code, &log)) {
      log_err("compile_check", "hiprtc: %s", log.c_str());
      return -1;
    }
    if (next == std::string::npos) break;
    pos = all.find('\n', next + 1);
    if (pos == std::string::npos) break;
    pos++;
  }
  return 0;
}

void poly_hip_free_string(char *s) { free(s); }

int poly_hip_check_index_simplification(PolyUOp *scheduled_root, int samples) {
  KernelGraph g;
  if (!scheduled_root || !g.build(scheduled_root)) return -1;
  std::string bad;
  int n = g.check_lins(samples > 0 ? samples : 4096, &bad);
  if (n > 0) log_err("render_hip", "index simplification self-check: %d mismatches, first: %s", n, bad.c_str());
  return n;
}

}  // extern "C"
