// plan_hip: MI355X-native counterparts of poly_compile_schedule /
// poly_compiled_plan_run / poly_compiled_plan_free (src/exec_plan.c:801-1096).
//
// What differs from the reference plan, by design:
//   * intermediates live in ONE device arena; slots whose lifetimes (first
//     write .. last use in execution order) do not overlap share memory, so a
//     12-layer transformer keeps a few activations resident instead of all;
//   * nothing is zero-filled per run unless a slot's producer does not cover
//     it (the reference memsets every intermediate on every run,
//     src/exec_plan.c:946-963);
//   * kernels are enqueued on one stream with no per-kernel synchronisation and
//     no per-launch allocation (src/exec_plan.c:590-607 does both);
//   * the launch sequence is captured into a hipGraph and replayed while the
//     bound pointers and variable values repeat.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <memory>

#include "polygrad_hip.h"
#include "runtime_hip.h"

using namespace polyhip;

namespace {

struct GraphEntry {
  uint64_t key = 0;
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  uint64_t last_use = 0;
};

const char *const kFillSrc = R"HIP(
extern "C" __global__ void __launch_bounds__(256) poly_fill0(unsigned int* p, long long n_words) {
  long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  long long stride = (long long)gridDim.x * 256;
  for (; i < n_words; i += stride) p[i] = 0u;
}
)HIP";

}  // namespace

struct PolyHipPlan {
  const PolySchedule *sched = nullptr;
  std::vector<HipRunner *> runners;          // by item index
  std::vector<void *> slot_ptr;              // device pointer per slot (intermediates fixed)
  std::vector<size_t> slot_off;
  std::vector<char> slot_needs_zero;
  void *arena = nullptr;
  size_t arena_bytes = 0;
  std::vector<std::vector<void *>> kargs;    // per item: args array handed to runner_launch
  std::vector<std::vector<int>> var_vals;    // per item: storage for var ints
  std::vector<PolyVarBinding> merged;
  Program *fill = nullptr;
  bool use_graph = true;
  std::vector<GraphEntry> graphs;
  uint64_t tick = 0;
  ~PolyHipPlan() {
    for (GraphEntry &g : graphs) {
      if (g.exec) (void)hipGraphExecDestroy(g.exec);
      if (g.graph) (void)hipGraphDestroy(g.graph);
    }
    for (HipRunner *r : runners) runner_destroy(r);
    if (fill) program_destroy(fill);
    if (arena) runtime_free(arena);
  }
};

namespace {

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Does the producer of `slot` write every element?  Counts, over every STORE
// into the slot's PARAM, the product of the extents of the store's ranges when
// the store is ungated and its index is injective enough to be a full cover
// (affine with non-zero coefficient on every range).
bool slot_fully_written(const PolySchedule *s, int slot, const std::vector<KernelGraph> &graphs) {
  double covered = 0;
  for (int k = 0; k < s->n_items; k++) {
    const PolyExecItem &it = s->items[k];
    const KernelGraph &g = graphs[(size_t)k];
    for (const StoreInfo &st : g.stores) {
      int p = g.param_slot(st.param);
      if (p < 0 || p >= it.n_buf_slots || it.buf_slot_indices[p] != slot) continue;
      if (st.gate >= 0) continue;
      int li = g.n(g.n(st.index).src[1]).lin;
      if (li < 0) continue;
      double n = 1;
      bool ok = true;
      for (int r : st.ranges) {
        bool aff;
        int64_t c = g.lin_range_coef(g.lins[(size_t)li], r, &aff);
        if (!aff || c == 0 || g.ranges[(size_t)r].extent < 0) { ok = false; break; }
        n *= (double)g.ranges[(size_t)r].extent;
      }
      if (ok) covered += n;
    }
  }
  return covered >= (double)s->buf_slots[slot].numel;
}

int enqueue_all(PolyHipPlan *plan) {
  const PolySchedule *s = plan->sched;
  // zero-fill the few slots whose producers leave holes
  for (int i = 0; i < s->n_buf_slots; i++) {
    if (!plan->slot_needs_zero[(size_t)i]) continue;
    void *p = plan->slot_ptr[(size_t)i];
    long long words = (long long)(align_up((size_t)std::max<int64_t>(s->buf_slots[i].nbytes, 4), 4) / 4);
    void *args[2] = {&p, &words};
    LaunchSpec ls;
    ls.grid[0] = (unsigned)std::min<long long>((words + 255) / 256, 65536);
    if (program_launch(plan->fill, args, ls) != 0) return -1;
  }
  for (int step = 0; step < s->n_items; step++) {
    int k = s->exec_order[step];
    std::vector<void *> &a = plan->kargs[(size_t)k];
    if (runner_launch(plan->runners[(size_t)k], a.data(), (int)a.size()) != 0) {
      log_err("plan_run", "kernel %d failed to launch", k);
      return -1;
    }
  }
  return 0;
}

}  // namespace

extern "C" {

PolyHipPlan *poly_hip_compile_schedule(PolyCtx *ctx, const PolySchedule *s) {
  (void)ctx;
  if (!s) return nullptr;
  if (runtime_init() != 0) return nullptr;
  std::unique_ptr<PolyHipPlan> plan(new PolyHipPlan());
  plan->sched = s;
  static int plan_counter = 0;
  std::vector<KernelGraph> graphs((size_t)s->n_items);
  plan->runners.assign((size_t)s->n_items, nullptr);
  for (int k = 0; k < s->n_items; k++) {
    const PolyExecItem &it = s->items[k];
    if (it.kind != POLY_EXEC_COMPUTE) {
      log_err("compile_schedule", "non-COMPUTE item %d not supported", k);
      return nullptr;
    }
    std::string name = strf("hip%d_k%d", plan_counter, k);
    if (!graphs[(size_t)k].build(it.root)) {
      log_err("compile_schedule", "kernel %d: %s", k, graphs[(size_t)k].error.c_str());
      return nullptr;
    }
    HipRunner *r = runner_create(it.root, name.c_str(), 0);
    if (!r) {
      log_err("compile_schedule", "backend 'hip' failed for kernel %d", k);
      return nullptr;
    }
    plan->runners[(size_t)k] = r;
    if (r->rk.n_params != it.n_buf_slots || r->rk.n_vars != it.n_var_uops) {
      log_err("compile_schedule", "kernel %d: %d params / %d vars in the graph, %d / %d in the schedule", k,
              r->rk.n_params, r->rk.n_vars, it.n_buf_slots, it.n_var_uops);
      return nullptr;
    }
  }
  plan_counter++;

  // ── lifetimes of intermediates in execution order ──────────────────────
  const int ns = s->n_buf_slots;
  std::vector<int> first((size_t)ns, -1), last((size_t)ns, -1);
  for (int step = 0; step < s->n_items; step++) {
    const PolyExecItem &it = s->items[s->exec_order[step]];
    for (int i = 0; i < it.n_buf_slots; i++) {
      int sl = it.buf_slot_indices[i];
      if (sl < 0 || sl >= ns) { log_err("compile_schedule", "bad slot index %d", sl); return nullptr; }
      if (first[(size_t)sl] < 0) first[(size_t)sl] = step;
      last[(size_t)sl] = step;
    }
  }
  // ── place intermediates in one arena; overlapping lifetimes never share ──
  struct Placed { size_t off, size; int first, last; };
  std::vector<Placed> placed;
  std::vector<int> order;
  for (int i = 0; i < ns; i++) if (s->buf_slots[i].is_intermediate) order.push_back(i);
  const bool no_alias = getenv("POLY_HIP_NO_ALIAS") != nullptr;
  std::sort(order.begin(), order.end(), [&](int a, int b) {
    if (s->buf_slots[a].nbytes != s->buf_slots[b].nbytes) return s->buf_slots[a].nbytes > s->buf_slots[b].nbytes;
    return a < b;
  });
  plan->slot_off.assign((size_t)ns, 0);
  size_t total = 0;
  for (int sl : order) {
    size_t size = align_up((size_t)std::max<int64_t>(s->buf_slots[sl].nbytes, 4), 256);
    int f = first[(size_t)sl], l = last[(size_t)sl];
    if (f < 0) { f = 0; l = s->n_items; }
    if (no_alias) { f = 0; l = s->n_items; }
    // candidate offsets: 0 and the end of every conflicting block
    std::vector<Placed> conflicts;
    for (const Placed &p : placed)
      if (!(p.last < f || l < p.first)) conflicts.push_back(p);
    std::sort(conflicts.begin(), conflicts.end(), [](const Placed &a, const Placed &b) { return a.off < b.off; });
    size_t off = 0;
    for (const Placed &p : conflicts) {
      if (off + size <= p.off) break;
      off = std::max(off, p.off + p.size);
    }
    placed.push_back({off, size, f, l});
    plan->slot_off[(size_t)sl] = off;
    total = std::max(total, off + size);
  }
  plan->arena_bytes = total;
  if (total > 0) {
    plan->arena = runtime_alloc(total);
    if (!plan->arena) return nullptr;
  }
  plan->slot_ptr.assign((size_t)ns, nullptr);
  plan->slot_needs_zero.assign((size_t)ns, 0);
  bool any_zero = false;
  for (int sl : order) {
    plan->slot_ptr[(size_t)sl] = (char *)plan->arena + plan->slot_off[(size_t)sl];
    if (!slot_fully_written(s, sl, graphs)) { plan->slot_needs_zero[(size_t)sl] = 1; any_zero = true; }
  }
  if (any_zero) {
    plan->fill = program_create(kFillSrc, "poly_fill0");
    if (!plan->fill) return nullptr;
  }
  plan->kargs.resize((size_t)s->n_items);
  plan->var_vals.resize((size_t)s->n_items);
  for (int k = 0; k < s->n_items; k++) {
    plan->kargs[(size_t)k].assign((size_t)(s->items[k].n_buf_slots + s->items[k].n_var_uops), nullptr);
    plan->var_vals[(size_t)k].assign((size_t)s->items[k].n_var_uops, 0);
  }
  return plan.release();
}

static int bind_args(PolyHipPlan *plan, void **slot_data, int n_slots, const PolyVarBinding *vb, int nvb,
                     uint64_t *key_out) {
  const PolySchedule *s = plan->sched;
  uint64_t key = 1469598103934665603ull;
  for (int i = 0; i < s->n_buf_slots; i++) {
    if (s->buf_slots[i].is_intermediate) continue;
    plan->slot_ptr[(size_t)i] = (i < n_slots && slot_data) ? slot_data[i] : nullptr;
    key = fnv1a(&plan->slot_ptr[(size_t)i], sizeof(void *), key);
  }
  // default vars first, runtime overrides win (src/exec_plan.c:984-996)
  plan->merged.clear();
  for (int i = 0; i < s->n_default_vars; i++) plan->merged.push_back(s->default_vars[i]);
  for (int i = 0; i < nvb; i++) {
    bool found = false;
    for (PolyVarBinding &m : plan->merged)
      if (m.var == vb[i].var) { m.value = vb[i].value; found = true; break; }
    if (!found) plan->merged.push_back(vb[i]);
  }
  for (int k = 0; k < s->n_items; k++) {
    const PolyExecItem &it = s->items[k];
    std::vector<void *> &a = plan->kargs[(size_t)k];
    for (int i = 0; i < it.n_buf_slots; i++) {
      void *p = plan->slot_ptr[(size_t)it.buf_slot_indices[i]];
      if (!p) {
        log_err("plan_run", "missing data for param %d (slot %d) in kernel %d", i, it.buf_slot_indices[i], k);
        return -1;
      }
      a[(size_t)i] = p;
    }
    for (int v = 0; v < it.n_var_uops; v++) {
      bool found = false;
      for (const PolyVarBinding &m : plan->merged)
        if (m.var == it.var_uops[v]) { plan->var_vals[(size_t)k][(size_t)v] = m.value; found = true; break; }
      if (!found) { log_err("plan_run", "no binding for DEFINE_VAR in kernel %d", k); return -1; }
      a[(size_t)(it.n_buf_slots + v)] = &plan->var_vals[(size_t)k][(size_t)v];
      key = fnv1a(&plan->var_vals[(size_t)k][(size_t)v], sizeof(int), key);
    }
  }
  *key_out = key;
  return 0;
}

int poly_hip_plan_run(PolyHipPlan *plan, void **slot_data, int n_slots, const PolyVarBinding *vb, int nvb) {
  if (!plan || !plan->sched) return -1;
  uint64_t key = 0;
  if (bind_args(plan, slot_data, n_slots, vb, nvb, &key) != 0) return -1;
  hipStream_t stream = (hipStream_t)runtime_stream();
  if (!plan->use_graph || getenv("POLY_HIP_NO_GRAPH")) return enqueue_all(plan);
  plan->tick++;
  for (GraphEntry &g : plan->graphs)
    if (g.key == key && g.exec) {
      g.last_use = plan->tick;
      if (hipGraphLaunch(g.exec, stream) != hipSuccess) { log_err("plan_run", "hipGraphLaunch failed"); return -1; }
      return 0;
    }
  // First sight of this binding: capture the launch sequence, then replay it.
  GraphEntry ge;
  ge.key = key;
  ge.last_use = plan->tick;
  if (hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal) != hipSuccess) {
    log_err("plan_run", "hipStreamBeginCapture failed; running without a graph");
    plan->use_graph = false;
    return enqueue_all(plan);
  }
  int rc = enqueue_all(plan);
  hipError_t e = hipStreamEndCapture(stream, &ge.graph);
  if (rc != 0 || e != hipSuccess || !ge.graph) {
    if (ge.graph) (void)hipGraphDestroy(ge.graph);
    log_err("plan_run", "graph capture failed; running without a graph");
    plan->use_graph = false;
    return rc != 0 ? rc : enqueue_all(plan);
  }
  if (hipGraphInstantiate(&ge.exec, ge.graph, nullptr, nullptr, 0) != hipSuccess) {
    (void)hipGraphDestroy(ge.graph);
    log_err("plan_run", "hipGraphInstantiate failed; running without a graph");
    plan->use_graph = false;
    return enqueue_all(plan);
  }
  if (plan->graphs.size() >= 4) {
    size_t victim = 0;
    for (size_t i = 1; i < plan->graphs.size(); i++)
      if (plan->graphs[i].last_use < plan->graphs[victim].last_use) victim = i;
    (void)hipGraphExecDestroy(plan->graphs[victim].exec);
    (void)hipGraphDestroy(plan->graphs[victim].graph);
    plan->graphs.erase(plan->graphs.begin() + (long)victim);
  }
  plan->graphs.push_back(ge);
  if (hipGraphLaunch(ge.exec, stream) != hipSuccess) { log_err("plan_run", "hipGraphLaunch failed"); return -1; }
  return 0;
}

void poly_hip_plan_free(PolyHipPlan *plan) {
  if (!plan) return;
  runtime_sync();
  delete plan;
}

int poly_hip_plan_n_kernels(const PolyHipPlan *plan) { return plan ? (int)plan->runners.size() : -1; }

int poly_hip_plan_kernel_info(const PolyHipPlan *plan, int cap, int *klass, double *bytes, double *flops) {
  if (!plan) return -1;
  const PolySchedule *s = plan->sched;
  for (int step = 0; step < s->n_items && step < cap; step++) {
    const HipRunner *r = plan->runners[(size_t)s->exec_order[step]];
    if (klass) klass[step] = (int)r->rk.klass;
    if (bytes) bytes[step] = r->rk.bytes;
    if (flops) flops[step] = r->rk.flops;
  }
  return s->n_items;
}

int poly_hip_plan_profile(PolyHipPlan *plan, void **slot_data, int n_slots, float *ms_out, int cap) {
  if (!plan) return -1;
  uint64_t key;
  if (bind_args(plan, slot_data, n_slots, nullptr, 0, &key) != 0) return -1;
  const PolySchedule *s = plan->sched;
  hipStream_t stream = (hipStream_t)runtime_stream();
  std::vector<hipEvent_t> ev((size_t)s->n_items + 1);
  for (hipEvent_t &e : ev) if (hipEventCreate(&e) != hipSuccess) return -1;
  int rc = 0;
  (void)hipEventRecord(ev[0], stream);
  for (int step = 0; step < s->n_items && rc == 0; step++) {
    int k = s->exec_order[step];
    std::vector<void *> &a = plan->kargs[(size_t)k];
    rc = runner_launch(plan->runners[(size_t)k], a.data(), (int)a.size());
    (void)hipEventRecord(ev[(size_t)step + 1], stream);
  }
  (void)hipStreamSynchronize(stream);
  for (int step = 0; step < s->n_items && step < cap && rc == 0; step++)
    (void)hipEventElapsedTime(&ms_out[step], ev[(size_t)step], ev[(size_t)step + 1]);
  for (hipEvent_t &e : ev) (void)hipEventDestroy(e);
  return rc == 0 ? s->n_items : -1;
}

char *poly_hip_plan_kernel_desc(const PolyHipPlan *plan, int step) {
  if (!plan || step < 0 || step >= plan->sched->n_items) return nullptr;
  const HipRunner *r = plan->runners[(size_t)plan->sched->exec_order[step]];
  static const char *const kn[] = {"elementwise", "row-reduce", "thread-reduce", "matmul-mfma", "gather", "copy"};
  std::string d = strf("%s %s: %s grid=%u,%u,%u bytes=%.0f flops=%.0f", r->name.c_str(), kn[(int)r->rk.klass],
                       r->rk.strategy.c_str(), r->rk.launch.grid[0], r->rk.launch.grid[1], r->rk.launch.grid[2],
                       r->rk.bytes, r->rk.flops);
  char *p = (char *)malloc(d.size() + 1);
  if (p) memcpy(p, d.c_str(), d.size() + 1);
  return p;
}

void *poly_hip_plan_slot_ptr(const PolyHipPlan *plan, int slot) {
  if (!plan || slot < 0 || slot >= (int)plan->slot_ptr.size()) return nullptr;
  return plan->slot_ptr[(size_t)slot];
}

void poly_hip_plan_set_graph(PolyHipPlan *plan, int enabled) { if (plan) plan->use_graph = enabled != 0; }
size_t poly_hip_plan_workspace_bytes(const PolyHipPlan *plan) { return plan ? plan->arena_bytes : 0; }

}  // extern "C"
