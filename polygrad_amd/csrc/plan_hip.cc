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
//     bound pointers and variable values repeat; in the graph, small launches that are
//     chains of dependent steps run on a second stream beside the main sequence;
//   * kernel groups that fusion.cc recognises run as one launch and their
//     intermediates get no memory at all.
#include <hip/hip_runtime.h>
#include <unistd.h>

#include <algorithm>
#include <array>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>

#include "fusion.h"
#include "polygrad_hip.h"
#include "runtime_hip.h"

using namespace polyhip;

namespace {

// One instantiated graph of the plan's launch sequence, bound to one set of buffers and
// variable values (compared value by value, not by a hash of them).
struct GraphEntry {
  std::vector<uint64_t> bound;
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

// Reads one word of every 64 bytes of a buffer and drops it: what the launch leaves behind
// is the buffer in the memory-side cache.
const char *const kTouchSrc = R"HIP(
extern "C" __global__ void __launch_bounds__(256) poly_touch(const unsigned int* p, long long n_lines) {
  long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  const long long stride = (long long)gridDim.x * 256;
  unsigned int a = 0;
  for (; i < n_lines; i += stride) a ^= p[i * 16];
  asm volatile("" ::"v"(a));
}
)HIP";

}  // namespace

// One launch of the plan: a scheduled kernel, or a fused group of them.
struct Unit {
  HipRunner *runner = nullptr;
  int item = -1;                 // schedule item (also for a fused group: the item it runs in place of)
  std::vector<int> slots;        // buffer slot per kernel argument
  int n_vars = 0;                // DEFINE_VAR arguments of the kernel
  std::vector<const PolyUOp *> var_uops;   // which variable each of them is
  int n_items = 1;               // schedule items this launch stands for
  bool repeatable = false;       // writes no buffer it also reads: running it twice changes nothing
  std::vector<int> writes;       // slots the launch writes
};

struct PolyHipPlan {
  const PolySchedule *sched = nullptr;
  std::vector<Unit> units;                   // in execution order
  std::vector<void *> slot_ptr;              // device pointer per slot (intermediates fixed)
  std::vector<size_t> slot_off;
  std::vector<char> slot_needs_zero;
  std::vector<void *> vetted_slot;              // per external slot: the last pointer found to be device memory
  std::vector<std::vector<int>> fills_before;   // per unit: slots to clear right before it runs
  void *arena = nullptr;
  size_t arena_bytes = 0;
  void *scratch_pool = nullptr;              // shared by the two-stage kernels of the plan (they run one after the other)
  size_t scratch_bytes = 0;
  size_t kept_scratch_bytes = 0;            // scratch memory of first stages that later launches read
  std::vector<std::vector<void *>> kargs;    // per unit: args array handed to runner_launch
  std::vector<std::vector<int>> var_vals;    // per unit: storage for var ints
  std::vector<PolyVarBinding> merged;
  // Launches that a captured graph runs beside the main sequence, on further streams: small
  // launches whose time is a dependent chain, not throughput (the in-order adders of the
  // bf16 column sums: 1024 threads for 48 us each, 194 of them in a 24-layer training step).
  // on_side[u]: 0 = main sequence, k = side stream k - 1; waits[u]: launches on other streams
  // that u's buffers depend on (those that an earlier wait of u's stream does not already
  // cover); records[u]: someone waits for u.
  std::vector<char> on_side;
  std::vector<std::vector<int>> waits;
  std::vector<char> records;
  std::vector<hipEvent_t> events;            // per launch (those with records), then fork and one join per side stream
  bool forked = false;
  int n_side_streams = 0;
  void *side_scratch_pool[kSideStreams] = {nullptr, nullptr, nullptr};   // the two-stage kernels of a side stream share one
  Program *fill = nullptr;
  // Buffers that no launch of the plan writes (weights) and that a matrix product reads are
  // read once by a small launch shortly before the product: it then finds them in the
  // memory-side cache instead of waiting for HBM with the first tiles of every workgroup (a
  // product of 8192 x 3072 x 768 whose 4.7 MB of weights come from HBM takes 54 us, 43 us
  // after such a read, which itself takes 2-3 us).  touch_at[u]: slots to read right
  // before launch u.
  std::vector<std::vector<int>> touch_at;
  Program *touch = nullptr;
  bool use_graph = true;
  bool tuned = false;            // candidates of the tunable kernels have been timed (or there are none)
  // The launch sequence is captured once (`captured`, with the kernel node of every launch
  // in `launches`); a binding the plan has not seen gets a graph instantiated from it whose
  // kernel nodes receive the new argument values, not a capture of its own.
  hipGraph_t captured = nullptr;
  GraphLaunches launches;
  bool captured_forked = false;              // the capture put launches on side streams
  std::vector<GraphEntry> graphs;
  std::vector<uint64_t> bound_now;           // the current binding: external pointers, then variable values
  uint64_t tick = 0;
  long long n_captures = 0, n_rebinds = 0;   // (how often the sequence was captured / rebound by updating nodes)
  ~PolyHipPlan() {
    for (GraphEntry &g : graphs)
      if (g.exec) (void)hipGraphExecDestroy(g.exec);
    if (captured) (void)hipGraphDestroy(captured);
    for (Unit &u : units) runner_destroy(u.runner);
    if (fill) program_destroy(fill);
    if (touch) program_destroy(touch);
    if (arena) runtime_free(arena);
    if (scratch_pool) runtime_free(scratch_pool);
    for (void *p : side_scratch_pool) if (p) runtime_free(p);
    for (hipEvent_t e : events) if (e) (void)hipEventDestroy(e);
  }
};

namespace {

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Do the producers of `slot` write every element?  Every ungated STORE into the slot's
// PARAM whose index is affine in its ranges with strides that nest (sorted by stride,
// each stride is the previous stride times the previous extent, the smallest is 1)
// writes exactly one contiguous interval of elements; the slot is covered when the union
// of those intervals is [0, numel).  Gated stores, strided stores and indices with
// divisions count for nothing: the answer errs towards "needs a fill".
bool slot_fully_written(const PolySchedule *s, int slot, const std::vector<KernelGraph> &graphs) {
  std::vector<std::pair<int64_t, int64_t>> spans;    // [first, end)
  for (int k = 0; k < s->n_items; k++) {
    const PolyExecItem &it = s->items[k];
    const KernelGraph &g = graphs[(size_t)k];
    for (const StoreInfo &st : g.stores) {
      int p = g.param_slot(st.param);
      if (p < 0 || p >= it.n_buf_slots || it.buf_slot_indices[p] != slot) continue;
      if (st.gate >= 0) continue;
      int li = g.n(g.n(st.index).src[1]).lin;
      if (li < 0) continue;
      const Lin &l = g.lins[(size_t)li];
      if (!g.lin_is_affine(l)) continue;
      std::vector<std::pair<int64_t, int64_t>> dims;   // (|stride|, extent)
      int64_t base = l.c0;
      bool ok = true;
      uint64_t seen = 0;
      for (int r : st.ranges) {
        bool aff;
        int64_t c = g.lin_range_coef(l, r, &aff);
        const int64_t ext = g.ranges[(size_t)r].extent;
        if (!aff || ext <= 0 || r >= 64) { ok = false; break; }
        seen |= 1ull << r;
        if (c == 0 || ext == 1) continue;              // rewrites the same elements / a single value
        if (c < 0) { base += c * (ext - 1); c = -c; }  // walks downwards: the interval starts at its last step
        dims.push_back({c, ext});
      }
      // anything else the index depends on (a variable, a range of an enclosing loop)
      if (ok && (g.lin_deps(l) & ~seen) != 0) ok = false;
      if (ok) for (const Term &t : l.terms) if (g.atoms[(size_t)t.atom].kind != Atom::RANGE) ok = false;
      if (!ok) continue;
      std::sort(dims.begin(), dims.end());
      int64_t expect = 1;
      for (const auto &d : dims) {
        if (d.first != expect) { ok = false; break; }
        expect *= d.second;
      }
      if (ok) spans.push_back({base, base + expect});
    }
  }
  std::sort(spans.begin(), spans.end());
  int64_t covered_to = 0;
  for (const auto &sp : spans) {
    if (sp.first > covered_to) break;
    covered_to = std::max(covered_to, sp.second);
  }
  return covered_to >= s->buf_slots[slot].numel;
}

// The fill kernel over one slot (a slot whose producers leave holes reads as zero there,
// as every intermediate does in the reference, src/exec_plan.c:946-963).
int launch_fill(PolyHipPlan *plan, int slot) {
  const PolySchedule *s = plan->sched;
  void *p = plan->slot_ptr[(size_t)slot];
  long long words = (long long)(align_up((size_t)std::max<int64_t>(s->buf_slots[slot].nbytes, 4), 4) / 4);
  void *args[2] = {&p, &words};
  LaunchSpec ls;
  ls.grid[0] = (unsigned)std::min<long long>((words + 255) / 256, 65536);
  return program_launch(plan->fill, args, ls);
}

// Launches unit `u` after the fills that belong in front of it.  A slot shares its bytes
// with intermediates that die before its first use, so it can only be cleared then.
// The touches that belong in front of launch `u`, as launches of the main sequence.  (On a
// stream of their own, beside the launch before the product, they cost more than they
// saved: every edge between two streams of a captured graph costs a few microseconds, and
// the attention kernel ran 7 us longer with a touch beside it.)
void launch_touches(PolyHipPlan *plan, size_t u) {
  if (u >= plan->touch_at.size() || plan->touch_at[u].empty() || !plan->touch) return;
  for (int slot : plan->touch_at[u]) {
    void *p = plan->slot_ptr[(size_t)slot];
    long long lines = (long long)(plan->sched->buf_slots[slot].nbytes / 64);
    if (!p || lines <= 0) continue;
    void *args[2] = {&p, &lines};
    LaunchSpec ls;
    ls.grid[0] = (unsigned)std::min<long long>((lines + 255) / 256, 2048);
    (void)program_launch(plan->touch, args, ls);
  }
}

int launch_unit(PolyHipPlan *plan, size_t u) {
  launch_touches(plan, u);
  for (int slot : plan->fills_before[u])
    if (launch_fill(plan, slot) != 0) return -1;
  std::vector<void *> &a = plan->kargs[u];
  return runner_launch(plan->units[u].runner, a.data(), (int)a.size());
}

int enqueue_all(PolyHipPlan *plan) {
  int rc = 0;
  for (size_t u = 0; u < plan->units.size() && rc == 0; u++) {
    if (launch_unit(plan, u) != 0) {
      log_err("plan_run", "kernel %d failed to launch", plan->units[u].item);
      rc = -1;
    }
  }
  return rc;
}

// The same launches under stream capture, with those marked on_side going to the side
// streams: each joins the capture by waiting for an event recorded at the start of the main
// sequence, every dependence between two streams is an event recorded behind the producer
// and waited for in front of the consumer (edges of the graph), and the main stream waits
// for the last launch of every side stream before the capture ends.
int enqueue_captured(PolyHipPlan *plan) {
  hipStream_t main_s = (hipStream_t)runtime_stream();
  hipStream_t side_s[kSideStreams];
  const int ns = plan->n_side_streams;
  for (int k = 0; k < ns; k++) {
    side_s[k] = (hipStream_t)runtime_side_stream(k);
    if (!side_s[k]) return enqueue_all(plan);
  }
  const size_t n = plan->units.size();
  if (plan->events.size() != n + 1 + kSideStreams) plan->events.assign(n + 1 + kSideStreams, nullptr);
  auto event = [&](size_t i) -> hipEvent_t {
    if (!plan->events[i] && hipEventCreateWithFlags(&plan->events[i], hipEventDisableTiming) != hipSuccess) plan->events[i] = nullptr;
    return plan->events[i];
  };
  int rc = 0;
  hipEvent_t fork = event(n);
  if (!fork || hipEventRecord(fork, main_s) != hipSuccess) rc = -1;
  int joined = 0;       // side streams that are part of the capture
  for (; joined < ns && rc == 0; joined++)
    if (hipStreamWaitEvent(side_s[joined], fork, 0) != hipSuccess) { rc = -1; break; }
  for (size_t u = 0; u < n && rc == 0; u++) {
    hipStream_t st = plan->on_side[u] ? side_s[plan->on_side[u] - 1] : main_s;
    for (int w : plan->waits[u]) {
      hipEvent_t e = event((size_t)w);
      if (!e || hipStreamWaitEvent(st, e, 0) != hipSuccess) { rc = -1; break; }
    }
    if (rc != 0) break;
    runtime_launch_on(plan->on_side[u] ? (void *)st : nullptr);
    if (launch_unit(plan, u) != 0) {
      log_err("plan_run", "kernel %d failed to launch", plan->units[u].item);
      rc = -1;
      break;
    }
    if (plan->records[u]) {
      hipEvent_t e = event(u);
      if (!e || hipEventRecord(e, st) != hipSuccess) { rc = -1; break; }
    }
  }
  runtime_launch_on(nullptr);
  // (the side streams rejoin whatever happened, or the capture cannot end)
  for (int k = 0; k < joined; k++) {
    hipEvent_t join = event(n + 1 + (size_t)k);
    if (!join || hipEventRecord(join, side_s[k]) != hipSuccess || hipStreamWaitEvent(main_s, join, 0) != hipSuccess) rc = -1;
  }
  return rc;
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
  for (int k = 0; k < s->n_items; k++) {
    const PolyExecItem &it = s->items[k];
    if (it.kind != POLY_EXEC_COMPUTE) {
      log_err("compile_schedule", "non-COMPUTE item %d not supported", k);
      return nullptr;
    }
    if (!graphs[(size_t)k].build(it.root)) {
      log_err("compile_schedule", "kernel %d: %s", k, graphs[(size_t)k].error.c_str());
      return nullptr;
    }
  }
  // kernel groups that run as one launch
  std::vector<FusedGroup> groups;
  find_fused_groups(s, graphs, &groups);
  std::vector<int> group_of((size_t)s->n_items, -1);
  std::vector<char> internal((size_t)s->n_buf_slots, 0);
  for (size_t gi = 0; gi < groups.size(); gi++) {
    for (int it : groups[gi].items) group_of[(size_t)it] = (int)gi;
    for (int sl : groups[gi].internal_slots) internal[(size_t)sl] = 1;
  }
  for (int step = 0; step < s->n_items; step++) {
    const int k = s->exec_order[step];
    const PolyExecItem &it = s->items[k];
    std::string name = strf("hip%d_k%d", plan_counter, k);
    Unit u;
    u.item = k;
    if (group_of[(size_t)k] >= 0) {
      FusedGroup &fg = groups[(size_t)group_of[(size_t)k]];
      if (fg.launch_item != k) continue;   // runs as part of the group, later
      u.runner = runner_from_rendered(fg.rk, name.c_str(), false);
      u.slots = fg.arg_slots;
      u.n_items = (int)fg.items.size();
    } else {
      {
        // (which of the kernel's buffers are inputs of the plan that nothing in it writes)
        uint64_t mask = 0;
        for (int p = 0; p < it.n_buf_slots && p < 64; p++) {
          const int sl = it.buf_slot_indices[p];
          bool written = s->buf_slots[sl].is_intermediate;
          for (int k2 = 0; k2 < s->n_items && !written; k2++) {
            const PolyExecItem &o = s->items[k2];
            const KernelGraph &g2 = graphs[(size_t)k2];
            for (size_t q = 0; q < g2.params.size() && (int)q < o.n_buf_slots; q++)
              if (o.buf_slot_indices[q] == sl && g2.params[q].written) written = true;
          }
          if (!written) mask |= (uint64_t)1 << p;
        }
        matmul_hint_input_params(mask);
        matmul_hint_param_kinds(matmul_param_kinds_of(s, graphs, k, {}));
        u.runner = runner_create(it.root, name.c_str(), 0);
        matmul_hint_input_params(0);
        matmul_hint_param_kinds({});
      }
      // (a kernel may use fewer variables than the schedule lists for it: a buffer sized by
      // a variable that the kernel itself walks over its full allocation)
      if (u.runner && (u.runner->rk.n_params != it.n_buf_slots || u.runner->rk.n_vars > it.n_var_uops)) {
        log_err("compile_schedule", "kernel %d: %d params / %d vars in the graph, %d / %d in the schedule", k,
                u.runner->rk.n_params, u.runner->rk.n_vars, it.n_buf_slots, it.n_var_uops);
        runner_destroy(u.runner);
        return nullptr;
      }
      u.slots.assign(it.buf_slot_indices, it.buf_slot_indices + it.n_buf_slots);
      u.n_vars = u.runner ? u.runner->rk.n_vars : 0;
      if (u.runner) for (const void *v : u.runner->rk.var_uops) u.var_uops.push_back((const PolyUOp *)v);
    }
    if (!u.runner) {
      log_err("compile_schedule", "backend 'hip' failed for kernel %d", k);
      return nullptr;
    }
    // which buffers the launch writes and which it reads (buffers internal to a group are
    // neither); tuning may only repeat a launch whose two sets are disjoint
    {
      std::vector<int> members;
      if (group_of[(size_t)k] >= 0) members = groups[(size_t)group_of[(size_t)k]].items;
      else members.push_back(k);
      std::vector<char> wr((size_t)s->n_buf_slots, 0), rd((size_t)s->n_buf_slots, 0);
      for (int m : members) {
        const PolyExecItem &mi = s->items[m];
        const KernelGraph &g = graphs[(size_t)m];
        for (size_t p = 0; p < g.params.size() && (int)p < mi.n_buf_slots; p++) {
          const int sl = mi.buf_slot_indices[p];
          if (sl < 0 || sl >= s->n_buf_slots || internal[(size_t)sl]) continue;
          if (g.params[p].written) wr[(size_t)sl] = 1;
          if (g.params[p].read) rd[(size_t)sl] = 1;
        }
      }
      u.repeatable = true;
      for (int sl = 0; sl < s->n_buf_slots; sl++) {
        if (wr[(size_t)sl] && rd[(size_t)sl]) u.repeatable = false;
        if (wr[(size_t)sl]) u.writes.push_back(sl);
      }
    }
    plan->units.push_back(u);
  }
  plan_counter++;

  const int n_units = (int)plan->units.size();
  // Which launches may run beside the main sequence (what orders the two streams follows
  // further down, once the intermediates have their places).
  plan->on_side.assign((size_t)n_units, 0);
  plan->waits.assign((size_t)n_units, std::vector<int>());
  plan->records.assign((size_t)n_units, 0);
  // (chain_of: which seed a side launch follows; the chains are dealt to the side streams in
  // turn once it is known how many streams pay, further down)
  std::vector<int> chain_of((size_t)n_units, -1);
  if (!getenv("POLY_HIP_NO_SIDE_STREAM") && n_units > 1) {
    auto threads_of = [](const LaunchSpec &l) {
      return (uint64_t)l.grid[0] * l.grid[1] * l.grid[2] * l.block[0] * l.block[1] * l.block[2];
    };
    // The seeds are the small thread reductions (each is one dependent chain on a handful of
    // waves: several run side by side); a small launch of any kind that reads what a side
    // launch left (the cast of a column sum, the optimizer update of a bias) follows its
    // producer on the same stream, so that the main sequence does not wait for the chain one
    // step later.
    std::vector<int> side_wrote((size_t)s->n_buf_slots, 0);     // the chain (1-based) that the slot's current contents come from
    int next = 0;
    for (int ui = 0; ui < n_units; ui++) {
      const Unit &u = plan->units[(size_t)ui];
      const HipRunner *r = u.runner;
      // (several column sums as one launch are still a chain: up to 65 536 threads there)
      const uint64_t most = r->rk.klass == KernelClass::THREAD_REDUCE ? 65536 : 16384;
      bool small = threads_of(r->rk.launch) <= most && r->guards.empty() && r->rk.variants.size() < 2 && r->rk.pres_key.empty() && r->rk.scratch_of_item < 0;
      for (const RenderedKernel::Pre &pk : r->rk.pres) small = small && (r->rk.klass == KernelClass::THREAD_REDUCE || threads_of(pk.launch) <= 16384);
      int follows = 0;
      for (int sl : u.slots) if (!follows) follows = side_wrote[(size_t)sl];
      int side = 0;
      if (small && follows) side = follows;
      else if (small && r->rk.klass == KernelClass::THREAD_REDUCE) side = 1 + next++;
      if (side) { plan->on_side[(size_t)ui] = 1; chain_of[(size_t)ui] = side - 1; plan->forked = true; }
      for (int sl : u.writes) side_wrote[(size_t)sl] = side;
    }
    // (a plan that is mostly such launches is one chain of small steps: nothing to run beside)
    int n_side = 0;
    for (int ui = 0; ui < n_units; ui++) n_side += plan->on_side[(size_t)ui] != 0;
    if (2 * n_side > n_units) { plan->on_side.assign((size_t)n_units, 0); plan->forked = false; }
  }
  // ── lifetimes of intermediates in execution order ──────────────────────
  const int ns = s->n_buf_slots;
  std::vector<int> first((size_t)ns, -1), last((size_t)ns, -1);
  for (int step = 0; step < n_units; step++) {
    for (int sl : plan->units[(size_t)step].slots) {
      if (sl < 0 || sl >= ns) { log_err("compile_schedule", "bad slot index %d", sl); return nullptr; }
      if (first[(size_t)sl] < 0) first[(size_t)sl] = step;
      last[(size_t)sl] = step;
    }
  }
  // What a side launch reads or writes keeps its place to the end of the sequence: the main
  // sequence runs on meanwhile, and a later launch given the same bytes would have to wait
  // for the side stream.  A wait by the main sequence in the middle of the graph costs far
  // more than the wait itself (one such wait made the 24-layer training step 2 ms slower),
  // the memory little (the buffers are the terms of the column sums, alive up to their
  // adder anyway, and the sums).  POLY_HIP_SIDE_KEEP=n releases buffers above 64 KB n
  // launches after their side launch instead.
  if (plan->forked) {
    int keep_for = n_units;
    if (const char *e = measurement_env("POLY_HIP_SIDE_KEEP")) keep_for = std::max(0, atoi(e));
    for (int step = 0; step < n_units; step++) {
      if (!plan->on_side[(size_t)step]) continue;
      for (int sl : plan->units[(size_t)step].slots) {
        if (!s->buf_slots[sl].is_intermediate) continue;
        const int keep = s->buf_slots[sl].nbytes <= 65536 ? n_units : std::min(n_units, step + keep_for);
        last[(size_t)sl] = std::max(last[(size_t)sl], keep);
      }
    }
  }
  // ── place intermediates in one arena; overlapping lifetimes never share ──
  struct Placed { size_t off, size; int first, last; };
  std::vector<Placed> placed;
  std::vector<int> order;
  for (int i = 0; i < ns; i++) if (s->buf_slots[i].is_intermediate && !internal[(size_t)i]) order.push_back(i);
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
    if (f < 0) { f = 0; l = n_units; }
    if (no_alias) { f = 0; l = n_units; }
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
  plan->fills_before.assign((size_t)n_units, std::vector<int>());
  bool any_zero = false;
  for (int sl : order) {
    plan->slot_ptr[(size_t)sl] = (char *)plan->arena + plan->slot_off[(size_t)sl];
    if (first[(size_t)sl] < 0 || slot_fully_written(s, sl, graphs)) continue;
    plan->slot_needs_zero[(size_t)sl] = 1;
    plan->fills_before[(size_t)first[(size_t)sl]].push_back(sl);
    any_zero = true;
    if (getenv("POLY_HIP_DEBUG"))
      fprintf(stderr, "polygrad: compile_schedule: slot %d (%lld bytes) is not fully written by its producers: cleared before launch %d\n",
              sl, (long long)s->buf_slots[sl].nbytes, first[(size_t)sl]);
  }
  if (any_zero) {
    plan->fill = program_create(kFillSrc, "poly_fill0");
    if (!plan->fill) return nullptr;
  }
  // First stages whose result depends only on buffers that nothing writes in between run
  // once: the first launch of such a family keeps its scratch memory to itself, the later
  // ones read it and skip their first stages.
  std::vector<char> keeps_scratch((size_t)n_units, 0);
  // Launches that leave values in the scratch memory of a later launch (a product's block
  // maxima for the attention kernel that reads its keys): writer_for[reader] = writer.
  std::vector<int> writer_for((size_t)n_units, -1);
  for (int ui = 0; ui < n_units; ui++) {
    const RenderedKernel &rk = plan->units[(size_t)ui].runner->rk;
    if (rk.scratch_of_item < 0) continue;
    int reader = -1;
    for (int r = ui + 1; r < n_units && reader < 0; r++)
      if (plan->units[(size_t)r].item == rk.scratch_of_item) reader = r;
    if (reader < 0 || plan->units[(size_t)reader].runner->rk.scratch_bytes < rk.scratch_offset + rk.scratch_bytes || plan->on_side[(size_t)ui] ||
        plan->on_side[(size_t)reader]) {
      log_err("compile_schedule", "launch %d leaves values for the launch of kernel %d, which is not a later launch of the main sequence with room for them", ui,
              rk.scratch_of_item);
      return nullptr;
    }
    writer_for[(size_t)reader] = ui;
  }
  if (!getenv("POLY_HIP_NO_SHARED_FIRST_STAGE")) {
    std::map<std::pair<std::string, std::vector<int>>, int> leader_of;
    std::map<std::pair<std::string, std::vector<int>>, int> last_member;      // the latest launch that reads a family's scratch memory
    for (int ui = 0; ui < n_units; ui++) {
      HipRunner *r = plan->units[(size_t)ui].runner;
      if (r->rk.pres_key.empty() || r->pres.empty()) continue;
      std::vector<int> read_slots;
      bool known = true;
      for (int a : r->rk.pre_reads) {
        if (a < 0 || a >= (int)plan->units[(size_t)ui].slots.size()) { known = false; break; }
        read_slots.push_back(plan->units[(size_t)ui].slots[(size_t)a]);
      }
      if (!known) continue;
      const auto key = std::make_pair(r->rk.pres_key, read_slots);
      auto it = leader_of.find(key);
      bool reuse = it != leader_of.end();
      for (int w = reuse ? it->second : ui; reuse && w < ui; w++)
        for (int sl : plan->units[(size_t)w].writes)
          if (std::find(read_slots.begin(), read_slots.end(), sl) != read_slots.end()) reuse = false;
      // (values left by another launch arrive after the family's last reader is done, or this
      // launch keeps scratch memory of its own)
      if (reuse && writer_for[(size_t)ui] >= 0 && writer_for[(size_t)ui] < last_member[key]) reuse = false;
      if (reuse && plan->units[(size_t)it->second].runner->rk.scratch_bytes < r->rk.scratch_bytes) reuse = false;
      last_member[key] = ui;
      if (!reuse) { leader_of[key] = ui; continue; }
      HipRunner *lead = plan->units[(size_t)it->second].runner;
      if (runner_ensure_scratch(lead) != 0) return nullptr;
      runner_share_scratch(r, lead->scratch);
      r->skip_pres = true;
      if (!keeps_scratch[(size_t)it->second]) plan->kept_scratch_bytes += lead->rk.scratch_bytes;
      keeps_scratch[(size_t)it->second] = keeps_scratch[(size_t)ui] = 1;
      if (getenv("POLY_HIP_DEBUG"))
        fprintf(stderr, "polygrad: compile_schedule: launch %d reads what the first stage of launch %d leaves\n", ui, it->second);
    }
  }
  // (the writers get their readers' scratch memory, which starts as NaN bounds)
  for (int ri = 0; ri < n_units; ri++) {
    const int wi = writer_for[(size_t)ri];
    if (wi < 0) continue;
    HipRunner *reader = plan->units[(size_t)ri].runner, *writer = plan->units[(size_t)wi].runner;
    if (!reader->scratch) {
      if (runner_ensure_scratch(reader) != 0) return nullptr;
      plan->kept_scratch_bytes += reader->rk.scratch_bytes;
      keeps_scratch[(size_t)ri] = 1;
    }
    keeps_scratch[(size_t)wi] = 1;
    void *at = (char *)reader->scratch + writer->rk.scratch_offset;
    if (runtime_memset(at, 0xff, writer->rk.scratch_bytes) != 0) return nullptr;
    runner_share_scratch(writer, at);
  }
  // What orders the two streams.
  if (plan->forked) {
    // what a launch touches, as byte ranges: intermediates by their place in the arena (two
    // slots that share bytes are one resource), every other slot as a range of its own
    struct Span { uint64_t lo, hi; bool w; };
    std::vector<std::vector<Span>> spans((size_t)n_units);
    for (int ui = 0; ui < n_units; ui++) {
      const Unit &u = plan->units[(size_t)ui];
      for (int sl : u.slots) {
        const bool in_arena = s->buf_slots[sl].is_intermediate && !internal[(size_t)sl];
        const uint64_t lo = in_arena ? (uint64_t)plan->slot_off[(size_t)sl] : ((uint64_t)(sl + 1) << 44);
        const uint64_t size = (uint64_t)std::max<int64_t>(s->buf_slots[sl].nbytes, 4);
        bool w = std::find(u.writes.begin(), u.writes.end(), sl) != u.writes.end();
        for (int f : plan->fills_before[(size_t)ui]) w = w || f == sl;
        spans[(size_t)ui].push_back({lo, lo + size, w});
      }
    }
    auto conflict = [&](int a, int b) {
      for (const Span &x : spans[(size_t)a])
        for (const Span &y : spans[(size_t)b])
          if ((x.w || y.w) && x.lo < y.hi && y.lo < x.hi) return true;
      return false;
    };
    // A wait between the streams costs a few microseconds of its own: worth it when the
    // side launches run for long stretches without one (a handful of waits for 388 launches
    // in the 24-layer training step), not when every other side launch needs one (an MLP
    // step of 22 launches came out 13 % slower on two streams).  The most side streams
    // whose waits stay under one for eight side launches are taken.
    int n_on_side = 0, n_waits = 0, n_main_waits = 0;
    for (int i = 0; i < n_units; i++) n_on_side += plan->on_side[(size_t)i] != 0;
    // (two by default: on three the 24-layer step came out 1.6-3 ms slower than on two, with
    // four hardware queues for the process and with eight alike -- the chains slow each
    // other down, an adder that takes 48 us alone takes up to 110 us beside others)
    int max_streams = 2;
    if (const char *e = getenv("POLY_HIP_SIDE_STREAMS")) max_streams = std::max(1, std::min(kSideStreams, atoi(e)));
    for (int n_streams = max_streams; n_streams >= 1; n_streams--) {
      plan->n_side_streams = 0;
      for (int i = 0; i < n_units; i++) {
        plan->on_side[(size_t)i] = chain_of[(size_t)i] < 0 ? 0 : (char)(1 + chain_of[(size_t)i] % n_streams);
        plan->n_side_streams = std::max(plan->n_side_streams, (int)plan->on_side[(size_t)i]);
      }
      plan->waits.assign((size_t)n_units, std::vector<int>());
      plan->records.assign((size_t)n_units, 0);
      // synced[a][b]: the latest launch of stream b that stream a has waited for
      int synced[kSideStreams + 1][kSideStreams + 1];
      for (auto &row : synced) for (int &v : row) v = -1;
      n_waits = n_main_waits = 0;
      for (int i = 0; i < n_units; i++) {
        const int me = plan->on_side[(size_t)i];
        for (int other = 0; other <= plan->n_side_streams; other++) {
          if (other == me) continue;
          for (int j = i - 1; j > synced[me][other]; j--) {
            if (plan->on_side[(size_t)j] != other || !conflict(i, j)) continue;
            plan->waits[(size_t)i].push_back(j);
            plan->records[(size_t)j] = 1;
            synced[me][other] = j;
            n_waits++;
            n_main_waits += me == 0;
            break;
          }
        }
      }
      if (8 * n_main_waits <= n_on_side) break;
      if (getenv("POLY_HIP_DEBUG"))
        fprintf(stderr, "polygrad: compile_schedule: the main sequence would wait %d times for %d side launches on %d side streams: too many\n", n_main_waits, n_on_side, n_streams);
      if (n_streams == 1) {   // everything stays on one stream
        plan->on_side.assign((size_t)n_units, 0);
        plan->waits.assign((size_t)n_units, std::vector<int>());
        plan->records.assign((size_t)n_units, 0);
        plan->n_side_streams = 0;
        plan->forked = false;
      }
    }
    if (plan->forked) {
      const bool debug = getenv("POLY_HIP_DEBUG") != nullptr;
      if (debug) {
        fprintf(stderr, "polygrad: compile_schedule: %d of %d launches on %d side streams, %d waits between the streams, %d of them by the main sequence\n",
                n_on_side, n_units, plan->n_side_streams, n_waits, n_main_waits);
        for (int i = 0; i < n_units; i++)
          for (int w : plan->waits[(size_t)i])
            if (plan->on_side[(size_t)i] == 0 || n_waits <= 16) fprintf(stderr, "polygrad: compile_schedule: launch %d (stream %d) waits for launch %d (stream %d)\n", i, plan->on_side[(size_t)i], w,
                    plan->on_side[(size_t)w]);
      }
      // Every pair of launches on different streams that touch the same bytes, one of them
      // writing, must be ordered by the waits: checked here from scratch, pair by pair,
      // whenever a plan is forked (cheap next to compiling its kernels).  A plan that fails
      // runs on one stream.
      // seen[i][b]: latest launch of stream b known to be over when i starts
      std::vector<std::array<int, kSideStreams + 1>> seen((size_t)n_units);
      int last_on[kSideStreams + 1];
      for (int &v : last_on) v = -1;
      long long unordered = 0, pairs = 0;
      for (int i = 0; i < n_units; i++) {
        const int me = plan->on_side[(size_t)i];
        for (int b = 0; b <= kSideStreams; b++) seen[(size_t)i][(size_t)b] = last_on[me] >= 0 ? seen[(size_t)last_on[me]][(size_t)b] : -1;
        for (int w : plan->waits[(size_t)i]) {
          int &v = seen[(size_t)i][(size_t)plan->on_side[(size_t)w]];
          v = std::max(v, w);
        }
        last_on[me] = i;
        for (int j = 0; j < i; j++) {
          const int sj = plan->on_side[(size_t)j];
          if (sj != me && conflict(i, j)) { pairs++; if (j > seen[(size_t)i][(size_t)sj]) unordered++; }
        }
      }
      if (debug) fprintf(stderr, "polygrad: compile_schedule: %lld pairs of launches across the streams share bytes, %lld of them unordered\n", pairs, unordered);
      if (unordered != 0) {
        log_err("compile_schedule", "%lld pairs of launches on different streams share bytes without an order between them: everything stays on one stream", unordered);
        plan->on_side.assign((size_t)n_units, 0);
        plan->waits.assign((size_t)n_units, std::vector<int>());
        plan->records.assign((size_t)n_units, 0);
        plan->n_side_streams = 0;
        plan->forked = false;
      }
    }
  }
  // one scratch pool for all other two-stage kernels of a stream: the largest need
  {
    int users = 0, side_users[kSideStreams] = {0, 0, 0};
    size_t side_bytes[kSideStreams] = {0, 0, 0};
    for (int ui = 0; ui < n_units; ui++) {
      const Unit &u = plan->units[(size_t)ui];
      if (u.runner->rk.scratch_bytes == 0 || keeps_scratch[(size_t)ui]) continue;
      const int st = plan->on_side[(size_t)ui];
      if (st) { side_users[st - 1]++; side_bytes[st - 1] = std::max(side_bytes[st - 1], u.runner->rk.scratch_bytes); }
      else { users++; plan->scratch_bytes = std::max(plan->scratch_bytes, u.runner->rk.scratch_bytes); }
    }
    if (users > 1) {
      plan->scratch_pool = runtime_alloc(plan->scratch_bytes);
      if (!plan->scratch_pool) return nullptr;
      for (int ui = 0; ui < n_units; ui++)
        if (!keeps_scratch[(size_t)ui] && !plan->on_side[(size_t)ui]) runner_share_scratch(plan->units[(size_t)ui].runner, plan->scratch_pool);
    }
    for (int k = 0; k < kSideStreams; k++) {
      if (side_users[k] > 1) {
        plan->side_scratch_pool[k] = runtime_alloc(side_bytes[k]);
        if (!plan->side_scratch_pool[k]) return nullptr;
        for (int ui = 0; ui < n_units; ui++)
          if (!keeps_scratch[(size_t)ui] && plan->on_side[(size_t)ui] == k + 1) runner_share_scratch(plan->units[(size_t)ui].runner, plan->side_scratch_pool[k]);
      }
      plan->kept_scratch_bytes += side_bytes[k];
    }
    // a lone user owns its scratch memory; it must exist before the launches are captured
    for (Unit &u : plan->units) if (runner_ensure_scratch(u.runner) != 0) return nullptr;
  }
  // Which buffers are read ahead of which launch: the inputs of a matrix product that no
  // launch of the plan writes (the weights), from 128 KB up, `lead` launches ahead of it,
  // and not again while an earlier touch is recent.
  plan->touch_at.assign((size_t)n_units, std::vector<int>());
  if (!getenv("POLY_HIP_NO_PREFETCH")) {
    int lead = 1;
    if (const char *e = measurement_env("POLY_HIP_PREFETCH_LEAD")) lead = std::max(0, atoi(e));
    int64_t most = 128ll << 20;
    if (const char *e = measurement_env("POLY_HIP_PREFETCH_MAX_MB")) most = (int64_t)std::max(0, atoi(e)) << 20;
    std::vector<char> written((size_t)ns, 0);
    for (const Unit &u : plan->units) for (int sl : u.writes) written[(size_t)sl] = 1;
    std::vector<int> touched_for((size_t)ns, -1000);
    bool any = false;
    for (int t = 0; t < n_units; t++) {
      const Unit &u = plan->units[(size_t)t];
      if (u.runner->rk.klass != KernelClass::MATMUL_MFMA || plan->on_side[(size_t)t] || u.runner->rk.reads_b_ahead) continue;
      for (int sl : u.slots) {
        const PolyScheduleBufSlot &b = s->buf_slots[sl];
        if (b.is_intermediate || written[(size_t)sl] || b.nbytes < (128 << 10) || b.nbytes > most) continue;
        if (t - touched_for[(size_t)sl] <= 8) continue;
        touched_for[(size_t)sl] = t;
        auto &at = plan->touch_at[(size_t)std::max(0, t - lead)];
        if (std::find(at.begin(), at.end(), sl) == at.end()) at.push_back(sl);
        any = true;
      }
    }
    if (any) {
      plan->touch = program_create(kTouchSrc, "poly_touch");
      if (!plan->touch) return nullptr;
    }
  }
  plan->kargs.resize((size_t)n_units);
  plan->var_vals.resize((size_t)n_units);
  for (int u = 0; u < n_units; u++) {
    plan->kargs[(size_t)u].assign(plan->units[(size_t)u].slots.size() + (size_t)plan->units[(size_t)u].n_vars, nullptr);
    plan->var_vals[(size_t)u].assign((size_t)plan->units[(size_t)u].n_vars, 0);
  }
  return plan.release();
}

static int bind_args(PolyHipPlan *plan, void **slot_data, int n_slots, const PolyVarBinding *vb, int nvb,
                     uint64_t *key_out) {
  const PolySchedule *s = plan->sched;
  uint64_t key = 1469598103934665603ull;
  plan->bound_now.clear();
  if (plan->vetted_slot.size() != (size_t)s->n_buf_slots) plan->vetted_slot.assign((size_t)s->n_buf_slots, nullptr);
  for (int i = 0; i < s->n_buf_slots; i++) {
    if (s->buf_slots[i].is_intermediate) continue;
    plan->slot_ptr[(size_t)i] = (i < n_slots && slot_data) ? slot_data[i] : nullptr;
    plan->bound_now.push_back((uint64_t)(uintptr_t)plan->slot_ptr[(size_t)i]);
    key = fnv1a(&plan->slot_ptr[(size_t)i], sizeof(void *), key);
    // A host address in a device plan (the frontend's constant registry, src/frontend.c:2231-2232,
    // or a training step's loss slot, src/instance.c:1299-1311) would fault in the first kernel
    // that touches it; looked up once per new pointer, outside any stream capture.
    void *p = plan->slot_ptr[(size_t)i];
    if (p && p != plan->vetted_slot[(size_t)i]) {
      if (!runtime_device_can_read(p)) {
        log_err("plan_run", "slot %d (%p) is not device memory; upload it with the allocator's copy_in first", i, p);
        return -1;
      }
      plan->vetted_slot[(size_t)i] = p;
    }
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
  for (size_t u = 0; u < plan->units.size(); u++) {
    const Unit &un = plan->units[u];
    const PolyExecItem &it = s->items[un.item];
    std::vector<void *> &a = plan->kargs[u];
    for (size_t i = 0; i < un.slots.size(); i++) {
      void *p = plan->slot_ptr[(size_t)un.slots[i]];
      if (!p) {
        log_err("plan_run", "missing data for param %zu (slot %d) in kernel %d", i, un.slots[i], un.item);
        return -1;
      }
      a[i] = p;
      if (i < un.runner->vetted.size()) un.runner->vetted[i] = p;     // vetted above, or the plan's own arena
    }
    (void)it;
    for (int v = 0; v < un.n_vars; v++) {
      bool found = false;
      for (const PolyVarBinding &m : plan->merged)
        if (m.var == un.var_uops[(size_t)v]) { plan->var_vals[u][(size_t)v] = m.value; found = true; break; }
      if (!found) { log_err("plan_run", "no binding for DEFINE_VAR in kernel %d", un.item); return -1; }
      a[un.slots.size() + (size_t)v] = &plan->var_vals[u][(size_t)v];
      plan->bound_now.push_back((uint64_t)(uint32_t)plan->var_vals[u][(size_t)v]);
      key = fnv1a(&plan->var_vals[u][(size_t)v], sizeof(int), key);
    }
  }
  *key_out = key;
  return 0;
}

// ── on-device tuning ──────────────────────────────────────────────────────
//
// The reference searches kernel configurations by timing candidates on the machine
// and keeps the winners on disk (src/codegen.c:1012-1105 times one candidate, :1108-1195
// is the cache, :1207-1330 the search; enabled by POLY_BEAM, src/render_c.c:839).  Here the
// candidates are the tile shapes and pipeline depths of the matmul template: with
// POLY_BEAM > 0 every matmul launch of a plan carries them, and the first run of the plan
// -- the first moment all its buffers exist -- times each one on the launch's own
// arguments and keeps the fastest.  Decisions are remembered per process and in the
// cache directory, keyed by the text of all candidates.

static float time_runner(HipRunner *r, std::vector<void *> &args, hipEvent_t e0, hipEvent_t e1) {
  hipStream_t stream = (hipStream_t)runtime_stream();
  if (runner_launch(r, args.data(), (int)args.size()) != 0) return -1.0f;     // warm-up, loads the code
  if (hipStreamSynchronize(stream) != hipSuccess) return -1.0f;
  float best = -1.0f;
  const int reps = 3;
  for (int round = 0; round < 3; round++) {
    (void)hipEventRecord(e0, stream);
    for (int i = 0; i < reps; i++) if (runner_launch(r, args.data(), (int)args.size()) != 0) return -1.0f;
    (void)hipEventRecord(e1, stream);
    if (hipStreamSynchronize(stream) != hipSuccess) return -1.0f;
    float ms = 0;
    if (hipEventElapsedTime(&ms, e0, e1) != hipSuccess) return -1.0f;
    ms /= reps;
    if (best < 0 || ms < best) best = ms;
  }
  return best;
}

// The first run of a plan with tuning enabled: the launches go out one by one in
// execution order, and each tunable one is timed in all its candidates at the moment its
// inputs hold their real values (matrix-pipe speed depends on the data: zeros run a third
// faster than random values at the same instruction stream, so timing on untouched
// buffers would rank by the wrong clock).  Every candidate writes the same values, so the
// buffers are as after a plain run.
static int tuned_first_run(PolyHipPlan *plan) {
  plan->tuned = true;
  static std::map<uint64_t, std::string> decided;   // per process: identical kernels are timed once
  const std::string dir = runtime_cache_dir();
  hipEvent_t e0 = nullptr, e1 = nullptr;
  int rc = 0;
  for (size_t ui = 0; ui < plan->units.size() && rc == 0; ui++) {
    Unit &u = plan->units[ui];
    for (int slot : plan->fills_before[ui]) if (launch_fill(plan, slot) != 0) rc = -1;
    if (rc != 0) break;
    HipRunner *r = u.runner;
    std::vector<void *> &args = plan->kargs[ui];
    const std::vector<RenderedKernel::Variant> &vs = r->rk.variants;
    if (vs.size() < 2 || !u.repeatable || !r->guards.empty()) {
      rc = runner_launch(r, args.data(), (int)args.size());
      continue;
    }
    uint64_t key = 1469598103934665603ull;
    for (const RenderedKernel::Variant &v : vs) key = fnv1a(v.source.data(), v.source.size(), key);
    std::string choice;
    auto it = decided.find(key);
    if (it != decided.end()) choice = it->second;
    const std::string path = dir.empty() ? "" : strf("%s/%016llx.tune", dir.c_str(), (unsigned long long)key);
    if (choice.empty() && !path.empty()) {
      if (FILE *f = fopen(path.c_str(), "r")) {
        char buf[64] = {0};
        if (fscanf(f, "%63s", buf) == 1) choice = buf;
        fclose(f);
      }
    }
    int pick = -1;
    for (size_t i = 0; i < vs.size(); i++) if (vs[i].label == choice) pick = (int)i;
    if (pick < 0) {
      if (!e0 && (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess)) { rc = -1; break; }
      float best = -1.0f;
      std::string report;
      for (size_t i = 0; i < vs.size(); i++) {
        if (runner_use_variant(r, (int)i) != 0) continue;    // a candidate that does not compile is no candidate
        const float ms = time_runner(r, args, e0, e1);
        report += strf(" %s=%.4f", vs[i].label.c_str(), ms);
        if (ms > 0 && (best < 0 || ms < best)) { best = ms; pick = (int)i; }
      }
      if (pick < 0) pick = 0;
      if (getenv("POLY_HIP_DEBUG"))
        fprintf(stderr, "polygrad: tune: %s -> %s (ms:%s)\n", vs[0].strategy.c_str(), vs[(size_t)pick].label.c_str(), report.c_str());
      if (!path.empty()) {
        const std::string tmp = path + strf(".%d.tmp", (int)getpid());
        if (FILE *f = fopen(tmp.c_str(), "w")) {
          fprintf(f, "%s\n", vs[(size_t)pick].label.c_str());
          fclose(f);
          rename(tmp.c_str(), path.c_str());
        }
      }
    }
    decided[key] = vs[(size_t)pick].label;
    if (runner_use_variant(r, pick) != 0 && runner_use_variant(r, 0) != 0) { rc = -1; break; }
    rc = runner_launch(r, args.data(), (int)args.size());
  }
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  if (rc != 0) log_err("plan_run", "tuning run failed");
  return rc;
}

int poly_hip_plan_run(PolyHipPlan *plan, void **slot_data, int n_slots, const PolyVarBinding *vb, int nvb) {
  if (!plan || !plan->sched) return -1;
  uint64_t key = 0;
  if (bind_args(plan, slot_data, n_slots, vb, nvb, &key) != 0) return -1;
  if (!plan->tuned) {
    bool any = false;
    for (const Unit &u : plan->units) any = any || u.runner->rk.variants.size() > 1;
    if (any) return tuned_first_run(plan);
    plan->tuned = true;
  }
  hipStream_t stream = (hipStream_t)runtime_stream();
  if (!plan->use_graph || getenv("POLY_HIP_NO_GRAPH")) return enqueue_all(plan);
  plan->tick++;
  (void)key;
  for (GraphEntry &g : plan->graphs)
    if (g.exec && g.bound == plan->bound_now) {
      g.last_use = plan->tick;
      if (hipGraphLaunch(g.exec, stream) != hipSuccess) { log_err("plan_run", "hipGraphLaunch failed"); return -1; }
      return 0;
    }
  // (the order between the streams was worked out with every bound buffer a resource of its
  // own: two bound buffers that share bytes put everything on one stream)
  bool disjoint = true;
  if (plan->forked) {
    std::vector<std::pair<uintptr_t, uintptr_t>> ext;
    for (int i = 0; i < plan->sched->n_buf_slots; i++)
      if (!plan->sched->buf_slots[i].is_intermediate && plan->slot_ptr[(size_t)i])
        ext.push_back({(uintptr_t)plan->slot_ptr[(size_t)i], (uintptr_t)plan->slot_ptr[(size_t)i] + (uintptr_t)std::max<int64_t>(plan->sched->buf_slots[i].nbytes, 4)});
    std::sort(ext.begin(), ext.end());
    for (size_t i = 1; i < ext.size(); i++) if (ext[i].first < ext[i - 1].second) disjoint = false;
  }
  auto keep = [&](GraphEntry &ge) {
    if (plan->graphs.size() >= 4) {
      size_t victim = 0;
      for (size_t i = 1; i < plan->graphs.size(); i++)
        if (plan->graphs[i].last_use < plan->graphs[victim].last_use) victim = i;
      (void)hipGraphExecDestroy(plan->graphs[victim].exec);
      plan->graphs.erase(plan->graphs.begin() + (long)victim);
    }
    plan->graphs.push_back(ge);
  };
  GraphEntry ge;
  ge.bound = plan->bound_now;
  ge.last_use = plan->tick;
  // A binding the plan has not run with, and the sequence is captured already: a graph
  // instantiated from the capture, every kernel node given the arguments of this binding
  // (the launches are walked as for a capture, but each call only updates its node).
  if (plan->captured && !plan->launches.failed && !getenv("POLY_HIP_NO_GRAPH_REBIND") && (!plan->captured_forked || disjoint)) {
    if (hipGraphInstantiate(&ge.exec, plan->captured, nullptr, nullptr, 0) == hipSuccess) {
      plan->launches.exec = (void *)ge.exec;
      plan->launches.next = 0;
      runtime_graph_update(&plan->launches);
      int rc = 0;
      for (size_t u = 0; u < plan->units.size() && rc == 0; u++) rc = launch_unit(plan, u);
      runtime_graph_update(nullptr);
      const bool ok = rc == 0 && !plan->launches.failed && plan->launches.next == plan->launches.nodes.size();
      plan->launches.failed = false;      // (a failed update says nothing about the capture)
      if (ok) {
        plan->n_rebinds++;
        keep(ge);
        if (hipGraphLaunch(ge.exec, stream) != hipSuccess) { log_err("plan_run", "hipGraphLaunch failed"); return -1; }
        return 0;
      }
      (void)hipGraphExecDestroy(ge.exec);
      ge.exec = nullptr;
      log_err("plan_run", "the captured graph could not be bound to new buffers by updating its nodes; capturing again");
    }
    // the capture is replaced below
    for (GraphEntry &g : plan->graphs) if (g.exec) (void)hipGraphExecDestroy(g.exec);
    plan->graphs.clear();
    (void)hipGraphDestroy(plan->captured);
    plan->captured = nullptr;
  } else if (plan->captured) {
    // (bound buffers that overlap under a forked capture, or rebinding switched off: this
    // binding gets a capture of its own, which replaces the old one)
    for (GraphEntry &g : plan->graphs) if (g.exec) (void)hipGraphExecDestroy(g.exec);
    plan->graphs.clear();
    (void)hipGraphDestroy(plan->captured);
    plan->captured = nullptr;
  }
  // First sight of the sequence: capture it, then replay it.
  if (hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal) != hipSuccess) {
    log_err("plan_run", "hipStreamBeginCapture failed; running without a graph");
    plan->use_graph = false;
    return enqueue_all(plan);
  }
  plan->launches = GraphLaunches();
  runtime_graph_record(&plan->launches);
  plan->captured_forked = plan->forked && disjoint;
  int rc = plan->captured_forked ? enqueue_captured(plan) : enqueue_all(plan);
  runtime_graph_record(nullptr);
  hipError_t e = hipStreamEndCapture(stream, &plan->captured);
  if (rc != 0 || e != hipSuccess || !plan->captured) {
    if (plan->captured) (void)hipGraphDestroy(plan->captured);
    plan->captured = nullptr;
    log_err("plan_run", "graph capture failed; running without a graph");
    plan->use_graph = false;
    return rc != 0 ? rc : enqueue_all(plan);
  }
  plan->n_captures++;
  if (hipGraphInstantiate(&ge.exec, plan->captured, nullptr, nullptr, 0) != hipSuccess) {
    (void)hipGraphDestroy(plan->captured);
    plan->captured = nullptr;
    log_err("plan_run", "hipGraphInstantiate failed; running without a graph");
    plan->use_graph = false;
    return enqueue_all(plan);
  }
  keep(ge);
  if (hipGraphLaunch(ge.exec, stream) != hipSuccess) { log_err("plan_run", "hipGraphLaunch failed"); return -1; }
  return 0;
}

int poly_hip_fused_groups(const PolySchedule *s, int index, char **source_out, int *n_items_out) {
  if (!s) return -1;
  std::vector<KernelGraph> graphs((size_t)s->n_items);
  for (int k = 0; k < s->n_items; k++)
    if (s->items[k].kind != POLY_EXEC_COMPUTE || !graphs[(size_t)k].build(s->items[k].root)) return -1;
  std::vector<FusedGroup> groups;
  find_fused_groups(s, graphs, &groups);
  if (index >= 0 && index < (int)groups.size()) {
    if (n_items_out) *n_items_out = (int)groups[(size_t)index].items.size();
    if (source_out) {
      // the main kernel, then the kernels that fill its tables and those that run ahead of
      // it, as separate translation units
      std::string src = groups[(size_t)index].rk.source;
      for (const RenderedKernel::Table &t : groups[(size_t)index].rk.tables) src += "\n// ---- table " + t.entry + "\n" + t.source;
      for (const RenderedKernel::Pre &pk : groups[(size_t)index].rk.pres) {
        char head[160];
        snprintf(head, sizeof head, "\n// ---- first stage ---- grid=%u,%u block=%u scratch=%zu\n", pk.launch.grid[0], pk.launch.grid[1],
                 pk.launch.block[0], groups[(size_t)index].rk.scratch_bytes);
        src += head + pk.source;
      }
      if (groups[(size_t)index].rk.pres.empty() && groups[(size_t)index].rk.scratch_bytes > 0)     // scratch memory without a first stage
        src += strf("\n// ---- scratch ---- bytes=%zu\n", groups[(size_t)index].rk.scratch_bytes);
      const std::vector<RenderedKernel::Variant> &vs = groups[(size_t)index].rk.variants;
      for (size_t i = 1; i < vs.size(); i++) src += "\n// ---- variant " + vs[i].label + "\n" + vs[i].source;
      *source_out = (char *)malloc(src.size() + 1);
      if (*source_out) memcpy(*source_out, src.c_str(), src.size() + 1);
    }
  }
  return (int)groups.size();
}

int poly_hip_fused_group_launch(const PolySchedule *s, int index, int *slots_out, int cap, int *launch_out) {
  if (!s) return -1;
  std::vector<KernelGraph> graphs((size_t)s->n_items);
  for (int k = 0; k < s->n_items; k++)
    if (s->items[k].kind != POLY_EXEC_COMPUTE || !graphs[(size_t)k].build(s->items[k].root)) return -1;
  std::vector<FusedGroup> groups;
  find_fused_groups(s, graphs, &groups);
  if (index < 0 || index >= (int)groups.size()) return -1;
  const FusedGroup &fg = groups[(size_t)index];
  for (size_t i = 0; i < fg.arg_slots.size() && (int)i < cap; i++) if (slots_out) slots_out[i] = fg.arg_slots[i];
  if (launch_out) {
    for (int i = 0; i < 3; i++) launch_out[i] = (int)fg.rk.launch.grid[i];
    launch_out[3] = (int)fg.rk.launch.block[0];
  }
  return (int)fg.arg_slots.size();
}

int poly_hip_unwritten_slots(const PolySchedule *s, int *slots_out, int cap) {
  if (!s) return -1;
  std::vector<KernelGraph> graphs((size_t)s->n_items);
  for (int k = 0; k < s->n_items; k++)
    if (s->items[k].kind != POLY_EXEC_COMPUTE || !graphs[(size_t)k].build(s->items[k].root)) return -1;
  std::vector<FusedGroup> groups;
  find_fused_groups(s, graphs, &groups);
  std::vector<char> internal((size_t)s->n_buf_slots, 0);
  for (const FusedGroup &fg : groups) for (int sl : fg.internal_slots) internal[(size_t)sl] = 1;
  int n = 0;
  for (int sl = 0; sl < s->n_buf_slots; sl++) {
    if (!s->buf_slots[sl].is_intermediate || internal[(size_t)sl] || slot_fully_written(s, sl, graphs)) continue;
    if (slots_out && n < cap) slots_out[n] = sl;
    n++;
  }
  return n;
}

void poly_hip_plan_free(PolyHipPlan *plan) {
  if (!plan) return;
  runtime_sync();
  delete plan;
}

int poly_hip_plan_n_kernels(const PolyHipPlan *plan) { return plan ? (int)plan->units.size() : -1; }

int poly_hip_plan_kernel_info(const PolyHipPlan *plan, int cap, int *klass, double *bytes, double *flops) {
  if (!plan) return -1;
  const int n = (int)plan->units.size();
  for (int step = 0; step < n && step < cap; step++) {
    const HipRunner *r = plan->units[(size_t)step].runner;
    if (klass) klass[step] = (int)r->rk.klass;
    if (bytes) bytes[step] = r->rk.bytes;
    if (flops) flops[step] = r->rk.flops;
  }
  return n;
}

int poly_hip_plan_profile(PolyHipPlan *plan, void **slot_data, int n_slots, float *ms_out, int cap) {
  if (!plan) return -1;
  uint64_t key;
  if (bind_args(plan, slot_data, n_slots, nullptr, 0, &key) != 0) return -1;
  if (!plan->tuned) {
    bool any = false;
    for (const Unit &u : plan->units) any = any || u.runner->rk.variants.size() > 1;
    if (any && tuned_first_run(plan) != 0) return -1;
    plan->tuned = true;
  }
  // One pass of the launches in order on the one stream, every kernel launch with the pair
  // of events its own dispatch stamps (runtime_time_launches): a step's time is the sum of
  // the durations of its kernels (a fill or a first stage in front of it included), as a
  // profiler's kernel trace would give them, without the gaps between launches.
  const int n = (int)plan->units.size();
  hipStream_t stream = (hipStream_t)runtime_stream();
  LaunchTimes times;
  std::vector<size_t> first((size_t)n + 1, 0);
  int rc = 0;
  runtime_time_launches(&times);
  for (int step = 0; step < n && rc == 0; step++) {
    first[(size_t)step] = times.events.size();
    rc = launch_unit(plan, (size_t)step);
  }
  runtime_time_launches(nullptr);
  first[(size_t)n] = times.events.size();
  if (times.failed) rc = -1;
  if (hipStreamSynchronize(stream) != hipSuccess) rc = -1;
  for (int step = 0; step < n && step < cap && rc == 0; step++) {
    float total = 0;
    for (size_t i = first[(size_t)step]; i + 1 < first[(size_t)step + 1]; i += 2) {
      float ms = 0;
      if (hipEventElapsedTime(&ms, (hipEvent_t)times.events[i], (hipEvent_t)times.events[i + 1]) != hipSuccess) { rc = -1; break; }
      total += ms;
    }
    ms_out[step] = total;
  }
  for (void *e : times.events) (void)hipEventDestroy((hipEvent_t)e);
  return rc == 0 ? n : -1;
}

char *poly_hip_plan_kernel_desc(const PolyHipPlan *plan, int step) {
  if (!plan || step < 0 || step >= (int)plan->units.size()) return nullptr;
  const HipRunner *r = plan->units[(size_t)step].runner;
  std::string d = strf("%s %s: %s grid=%u,%u,%u bytes=%.0f flops=%.0f", r->name.c_str(), kernel_class_name(r->rk.klass),
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
int poly_hip_plan_side_launches(const PolyHipPlan *plan) {
  int n = 0;
  if (plan) for (char c : plan->on_side) n += c != 0;
  return n;
}

void poly_hip_plan_graph_counts(const PolyHipPlan *plan, long long *captures, long long *rebinds) {
  if (captures) *captures = plan ? plan->n_captures : 0;
  if (rebinds) *rebinds = plan ? plan->n_rebinds : 0;
}

size_t poly_hip_plan_workspace_bytes(const PolyHipPlan *plan) { return plan ? plan->arena_bytes + plan->scratch_bytes + plan->kept_scratch_bytes : 0; }

}  // extern "C"
