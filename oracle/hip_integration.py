#!/usr/bin/env python3
"""Applies the HIP-backend integration edits (a device id, a table row, the whole-plan hook) to a
SCRATCH COPY of the polygrad source tree.  Test infrastructure: `make -C oracle ref_hip`
copies the tree to a temporary directory, runs this script on the copy, compiles it into
oracle/_ref/libpolygrad_hip_ref.so linked against libpolygrad_hip.so, and deletes the
copy.  Nothing of the reference is stored in this repository; the script only names the
places where the new lines go (short anchors) and carries the new lines themselves.

    python3 hip_integration.py <copy-of-the-reference-tree>

Edits (file: what):
  src/exec_plan.h         POLY_DEVICE_HIP appended to PolyDeviceId; PolyCompiledPlan gets
                          `backend_plan` (whole-plan hook) and `hip_needs_zero`
  src/exec_plan.c         BACKENDS[POLY_DEVICE_HIP] row; poly_compile_schedule /
                          poly_compiled_plan_run / poly_compiled_plan_free hand the whole
                          schedule to the backend (POLY_HIP_PER_KERNEL=1 keeps the
                          kernel-by-kernel path through the table row); per-run clearing
                          of the intermediates their kernels leave holes in
  src/frontend_internal.h POLY_MAX_REALIZE_BUFS 256 -> 2048, POLY_MAX_STRUCT_NODES
                          8192 -> 65536 (a 24-layer transformer has 297 buffers)
  src/frontend.c          poly_realize / poly_realize_ex on HIP: host-resident bindings
                          and registry constants are staged through the allocator
  src/instance.c          set_device availability check; param_data / buf_data return
                          NULL for HIP-resident buffers; train_step keeps loss, moments
                          and bias corrections in device memory
"""
import os
import re
import sys


def edit(path, anchor, new, where="after", count=1, regex=False):
    """Inserts `new` before/after the text `anchor` (or replaces it); the anchor must
    occur exactly `count` times."""
    s = open(path).read()
    pat = anchor if regex else re.escape(anchor)
    found = list(re.finditer(pat, s))
    if len(found) != count:
        sys.exit(f"{path}: anchor {anchor!r} found {len(found)} times, expected {count}")
    for m in reversed(found):
        a, b = m.span()
        if where == "after":
            s = s[:b] + new + s[b:]
        elif where == "before":
            s = s[:a] + new + s[a:]
        elif where == "replace":
            s = s[:a] + (m.expand(new) if regex else new) + s[b:]
        else:
            raise ValueError(where)
    open(path, "w").write(s)


HIP_PROTOS = r'''
#ifdef POLY_HAS_HIP
/* libpolygrad_hip.so (include/polygrad_hip.h), restated so this file needs no new include */
int  poly_hip_lower_item(PolyCtx *, PolyUOp *, const char *, PolyRunner *);
int  poly_hip_execute(PolyRunner *, void **, int);
void poly_hip_free_runner(PolyRunner *);
const PolyAllocator *poly_hip_get_allocator(void);
int  poly_hip_memset(void *, int, size_t);
typedef struct PolyHipPlan PolyHipPlan;
PolyHipPlan *poly_hip_compile_schedule(PolyCtx *, const PolySchedule *);
int  poly_hip_plan_run(PolyHipPlan *, void **, int, const struct PolyVarBinding *, int);
void poly_hip_plan_free(PolyHipPlan *);
int  poly_hip_unwritten_slots(const PolySchedule *, int *, int);
#endif
'''

HIP_ROW = r'''#ifdef POLY_HAS_HIP
  [POLY_DEVICE_HIP]   = { "hip",    POLY_DEVICE_HIP,   false,
                          poly_hip_lower_item, poly_hip_execute, poly_hip_free_runner,
                          poly_hip_get_allocator },
#else
  [POLY_DEVICE_HIP]   = { NULL, POLY_DEVICE_HIP, false, NULL, NULL, NULL, NULL },
#endif
'''

COMPILE_HOOK = r'''
#ifdef POLY_HAS_HIP
  /* The backend takes the schedule whole (buffer aliasing, kernel fusion, hipGraph);
   * POLY_HIP_PER_KERNEL=1 keeps the generic path below, one runner per kernel. */
  if (device == POLY_DEVICE_HIP && !getenv("POLY_HIP_PER_KERNEL")) {
    plan->backend_plan = poly_hip_compile_schedule(ctx, schedule);
    if (!plan->backend_plan) { free(plan->runners); free(plan); return NULL; }
    plan->n_runners = 0;
    return plan;
  }
#endif
'''

ZERO_LIST = r'''
#ifdef POLY_HAS_HIP
  /* Which intermediates their kernels do not write completely: only those are cleared
   * per run on this device (index = position among the intermediates). */
  if (device == POLY_DEVICE_HIP && plan->n_intermediates > 0) {
    int *holes = calloc((size_t)schedule->n_buf_slots, sizeof(int));
    int n_holes = holes ? poly_hip_unwritten_slots(schedule, holes, schedule->n_buf_slots) : 0;
    plan->hip_needs_zero = calloc((size_t)plan->n_intermediates, 1);
    if (!holes || !plan->hip_needs_zero || n_holes < 0) { free(holes); goto cleanup; }
    int idx = 0;
    for (int i = 0; i < schedule->n_buf_slots; i++) {
      if (!schedule->buf_slots[i].is_intermediate) continue;
      for (int h = 0; h < n_holes; h++) if (holes[h] == i) plan->hip_needs_zero[idx] = 1;
      idx++;
    }
    free(holes);
  }
#endif
'''

RUN_HOOK = r'''
#ifdef POLY_HAS_HIP
  if (plan->backend_plan)
    return poly_hip_plan_run((PolyHipPlan *)plan->backend_plan, slot_data, n_slots,
                             var_bindings, n_var_bindings);
#endif
'''

ZERO_BRANCH = r'''
#ifdef POLY_HAS_HIP
    else if (h->domain == POLY_DEVICE_HIP) {
      if (plan->hip_needs_zero && plan->hip_needs_zero[i]) poly_hip_memset(h->ptr, 0, h->nbytes);
    }
#endif
'''

FREE_HOOK = r'''
#ifdef POLY_HAS_HIP
  if (plan->backend_plan) poly_hip_plan_free((PolyHipPlan *)plan->backend_plan);
  free(plan->hip_needs_zero);
#endif
'''

STAGING = r'''
#ifdef POLY_HAS_HIP
/* poly_realize on the HIP device: slots whose binding is host memory (CPU-domain
 * handles such as the loss and gradient outputs of poly_instance_value_and_grad, or the
 * constants of the registry) get a device copy for the run; host bindings are copied
 * back afterwards, registry constants stay uploaded for the life of the process. */
typedef struct { void *host, *dev; size_t nbytes; } HipStaged;
typedef struct { HipStaged *v; int n; } HipStagedList;
typedef struct { PolyCtx *ctx; PolyUOp *buf; void *dev; } HipConstCopy;
static HipConstCopy *g_hip_consts = NULL;
static int g_hip_consts_n = 0, g_hip_consts_cap = 0;

static void *hip_const_device_copy(PolyCtx *ctx, PolyUOp *buf, const void *host, size_t nbytes) {
  for (int i = 0; i < g_hip_consts_n; i++)
    if (g_hip_consts[i].ctx == ctx && g_hip_consts[i].buf == buf) return g_hip_consts[i].dev;
  const PolyBackendDesc *be = poly_backend_get(POLY_DEVICE_HIP);
  if (!be) return NULL;
  const PolyAllocator *a = be->get_allocator();
  void *dev = a->alloc(nbytes, a->dev_ctx);
  if (!dev || a->copy_in(dev, host, nbytes, a->dev_ctx) != 0) return NULL;
  if (g_hip_consts_n == g_hip_consts_cap) {
    int cap = g_hip_consts_cap ? 2 * g_hip_consts_cap : 16;
    HipConstCopy *nv = realloc(g_hip_consts, (size_t)cap * sizeof(*nv));
    if (!nv) return dev;
    g_hip_consts = nv;
    g_hip_consts_cap = cap;
  }
  g_hip_consts[g_hip_consts_n++] = (HipConstCopy){ ctx, buf, dev };
  return dev;
}

static int hip_stage_slots(PolyCtx *ctx, const PolySchedule *sched, PolyBufferBinding *bindings,
                           int n_bindings, void **slot_data, HipStagedList *staged) {
  const PolyBackendDesc *be = poly_backend_get(POLY_DEVICE_HIP);
  if (!be) return -1;
  const PolyAllocator *a = be->get_allocator();
  staged->v = calloc((size_t)(sched->n_buf_slots > 0 ? sched->n_buf_slots : 1), sizeof(HipStaged));
  staged->n = 0;
  if (!staged->v) return -1;
  for (int s = 0; s < sched->n_buf_slots; s++) {
    if (sched->buf_slots[s].is_intermediate || !slot_data[s]) continue;
    PolyUOp *slot_uop = sched->buf_slots[s].buf_uop;
    size_t nbytes = (size_t)sched->buf_slots[s].nbytes;
    int bound = -1;
    for (int j = 0; j < n_bindings; j++) if (bindings[j].buffer == slot_uop) { bound = j; break; }
    if (bound < 0) {                      /* filled from the constant registry: host memory */
      slot_data[s] = hip_const_device_copy(ctx, slot_uop, slot_data[s], nbytes);
      if (!slot_data[s]) return -1;
      continue;
    }
    if (bindings[bound].handle.domain == POLY_DEVICE_HIP) continue;
    void *dev = a->alloc(nbytes, a->dev_ctx);
    if (!dev || a->copy_in(dev, slot_data[s], nbytes, a->dev_ctx) != 0) return -1;
    staged->v[staged->n++] = (HipStaged){ slot_data[s], dev, nbytes };
    slot_data[s] = dev;
  }
  return 0;
}

static void hip_unstage_slots(HipStagedList *staged, int run_ok) {
  const PolyBackendDesc *be = poly_backend_get(POLY_DEVICE_HIP);
  const PolyAllocator *a = be ? be->get_allocator() : NULL;
  for (int i = 0; a && i < staged->n; i++) {
    if (run_ok) a->copy_out(staged->v[i].host, staged->v[i].dev, staged->v[i].nbytes, a->dev_ctx);
    a->free(staged->v[i].dev, a->dev_ctx);
  }
  free(staged->v);
  staged->v = NULL;
  staged->n = 0;
}
#endif
'''

INSTANCE_HELPERS = r'''
#ifdef POLY_HAS_HIP
int poly_hip_available(void);
#endif
'''

TRAIN_MIGRATE = r'''
#ifdef POLY_HAS_HIP
  /* Training state created after set_device(HIP) starts out in host memory: move the
   * moments and the bias corrections to the device the parameters live on, and give the
   * loss a device cell to be written to. */
  if (inst->buf_handles[0].domain == POLY_DEVICE_HIP) {
    const PolyAllocator *ha = poly_backend_get(POLY_DEVICE_HIP)->get_allocator();
    if (!ts->loss_dev) {
      ts->loss_dev = ha->alloc(sizeof(float), ha->dev_ctx);
      if (!ts->loss_dev) return -1;
    }
    for (int i = 0; i < ts->n_moment_bufs; i++) {
      PolyBufferHandle *hs[2] = { &ts->m_handles[i], &ts->v_handles[i] };
      float *src[2] = { ts->m_datas[i], ts->v_datas[i] };
      for (int k = 0; k < 2; k++) {
        if (hs[k]->domain == POLY_DEVICE_HIP) continue;
        void *p = ha->alloc(hs[k]->nbytes, ha->dev_ctx);
        if (!p || (src[k] && ha->copy_in(p, src[k], hs[k]->nbytes, ha->dev_ctx) != 0)) return -1;
        *hs[k] = (PolyBufferHandle){ .ptr = p, .nbytes = hs[k]->nbytes, .domain = POLY_DEVICE_HIP, .owned = true };
      }
    }
    if (ts->n_moment_bufs > 0 && ts->bc1_handle.domain != POLY_DEVICE_HIP) {
      void *b1 = ha->alloc(sizeof(float), ha->dev_ctx), *b2 = ha->alloc(sizeof(float), ha->dev_ctx);
      if (!b1 || !b2) return -1;
      ha->copy_in(b1, &ts->bc1_data, sizeof(float), ha->dev_ctx);
      ha->copy_in(b2, &ts->bc2_data, sizeof(float), ha->dev_ctx);
      ts->bc1_handle = (PolyBufferHandle){ .ptr = b1, .nbytes = sizeof(float), .domain = POLY_DEVICE_HIP, .owned = true };
      ts->bc2_handle = (PolyBufferHandle){ .ptr = b2, .nbytes = sizeof(float), .domain = POLY_DEVICE_HIP, .owned = true };
    }
  }
#endif
'''

TRAIN_LOSS_READBACK = r'''
#ifdef POLY_HAS_HIP
  if (ret == 0 && ts->loss_dev && inst->buf_handles[0].domain == POLY_DEVICE_HIP) {
    const PolyAllocator *ha = poly_backend_get(POLY_DEVICE_HIP)->get_allocator();
    ret = ha->copy_out(&ts->loss_data, ts->loss_dev, sizeof(float), ha->dev_ctx);
  }
#endif
'''


def main(root):
    src = os.path.join(root, "src")
    h = os.path.join(src, "exec_plan.h")
    edit(h, r"(POLY_DEVICE_X64_JIT,[^\n]*\n)", r"\1  POLY_DEVICE_HIP,      /* AMD GPU (gfx950): libpolygrad_hip.so */\n", "replace", regex=True)
    edit(h, "} PolyCompiledPlan;", "  void *backend_plan;       /* HIP: the whole schedule compiled by the backend, or NULL */\n"
                                   "  char *hip_needs_zero;     /* HIP, per-kernel path: [n_intermediates] cleared per run */\n", "before")

    c = os.path.join(src, "exec_plan.c")
    edit(c, "static const PolyBackendDesc BACKENDS[] = {", HIP_PROTOS + "\n", "before")
    edit(c, "};\n\n#define N_BACKENDS", HIP_ROW, "before")
    edit(c, "  if (!plan->runners) { free(plan); return NULL; }\n", COMPILE_HOOK)
    edit(c, "  /* ── Allocate persistent per-kernel args arrays", ZERO_LIST + "\n", "before")
    edit(c, "  const PolyBackendDesc *backend = poly_backend_get(plan->device);\n  if (!backend) return -1;\n", RUN_HOOK)
    edit(c, "      memset(h->ptr, 0, h->nbytes);\n    }\n", ZERO_BRANCH)
    edit(c, "  if (!plan) return;\n\n  const PolyBackendDesc *backend = poly_backend_get(plan->device);\n", FREE_HOOK)

    fi = os.path.join(src, "frontend_internal.h")
    edit(fi, "#define POLY_MAX_REALIZE_BUFS 256", "#define POLY_MAX_REALIZE_BUFS 2048", "replace")
    edit(fi, "#define POLY_MAX_STRUCT_NODES 8192", "#define POLY_MAX_STRUCT_NODES 65536", "replace")

    f = os.path.join(src, "frontend.c")
    edit(f, "static void **build_slot_data_from_bindings(", STAGING + "\n", "before")
    call = "  void **slot_data = build_slot_data_from_bindings(ctx, sched, bindings, n_bindings);\n  if (!slot_data) return -1;\n"
    stage = ("#ifdef POLY_HAS_HIP\n  HipStagedList hip_staged = { NULL, 0 };\n"
             "  if (device == POLY_DEVICE_HIP && hip_stage_slots(ctx, sched, bindings, n_bindings, slot_data, &hip_staged) != 0) {\n"
             "    fprintf(stderr, \"polygrad: realize: staging host buffers for the HIP device failed\\n\");\n"
             "    hip_unstage_slots(&hip_staged, 0);\n    free(slot_data);\n    return -1;\n  }\n#endif\n")
    edit(f, call, stage, count=2)
    unstage = "#ifdef POLY_HAS_HIP\n  if (device == POLY_DEVICE_HIP) hip_unstage_slots(&hip_staged, ret == 0);\n#endif\n"
    edit(f, "  int ret = poly_compiled_plan_run(plan, slot_data, sched->n_buf_slots, NULL, 0);\n", unstage)
    edit(f, "  int ret = poly_compiled_plan_run(plan, slot_data, sched->n_buf_slots,\n"
            "                                   var_bindings, n_var_bindings);\n", unstage)

    i = os.path.join(src, "instance.c")
    edit(i, "/* ── Slot table cache ─", INSTANCE_HELPERS + "\n", "before")
    edit(i, "  float loss_data;                  /* scalar loss value after step */\n",
         "  void *loss_dev;                   /* HIP: device cell the loss is written to */\n")
    edit(i, "  const PolyAllocator *alloc = backend->get_allocator();\n\n  /* Bulk rematerialization",
         "#ifdef POLY_HAS_HIP\n  if (resolved == POLY_DEVICE_HIP && !poly_hip_available()) {\n"
         "    fprintf(stderr, \"poly_instance_set_device: HIP not available\\n\");\n    return -1;\n  }\n#endif\n\n", "before")
    edit(i, r"(\.domain == POLY_DEVICE_CUDA)\)\n    return NULL;", r"\1\n      || inst->buf_handles[BI].domain == POLY_DEVICE_HIP)\n    return NULL;",
         "replace", count=2, regex=True)
    s = open(i).read()
    # the two NULL-return tests index buf_handles differently (bi / i): name the right one
    parts = s.split("inst->buf_handles[BI]")
    assert len(parts) == 3
    s = parts[0] + "inst->buf_handles[bi]" + parts[1] + "inst->buf_handles[i]" + parts[2]
    open(i, "w").write(s)
    edit(i, "  TrainState *ts = inst->train;\n  OptimState *o = &inst->optim;\n  int np = inst->n_params;\n", TRAIN_MIGRATE)
    edit(i, "    extra_ptrs[0] = &ts->loss_data;\n",
         "    extra_ptrs[0] = (ts->loss_dev && inst->buf_handles[0].domain != POLY_DEVICE_CPU) ? ts->loss_dev : (void *)&ts->loss_data;\n", "replace")
    edit(i, "      extra_ptrs[1 + 2*np] = &ts->bc1_data;\n", "      extra_ptrs[1 + 2*np] = ts->bc1_handle.ptr;\n", "replace")
    edit(i, "      extra_ptrs[1 + 2*np + 1] = &ts->bc2_data;\n", "      extra_ptrs[1 + 2*np + 1] = ts->bc2_handle.ptr;\n", "replace")
    edit(i, "  int ret = poly_compiled_plan_run(c->plan, c->slot_data, c->n_slots, NULL, 0);\n  if (ret != 0) { o->step--; return ret; }\n",
         TRAIN_LOSS_READBACK, "before")
    # the readback goes between the run and its error check
    s = open(i).read()
    run_line = "  int ret = poly_compiled_plan_run(c->plan, c->slot_data, c->n_slots, NULL, 0);\n"
    s = s.replace(TRAIN_LOSS_READBACK + run_line, run_line + TRAIN_LOSS_READBACK)
    open(i, "w").write(s)
    print("HIP integration edits applied to", root)


if __name__ == "__main__":
    if len(sys.argv) != 2 or not os.path.isdir(os.path.join(sys.argv[1], "src")):
        sys.exit(__doc__)
    main(sys.argv[1])
