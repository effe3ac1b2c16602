/*
 * polygrad_hip.h -- C ABI of the MI355X (gfx950) device backend for polygrad.
 *
 * The library (libpolygrad_hip.so) is a drop-in device backend for the seam
 * polygrad defines at src/exec_plan.h:264-283 (PolyBackendDesc): one row of
 * the BACKENDS[] table (src/exec_plan.c:753-787) plus the allocator that
 * poly_compile_schedule / PolyInstance call through.  Every entry point takes
 * plain pointers and sizes; none takes or returns a C++ or torch type.
 *
 * Conventions follow the reference: 0 on success, negative int or NULL on
 * failure with a "polygrad: <area>: ..." line on stderr, never abort; callers
 * are single-threaded (src/exec_plan.h:220).  There is no host fallback: when
 * no HIP device or no hiprtc is available every compute entry point fails.
 */
#ifndef POLYGRAD_HIP_H
#define POLYGRAD_HIP_H

#include "polygrad_abi.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ── Backend vtable (replaces the CUDA row, src/exec_plan.c:766-768) ────── */

/* Descriptor to place at BACKENDS[POLY_DEVICE_HIP]; replaces the role of the
 * static "cuda" descriptor at src/exec_plan.c:766-768. */
const PolyBackendDesc *poly_hip_backend_desc(void);

/* Replaces cuda_lower_item (src/exec_plan.c:529-582): scheduled kernel SINK ->
 * HIP C -> code object -> runner.  Sets kind, handle, grid, block only. */
int poly_hip_lower_item(PolyCtx *ctx, PolyUOp *scheduled_root, const char *fn_name,
                        PolyRunner *runner_out);

/* Replaces cuda_execute (src/exec_plan.c:584-609): args[0..n_params) are device
 * pointers, followed by one pointer-to-host-int per DEFINE_VAR
 * (src/exec_plan.c:1026-1041).  Launches on the backend stream and returns
 * without waiting; copy_out / poly_hip_sync make results visible. */
int poly_hip_execute(PolyRunner *runner, void **args, int n_args);

/* No counterpart in the reference.  For callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc):
 * poly_hip_execute for a runner whose kernel runs in two stages (partial sums, split-K
 * accumulators, operand planes), with the stage-one results in a static device array of
 * POLY_HIP_STATIC_SCRATCH_BYTES inside the library instead of memory the runner
 * allocates on its first poly_hip_execute.  Calls no hipMalloc/hipFree once
 * poly_hip_init() (or a first call on the device) has looked the array up.  Returns -1
 * with a "polygrad: execute_static:" message when the kernel needs more scratch than the
 * array holds; a one-stage kernel is simply launched.  Every call on a GPU uses the
 * same array: calls that overlap on one GPU (other streams, other threads) race. */
#define POLY_HIP_STATIC_SCRATCH_BYTES (32u << 20)
int poly_hip_execute_static(PolyRunner *runner, void **args, int n_args);

/* Replaces cuda_free_runner (src/exec_plan.c:611-617). */
void poly_hip_free_runner(PolyRunner *runner);

/* Replaces cuda_get_allocator / POLY_CUDA_ALLOCATOR (src/exec_plan.c:267-303,
 * 619-621).  copy_between is implemented (device to device). */
const PolyAllocator *poly_hip_get_allocator(void);

/* ── Runtime (replaces src/runtime_cuda.c:192-435) ──────────────────────── */

/* poly_cuda_init / poly_cuda_available (runtime_cuda.c:192-243). 0 = usable. */
int poly_hip_init(void);
int poly_hip_available(void);
/* poly_cuda_alloc/free (runtime_cuda.c:245-262). NULL on failure. */
void *poly_hip_alloc(size_t nbytes);
void poly_hip_free(void *dptr);
/* poly_cuda_copy_htod/dtoh (runtime_cuda.c:264-286). Synchronous on return. */
int poly_hip_copy_htod(void *dst, const void *src, size_t nbytes);
int poly_hip_copy_dtoh(void *dst, const void *src, size_t nbytes);
int poly_hip_copy_dtod(void *dst, const void *src, size_t nbytes);
/* poly_cuda_memset (runtime_cuda.c:426-435). Asynchronous on the stream. */
int poly_hip_memset(void *dptr, int value, size_t nbytes);
/* poly_cuda_sync (runtime_cuda.c:408-416). */
int poly_hip_sync(void);
/* The HIP stream (hipStream_t) all launches go to; callers that own device
 * memory on another stream order against it with events. */
void *poly_hip_stream(void);

/* poly_cuda_compile / launch / program_destroy (runtime_cuda.c:288-406, 418-424).
 * Compiles HIP C with hiprtc for gfx950; identical sources share one module. */
typedef struct PolyHipProgram PolyHipProgram;
PolyHipProgram *poly_hip_compile(const char *source, const char *entry);
int poly_hip_launch(PolyHipProgram *prog, void **kernel_args, int n_args,
                    unsigned gx, unsigned gy, unsigned gz,
                    unsigned bx, unsigned by, unsigned bz, unsigned lds_bytes);
void poly_hip_program_destroy(PolyHipProgram *prog);

/* ── Rendering without a device (render-only tests, dumps) ──────────────── */

/* Lowers one scheduled kernel root to HIP C.  Returns a malloc'd string (free
 * with poly_hip_free_string) or NULL.  Mirrors the render-only use of
 * poly_render_cuda (src/render_cuda.c:196) in the reference's tests.
 * launch_out, when non-NULL, receives grid[3], block[3], lds bytes (7 ints).
 * flags: bit0 disable templates, bit1 disable vectorisation, bit2 disable
 * cooperative reductions. */
char *poly_hip_render(PolyUOp *scheduled_root, const char *fn_name, int flags, int *launch_out);
/* One-line description of how the kernel was lowered ("row-reduce G=64 ..."). */
char *poly_hip_describe(PolyUOp *scheduled_root, int flags);
/* Compiles source for gfx950 with hiprtc only (no device needed). 0 = ok. */
int poly_hip_compile_check(const char *source);
void poly_hip_free_string(char *s);
/* Self-check used by the CPU tests: evaluates every integer index expression of
 * the kernel both as written and in the simplified form the renderer emits, at
 * `samples` points of the iteration space.  Returns the number of mismatches
 * (0 = consistent), <0 on a malformed root.  No reference counterpart: the
 * reference relies on its symbolic pass (src/sym.c) being right. */
int poly_hip_check_index_simplification(PolyUOp *scheduled_root, int samples);

/* ── Plan level (replaces src/exec_plan.c:801-1096 for this device) ─────── */

/* MI355X-native counterparts of poly_compile_schedule / poly_compiled_plan_run /
 * poly_compiled_plan_free.  Differences from the reference, all internal:
 * intermediates that are dead share memory, only the intermediates that their
 * producers leave holes in are cleared per run (poly_hip_unwritten_slots), launches are
 * asynchronous on one stream and the launch sequence is replayed from a
 * hipGraph when the bound pointers repeat (in that graph, small launches that are
 * chains of dependent steps may run on side branches beside the others, ordered by
 * the buffers they share: poly_hip_plan_side_launches). */
typedef struct PolyHipPlan PolyHipPlan;
PolyHipPlan *poly_hip_compile_schedule(PolyCtx *ctx, const PolySchedule *schedule);
/* slot_data[i]: device pointer for every external slot (ignored for
 * intermediates).  Returns after enqueueing; poly_hip_sync() waits.
 * With POLY_BEAM > 0 in the environment at compile and run time (the switch of
 * the reference's kernel search, src/render_c.c:839; its timing loop and disk
 * cache are src/codegen.c:1012-1195), the first run goes through the launches
 * in order and times every matmul in each tile shape of the template, on its
 * own buffers once they hold their real values; it keeps the fastest and
 * records the decision in the cache directory. */
int poly_hip_plan_run(PolyHipPlan *plan, void **slot_data, int n_slots,
                      const PolyVarBinding *var_bindings, int n_var_bindings);
void poly_hip_plan_free(PolyHipPlan *plan);
/* Kernel groups of `schedule` that poly_hip_compile_schedule runs as ONE launch
 * (attention: scores, scale/mask, row max, row sum, normalise, weighted sum of
 * values -- src/modelzoo/models/gpt2.c:411-441 builds it as separate realized
 * tensors).  Returns their number, <0 on a malformed schedule; needs no device.
 * For 0 <= index < count, *n_items_out receives how many scheduled kernels the
 * group replaces and *source_out its HIP source (free with poly_hip_free_string);
 * kernels that fill the group's tables follow the main kernel, each after a line
 * starting with "// ---- ".
 * No reference counterpart: the reference launches every scheduled kernel. */
int poly_hip_fused_groups(const PolySchedule *schedule, int index, char **source_out, int *n_items_out);
/* How group `index` is launched, for checking its indexing away from the GPU: the
 * buffer slot of each kernel argument in order (at most cap entries written to
 * slots_out; tables and flags the kernel takes after them are not listed) and
 * launch_out[0..3] = grid x, y, z and workgroup size.  Returns the number of buffer
 * arguments, <0 on error.  No reference counterpart. */
int poly_hip_fused_group_launch(const PolySchedule *schedule, int index, int *slots_out, int cap, int *launch_out);
/* Intermediate slots of `schedule` that its kernels do not write completely (padded or
 * gated stores): poly_hip_compile_schedule clears each of them with a fill kernel right
 * before its first use on every run, which is what keeps the reference's rule that an
 * intermediate reads as zero where nothing was stored (src/exec_plan.c:946-963 zeroes
 * all of them, every run).  At most cap slot numbers go to slots_out; returns how many
 * there are, <0 on a malformed schedule.  Needs no device. */
int poly_hip_unwritten_slots(const PolySchedule *schedule, int *slots_out, int cap);
/* Introspection for benches and tests. */
int poly_hip_plan_n_kernels(const PolyHipPlan *plan);
/* Fills at most cap entries; per kernel (in execution order): class id
 * (0 elementwise, 1 row-reduce, 2 thread-reduce, 3 matmul-mfma, 4 gather,
 * 5 copy, 6 attention-mfma), algorithmic bytes, flops.  A "kernel" here is one
 * launch: a fused group counts once.  Returns the number of launches. */
int poly_hip_plan_kernel_info(const PolyHipPlan *plan, int cap, int *klass, double *bytes,
                              double *flops);
/* Runs the plan once, launch by launch on the backend stream, and times every
 * kernel with the pair of HIP events its own dispatch stamps at its start and end
 * (hipExtModuleLaunchKernel): ms_out[k], k in execution order, is the sum over the
 * kernels of launch k (a fill or first stage in front of it included) -- what a
 * profiler's kernel trace reports, without the waits between launches.  Returns
 * the number of launches or <0. */
int poly_hip_plan_profile(PolyHipPlan *plan, void **slot_data, int n_slots, float *ms_out, int cap);
/* Malloc'd description ("lower0_k3 matmul-mfma ...") of kernel k; free with
 * poly_hip_free_string. */
char *poly_hip_plan_kernel_desc(const PolyHipPlan *plan, int k);
/* Device address of an intermediate slot (tests compare intermediates). */
void *poly_hip_plan_slot_ptr(const PolyHipPlan *plan, int slot);
/* Enable (1, default) or disable (0) hipGraph replay for this plan. */
void poly_hip_plan_set_graph(PolyHipPlan *plan, int enabled);
size_t poly_hip_plan_workspace_bytes(const PolyHipPlan *plan);
/* How many launches of the plan its captured graph runs on side streams beside the
 * main sequence (small launches that are a chain of dependent steps; 0 for most plans).
 * No counterpart in the reference, whose plans run kernel by kernel with a sync after
 * each (src/exec_plan.c:1000-1057). */
int poly_hip_plan_side_launches(const PolyHipPlan *plan);
/* How the plan's graph met the bindings it has run with: *captures = times the launch
 * sequence went through stream capture, *rebinds = times a binding (a set of buffer
 * addresses and variable values) not seen before was served by instantiating the
 * captured graph again and giving every kernel node the new argument values.  A binding
 * seen before (all values compared, up to four kept) replays its graph and counts in
 * neither.  No counterpart in the reference (src/exec_plan.c:1000-1057 has no graphs). */
void poly_hip_plan_graph_counts(const PolyHipPlan *plan, long long *captures, long long *rebinds);

/* ── Serialized schedules ("plan files") ─────────────────────────────────── */

/* A PolySchedule is "internal only, not serialized" in the reference
 * (src/exec_plan.h:149); these two calls add a portable container so a
 * schedule produced once by polygrad's scheduler can be compiled for the GPU
 * without the frontend present.  names[i] (may be NULL) labels external
 * slot i. */
int poly_hip_planfile_save(const PolySchedule *schedule, const char *const *names, const char *path);
typedef struct PolyHipPlanFile PolyHipPlanFile;
PolyHipPlanFile *poly_hip_planfile_load(const char *path);
const PolySchedule *poly_hip_planfile_schedule(const PolyHipPlanFile *pf);
/* Name given at save time to external slot i, or "". */
const char *poly_hip_planfile_slot_name(const PolyHipPlanFile *pf, int slot);
void poly_hip_planfile_free(PolyHipPlanFile *pf);

#ifdef __cplusplus
}
#endif
#endif /* POLYGRAD_HIP_H */
