/*
 * polygrad_abi.h -- the slice of polygrad's in-memory ABI that a device backend
 * consumes, re-declared so that this backend builds without polygrad's headers.
 *
 * Every type below must stay layout-identical (x86-64 SysV) to the reference
 * declaration it cites; tests/test_render_cpu.py checks sizes and offsets
 * against the real library where it is available.  Names are kept identical
 * on purpose: a translation unit inside polygrad that includes both this file
 * and polygrad's own headers must define POLYGRAD_ABI_USE_NATIVE_HEADERS and
 * include polygrad.h / exec_plan.h / frontend.h first.
 *
 * Reference declarations (paths relative to the polygrad tree):
 *   PolyOps            src/polygrad.h:24-129
 *   PolyAddrSpace      src/polygrad.h:183-187
 *   PolyDType          src/polygrad.h:189-200
 *   PolyAxisType       src/polygrad.h:232-243
 *   PolyArgKind/Arg    src/polygrad.h:247-276
 *   PolyUOp            src/polygrad.h:364-372
 *   PolyDeviceId       src/exec_plan.h:28-36
 *   PolyBufferHandle   src/exec_plan.h:78-83
 *   PolyAllocator      src/exec_plan.h:91-101
 *   PolyScheduleBufSlot src/exec_plan.h:109-116
 *   PolyExecItem       src/exec_plan.h:128-145
 *   PolySchedule       src/exec_plan.h:153-176
 *   PolyRunner         src/exec_plan.h:190-211
 *   PolyBackendDesc    src/exec_plan.h:264-283
 *   PolyVarBinding     src/frontend.h:88-91
 */
#ifndef POLYGRAD_ABI_H
#define POLYGRAD_ABI_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifndef POLYGRAD_ABI_USE_NATIVE_HEADERS

#ifdef __cplusplus
extern "C" {
#endif

/* Op codes.  Only the numeric values matter; they start at 1 and follow the
 * reference enum order exactly. */
typedef enum {
  POLY_OP_DEFINE_VAR = 1, POLY_OP_BIND, POLY_OP_SPECIAL, POLY_OP_DEFINE_LOCAL, POLY_OP_DEFINE_REG,
  POLY_OP_NOOP, POLY_OP_REWRITE_ERROR, POLY_OP_PARAM, POLY_OP_CALL, POLY_OP_PROGRAM, POLY_OP_LINEAR,
  POLY_OP_SOURCE, POLY_OP_BINARY, POLY_OP_SINK, POLY_OP_AFTER, POLY_OP_GROUP, POLY_OP_GEP,
  POLY_OP_VECTORIZE,
  POLY_OP_INDEX, POLY_OP_LOAD, POLY_OP_STORE,
  POLY_OP_WMMA,
  POLY_OP_CAST, POLY_OP_BITCAST, POLY_OP_EXP2, POLY_OP_LOG2, POLY_OP_SIN, POLY_OP_SQRT,
  POLY_OP_RECIPROCAL, POLY_OP_NEG, POLY_OP_TRUNC,
  POLY_OP_ADD, POLY_OP_MUL, POLY_OP_SHL, POLY_OP_SHR, POLY_OP_IDIV, POLY_OP_MAX, POLY_OP_MOD,
  POLY_OP_CMPLT, POLY_OP_CMPNE, POLY_OP_CMPEQ, POLY_OP_XOR, POLY_OP_OR, POLY_OP_AND,
  POLY_OP_THREEFRY, POLY_OP_SUB, POLY_OP_FDIV, POLY_OP_POW,
  POLY_OP_WHERE, POLY_OP_MULACC,
  POLY_OP_BARRIER, POLY_OP_RANGE, POLY_OP_IF, POLY_OP_END, POLY_OP_ENDIF, POLY_OP_VCONST,
  POLY_OP_CONST, POLY_OP_CUSTOM, POLY_OP_CUSTOMI, POLY_OP_INS,
  POLY_OP_UNIQUE, POLY_OP_DEVICE, POLY_OP_ASSIGN, POLY_OP_LUNIQUE, POLY_OP_CONTIGUOUS,
  POLY_OP_CONTIGUOUS_BACKWARD, POLY_OP_DETACH, POLY_OP_BUFFERIZE, POLY_OP_COPY, POLY_OP_BUFFER,
  POLY_OP_BUFFER_VIEW, POLY_OP_MSELECT, POLY_OP_MSTACK, POLY_OP_ENCDEC, POLY_OP_RESHAPE,
  POLY_OP_PERMUTE, POLY_OP_EXPAND, POLY_OP_PAD, POLY_OP_SHRINK, POLY_OP_FLIP, POLY_OP_MULTI,
  POLY_OP_REDUCE_AXIS, POLY_OP_REDUCE, POLY_OP_ALLREDUCE, POLY_OP_UNROLL, POLY_OP_CONTRACT,
  POLY_OP_VCAT, POLY_OP_PTRCAT,
  POLY_OP_COUNT
} PolyOps;

typedef enum { POLY_ADDR_GLOBAL = 0, POLY_ADDR_LOCAL, POLY_ADDR_REG } PolyAddrSpace;

/* A dtype is identified by (priority, bitsize, name); bf16 is priority 12 with
 * name "__bf16", fp16 priority 11 "__fp16" (src/dtype.c:14-28). */
typedef struct {
  int8_t priority;
  uint16_t bitsize;
  const char *name;
  char fmt;
  uint16_t count;
  bool is_ptr;
  PolyAddrSpace addrspace;
  uint16_t vcount;
  int64_t ptr_size;
} PolyDType;

typedef enum {
  POLY_AXIS_GLOBAL = 0, POLY_AXIS_WARP, POLY_AXIS_LOCAL, POLY_AXIS_LOOP, POLY_AXIS_GROUP_REDUCE,
  POLY_AXIS_REDUCE, POLY_AXIS_UPCAST, POLY_AXIS_UNROLL, POLY_AXIS_THREAD, POLY_AXIS_PLACEHOLDER
} PolyAxisType;

typedef enum {
  POLY_ARG_NONE = 0, POLY_ARG_INT, POLY_ARG_FLOAT, POLY_ARG_BOOL, POLY_ARG_INT_TUPLE,
  POLY_ARG_PAIR_TUPLE, POLY_ARG_STRING, POLY_ARG_OPS, POLY_ARG_REDUCE_AXIS, POLY_ARG_RANGE,
  POLY_ARG_DEFINE_VAR, POLY_ARG_INVALID
} PolyArgKind;

typedef struct {
  PolyArgKind kind;
  union {
    int64_t i;
    double f;
    bool b;
    struct { int64_t *vals; int n; } int_tuple;
    struct { int64_t (*pairs)[2]; int n; } pair_tuple;
    const char *str;
    PolyOps ops;
    struct { PolyOps op; int64_t *axes; int n; } reduce_axis;
    struct { int64_t axis_id; PolyAxisType axis_type; int64_t *extra; int n_extra; } range;
    struct { const char *name; int64_t min_val; int64_t max_val; } define_var;
  };
} PolyArg;

typedef struct PolyUOp PolyUOp;
struct PolyUOp {
  PolyOps op;
  PolyDType dtype;
  PolyUOp **src;
  uint16_t n_src;
  PolyArg arg;
  int32_t tag;
  uint32_t hash;
};

typedef struct PolyCtx PolyCtx; /* opaque: owns every UOp it created */

typedef enum {
  POLY_DEVICE_AUTO = 0, POLY_DEVICE_CPU, POLY_DEVICE_INTERP, POLY_DEVICE_CUDA,
  POLY_DEVICE_WASM_JIT, POLY_DEVICE_WEBGPU, POLY_DEVICE_X64_JIT,
  /* Appended by this backend; existing members keep their values because JS and
   * Python pass device ids as raw integers. */
  POLY_DEVICE_HIP = 7
} PolyDeviceId;

typedef enum { POLY_MODE_CALL = 0, POLY_MODE_VALUE_AND_GRAD } PolyCompileMode;
typedef enum { POLY_EXEC_COMPUTE, POLY_EXEC_COPY, POLY_EXEC_VIEW, POLY_EXEC_ENCDEC } PolyExecItemKind;
typedef enum {
  POLY_RUNNER_COMPILED, POLY_RUNNER_COPY, POLY_RUNNER_VIEW, POLY_RUNNER_ENCDEC, POLY_RUNNER_INTERP
} PolyRunnerKind;

typedef struct {
  void *ptr;
  size_t nbytes;
  PolyDeviceId domain;
  bool owned;
} PolyBufferHandle;

typedef struct {
  void *(*alloc)(size_t nbytes, void *dev_ctx);
  void (*free)(void *handle, void *dev_ctx);
  int (*copy_in)(void *dst_handle, const void *host_src, size_t nbytes, void *dev_ctx);
  int (*copy_out)(void *host_dst, const void *src_handle, size_t nbytes, void *dev_ctx);
  int (*copy_between)(void *dst_handle, const void *src_handle, size_t nbytes, void *dev_ctx);
  void *dev_ctx;
} PolyAllocator;

typedef struct PolyVarBinding {
  PolyUOp *var;
  int32_t value;
} PolyVarBinding;

typedef struct {
  PolyDType dtype;
  int64_t numel;
  int64_t nbytes;
  PolyUOp *buf_uop;
  bool is_intermediate;
  int external_buf_idx;
} PolyScheduleBufSlot;

typedef struct {
  PolyExecItemKind kind;
  PolyUOp *root;
  int *buf_slot_indices;
  int n_buf_slots;
  struct PolyVarBinding *fixedvars;
  int n_fixedvars;
  PolyUOp **var_uops;
  int n_var_uops;
} PolyExecItem;

typedef struct {
  const char *entrypoint_name;
  PolyCompileMode mode;
  uint32_t graph_hash;
  PolyScheduleBufSlot *buf_slots;
  int n_buf_slots;
  PolyExecItem *items;
  int n_items;
  int *exec_order;
  struct PolyVarBinding *default_vars;
  int n_default_vars;
  int loss_buf_slot;
  int *grad_buf_slots;
} PolySchedule;

typedef struct {
  PolyRunnerKind kind;
  void *handle;
  int handle_size;
  int (*execute)(void *self, void **args, int n_args);
  void (*free_handle)(void *self);
  int grid[3];
  int block[3];
  int *param_to_slot;
  int n_params;
  int *var_indices;
  int n_vars;
} PolyRunner;

typedef struct {
  const char *name;
  PolyDeviceId id;
  bool host_executed;
  int (*lower_item)(PolyCtx *ctx, PolyUOp *scheduled_root, const char *fn_name,
                    PolyRunner *runner_out);
  int (*execute)(PolyRunner *runner, void **args, int n_args);
  void (*free_runner)(PolyRunner *runner);
  const PolyAllocator *(*get_allocator)(void);
} PolyBackendDesc;

#ifdef __cplusplus
}
#endif

#else /* POLYGRAD_ABI_USE_NATIVE_HEADERS */
#ifndef POLY_DEVICE_HIP
#define POLY_DEVICE_HIP ((PolyDeviceId)7)
#endif
#endif

/* Scalar dtype codes used by the serialized plan format and by the FFI dtype
 * table of the reference (src/frontend.c:124-129), plus the index dtype. */
enum {
  POLYHIP_DT_VOID = 0, POLYHIP_DT_BOOL, POLYHIP_DT_INT8, POLYHIP_DT_UINT8, POLYHIP_DT_INT16,
  POLYHIP_DT_UINT16, POLYHIP_DT_INT32, POLYHIP_DT_UINT32, POLYHIP_DT_INT64, POLYHIP_DT_UINT64,
  POLYHIP_DT_FLOAT16, POLYHIP_DT_BFLOAT16, POLYHIP_DT_FLOAT32, POLYHIP_DT_FLOAT64,
  POLYHIP_DT_INDEX, POLYHIP_DT_COUNT
};

#endif /* POLYGRAD_ABI_H */
