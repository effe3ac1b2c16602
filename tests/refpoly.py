"""Test-only ctypes binding of the REAL reference library (oracle/_ref/libpolygrad.so).

Used by tests, smoke and the CPU-baseline leg of the bench as (a) the caller
that produces scheduled kernel graphs exactly as polygrad's frontend and
scheduler do and (b) the checker (the reference CPU backend via poly_realize).
Nothing in the product path imports this module.

The library is built by `make -C oracle ref` from the reference sources where
they lie; it cannot be built on a machine without the reference tree, but the
built file travels with the repository snapshot.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
REF_LIB = os.path.join(_HERE, "..", "oracle", "_ref", "libpolygrad.so")
# The same sources with the HIP backend wired in (oracle/hip_integration.py,
# `make -C oracle ref_hip`): the reference's own callers driving libpolygrad_hip.so.
HIP_REF_LIB = os.path.join(_HERE, "..", "oracle", "_ref", "libpolygrad_hip_ref.so")

# dtype ids of the reference's FFI table (src/frontend.c:124-129)
VOID, BOOL, I8, U8, I16, U16, I32, U32, I64, U64, F16, BF16, F32, F64 = range(14)
NP_DTYPE = {BOOL: np.bool_, I8: np.int8, U8: np.uint8, I16: np.int16, U16: np.uint16, I32: np.int32,
            U32: np.uint32, I64: np.int64, U64: np.uint64, F16: np.float16, BF16: np.uint16,
            F32: np.float32, F64: np.float64}
ITEMSIZE = {BOOL: 1, I8: 1, U8: 1, I16: 2, U16: 2, I32: 4, U32: 4, I64: 8, U64: 8, F16: 2, BF16: 2, F32: 4, F64: 8}

# op codes (src/polygrad.h:24-129)
OPS = ("DEFINE_VAR BIND SPECIAL DEFINE_LOCAL DEFINE_REG NOOP REWRITE_ERROR PARAM CALL PROGRAM LINEAR SOURCE "
       "BINARY SINK AFTER GROUP GEP VECTORIZE INDEX LOAD STORE WMMA CAST BITCAST EXP2 LOG2 SIN SQRT RECIPROCAL "
       "NEG TRUNC ADD MUL SHL SHR IDIV MAX MOD CMPLT CMPNE CMPEQ XOR OR AND THREEFRY SUB FDIV POW WHERE MULACC "
       "BARRIER RANGE IF END ENDIF VCONST CONST").split()
OP = {name: i + 1 for i, name in enumerate(OPS)}

DEVICE_CPU, DEVICE_INTERP, DEVICE_HIP = 1, 2, 7


class PolyDType(C.Structure):
    _fields_ = [("priority", C.c_int8), ("bitsize", C.c_uint16), ("name", C.c_char_p),
                ("fmt", C.c_char), ("count", C.c_uint16), ("is_ptr", C.c_bool),
                ("addrspace", C.c_int), ("vcount", C.c_uint16), ("ptr_size", C.c_int64)]


class PolyBufferHandle(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("nbytes", C.c_size_t), ("domain", C.c_int), ("owned", C.c_bool)]


class PolyBufferBinding(C.Structure):
    _fields_ = [("buffer", C.c_void_p), ("handle", PolyBufferHandle)]


class PolyIOBinding(C.Structure):
    _fields_ = [("name", C.c_char_p), ("data", C.c_void_p)]


_libs = {}


def available():
    return os.path.exists(REF_LIB)


def hip_ref_available():
    return os.path.exists(HIP_REF_LIB)


def lib(path=None):
    path = os.path.abspath(path or REF_LIB)
    if path in _libs:
        return _libs[path]
    L = C.CDLL(path)
    P = C.c_void_p
    I64P = C.POINTER(C.c_int64)
    sig = {
        "poly_ctx_new": (P, []), "poly_ctx_destroy": (None, [P]),
        "poly_const_float": (P, [P, C.c_double]), "poly_const_int": (P, [P, C.c_int64]),
        "poly_const_typed": (P, [P, PolyDType, C.c_double]),
        "poly_alu1": (P, [P, C.c_int, P]), "poly_alu2": (P, [P, C.c_int, P, P]),
        "poly_alu3": (P, [P, C.c_int, P, P, P]),
        "poly_store_val": (P, [P, P, P]), "poly_sink1": (P, [P, P]),
        "poly_sink_n": (P, [P, C.POINTER(P), C.c_int]), "poly_assign": (P, [P, P, P]),
        "poly_buffer_by_id": (P, [P, C.c_int64, C.c_int]), "poly_cast_by_id": (P, [P, P, C.c_int]),
        "poly_reshape": (P, [P, P, I64P, C.c_int]), "poly_expand": (P, [P, P, I64P, C.c_int]),
        "poly_permute": (P, [P, P, I64P, C.c_int]), "poly_reduce_axis": (P, [P, C.c_int, P, I64P, C.c_int]),
        "poly_shrink": (P, [P, P, I64P, C.c_int]), "poly_pad": (P, [P, P, I64P, C.c_int]),
        "poly_flip": (P, [P, P, I64P, C.c_int]),
        "poly_dot": (P, [P, P, I64P, C.c_int, P, I64P, C.c_int, I64P, C.POINTER(C.c_int)]),
        "poly_softmax": (P, [P, P, I64P, C.c_int, C.c_int]),
        "poly_log_softmax": (P, [P, P, I64P, C.c_int, C.c_int]),
        "poly_layernorm": (P, [P, P, I64P, C.c_int, C.c_int, C.c_double, I64P, C.POINTER(C.c_int)]),
        "poly_sum_reduce": (P, [P, P, I64P, C.c_int, C.c_int, C.c_int, I64P, C.POINTER(C.c_int)]),
        "poly_max_reduce": (P, [P, P, I64P, C.c_int, C.c_int, C.c_int, I64P, C.POINTER(C.c_int)]),
        "poly_mean_reduce": (P, [P, P, I64P, C.c_int, C.c_int, C.c_int, I64P, C.POINTER(C.c_int)]),
        "poly_cross_entropy": (P, [P, P, I64P, C.c_int, P, I64P, C.c_int, C.c_int, I64P, C.POINTER(C.c_int)]),
        "poly_gelu": (P, [P, P]), "poly_relu": (P, [P, P]), "poly_exp": (P, [P, P]), "poly_log": (P, [P, P]),
        "poly_sigmoid": (P, [P, P]), "poly_tanh_act": (P, [P, P]), "poly_sin": (P, [P, P]),
        "poly_clamp": (P, [P, P, C.c_double, C.c_double]), "poly_where_op": (P, [P, P, P, P]),
        "poly_eq": (P, [P, P, P]), "poly_maximum": (P, [P, P, P]),
        "poly_rand": (P, [P, I64P, C.c_int, C.c_uint64]),
        "poly_gather": (P, [P, P, I64P, C.c_int, P, I64P, C.c_int, I64P, C.POINTER(C.c_int)]),
        "poly_realize": (C.c_int, [P, P, C.POINTER(PolyBufferBinding), C.c_int]),
        "poly_schedule_for": (P, [P, P, C.c_int]), "poly_schedule_free": (None, [P]),
        "poly_compile_schedule": (P, [P, P, C.c_int]),
        "poly_compiled_plan_run": (C.c_int, [P, C.POINTER(P), C.c_int, P, C.c_int]),
        "poly_compiled_plan_free": (None, [P]),
        "poly_grad": (P, [P, P, P]),
        "poly_grad_many": (C.c_int, [P, P, P, C.POINTER(P), C.c_int, C.POINTER(P)]),
        "poly_const_buffer_data": (P, [P, P]),
        "poly_define_var": (P, [P, C.c_char_p, C.c_int64, C.c_int64]), "poly_bind_var": (P, [P, P, C.c_int64]),
        "poly_buffer_var": (P, [P, PolyDType, P, I64P, C.c_int]),
        "poly_op_name": (C.c_char_p, [C.c_int]),
        # PolyInstance (src/instance.h) and the MLP builder (src/model_mlp.h:31)
        "poly_mlp_instance": (P, [C.c_char_p, C.c_int]), "poly_instance_free": (None, [P]),
        "poly_instance_set_device": (C.c_int, [P, C.c_int]),
        "poly_instance_param_count": (C.c_int, [P]), "poly_instance_buf_count": (C.c_int, [P]),
        "poly_instance_param_data": (P, [P, C.c_int, I64P]), "poly_instance_buf_data": (P, [P, C.c_int, I64P]),
        "poly_instance_buf_role": (C.c_int, [P, C.c_int]), "poly_instance_buf_name": (C.c_char_p, [P, C.c_int]),
        "poly_instance_readback_buf": (C.c_int, [P, C.c_int, P, C.c_size_t]),
        "poly_instance_readback_param": (C.c_int, [P, C.c_int, P, C.c_size_t]),
        "poly_instance_forward": (C.c_int, [P, C.POINTER(PolyIOBinding), C.c_int]),
        "poly_instance_value_and_grad": (C.c_int, [P, C.c_char_p, C.POINTER(PolyIOBinding), C.c_int, C.POINTER(C.c_float)]),
        "poly_instance_train_step": (C.c_int, [P, C.POINTER(PolyIOBinding), C.c_int, C.POINTER(C.c_float)]),
        "poly_instance_set_optimizer": (C.c_int, [P, C.c_int] + [C.c_float] * 5),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    _libs[path] = L
    return L


def dtype_struct(dt, L=None):
    names = ["POLY_VOID", "POLY_BOOL", "POLY_INT8", "POLY_UINT8", "POLY_INT16", "POLY_UINT16", "POLY_INT32",
             "POLY_UINT32", "POLY_INT64", "POLY_UINT64", "POLY_FLOAT16", "POLY_BFLOAT16", "POLY_FLOAT32",
             "POLY_FLOAT64"]
    return PolyDType.in_dll(L or lib(), names[dt])


def _i64(vals):
    arr = (C.c_int64 * max(1, len(vals)))(*vals)
    return arr


class Ctx:
    """A reference PolyCtx plus the list of buffers created in it."""

    def __init__(self, hip_ref=False):
        """hip_ref: use the build of the reference that has the HIP backend in its table."""
        self.L = lib(HIP_REF_LIB if hip_ref else None)
        self.ctx = self.L.poly_ctx_new()
        self.buffers = []   # (T, name)

    def close(self):
        if self.ctx:
            self.L.poly_ctx_destroy(self.ctx)
            self.ctx = None

    # ── leaves ─────────────────────────────────────────────────────────────
    def buffer(self, shape, dt=F32, name=None):
        shape = tuple(int(s) for s in shape)
        n = int(np.prod(shape)) if shape else 1
        u = self.L.poly_buffer_by_id(self.ctx, n, dt)
        t = T(self, u, (n,), dt, buf=u)
        self.buffers.append((t, name or f"buf{len(self.buffers)}"))
        return t.reshape(shape) if shape != (n,) else t

    def define_var(self, name, lo, hi):
        """A DEFINE_VAR UOp (symbolic size in [lo, hi])."""
        self._keep = getattr(self, "_keep", [])
        b = name.encode()
        self._keep.append(b)
        return self.L.poly_define_var(self.ctx, b, lo, hi)

    def buffer_var(self, var, max_val, inner=(), dt=F32, name=None):
        """A buffer whose leading dimension is the variable `var` (allocated for max_val),
        as poly_buffer_var builds it (src/frontend.c:163-179)."""
        u = self.L.poly_buffer_var(self.ctx, dtype_struct(dt, self.L), var, _i64(inner) if inner else None, len(inner))
        t = T(self, u, (max_val,) + tuple(inner), dt, buf=u)
        self.buffers.append((t, name or f"buf{len(self.buffers)}"))
        return t

    def const(self, v, dt=F32):
        if dt in (F32,):
            return T(self, self.L.poly_const_float(self.ctx, float(v)), (), dt)
        return T(self, self.L.poly_const_typed(self.ctx, dtype_struct(dt, self.L), float(v)), (), dt)

    def sink(self, *pairs):
        """pairs: (out_buffer T, value T) -> tensor-level SINK."""
        stores = []
        for out, val in pairs:
            flat = val.reshape((int(np.prod(val.shape)) if val.shape else 1,))
            stores.append(self.L.poly_store_val(self.ctx, out.buf, flat.u))
        if len(stores) == 1:
            return self.L.poly_sink1(self.ctx, stores[0])
        arr = (C.c_void_p * len(stores))(*stores)
        return self.L.poly_sink_n(self.ctx, arr, len(stores))

    def sink_assign(self, *pairs):
        """pairs: (target buffer T, value T) -> SINK of ASSIGNs (in-place updates)."""
        srcs = []
        for tgt, val in pairs:
            flat = val.reshape((int(np.prod(val.shape)),))
            srcs.append(self.L.poly_assign(self.ctx, tgt.buf, flat.u))
        arr = (C.c_void_p * len(srcs))(*srcs)
        return self.L.poly_sink_n(self.ctx, arr, len(srcs))

    def sink_mixed(self, stores, assigns):
        """One SINK holding plain stores (out buffer, value) and in-place updates (target, value)."""
        srcs = []
        for out, val in stores:
            flat = val.reshape((int(np.prod(val.shape)) if val.shape else 1,))
            srcs.append(self.L.poly_store_val(self.ctx, out.buf, flat.u))
        for tgt, val in assigns:
            flat = val.reshape((int(np.prod(val.shape)),))
            srcs.append(self.L.poly_assign(self.ctx, tgt.buf, flat.u))
        arr = (C.c_void_p * len(srcs))(*srcs)
        return self.L.poly_sink_n(self.ctx, arr, len(srcs))

    # ── running the reference ──────────────────────────────────────────────
    def realize_cpu(self, sink, arrays):
        """Runs the reference CPU backend (fork+clang JIT). arrays: {buffer T: ndarray}."""
        n = len(arrays)
        b = (PolyBufferBinding * n)()
        keep = []
        for i, (t, a) in enumerate(arrays.items()):
            assert a.flags["C_CONTIGUOUS"]
            keep.append(a)
            b[i].buffer = t.buf
            b[i].handle = PolyBufferHandle(a.ctypes.data, a.nbytes, DEVICE_CPU, False)
        rc = self.L.poly_realize(self.ctx, sink, b, n)
        if rc != 0:
            raise RuntimeError("reference poly_realize failed")

    def realize_bound(self, sink, handles):
        """poly_realize with explicit handles: {buffer T: (pointer, nbytes, device domain)}
        -- the form the reference's own device tests use (test/test_cuda.c:438-516)."""
        n = len(handles)
        b = (PolyBufferBinding * n)()
        for i, (t, (ptr, nbytes, domain)) in enumerate(handles.items()):
            b[i].buffer = t.buf
            b[i].handle = PolyBufferHandle(ptr, nbytes, domain, False)
        return self.L.poly_realize(self.ctx, sink, b, n)

    def schedule(self, sink):
        s = self.L.poly_schedule_for(self.ctx, sink, 0)
        if not s:
            raise RuntimeError("reference poly_schedule_for failed")
        return s

    def run_schedule_ref(self, sched, slot_arrays, device=DEVICE_CPU):
        """poly_compile_schedule + poly_compiled_plan_run on a reference device."""
        plan = self.L.poly_compile_schedule(self.ctx, sched, device)
        if not plan:
            raise RuntimeError("reference poly_compile_schedule failed")
        n = len(slot_arrays)
        data = (C.c_void_p * n)(*[a.ctypes.data if a is not None else None for a in slot_arrays])
        rc = self.L.poly_compiled_plan_run(plan, data, n, None, 0)
        self.L.poly_compiled_plan_free(plan)
        if rc != 0:
            raise RuntimeError("reference poly_compiled_plan_run failed")


class T:
    """A tensor-level UOp with its shape, in the reference's graph."""

    def __init__(self, c, u, shape, dt, buf=None):
        if not u:
            raise RuntimeError("reference returned NULL while building the graph")
        self.c, self.u, self.shape, self.dt, self.buf = c, u, tuple(shape), dt, buf

    def __hash__(self):
        return hash(self.buf or self.u)

    def __eq__(self, o):
        return isinstance(o, T) and (self.buf or self.u) == (o.buf or o.u)

    def _new(self, u, shape=None, dt=None):
        return T(self.c, u, self.shape if shape is None else shape, self.dt if dt is None else dt, buf=self.buf)

    # movement
    def reshape(self, shape):
        shape = tuple(int(s) for s in shape)
        return self._new(self.c.L.poly_reshape(self.c.ctx, self.u, _i64(shape), len(shape)), shape)

    def expand(self, shape):
        shape = tuple(int(s) for s in shape)
        return self._new(self.c.L.poly_expand(self.c.ctx, self.u, _i64(shape), len(shape)), shape)

    def permute(self, perm):
        shape = tuple(self.shape[p] for p in perm)
        return self._new(self.c.L.poly_permute(self.c.ctx, self.u, _i64(perm), len(perm)), shape)

    def shrink(self, pairs):
        flat = [v for p in pairs for v in p]
        shape = tuple(e - s for s, e in pairs)
        return self._new(self.c.L.poly_shrink(self.c.ctx, self.u, _i64(flat), len(pairs)), shape)

    def pad(self, pairs):
        flat = [v for p in pairs for v in p]
        shape = tuple(d + b + a for d, (b, a) in zip(self.shape, pairs))
        return self._new(self.c.L.poly_pad(self.c.ctx, self.u, _i64(flat), len(pairs)), shape)

    def flip(self, axes):
        return self._new(self.c.L.poly_flip(self.c.ctx, self.u, _i64(axes), len(axes)))

    def contiguous(self):
        # CONTIGUOUS is op 65 in the reference enum; poly_alu1 builds a unary node of any op
        return self._new(self.c.L.poly_alu1(self.c.ctx, 65, self.u))

    def cast(self, dt):
        return self._new(self.c.L.poly_cast_by_id(self.c.ctx, self.u, dt), dt=dt)

    # elementwise
    def _bin(self, op, o, dt=None):
        if not isinstance(o, T):
            o = self.c.const(o, self.dt)
        shape = self.shape if len(self.shape) >= len(o.shape) else o.shape
        return T(self.c, self.c.L.poly_alu2(self.c.ctx, OP[op], self.u, o.u), shape, self.dt if dt is None else dt)

    def __add__(self, o): return self._bin("ADD", o)
    def __sub__(self, o): return self._bin("SUB", o)
    def __mul__(self, o): return self._bin("MUL", o)
    def __truediv__(self, o): return self._bin("FDIV", o)
    def lt(self, o): return self._bin("CMPLT", o, BOOL)
    def ne(self, o): return self._bin("CMPNE", o, BOOL)
    def maximum(self, o): return self._bin("MAX", o)
    def idiv(self, o): return self._bin("IDIV", o)
    def mod(self, o): return self._bin("MOD", o)
    def bxor(self, o): return self._bin("XOR", o)
    def band(self, o): return self._bin("AND", o)
    def bor(self, o): return self._bin("OR", o)
    def shl(self, o): return self._bin("SHL", o)
    def shr(self, o): return self._bin("SHR", o)

    def eq(self, o):
        return T(self.c, self.c.L.poly_eq(self.c.ctx, self.u, o.u), self.shape, BOOL)

    def un(self, op):
        return self._new(self.c.L.poly_alu1(self.c.ctx, OP[op], self.u))

    def where(self, a, b):
        if not isinstance(a, T): a = self.c.const(a, b.dt if isinstance(b, T) else F32)
        if not isinstance(b, T): b = self.c.const(b, a.dt)
        return T(self.c, self.c.L.poly_where_op(self.c.ctx, self.u, a.u, b.u), self.shape, a.dt)

    def _f1(self, name):
        return self._new(getattr(self.c.L, name)(self.c.ctx, self.u))

    def gelu(self): return self._f1("poly_gelu")
    def relu(self): return self._f1("poly_relu")
    def exp(self): return self._f1("poly_exp")
    def log(self): return self._f1("poly_log")
    def sigmoid(self): return self._f1("poly_sigmoid")
    def tanh(self): return self._f1("poly_tanh_act")
    def sin(self): return self._f1("poly_sin")
    def exp2(self): return self.un("EXP2")
    def log2(self): return self.un("LOG2")
    def sqrt(self): return self.un("SQRT")

    def clamp(self, lo, hi):
        return self._new(self.c.L.poly_clamp(self.c.ctx, self.u, float(lo), float(hi)))

    # reductions and composed ops
    def _red(self, fn, axis, keepdim=False):
        out = (C.c_int64 * 16)()
        nd = C.c_int(0)
        axis = axis % len(self.shape)
        u = getattr(self.c.L, fn)(self.c.ctx, self.u, _i64(self.shape), len(self.shape), axis, 1 if keepdim else 0, out, C.byref(nd))
        return self._new(u, tuple(out[i] for i in range(nd.value)))

    def sum(self, axis=-1, keepdim=False): return self._red("poly_sum_reduce", axis, keepdim)
    def max(self, axis=-1, keepdim=False): return self._red("poly_max_reduce", axis, keepdim)
    def mean(self, axis=-1, keepdim=False): return self._red("poly_mean_reduce", axis, keepdim)

    def reduce_axes(self, op, axes):
        """Raw REDUCE_AXIS over several axes (kept as size-1 dims)."""
        shape = tuple(1 if i in axes else d for i, d in enumerate(self.shape))
        return self._new(self.c.L.poly_reduce_axis(self.c.ctx, OP[op], self.u, _i64(axes), len(axes)), shape)

    def softmax(self, axis=-1):
        return self._new(self.c.L.poly_softmax(self.c.ctx, self.u, _i64(self.shape), len(self.shape), axis))

    def log_softmax(self, axis=-1):
        return self._new(self.c.L.poly_log_softmax(self.c.ctx, self.u, _i64(self.shape), len(self.shape), axis))

    def layernorm(self, eps=1e-5):
        out = (C.c_int64 * 16)()
        nd = C.c_int(0)
        u = self.c.L.poly_layernorm(self.c.ctx, self.u, _i64(self.shape), len(self.shape), -1, float(eps), out, C.byref(nd))
        return self._new(u, tuple(out[i] for i in range(nd.value)))

    def dot(self, w):
        out = (C.c_int64 * 16)()
        nd = C.c_int(0)
        u = self.c.L.poly_dot(self.c.ctx, self.u, _i64(self.shape), len(self.shape), w.u, _i64(w.shape), len(w.shape), out, C.byref(nd))
        return T(self.c, u, tuple(out[i] for i in range(nd.value)), self.dt)

    def cross_entropy(self, target, axis=-1):
        out = (C.c_int64 * 16)()
        nd = C.c_int(0)
        u = self.c.L.poly_cross_entropy(self.c.ctx, self.u, _i64(self.shape), len(self.shape), target.u,
                                        _i64(target.shape), len(target.shape), axis, out, C.byref(nd))
        return T(self.c, u, tuple(out[i] for i in range(nd.value)), self.dt)


# ── bf16 helpers (numpy has no bfloat16) ───────────────────────────────────
def f32_to_bf16_bits(a):
    """Round-to-nearest-even conversion of float32 to bfloat16 bit patterns (uint16)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    u = a.view(np.uint32).astype(np.uint64)
    nan = np.isnan(a)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    r[nan] = 0x7FC0
    return r


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)
