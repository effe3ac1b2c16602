"""Shared helpers for the parity tests: run one tensor-level graph through the
reference CPU backend and through the HIP backend (C ABI), and compare."""
import ctypes as C

import numpy as np

import refpoly as R
from polygrad_amd import HipPlan, _ffi

_TORCH_DT = None


def torch_dtype(dt):
    import torch
    global _TORCH_DT
    if _TORCH_DT is None:
        _TORCH_DT = {R.BOOL: torch.bool, R.I8: torch.int8, R.U8: torch.uint8, R.I16: torch.int16,
                     R.U16: torch.int16, R.I32: torch.int32, R.U32: torch.int32, R.I64: torch.int64,
                     R.U64: torch.int64, R.F16: torch.float16, R.BF16: torch.int16, R.F32: torch.float32,
                     R.F64: torch.float64}
    return _TORCH_DT[dt]


def to_device(a):
    """numpy -> CUDA tensor with the same bytes (dtypes torch lacks are carried as same-size ints)."""
    import torch
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).cuda()
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).cuda()
    if a.dtype == np.uint64:
        return torch.from_numpy(a.view(np.int64)).cuda()
    return torch.from_numpy(a).cuda()


def from_device(t, np_dtype):
    a = t.cpu().numpy()
    return a.view(np_dtype) if a.dtype != np_dtype else a


def schedule_slots(c, sched):
    """External slot index -> buffer T, matched through the slot's BUFFER UOp pointer."""
    s = C.cast(sched, C.POINTER(_ffi.PolySchedule)).contents
    by_ptr = {t.buf: (t, name) for t, name in c.buffers}
    out = {}
    for i in range(s.n_buf_slots):
        sl = s.buf_slots[i]
        if not sl.is_intermediate:
            out[i] = by_ptr.get(sl.buf_uop)
    return out, s.n_buf_slots


def constant_slots(c, sched):
    """External slots that are not caller buffers but constants the reference frontend
    created itself (poly_arange inside poly_cross_entropy, src/frontend.c:1213, registered
    at :253): slot index -> float32 array, read through poly_const_buffer_data
    (src/frontend.h:156), which is how poly_realize fills them (src/frontend.c:2232)."""
    s = C.cast(sched, C.POINTER(_ffi.PolySchedule)).contents
    known = {t.buf for t, _ in c.buffers}
    out = {}
    for i in range(s.n_buf_slots):
        sl = s.buf_slots[i]
        if sl.is_intermediate or sl.buf_uop in known:
            continue
        p = c.L.poly_const_buffer_data(c.ctx, sl.buf_uop)
        if p:
            assert sl.nbytes == 4 * sl.numel, "registry constants are float32"
            out[i] = np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_float)), shape=(int(sl.numel),)).copy()
    return out


def constant_name(a):
    """Plan files carry no data: a registry constant is stored by a name that says how to
    rebuild it (only aranges occur)."""
    if np.array_equal(a, np.arange(a.size, dtype=np.float32)):
        return f"__arange_{a.size}"
    raise RuntimeError("registry constant that is not an arange")


def run_hip(c, sink, arrays, graph=True, repeats=1):
    """Runs `sink` on the GPU through the plan-level C ABI.  arrays: {buffer T: ndarray}
    (inputs and outputs).  Returns {buffer T: ndarray} with device contents after the run."""
    import torch
    sched = c.schedule(sink)
    slots, n = schedule_slots(c, sched)
    names = [None] * n
    for i, tn in slots.items():
        if tn is not None:
            names[i] = tn[1]
    consts = constant_slots(c, sched)
    for i, a in consts.items():
        names[i] = constant_name(a)
    plan = HipPlan(sched, ctx=c.ctx, names=names)
    dev = [None] * n
    owner = {}
    for i, tn in slots.items():
        if tn is None and i in consts:
            dev[i] = to_device(consts[i])
            continue
        if tn is None:
            raise RuntimeError(f"external slot {i} has no known buffer")
        t = tn[0]
        if t not in arrays:
            raise RuntimeError(f"no array bound for buffer {tn[1]}")
        dev[i] = to_device(arrays[t])
        owner[i] = t
    torch.cuda.synchronize()
    plan.set_graph(graph)
    for _ in range(repeats):
        plan.run(dev)
    out = {owner[i]: from_device(dev[i], arrays[owner[i]].dtype) for i in owner}
    info = plan.kernel_info()
    run_hip.side_launches = plan.side_launches()      # of the last plan run (tests of the second stream read it)
    plan.close()
    c.L.poly_schedule_free(sched)
    return out, info


def run_ref(c, sink, arrays):
    """Runs `sink` on the reference CPU backend, in place on copies; returns the copies."""
    copies = {t: np.array(a, copy=True) for t, a in arrays.items()}
    c.realize_cpu(sink, copies)
    return copies


def assert_close(got, want, rtol, atol=0.0, what=""):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    both_nan = np.isnan(got) & np.isnan(want)
    same_inf = np.isinf(got) & np.isinf(want) & (np.sign(got) == np.sign(want))
    ok = both_nan | same_inf | (np.abs(got - want) <= atol + rtol * np.abs(want))
    if not ok.all():
        bad = np.argwhere(~ok)
        i = tuple(bad[0])
        raise AssertionError(f"{what}: {len(bad)} of {got.size} elements differ beyond rtol={rtol} atol={atol}; "
                             f"first at {i}: got {got[i]!r} want {want[i]!r}")
