"""The drop-in boundary itself: every fixture schedule is driven through the
PolyBackendDesc row (lower_item / execute / free_runner / get_allocator) in the
order the reference's poly_compile_schedule (src/exec_plan.c:801-932) and
poly_compiled_plan_run (src/exec_plan.c:934-1060) use it -- one lower_item per
kernel, intermediates from allocator->alloc, args[i] = pointer of PARAM i,
one execute per kernel in exec_order, results through allocator->copy_out."""
import ctypes as C

import numpy as np
import pytest

import fixtures as F
from hipharness import assert_close
from polygrad_amd import _ffi
from test_gpu_fixtures import BIT_EXACT, STATEFUL, TOL

pytestmark = pytest.mark.gpu


def run_through_vtable(fx):
    lib = _ffi.load()
    desc = lib.poly_hip_backend_desc().contents
    assert desc.name == b"hip" and not desc.host_executed
    alloc = desc.get_allocator().contents
    sched = C.cast(fx.plan.schedule, C.POINTER(_ffi.PolySchedule)).contents

    # compile: one runner per item (exec_plan.c:826-858)
    runners = []
    for k in range(sched.n_items):
        item = sched.items[k]
        r = _ffi.PolyRunner()
        r.kind = 99
        rc = desc.lower_item(None, item.root, f"lower0_k{k}".encode(), C.byref(r))
        assert rc == 0 and r.handle, f"{fx.name}: lower_item failed for kernel {k}"
        assert r.kind == 0, "runner kind must be POLY_RUNNER_COMPILED"
        runners.append(r)

    # buffers: externals uploaded by the caller, intermediates from the allocator (exec_plan.c:860-881)
    ptr = [None] * fx.n_slots
    for i in range(fx.n_slots):
        slot = sched.buf_slots[i]
        p = alloc.alloc(max(int(slot.nbytes), 1), alloc.dev_ctx)
        assert p, "allocator returned NULL"
        ptr[i] = p
        if not slot.is_intermediate:
            a = np.ascontiguousarray(fx.inputs[i])
            assert alloc.copy_in(p, a.ctypes.data, a.nbytes, alloc.dev_ctx) == 0

    # run: args in PARAM order, kernels in exec_order (exec_plan.c:1010-1056)
    for _ in range(1 if fx.name in STATEFUL else 2):
        for e in range(sched.n_items):
            k = sched.exec_order[e]
            item = sched.items[k]
            assert item.n_var_uops == 0
            args = (C.c_void_p * item.n_buf_slots)(*[ptr[item.buf_slot_indices[j]] for j in range(item.n_buf_slots)])
            assert desc.execute(C.byref(runners[k]), args, item.n_buf_slots) == 0

    out = {}
    for i in fx.external:
        a = np.empty_like(fx.inputs[i])
        assert alloc.copy_out(a.ctypes.data, ptr[i], a.nbytes, alloc.dev_ctx) == 0
        out[i] = a
    for r in runners:
        desc.free_runner(C.byref(r))
    for p in ptr:
        alloc.free(p, alloc.dev_ctx)
    return out


@pytest.mark.parametrize("name", F.case_names())
def test_fixture_through_backend_descriptor(name):
    fx = F.Fixture(name)
    got = run_through_vtable(fx)
    for slot in fx.external:
        want = fx.expected[slot]
        if name in BIT_EXACT:
            assert got[slot].tobytes() == want.tobytes(), f"{name}: slot {slot} not bit-exact"
        else:
            rtol, atol = TOL[name]
            assert_close(F.as_float(got[slot]), F.as_float(want), rtol=rtol, atol=atol, what=f"{name} slot {slot}")


def test_copy_between_and_zero_filled_alloc():
    lib = _ffi.load()
    alloc = lib.poly_hip_get_allocator().contents
    n = 1 << 20
    a = alloc.alloc(n, alloc.dev_ctx)
    b = alloc.alloc(n, alloc.dev_ctx)
    host = np.full(n, 7, np.uint8)
    assert alloc.copy_out(host.ctypes.data, a, n, alloc.dev_ctx) == 0
    assert not host.any(), "fresh allocations read as zero, like the reference's host allocator"
    src = (np.arange(n) % 251).astype(np.uint8)
    assert alloc.copy_in(a, src.ctypes.data, n, alloc.dev_ctx) == 0
    assert alloc.copy_between(b, a, n, alloc.dev_ctx) == 0
    assert alloc.copy_out(host.ctypes.data, b, n, alloc.dev_ctx) == 0
    assert host.tobytes() == src.tobytes()
    alloc.free(a, alloc.dev_ctx)
    alloc.free(b, alloc.dev_ctx)
