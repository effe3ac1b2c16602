"""Symbolic sizes: a RANGE bounded by a DEFINE_VAR, whose value arrives with every run
(src/exec_plan.c:1026-1041 passes it as a pointer to a host int; the plan-level entry
point takes PolyVarBinding pairs).  Mirrors test/test_nn.c:849-985 of the reference: one
compiled plan, run with several values of N; elements past N stay untouched."""
import ctypes as C

import numpy as np
import pytest

import refpoly as R
from hipharness import from_device, schedule_slots, to_device
from polygrad_amd import HipPlan

pytestmark = pytest.mark.gpu

NMAX = 5000


def build(reduce_it):
    c = R.Ctx()
    N = c.define_var("N", 1, NMAX)
    a = c.buffer_var(N, NMAX, name="a")
    if reduce_it:
        o = c.buffer((1,), name="o")
        val = (a * a).sum()
        store = c.L.poly_store_val(c.ctx, o.buf, val.reshape((1,)).u)
    else:
        o = c.buffer_var(N, NMAX, name="o")
        store = c.L.poly_store_val(c.ctx, o.buf, (a * c.const(2.0) + c.const(1.0)).u)
    sink = c.L.poly_sink1(c.ctx, store)
    sched = c.schedule(sink)
    slots, n = schedule_slots(c, sched)
    plan = HipPlan(sched, ctx=c.ctx, names=[slots[i][1] if i in slots and slots[i] else None for i in range(n)])
    return c, N, sched, slots, n, plan


def test_elementwise_with_symbolic_length():
    c, N, sched, slots, n, plan = build(False)
    g = np.random.default_rng(5)
    x = g.normal(0, 1, NMAX).astype(np.float32)
    for value in (4, 257, 4096, NMAX, 1):
        dev = [None] * n
        for i, (t, name) in slots.items():
            dev[i] = to_device(x if name == "a" else np.full(NMAX, -999.0, np.float32))
        plan.run(dev, var_bindings=[(N, value)])
        out = from_device([dev[i] for i, (t, name) in slots.items() if name == "o"][0], np.float32)
        assert np.array_equal(out[:value], x[:value] * np.float32(2.0) + np.float32(1.0)), value
        assert (out[value:] == -999.0).all(), f"N={value}: elements past N were written"
    # without a value for N (and no default in the schedule) the run is refused
    with pytest.raises(RuntimeError):
        plan.run(dev)
    plan.close()
    c.L.poly_schedule_free(sched)
    c.close()


def test_kernel_that_ignores_the_variable_of_its_buffer():
    """The frontend's reductions take explicit integer shapes, so a sum over a buffer sized by
    N walks the whole allocation: the schedule lists N for the kernel, the kernel has no use
    for it, and the plan must still bind and run it (variables are matched by identity, not
    by position)."""
    c, N, sched, slots, n, plan = build(True)
    g = np.random.default_rng(6)
    x = g.normal(0, 1, NMAX).astype(np.float32)
    want = float(np.sum(x.astype(np.float64) ** 2))
    for value in (1, 3000):
        dev = [None] * n
        for i, (t, name) in slots.items():
            dev[i] = to_device(x if name == "a" else np.zeros(1, np.float32))
        plan.run(dev, var_bindings=[(N, value)])
        out = from_device([dev[i] for i, (t, name) in slots.items() if name == "o"][0], np.float32)
        assert abs(float(out[0]) - want) <= 1e-4 * want, (value, out[0], want)
    plan.close()
    c.L.poly_schedule_free(sched)
    c.close()
