"""Corners of the boundary that the fixtures' ordinary inputs never reach: the byte fill
(poly_hip_memset, the counterpart of src/runtime_cuda.c:426-435), intermediates their
producers leave holes in (src/exec_plan.c:946-963 is the behaviour kept), buffer
aliasing on and off, host addresses handed in where device memory is expected
(src/frontend.c:2231-2232, src/instance.c:1299-1311 do that on any device), and the
embedding's generic twin (src/modelzoo/models/gpt2.c:93-153 is a masked sum: it has a
value for every input, arange or not)."""
import ctypes as C

import numpy as np
import pytest

import fixtures as F
from hipharness import from_device, to_device
from polygrad_amd import HipPlan, _ffi

pytestmark = pytest.mark.gpu


def test_memset_fills_bytes():
    lib = _ffi.load()
    n = (1 << 20) + 13
    p = lib.poly_hip_alloc(n)
    assert p
    host = np.empty(n, np.uint8)
    want = np.zeros(n, np.uint8)          # fresh allocations read as zero
    for value, off, cnt in ((0xAB, 0, n), (0x00, 5, 1000), (0x7F, n - 7, 7), (0x01, 4096, 0), (0xFF, 1, 3)):
        assert lib.poly_hip_memset(p + off, value, cnt) == 0
        assert lib.poly_hip_sync() == 0
        assert lib.poly_hip_copy_dtoh(host.ctypes.data, p, n) == 0
        want[off:off + cnt] = value
        assert host.tobytes() == want.tobytes(), f"memset value {value:#x} offset {off} count {cnt}"
    lib.poly_hip_free(p)


def _run(fx, inputs=None, runs=2):
    import torch
    plan = HipPlan(fx.plan.schedule, names=fx.plan.names, keepalive=fx.plan)
    dev = [None] * fx.n_slots
    for i in fx.external:
        dev[i] = to_device(fx.inputs[i] if inputs is None else inputs[i])
    torch.cuda.synchronize()
    for _ in range(runs):
        plan.run(dev)
    out = {i: from_device(dev[i], fx.inputs[i].dtype) for i in fx.external}
    work, info = plan.workspace_bytes(), plan.kernel_info()
    plan.close()
    return out, work, info


def test_partly_written_intermediate_reads_zero_where_nothing_was_stored(monkeypatch):
    """The intermediate that is only half written shares its bytes with one that died
    earlier: it can only be cleared right before its first use, on every run."""
    fx = F.Fixture("assembled_partial_store")
    out = (C.c_int * 8)()
    assert _ffi.load().poly_hip_unwritten_slots(fx.plan.schedule, out, 8) == 1
    # as lowered by default the first two kernels are one launch and their intermediate has
    # no memory at all; the results must be the same
    fused, _, info = _run(fx, runs=3)
    assert len(info) == 3, [k["desc"] for k in info]
    for i in fx.external:
        assert fused[i].tobytes() == fx.expected[i].tobytes(), f"slot {i} ({fx.plan.names[i]}), pointwise kernels as one launch"
    monkeypatch.setenv("POLY_HIP_NO_POINTWISE_GROUPS", "1")
    monkeypatch.setenv("POLY_HIP_NO_SIDE_BY_SIDE", "1")      # (kernels one by one, each at its place in the schedule)
    got, work, _ = _run(fx, runs=3)
    for i in fx.external:
        assert got[i].tobytes() == fx.expected[i].tobytes(), f"slot {i} ({fx.plan.names[i]})"
    monkeypatch.setenv("POLY_HIP_NO_ALIAS", "1")
    got2, work2, _ = _run(fx, runs=3)
    assert work < work2, "with aliasing the two intermediates share memory"
    for i in fx.external:
        assert got2[i].tobytes() == fx.expected[i].tobytes(), f"slot {i} without aliasing"


@pytest.mark.parametrize("name", ["gpt2_tiny_bf16", "gpt2_tiny_f32", "mlp_train_b32"])
def test_aliasing_changes_no_bit(monkeypatch, name):
    fx = F.Fixture(name)
    runs = 1 if name == "mlp_train_b32" else 2
    a, work_a, _ = _run(fx, runs=runs)
    monkeypatch.setenv("POLY_HIP_NO_ALIAS", "1")
    b, work_b, _ = _run(fx, runs=runs)
    assert work_a < work_b
    for i in fx.external:
        assert a[i].tobytes() == b[i].tobytes(), f"{name}: slot {i} ({fx.plan.names[i]}) depends on where its intermediates live"


def test_host_pointer_is_refused_not_dereferenced():
    """Through the descriptor row and through the plan: -1 and a message, no launch, and
    the next correct call works."""
    import torch
    lib = _ffi.load()
    fx = F.Fixture("kat_matmul_2x3x4")
    desc = lib.poly_hip_backend_desc().contents
    sched = C.cast(fx.plan.schedule, C.POINTER(_ffi.PolySchedule)).contents
    assert sched.n_items == 1
    item = sched.items[0]
    r = _ffi.PolyRunner()
    assert desc.lower_item(None, item.root, b"hostptr_k0", C.byref(r)) == 0
    slots = [item.buf_slot_indices[j] for j in range(item.n_buf_slots)]
    dev = {s: to_device(fx.inputs[s]) for s in slots}
    host = {s: np.array(fx.inputs[s], copy=True) for s in slots}
    torch.cuda.synchronize()
    for bad in range(len(slots)):
        args = (C.c_void_p * len(slots))(*[host[s].ctypes.data if j == bad else dev[s].data_ptr() for j, s in enumerate(slots)])
        assert desc.execute(C.byref(r), args, len(slots)) == -1, f"host pointer as param {bad} must be refused"
    args = (C.c_void_p * len(slots))(*[dev[s].data_ptr() for s in slots])
    assert desc.execute(C.byref(r), args, len(slots)) == 0
    assert lib.poly_hip_sync() == 0
    out = [s for s in fx.external if fx.plan.names[s] == "O"][0]
    np.testing.assert_allclose(from_device(dev[out], np.float32), fx.expected[out], rtol=1e-6)
    desc.free_runner(C.byref(r))

    plan = lib.poly_hip_compile_schedule(None, fx.plan.schedule)
    assert plan
    data = (C.c_void_p * fx.n_slots)()
    for s in fx.external:
        data[s] = dev[s].data_ptr()
    data[fx.external[1]] = host[fx.external[1]].ctypes.data
    assert lib.poly_hip_plan_run(plan, data, fx.n_slots, None, 0) == -1
    data[fx.external[1]] = dev[fx.external[1]].data_ptr()
    assert lib.poly_hip_plan_run(plan, data, fx.n_slots, None, 0) == 0
    assert lib.poly_hip_sync() == 0
    lib.poly_hip_plan_free(plan)


def _slot(fx, name):
    return [i for i in fx.external if fx.plan.names[i] == name][0]


@pytest.mark.parametrize("case", ["shuffled_arange", "tokens_out_of_range", "fractional_tokens", "duplicate_rows"])
def test_embedding_generic_twin_when_the_guard_fails(case):
    """The gather fast path is only valid when vocab_arange[v] == v; whatever else is
    bound, the result is the reference's masked sum over the vocabulary.  Checked on the
    tiny GPT-2 fixture's schedule against the CPU oracle (which reproduces the reference's
    outputs for this schedule bit for bit on the committed inputs)."""
    fx = F.Fixture("gpt2_tiny_f32")
    inputs = {i: np.array(a, copy=True) for i, a in fx.inputs.items()}
    va, x = _slot(fx, "vocab_arange"), _slot(fx, "x")
    g = np.random.default_rng(5)
    if case == "shuffled_arange":
        inputs[va] = g.permutation(inputs[va]).astype(np.float32)           # a relabelled vocabulary
    elif case == "tokens_out_of_range":
        inputs[x][::3] = np.float32(inputs[va].size + 4)                      # no row matches: zeros
        inputs[x][1::5] = np.float32(-2)
    elif case == "fractional_tokens":
        inputs[x][::2] += np.float32(0.5)                                     # equal to no arange entry
    elif case == "duplicate_rows":
        inputs[va][7] = inputs[va][3]                                          # two rows match token 3: their sum
        inputs[x][:4] = inputs[va][3]
    want = F.run_oracle_schedule(fx.plan.schedule, fx.n_slots, inputs)
    got, _, info = _run(fx, inputs=inputs)
    assert any(k["klass"] == "gather" for k in info), [k["klass"] for k in info]
    out = _slot(fx, "output")
    assert not np.array_equal(want[out], fx.expected[out]), "the altered inputs must change the logits"
    np.testing.assert_allclose(got[out], want[out], rtol=1e-4, atol=1e-5)


def test_embedding_with_a_relabelled_vocabulary_matches_the_live_reference():
    """The same through the reference itself where its library travels with the tests: the
    embedding graph alone (src/modelzoo/models/gpt2.c:93-153), arange buffer shuffled."""
    import graphs
    import refpoly as R
    from hipharness import run_hip, run_ref
    if not R.available():
        pytest.skip("reference library not built")
    V, D, B, T = 301, 48, 3, 20
    g = np.random.default_rng(9)
    c = R.Ctx()
    table, idx = c.buffer((V, D), name="wte"), c.buffer((B, T), name="x")
    ar, out = c.buffer((V,), name="vocab_arange"), c.buffer((B, T, D), name="out")
    sink = c.sink((out, graphs._embedding(c, table, V, D, idx, (B, T), ar, R.F32)))
    labels = g.permutation(V).astype(np.float32)
    labels[11] = labels[10]                        # one label twice, one missing
    tokens = g.integers(0, V, B * T).astype(np.float32)
    tokens[5] = 1e6
    tokens[6] += 0.25
    arrays = {table: g.normal(0, 1, V * D).astype(np.float32), idx: tokens, ar: labels, out: np.zeros(B * T * D, np.float32)}
    want = run_ref(c, sink, arrays)[out]
    got, info = run_hip(c, sink, arrays, repeats=2)
    assert any(k["klass"] == "gather" for k in info), [k["klass"] for k in info]
    np.testing.assert_allclose(got[out], want, rtol=1e-5, atol=1e-6)
    c.close()
