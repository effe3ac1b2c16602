"""Indexing of the generated kernels, checked without a GPU: every kernel of every
golden fixture and of the reduced training step runs on the host under
AddressSanitizer (tests/hostcheck.py), so an out-of-bounds load or store -- which on the
device may go unnoticed or fault the card -- fails here with the offending line."""
import ctypes as C
import os

import pytest

import fixtures as F
import hostcheck
import refpoly as R
from polygrad_amd import _ffi

pytestmark = pytest.mark.skipif(not os.path.exists(hostcheck.CLANG), reason="no host clang with AddressSanitizer")


def test_checker_sees_an_overrun(hiplib):
    fx = F.Fixture("bf16_matmul")
    jobs = list(hostcheck._jobs(hiplib, fx.plan.schedule, 1 << 21, None, False))
    what, main, grid, block, sizes, _ = jobs[0]
    hostcheck.check_kernel(main, hostcheck._entry_name(main), grid, block, sizes)
    with pytest.raises(AssertionError, match="out-of-bounds"):
        hostcheck.check_kernel(main, hostcheck._entry_name(main), grid, block, [sizes[0] // 2] + list(sizes[1:]))


def test_fixture_kernels_stay_in_bounds(hiplib):
    total = 0
    for name in F.case_names():
        fx = F.Fixture(name)            # owns the schedule's memory
        total += hostcheck.check_schedule(hiplib, fx.plan.schedule)
    assert total > 100


@pytest.mark.skipif(not R.available(), reason="reference library not built")
@pytest.mark.parametrize("B,T,D,H,V", [(1, 32, 64, 2, 97), (2, 64, 128, 4, 301), (1, 128, 128, 2, 97)])
def test_training_step_kernels_stay_in_bounds(B, T, D, H, V, hiplib):
    """The backward kernels of the one-block training step: among them the derivative of a
    pad, `where(valid, reduce(...), 0)`, whose index arithmetic goes negative on the masked
    positions (a modulus emitted as C's % read in front of its buffer there), and, at the
    larger size, the matmul-shaped reductions with computed operands and ragged extents."""
    import graphs
    c = R.Ctx()
    _, sink = graphs.gpt2_block_train_step(c, B, T, D, H, V)
    sched = c.schedule(sink)
    try:
        n = hostcheck.check_schedule(hiplib, sched)
    finally:
        c.L.poly_schedule_free(sched)
        c.close()
    assert n > 60


@pytest.mark.parametrize("name", ["mlp_train_f32_b4096", "gpt2_small_bf16_b1_t1024", "attention_bf16_b8_h12_t1024_d64",
                                  "matmul_bf16_b16_1024x1024x1024", "rowops_f32_8192_softmax"])
def test_benchmark_plan_kernels_stay_in_bounds(name, hiplib):
    """The benchmark plans at their real shapes (large launches sampled by workgroup):
    MFMA templates, the fused attention kernel, matmul epilogues, row chains, the two-stage
    reductions of the MLP step."""
    from polygrad_amd import PlanFile
    pf = PlanFile(os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "polygrad_amd", "plans", name + ".polyplan"))
    assert hostcheck.check_schedule(hiplib, pf.schedule) >= 1


@pytest.mark.skipif(not R.available(), reason="reference library not built")
def test_bf16_plane_kernels_stay_in_bounds(hiplib):
    """The four kernels of a matmul whose fp32 operand is cut into bf16 planes (two
    first-stage kernels writing the planes, the 16-bit MFMA template reading them with its
    K tiles dealt to three workgroups per output tile, the kernel adding their partial
    results behind the planes in scratch memory), with a depth that is not a multiple of
    the K tile."""
    import numpy as np
    import test_gpu_matmul as T
    c = R.Ctx()
    sink, _, _ = T._planes_case(c, np.random.default_rng(0))
    sched = c.schedule(sink)
    try:
        assert hostcheck.check_schedule(hiplib, sched) == 4
    finally:
        c.L.poly_schedule_free(sched)
        c.close()


@pytest.mark.skipif(not R.available(), reason="reference library not built")
@pytest.mark.parametrize("cols,bf", [(20001, False), (50257, False), (33333, True)])
def test_ragged_row_kernels_stay_in_bounds(cols, bf, hiplib):
    """Row sum and softmax over rows whose length is no multiple of the vector width:
    unaligned vector accesses up to the last full vector, single lanes for the rest."""
    c = R.Ctx()
    shape = (6, cols)
    x = c.buffer(shape, R.BF16 if bf else R.F32, name="x")
    xv = x.cast(R.F32) if bf else x
    s_out, o = c.buffer((6,), name="s"), c.buffer(shape, name="o")
    for out, val in ((s_out, xv.sum()), (o, xv.softmax())):
        sched = c.schedule(c.sink((out, val)))
        try:
            assert hostcheck.check_schedule(hiplib, sched) >= 1
        finally:
            c.L.poly_schedule_free(sched)
    c.close()


@pytest.mark.skipif(not R.available(), reason="reference library not built")
@pytest.mark.parametrize("tb", [False, True])
def test_split_k_matmul_stays_in_bounds(tb, hiplib):
    """A bf16 product with ragged M and N whose K tiles are dealt to two workgroups per
    tile: the template writing partial results to scratch memory and the adder."""
    import graphs
    c = R.Ctx()
    _, _, _, sink = graphs.matmul_bf16(c, 200, 328, 8192, transposed_b=tb)
    sched = c.schedule(sink)
    try:
        sp = C.cast(sched, C.POINTER(_ffi.PolySchedule)).contents
        assert "K dealt to 2" in _ffi.take_string(hiplib.poly_hip_describe(sp.items[0].root, 0))
        assert hostcheck.check_schedule(hiplib, sched) == 2
    finally:
        c.L.poly_schedule_free(sched)
        c.close()


@pytest.mark.skipif(not R.available(), reason="reference library not built")
@pytest.mark.parametrize("b,t,m,n,tm", [(4, 64, 256, 384, False), (4, 64, 256, 384, True), (3, 64, 136, 200, False)])
def test_matmul_over_two_reduce_ranges_stays_in_bounds(b, t, m, n, tm, hiplib):
    """dW = X^T dY summed over batch and position on the plain bf16 template: the two reduce
    ranges as one depth (nested strides) or as a depth of two levels (X stored time major),
    a row-contiguous A and a column-contiguous B, ragged M and N in the last case."""
    import graphs
    c = R.Ctx()
    _, _, _, sink = graphs.matmul_bf16_over_two_ranges(c, b, t, m, n, time_major_a=tm)
    sched = c.schedule(sink)
    try:
        sp = C.cast(sched, C.POINTER(_ffi.PolySchedule)).contents
        d = _ffi.take_string(hiplib.poly_hip_describe(sp.items[0].root, 0))
        assert d.startswith("matmul-mfma: mfma 32x32x16 bf16") and "A:m-major B:n-major" in d, d
        assert hostcheck.check_schedule(hiplib, sched) == 1
    finally:
        c.L.poly_schedule_free(sched)
        c.close()


@pytest.mark.skipif(not R.available(), reason="reference library not built")
@pytest.mark.parametrize("tb,batch", [(False, None), (True, None), (False, 3)])
def test_operand_read_in_place_beside_planes_stays_in_bounds(tb, batch, hiplib, monkeypatch):
    """fp32 x bf16 with the fp32 operand as three bf16 planes and the bf16 buffer read where
    it lies (rows along n, rows along k, per batch), K dealt to three workgroups per tile."""
    monkeypatch.setenv("POLY_HIP_BF16_SPLIT_MIN", "1048576")
    M, N, K = 256, 320, 4096 if batch is None else 2048
    c = R.Ctx()
    lead = () if batch is None else (batch,)
    A = c.buffer(lead + (M, K), R.F32, name="A")
    Bm = c.buffer(lead + ((N, K) if tb else (K, N)), R.BF16, name="B")
    O = c.buffer(lead + (M, N), R.F32, name="C")
    b = Bm.permute(tuple(range(len(lead))) + (len(lead) + 1, len(lead))) if tb else Bm
    sched = c.schedule(c.sink((O, (A * c.const(0.75)).dot(b.cast(R.F32)))))
    try:
        sp = C.cast(sched, C.POINTER(_ffi.PolySchedule)).contents
        assert "B read in place" in _ffi.take_string(hiplib.poly_hip_describe(sp.items[0].root, 0))
        assert hostcheck.check_schedule(hiplib, sched) == 3      # A's planes, the template, the adder of the partial results
    finally:
        c.L.poly_schedule_free(sched)
        c.close()


@pytest.mark.skipif(not R.available(), reason="reference library not built")
def test_slabs_that_share_operand_planes_stay_in_bounds(hiplib, monkeypatch):
    """The training step with the bf16-planes path taken at this small size: the second slab
    of the q/k/v derivative reads the first slab's planes of dS out of the scratch memory,
    rows along the depth."""
    import graphs
    monkeypatch.setenv("POLY_HIP_BF16_SPLIT_MIN", "1048576")
    c = R.Ctx()
    _, sink = graphs.gpt2_block_train_step(c, 1, 128, 128, 2, 97)
    sched = c.schedule(sink)
    try:
        sp = C.cast(sched, C.POINTER(_ffi.PolySchedule)).contents
        descs = [_ffi.take_string(hiplib.poly_hip_describe(sp.items[i].root, 0)) for i in range(sp.n_items)]
        slabs = [d for d in descs if "3 slabs of one output range" in d]
        assert len(slabs) == 1 and "rows and depth exchanged" in slabs[0], slabs
        assert hostcheck.check_schedule(hiplib, sched) > 60
    finally:
        c.L.poly_schedule_free(sched)
        c.close()


@pytest.mark.skipif(not R.available(), reason="reference library not built")
@pytest.mark.parametrize("rows,cols", [(512, 192), (1024, 100), (544, 192)])
def test_ordered_column_sum_stays_in_bounds(rows, cols, hiplib):
    """The order-preserving bf16 column sum (a kernel that writes the terms, one that adds
    them in order), with a column count that leaves the adder's last workgroup partly idle."""
    c = R.Ctx()
    x, w = (c.buffer((rows, cols), R.BF16, name=n) for n in "xw")
    s = c.buffer((rows, 1), R.F32, name="s")
    o = c.buffer((cols,), R.BF16, name="o")
    sched = c.schedule(c.sink((o, ((x.cast(R.F32) * s).cast(R.BF16) * w).sum(axis=0))))
    try:
        sp = C.cast(sched, C.POINTER(_ffi.PolySchedule)).contents
        assert "ordered reduce" in _ffi.take_string(hiplib.poly_hip_describe(sp.items[0].root, 0))
        assert hostcheck.check_schedule(hiplib, sched) == 2      # the terms kernel and the adder
    finally:
        c.L.poly_schedule_free(sched)
        c.close()
