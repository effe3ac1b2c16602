"""GPU parity, first tier: one graph per kernel class, HIP backend (through the
C ABI) against the reference CPU backend on the same seeded inputs.

Tolerances are the ones the task states: bit-exact for integer/index/movement
ops, rtol 1e-5 fp32 elementwise, rtol 1e-4 fp32 reductions and matmul, rtol 2e-2
for bf16/fp16."""
import numpy as np
import pytest

import refpoly as R
from hipharness import assert_close, run_hip, run_ref

pytestmark = [pytest.mark.gpu, pytest.mark.skipif(not R.available(), reason="reference library not built")]


def rng(seed):
    return np.random.default_rng(seed)


def test_fused_chain_fp32():
    c = R.Ctx()
    g = rng(1)
    shape = (256, 512)
    a, b, d, o = (c.buffer(shape, name=n) for n in "abdo")
    y = (a * b + d).exp2().clamp(-4, 4)
    sink = c.sink((o, y))
    arrays = {a: g.uniform(-1, 1, shape).astype(np.float32), b: g.uniform(-1, 1, shape).astype(np.float32),
              d: g.uniform(-1, 1, shape).astype(np.float32), o: np.zeros(shape, np.float32)}
    want = run_ref(c, sink, arrays)
    got, info = run_hip(c, sink, arrays)
    assert info[0]["klass"] == "elementwise"
    assert_close(got[o], want[o], rtol=1e-5, what="chain")
    c.close()


@pytest.mark.parametrize("cols,dt", [(20001, "f32"), (16387, "f32"), (50257, "f32"), (33333, "bf16")])
def test_ragged_long_rows_take_unaligned_vectors_and_a_scalar_tail(cols, dt):
    """Rows whose length is no multiple of the vector width (a vocabulary of 50257): row sum,
    row max and softmax read vectors at element alignment up to the last full one and leave
    the remaining elements to single lanes.  Every row starts at a different alignment; the
    last elements of each row carry the extreme values, so a dropped tail shows."""
    c = R.Ctx()
    g = rng(cols)
    rows = 24
    shape = (rows, cols)
    xf = g.uniform(-1, 1, shape).astype(np.float32)
    xf[:, -1] = 3.0          # the maximum of every row sits in the scalar tail
    xf[:, -2] = -2.5
    if dt == "bf16":
        x = c.buffer(shape, R.BF16, name="x")
        xv = x.cast(R.F32)
        xa = R.f32_to_bf16_bits(xf.ravel()).reshape(shape)
    else:
        x = c.buffer(shape, name="x")
        xv = x
        xa = xf
    s_out, m_out, o = c.buffer((rows,), name="sum"), c.buffer((rows,), name="max"), c.buffer(shape, name="o")
    atol = 1e-6 * float(np.abs(xf).sum(axis=1).max())
    for out, val, zero, what in ((s_out, xv.sum(), np.zeros(rows, np.float32), "sum"), (m_out, xv.max(), np.zeros(rows, np.float32), "max"),
                                 (o, xv.softmax(), np.zeros(shape, np.float32), "softmax")):
        sink = c.sink((out, val))
        sub = {x: xa, out: zero}
        want = run_ref(c, sink, sub)
        got, info = run_hip(c, sink, sub)
        assert any("tail" in k["desc"] for k in info), [k["desc"] for k in info]
        assert_close(got[out], want[out], rtol=1e-4, atol=atol if what == "sum" else 1e-9, what=f"{what} cols={cols} {dt}")
        if what == "max":
            assert np.array_equal(got[out], want[out])
    c.close()


@pytest.mark.parametrize("cols", [8, 100, 128, 1024, 4096, 5000])
def test_row_reductions_fp32(cols):
    c = R.Ctx()
    g = rng(2)
    shape = (96, cols)
    x = c.buffer(shape, name="x")
    s_out, m_out = c.buffer((96,), name="sum"), c.buffer((96,), name="max")
    arrays = {x: g.uniform(-1, 1, shape).astype(np.float32), s_out: np.zeros(96, np.float32), m_out: np.zeros(96, np.float32)}
    # A sum with cancellation is only defined to within the rounding of its
    # terms: the bound is rtol * sum(|x|) (the CPU's left-to-right order and the
    # GPU's tree order are both within it), which for same-sign data is plain rtol.
    atol = 1e-6 * float(np.abs(arrays[x]).sum(axis=1).max())
    for out, val in ((s_out, x.sum()), (m_out, x.max())):
        sink = c.sink((out, val))
        sub = {x: arrays[x], out: arrays[out]}
        want = run_ref(c, sink, sub)
        got, _ = run_hip(c, sink, sub)
        assert_close(got[out], want[out], rtol=1e-4, atol=atol, what=f"reduce cols={cols}")
    c.close()


def test_softmax_layernorm_fp32():
    c = R.Ctx()
    g = rng(3)
    shape = (64, 768)
    x = c.buffer(shape, name="x")
    o = c.buffer(shape, name="o")
    arrays = {x: g.normal(0, 1, shape).astype(np.float32), o: np.zeros(shape, np.float32)}
    for name, val in (("softmax", x.softmax()), ("layernorm", x.layernorm(1e-5))):
        sink = c.sink((o, val))
        want = run_ref(c, sink, arrays)
        got, info = run_hip(c, sink, arrays)
        assert_close(got[o], want[o], rtol=1e-4, atol=1e-6, what=name)
        assert any(k["klass"] == "row-reduce" for k in info)
    c.close()


def test_matmul_fp32_small():
    c = R.Ctx()
    g = rng(4)
    A, B, O = c.buffer((64, 48), name="A"), c.buffer((48, 80), name="B"), c.buffer((64, 80), name="O")
    sink = c.sink((O, A.dot(B)))
    arrays = {A: g.normal(0, 1, (64, 48)).astype(np.float32), B: g.normal(0, 1, (48, 80)).astype(np.float32),
              O: np.zeros((64, 80), np.float32)}
    want = run_ref(c, sink, arrays)
    got, _ = run_hip(c, sink, arrays)
    assert_close(got[O], want[O], rtol=1e-4, atol=1e-5, what="matmul")
    c.close()


def test_movement_ops_bit_exact():
    c = R.Ctx()
    g = rng(5)
    x = c.buffer((6, 10, 8), R.I32, name="x")
    o = c.buffer((8, 5, 8), R.I32, name="o")
    y = x.permute((2, 1, 0)).shrink(((0, 8), (2, 7), (1, 5))).pad(((0, 0), (0, 0), (2, 2))).flip((1,))
    sink = c.sink((o, y))
    arrays = {x: g.integers(-1000, 1000, (6, 10, 8)).astype(np.int32), o: np.zeros((8, 5, 8), np.int32)}
    want = run_ref(c, sink, arrays)
    got, _ = run_hip(c, sink, arrays)
    assert np.array_equal(got[o], want[o])
    c.close()


def test_graph_replay_matches_eager():
    c = R.Ctx()
    g = rng(6)
    shape = (32, 256)
    x, o = c.buffer(shape, name="x"), c.buffer(shape, name="o")
    sink = c.sink((o, x.softmax()))
    arrays = {x: g.normal(0, 1, shape).astype(np.float32), o: np.zeros(shape, np.float32)}
    eager, _ = run_hip(c, sink, arrays, graph=False)
    replay, _ = run_hip(c, sink, arrays, graph=True, repeats=4)
    assert np.array_equal(eager[o], replay[o])
    c.close()


@pytest.mark.parametrize("seed", range(6))
def test_random_graphs_match_reference(seed):
    """Random elementwise / movement / reduction graphs (the generator the oracle is pinned
    with) on the GPU against the reference CPU backend."""
    from test_oracle import _random_graph
    g = np.random.default_rng(1000 + seed)
    c = R.Ctx()
    x, y = c.buffer((6, 8), name="x"), c.buffer((6, 8), name="y")
    val, shape = _random_graph(c, R, g, x, y)
    o = c.buffer(shape, name="o")
    sink = c.sink((o, val))
    bx, by, bo = [t for t, _ in c.buffers]
    arrays = {bx: g.normal(0, 2, 48).astype(np.float32), by: g.normal(0, 2, 48).astype(np.float32),
              bo: np.zeros(int(np.prod(shape)), np.float32)}
    want = run_ref(c, sink, arrays)
    got, _ = run_hip(c, sink, arrays)
    c.close()
    scale = float(np.nanmax(np.abs(want[bo][np.isfinite(want[bo])]))) if np.isfinite(want[bo]).any() else 1.0
    assert_close(got[bo], want[bo], rtol=1e-4, atol=1e-5 * max(scale, 1.0), what=f"random graph {seed}")


@pytest.mark.parametrize("rows,cols", [(4096, 1024), (512, 192), (1024, 100), (500, 128), (544, 192), (608, 64)])
def test_bf16_column_sums_keep_the_reference_order(rows, cols):
    """Sums over the rows of a bf16 matrix accumulate in bf16: every addition rounds, so the
    result depends on the order.  The order-preserving lowering (a kernel that writes the
    terms, four per thread, and one that adds them in index order: blocks of 128 terms
    through alternating load sets, then a tail of single terms when the row count is no
    multiple of 128) must give the reference's bits; so must whatever lowering takes a
    shape it declines."""
    c = R.Ctx()
    g = rng(11)
    x = c.buffer((rows, cols), R.BF16, name="x")
    w = c.buffer((rows, cols), R.BF16, name="w")
    s = c.buffer((rows, 1), R.F32, name="s")
    o1, o2 = c.buffer((cols,), R.BF16, name="o1"), c.buffer((cols,), R.BF16, name="o2")
    bits = lambda shape: R.f32_to_bf16_bits(g.normal(0, 1, int(np.prod(shape))).astype(np.float32))
    arrays = {x: bits((rows, cols)), w: bits((rows, cols)), s: g.uniform(0.5, 2, rows).astype(np.float32)}
    for out, val in ((o1, x.sum(axis=0)), (o2, ((x.cast(R.F32) * s).cast(R.BF16) * w).sum(axis=0))):
        sink = c.sink((out, val))
        sub = {t: a for t, a in arrays.items()}
        sub[out] = np.zeros(cols, np.uint16)
        want = run_ref(c, sink, sub)
        got, info = run_hip(c, sink, sub)
        if rows >= 512 and rows % 32 == 0 and cols >= 64:
            assert any("ordered reduce" in i["desc"] for i in info), [i["desc"] for i in info]
        assert np.array_equal(np.asarray(got[out]).view(np.uint16), np.asarray(want[out]).view(np.uint16)), (rows, cols)
    c.close()
