"""GPU parity of the MFMA matmul template against the reference CPU backend:
bf16 / fp16 inputs, fp32 accumulate, every operand layout the template
distinguishes (k-major and row-major operands, batches, broadcast batch,
two-level K from merged heads, bias epilogue, ragged M and N)."""
import numpy as np
import pytest

import graphs
import refpoly as R
from hipharness import assert_close, run_hip, run_ref

pytestmark = [pytest.mark.gpu, pytest.mark.skipif(not R.available(), reason="reference library not built")]


def bf16(g, shape, scale=0.02):
    return R.f32_to_bf16_bits(g.normal(0, scale, int(np.prod(shape))).astype(np.float32))


def check(c, sink, arrays, out, what, rtol=1e-3, expect_mfma=True):
    want = run_ref(c, sink, arrays)
    got, info = run_hip(c, sink, arrays)
    if expect_mfma:
        assert any(k["klass"] == "matmul-mfma" for k in info), [k["desc"] for k in info]
    w, h = want[out], got[out]
    if w.dtype == np.uint16:
        w, h = R.bf16_bits_to_f32(w), R.bf16_bits_to_f32(h)
    # accumulation order differs: tolerance relative to the magnitude of the sums
    atol = rtol * float(np.abs(w).mean() + 1e-12)
    assert_close(h, w, rtol=rtol, atol=atol, what=what)


@pytest.mark.parametrize("m,n,k,tb", [(256, 512, 128, False), (256, 512, 128, True), (128, 192, 64, False),
                                       (200, 328, 192, True), (136, 128, 64, False), (64, 1000, 64, True)])
def test_matmul_bf16_layouts(m, n, k, tb):
    c = R.Ctx()
    g = np.random.default_rng(m * 7 + n)
    A, Bm, O, sink = graphs.matmul_bf16(c, m, n, k, transposed_b=tb)
    arrays = {A: bf16(g, (m, k)), Bm: bf16(g, (k, n)), O: np.zeros(m * n, np.float32)}
    check(c, sink, arrays, O, f"matmul {m}x{n}x{k} tb={tb}")
    c.close()


@pytest.mark.parametrize("tb", [False, True])
def test_matmul_bf16_deep_product_on_few_tiles_is_split_along_k(tb):
    """A deep product with few output tiles: the K tiles of a tile are dealt to several
    workgroups and a second kernel adds their fp32 partial results in split order (ragged
    M and N, so the partial stores meet both edges).  Against the reference, and against
    the unsplit kernel of the same graph (POLY_HIP_NO_SPLIT_K)."""
    import os
    m, n, k = 200, 328, 8192
    c = R.Ctx()
    g = np.random.default_rng(31 + tb)
    A, Bm, O, sink = graphs.matmul_bf16(c, m, n, k, transposed_b=tb)
    arrays = {A: bf16(g, (m, k), 1.0), Bm: bf16(g, (k, n), 1.0), O: np.zeros(m * n, np.float32)}
    want = run_ref(c, sink, arrays)
    got, info = run_hip(c, sink, arrays)
    assert any("K dealt to" in k_["desc"] and "32x32x16" in k_["desc"] for k_ in info), [k_["desc"] for k_ in info]
    os.environ["POLY_HIP_NO_SPLIT_K"] = "1"
    try:
        got1, info1 = run_hip(c, sink, arrays)
    finally:
        del os.environ["POLY_HIP_NO_SPLIT_K"]
    c.close()
    assert not any("K dealt to" in k_["desc"] for k_ in info1)
    w = want[O].astype(np.float64)
    bound = 1e-4 * float(np.abs(w).mean())
    assert_close(got[O], want[O], rtol=1e-4, atol=bound, what="split-K vs reference")
    assert_close(got1[O], want[O], rtol=1e-4, atol=bound, what="unsplit vs reference")
    assert float(np.abs(got[O].astype(np.float64) - got1[O]).max()) <= 2e-5 * float(np.abs(w).max())


@pytest.mark.parametrize("b,t,m,n,tm", [(4, 64, 256, 384, False), (4, 64, 256, 384, True), (3, 64, 136, 200, False)])
def test_matmul_bf16_reduce_over_two_ranges(b, t, m, n, tm):
    """dW = X^T dY summed over batch and position: the REDUCE runs over two ranges.  Where
    the strides of both operands nest they are one depth; where they do not (X stored time
    major) the depth has two levels.  Either way the operands are read where they lie: no
    launch that rewrites them first."""
    c = R.Ctx()
    g = np.random.default_rng(b * 1000 + m + tm)
    X, Y, O, sink = graphs.matmul_bf16_over_two_ranges(c, b, t, m, n, time_major_a=tm)
    arrays = {X: bf16(g, (b, t, m), 1.0), Y: bf16(g, (b, t, n), 1.0), O: np.zeros(m * n, np.float32)}
    want = run_ref(c, sink, arrays)
    got, info = run_hip(c, sink, arrays)
    c.close()
    assert len(info) == 1 and info[0]["klass"] == "matmul-mfma" and "planes" not in info[0]["desc"], [k_["desc"] for k_ in info]
    bound = 1e-4 * float(np.abs(want[O]).mean())
    assert_close(got[O], want[O], rtol=1e-4, atol=bound, what="two reduce ranges vs reference")
    # the definition, in float64 (the products of bf16 values are exact there)
    x = R.bf16_bits_to_f32(arrays[X]).astype(np.float64).reshape((t, b, m) if tm else (b, t, m))
    if tm:
        x = x.transpose(1, 0, 2)
    y = R.bf16_bits_to_f32(arrays[Y]).astype(np.float64).reshape(b, t, n)
    exact = np.einsum("btm,btn->mn", x, y)
    assert float(np.abs(got[O].reshape(m, n) - exact).max()) <= 1e-5 * float(np.abs(exact).max()) + 1e-4 * float(np.abs(exact).mean())


def test_matmul_broadcast_batch():
    c = R.Ctx()
    g = np.random.default_rng(11)
    A, Bm, O, sink = graphs.matmul_bf16(c, 128, 128, 64, batch=4)
    arrays = {A: bf16(g, (4, 128, 64)), Bm: bf16(g, (64, 128)), O: np.zeros(4 * 128 * 128, np.float32)}
    check(c, sink, arrays, O, "broadcast batch")
    c.close()


def test_matmul_fp16():
    c = R.Ctx()
    g = np.random.default_rng(12)
    A = c.buffer((128, 64), R.F16, name="A")
    B = c.buffer((64, 128), R.F16, name="B")
    O = c.buffer((128, 128), R.F32, name="C")
    sink = c.sink((O, A.cast(R.F32).dot(B.cast(R.F32))))
    arrays = {A: g.normal(0, 0.5, (128, 64)).astype(np.float16), B: g.normal(0, 0.5, (64, 128)).astype(np.float16),
              O: np.zeros((128, 128), np.float32)}
    check(c, sink, arrays, O, "fp16 matmul")
    c.close()


def test_attention_shaped_matmuls_with_bias_and_merged_heads():
    """The four matmul forms of one GPT-2 block at a reduced size: QK^T (both operands
    k-major, two batch dims with non-nesting strides), attn@V (row-major B), merged
    heads @ W + bias (A with a two-level K index), all with bf16 outputs."""
    B, T, H, hd = 2, 128, 2, 64
    D = H * hd
    c = R.Ctx()
    g = np.random.default_rng(13)
    q, k, v = (c.buffer((B, T, D), R.BF16, name=n) for n in "qkv")
    w = c.buffer((D, D), R.BF16, name="w")
    bias = c.buffer((D,), R.BF16, name="bias")
    scores_o = c.buffer((B, H, T, T), R.BF16, name="scores")
    ctx_o = c.buffer((B, H, T, hd), R.BF16, name="ctx")
    proj_o = c.buffer((B, T, D), R.BF16, name="proj")
    qh = q.reshape((B, T, H, hd)).permute((0, 2, 1, 3))
    kh = k.reshape((B, T, H, hd)).permute((0, 2, 1, 3))
    vh = v.reshape((B, T, H, hd)).permute((0, 2, 1, 3))
    scores = qh.cast(R.F32).dot(kh.permute((0, 1, 3, 2)).cast(R.F32)).cast(R.BF16)
    arr = {q: bf16(g, (B, T, D), 1.0), k: bf16(g, (B, T, D), 1.0), v: bf16(g, (B, T, D), 1.0),
           w: bf16(g, (D, D), 0.1), bias: bf16(g, (D,), 1.0)}
    a1 = {q: arr[q], k: arr[k], scores_o: np.zeros(B * H * T * T, np.uint16)}
    check(c, c.sink((scores_o, scores)), a1, scores_o, "QK^T", rtol=2e-2)
    attn = c.buffer((B, H, T, T), R.BF16, name="attn")
    ctxv = attn.cast(R.F32).dot(vh.cast(R.F32)).cast(R.BF16)
    a2 = {attn: bf16(g, (B, H, T, T), 0.1), v: arr[v], ctx_o: np.zeros(B * H * T * hd, np.uint16)}
    check(c, c.sink((ctx_o, ctxv)), a2, ctx_o, "attn@V", rtol=2e-2)
    ctx_in = c.buffer((B, H, T, hd), R.BF16, name="ctx_in")
    merged = ctx_in.permute((0, 2, 1, 3)).reshape((B, T, D))
    proj = merged.cast(R.F32).dot(w.cast(R.F32)).cast(R.BF16) + bias.reshape((1, 1, D)).expand((B, T, D))
    a3 = {ctx_in: bf16(g, (B, H, T, hd), 1.0), w: arr[w], bias: arr[bias], proj_o: np.zeros(B * T * D, np.uint16)}
    check(c, c.sink((proj_o, proj)), a3, proj_o, "merged heads @ W + bias", rtol=2e-2)
    c.close()


def test_full_size_row_block_matches_cpu_bit_pattern_of_sums():
    """At a benchmark shape (4096^3 is too slow on one CPU core) the CPU result of a
    row block is the full result for those rows: compare 8 rows of a 1024x4096x4096
    product computed on the GPU at full size with the CPU backend on the 8-row slice."""
    m, n, k = 1024, 4096, 4096
    g = np.random.default_rng(14)
    a_bits, b_bits = bf16(g, (m, k)), bf16(g, (k, n))
    c = R.Ctx()
    A, Bm, O, sink = graphs.matmul_bf16(c, m, n, k)
    got, info = run_hip(c, sink, {A: a_bits, Bm: b_bits, O: np.zeros(m * n, np.float32)})
    assert info[0]["klass"] == "matmul-mfma"
    c.close()
    rows = [0, 1, 127, 128, 500, 777, 1022, 1023]
    c = R.Ctx()
    A8, B8, O8, sink8 = graphs.matmul_bf16(c, 8, n, k)
    a8 = a_bits.reshape(m, k)[rows].reshape(-1)
    want = run_ref(c, sink8, {A8: a8, B8: b_bits, O8: np.zeros(8 * n, np.float32)})
    c.close()
    h = got[O].reshape(m, n)[rows]
    w = want[O8].reshape(8, n)
    assert_close(h, w, rtol=1e-4, atol=1e-4 * float(np.abs(w).mean()), what="row block of 1024x4096x4096")


@pytest.mark.parametrize("n,k,tb,how", [(2304, 64, False, "tile 128x192"), (2296, 128, False, "columns from 2048 on by a launch of 128x64 tiles"),
                                        (2296, 64, True, "columns from 2048 on by a launch of 128x64 tiles")])
def test_columns_left_over_by_whole_rounds_go_to_a_launch_of_small_tiles(n, k, tb, how):
    """8192 x 2304 in 128 x 256 tiles is 576 tiles, a round of 512 workgroups and an eighth:
    128 x 192 tiles when they divide N (768 tiles, a round and a half); otherwise the columns
    from 2048 on are computed by a launch of 128 x 64 tiles of their own (here with a ragged
    last tile).  Sampled rows against the CPU backend on those rows, and the whole result
    against the single launch of 128 x 256 tiles of the same graph (POLY_HIP_NO_TAIL_LAUNCH
    and POLY_HIP_MM_TILE)."""
    import os
    m = 8192
    g = np.random.default_rng(n + k)
    a_bits, b_bits = bf16(g, (m, k), 1.0), bf16(g, (k, n), 1.0)
    c = R.Ctx()
    A, Bm, O, sink = graphs.matmul_bf16(c, m, n, k, transposed_b=tb)
    arrays = {A: a_bits, Bm: b_bits, O: np.zeros(m * n, np.float32)}
    got, info = run_hip(c, sink, arrays)
    assert how in info[0]["desc"], info[0]["desc"]
    os.environ["POLY_HIP_NO_TAIL_LAUNCH"] = "1"
    os.environ["POLY_HIP_MM_TILE"] = "128,256,2,4"
    try:
        one, info1 = run_hip(c, sink, arrays)
    finally:
        del os.environ["POLY_HIP_NO_TAIL_LAUNCH"]
        del os.environ["POLY_HIP_MM_TILE"]
    c.close()
    assert "by a launch of" not in info1[0]["desc"] and "tile 128x256" in info1[0]["desc"]
    rows = [0, 1, 127, 128, 4095, 4096, 5000, 8063, 8064, 8191]
    c = R.Ctx()
    A8, B8, O8, sink8 = graphs.matmul_bf16(c, len(rows), n, k, transposed_b=tb)
    a8 = a_bits.reshape(m, k)[rows].reshape(-1)
    want = run_ref(c, sink8, {A8: a8, B8: b_bits, O8: np.zeros(len(rows) * n, np.float32)})
    c.close()
    w = want[O8].reshape(len(rows), n)
    bound = 1e-4 * float(np.abs(w).mean())
    assert_close(got[O].reshape(m, n)[rows], w, rtol=1e-4, atol=bound, what=f"rows of 8192x{n}x{k}")
    assert_close(got[O], one[O], rtol=1e-5, atol=bound, what="two launches vs one")


def test_matmul_of_computed_operands():
    """Matmul-shaped reductions that the plain templates do not take -- an fp32 operand
    against a bf16 one, arithmetic fused into an operand, a ragged depth, two reduce
    ranges, a flat output range shared by both operands -- run on the fp32 MFMA template
    with the operands evaluated on the way into LDS.  Products are exact fp32, so the
    tolerance is the fp32 reduction one."""
    g = np.random.default_rng(21)
    # (a) fp32 x bf16, K = 301 (not a multiple of the 16-deep K tile), relu fused into A
    c = R.Ctx()
    M, N, K = 96, 160, 301
    A = c.buffer((M, K), R.F32, name="A")
    Bm = c.buffer((K, N), R.BF16, name="B")
    O = c.buffer((M, N), R.F32, name="C")
    sink = c.sink((O, (A.relu() * c.const(0.5)).dot(Bm.cast(R.F32))))
    arrays = {A: g.normal(0, 1, (M, K)).astype(np.float32), Bm: bf16(g, (K, N), 1.0), O: np.zeros((M, N), np.float32)}
    want = run_ref(c, sink, arrays)
    got, info = run_hip(c, sink, arrays)
    c.close()
    assert any("operands as expressions" in k["desc"] for k in info), [k["desc"] for k in info]
    assert_close(got[O], want[O], rtol=1e-4, atol=1e-4 * float(np.abs(want[O]).mean()), what="fp32 x bf16, ragged K")
    # (b) weight-gradient form: dW[i, j] = sum over (b, t) of X[b, t, i] * dY[b, t, j], flat output
    c = R.Ctx()
    Bt, T, I, J = 3, 100, 64, 96
    X = c.buffer((Bt, T, I), R.BF16, name="X")
    dY = c.buffer((Bt, T, J), R.F32, name="dY")
    O = c.buffer((I * J,), R.F32, name="dW")
    xe = X.cast(R.F32).reshape((Bt, T, I, 1)).expand((Bt, T, I, J))
    ye = dY.reshape((Bt, T, 1, J)).expand((Bt, T, I, J))
    dw = (xe * ye).reduce_axes("ADD", [0, 1]).reshape((I * J,))
    sink = c.sink((O, dw))
    arrays = {X: bf16(g, (Bt, T, I), 1.0), dY: g.normal(0, 1, (Bt, T, J)).astype(np.float32), O: np.zeros(I * J, np.float32)}
    want = run_ref(c, sink, arrays)
    got, info = run_hip(c, sink, arrays)
    c.close()
    assert any("operands as expressions" in k["desc"] for k in info), [k["desc"] for k in info]
    assert_close(got[O], want[O], rtol=1e-4, atol=1e-4 * float(np.abs(want[O]).mean()), what="weight gradient over two ranges")


def _planes_case(c, g):
    """fp32 x bf16 with a ragged depth, large enough (2^30 multiply-adds) for the operands
    to be written as bf16 planes and multiplied on the bf16 MFMA."""
    M, N, K = 512, 512, 4100
    A = c.buffer((M, K), R.F32, name="A")
    Bm = c.buffer((K, N), R.BF16, name="B")
    O = c.buffer((M, N), R.F32, name="C")
    sink = c.sink((O, (A * c.const(1.5)).dot(Bm.cast(R.F32))))
    a = g.normal(0, 1, (M, K)).astype(np.float32)
    a[0, :8] = [1e-30, -3e30, 1.0 + 2.0 ** -20, 65504.0, 2.0 ** -126, 0.0, -0.0, 1e10]      # pieces at the edges of the exponent range
    arrays = {A: a, Bm: bf16(g, (K, N), 1.0), O: np.zeros((M, N), np.float32)}
    return sink, arrays, O


def test_matmul_of_fp32_operand_as_three_bf16_planes():
    """An fp32 operand is the sum of three bf16 pieces and a bf16 x bf16 product is exact
    in fp32, so the product runs on the bf16 MFMA over three K-long planes written by a
    first-stage kernel.  Held to the fp32 reduction tolerance against the reference, and
    compared with the fp32 MFMA path of the same kernel (POLY_HIP_NO_BF16_SPLIT)."""
    import os
    g = np.random.default_rng(22)
    c = R.Ctx()
    sink, arrays, O = _planes_case(c, g)
    want = run_ref(c, sink, arrays)
    got, info = run_hip(c, sink, arrays)
    assert any("bf16 planes" in k["desc"] for k in info), [k["desc"] for k in info]
    os.environ["POLY_HIP_NO_BF16_SPLIT"] = "1"
    try:
        got32, info32 = run_hip(c, sink, arrays)
    finally:
        del os.environ["POLY_HIP_NO_BF16_SPLIT"]
    c.close()
    assert any("mfma 32x32x2 f32, operands as expressions" in k["desc"] for k in info32), [k["desc"] for k in info32]
    w = want[O].astype(np.float64)
    # scale of the rounding error of any summation order: sum of |terms| ~ K * E|a| * E|b|
    bound = 1e-4 * float(np.abs(w).mean()) * 8
    assert_close(got[O], want[O], rtol=1e-4, atol=bound, what="three bf16 planes vs reference")
    assert_close(got32[O], want[O], rtol=1e-4, atol=bound, what="fp32 MFMA vs reference")
    # the two device paths agree far more closely than either needs to
    assert float(np.abs(got[O].astype(np.float64) - got32[O]).max()) <= 2e-5 * float(np.abs(w).max())


@pytest.mark.parametrize("tb,batch", [(False, None), (True, None), (False, 3)])
def test_plain_bf16_operand_beside_a_computed_one_is_read_in_place(tb, batch):
    """fp32 x bf16 with a depth of whole K tiles: the fp32 operand goes to three bf16 planes,
    the bf16 one is a buffer the template can read where it lies (rows along n, or along k
    when stored transposed; also per batch) and gets no plane.  Against the reference, and
    bit for bit against the same product with both operands as planes."""
    import os
    M, N, K = 256, 320, 4096 if batch is None else 2048
    g = np.random.default_rng(5 + tb)
    c = R.Ctx()
    lead = () if batch is None else (batch,)
    A = c.buffer(lead + (M, K), R.F32, name="A")
    Bm = c.buffer(lead + ((N, K) if tb else (K, N)), R.BF16, name="B")
    O = c.buffer(lead + (M, N), R.F32, name="C")
    b = Bm.permute(tuple(range(len(lead))) + (len(lead) + 1, len(lead))) if tb else Bm
    sink = c.sink((O, (A * c.const(0.75)).dot(b.cast(R.F32))))
    arrays = {A: g.normal(0, 1, lead + (M, K)).astype(np.float32), Bm: bf16(g, lead + (K, N), 1.0), O: np.zeros(lead + (M, N), np.float32)}
    os.environ["POLY_HIP_BF16_SPLIT_MIN"] = "1048576"
    try:
        want = run_ref(c, sink, arrays)
        got, info = run_hip(c, sink, arrays)
        assert any("B read in place" in k["desc"] for k in info), [k["desc"] for k in info]
        os.environ["POLY_HIP_NO_IN_PLACE_OPERAND"] = "1"
        try:
            planes, info1 = run_hip(c, sink, arrays)
        finally:
            del os.environ["POLY_HIP_NO_IN_PLACE_OPERAND"]
    finally:
        del os.environ["POLY_HIP_BF16_SPLIT_MIN"]
    c.close()
    assert any("bf16 planes" in k["desc"] and "in place" not in k["desc"] for k in info1), [k["desc"] for k in info1]
    bound = 1e-4 * float(np.abs(want[O]).mean()) * 8
    assert_close(got[O], want[O], rtol=1e-4, atol=bound, what="operand in place vs reference")
    assert got[O].tobytes() == planes[O].tobytes()
