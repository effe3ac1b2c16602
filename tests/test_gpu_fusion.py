"""Plan-level fusion on the GPU: the attention kernel group (scores, scale + mask,
row max, row sum, normalise, weighted sum of values) run as one launch, and pointwise
kernels run as the epilogue of the matmul that feeds them, must give what the separately
launched kernels give, and what the reference CPU backend gives."""
import os

import numpy as np
import pytest

import graphs
import refpoly as R
from hipharness import assert_close, run_hip, run_ref

pytestmark = pytest.mark.gpu


def small_gpt2(seed, qk_gain):
    """Two layers, two heads of 64 features, 256 positions: the smallest shape the fused
    kernel takes (128-query blocks, 64-key steps).  The q/k/v projection weights are
    scaled up so that the softmax is far from uniform."""
    cfg = graphs.GPT2Config(n_layer=2, n_head=2, d_model=128, vocab=211, ctx=256, batch=2)
    c = R.Ctx()
    sink, bufs = graphs.gpt2_forward(c, cfg, R.BF16)
    arrays = graphs.gpt2_inputs(cfg, bufs, seed=seed, wdt=R.BF16)
    for name, t in bufs.items():
        if name.endswith("attn.c_attn.weight"):
            w = R.bf16_bits_to_f32(arrays[t]) * qk_gain
            arrays[t] = R.f32_to_bf16_bits(w.astype(np.float32))
    return c, cfg, sink, bufs, arrays


def logits(arrays_out, bufs):
    return R.bf16_bits_to_f32(arrays_out[bufs["output"]]).astype(np.float64)


@pytest.mark.parametrize("form", ["online", "exact"])
@pytest.mark.parametrize("qk_gain", [1.0, 12.0])
def test_fused_attention_matches_unfused_and_reference(qk_gain, form):
    """form "online": the default single-pass fp32 softmax; "exact": the two-pass form that
    keeps every 16-bit rounding of the unfused kernels (POLY_HIP_EXACT_ATTENTION=1)."""
    c, cfg, sink, bufs, arrays = small_gpt2(seed=11, qk_gain=qk_gain)
    want = logits(run_ref(c, sink, arrays), bufs)
    if form == "exact":
        os.environ["POLY_HIP_EXACT_ATTENTION"] = "1"
    try:
        got, info = run_hip(c, sink, arrays)
    finally:
        os.environ.pop("POLY_HIP_EXACT_ATTENTION", None)
    assert sum(k["klass"] == "attention-mfma" for k in info) == cfg.n_layer, [k["klass"] for k in info]
    marker = "one pass" if form == "online" else "two passes"
    assert sum(marker in k["desc"] for k in info) == cfg.n_layer, [k["desc"] for k in info if k["klass"] == "attention-mfma"]
    os.environ["POLY_HIP_NO_FUSION"] = "1"
    try:
        plain, info_plain = run_hip(c, sink, arrays)
    finally:
        del os.environ["POLY_HIP_NO_FUSION"]
    assert not any(k["klass"] == "attention-mfma" for k in info_plain)
    # per layer: six attention kernels and the three copies that split q, k and v out of
    # the fused projection became one, three pointwise kernels (attention
    # residual, GELU, MLP residual) moved into the epilogue of the matmul in front of them,
    # and each LayerNorm (two per layer and the final one) runs its three kernels as one
    n_ln = 2 * cfg.n_layer + 1
    assert len(info_plain) == len(info) + (8 + 3) * cfg.n_layer + 2 * n_ln
    assert sum("in the epilogue" in k["desc"] for k in info) == 3 * cfg.n_layer
    assert sum("row chain of 3 kernels" in k["desc"] for k in info) == n_ln
    h, p = logits(got, bufs), logits(plain, bufs)
    scale = float(np.abs(want).max())
    assert np.isfinite(h).all()
    # With the projections scaled up the scores reach +-50 and one 16-bit rounding of an
    # activation moves a probability by tens of percent: the network amplifies the
    # rounding that the online form places differently, so that form gets three times the
    # absolute tolerance there and is judged against the fp32 network below.
    loose = 3.0 if (form == "online" and qk_gain > 1.0) else 1.0
    assert_close(h, p, rtol=2e-2, atol=2e-2 * scale * loose, what="fused vs separately launched kernels")
    assert_close(h, want, rtol=2e-2, atol=2e-2 * scale * loose, what="fused vs reference CPU backend")
    rms = lambda d: float(np.sqrt(np.mean(d ** 2)))
    if form == "exact":
        # same expressions per element; only the order of the fp32 sums differs
        assert float(np.mean(h != p)) < 0.05, "bf16 logits should rarely differ at all"
        assert rms(h - want) <= 1.5 * rms(p - want) + 1e-6 * scale
    else:
        # fewer roundings than the reference: judged against the same network in fp32
        sink32, bufs32 = graphs.gpt2_forward(c, cfg, R.F32)
        arr32 = {}
        for name, t in bufs32.items():
            a = arrays[bufs[name]]
            arr32[t] = R.bf16_bits_to_f32(a) if a.dtype == np.uint16 else a.astype(np.float32)
        truth = run_ref(c, sink32, arr32)[bufs32["output"]].astype(np.float64)
        e_gpu, e_ref = rms(h - truth), rms(want - truth)
        print(f"qk_gain {qk_gain}: rms error against the fp32 network: GPU {e_gpu:.3e}, reference {e_ref:.3e}; "
              f"max |GPU - reference| {np.abs(h - want).max():.3e} at scale {scale:.3e}")
        assert e_gpu <= 1.1 * e_ref, f"GPU rms error {e_gpu:.3e} vs reference rms error {e_ref:.3e} against the fp32 network"
    c.close()


@pytest.mark.parametrize("form", ["online", "online, mask looked at by every wave", "exact"])
def test_attention_with_infinite_mask_entries(form):
    """An additive mask handed in as a buffer, with -inf entries: causal; the first 64 keys
    hidden from the last 128 queries (their first key tiles are fully masked, so the running
    maximum starts at -inf); a band of keys hidden from everybody; one query with no key at
    all, whose output row is NaN in the reference.  The single-pass form runs both ways of
    finding the tiles whose mask entries are all one value: a first kernel that looks at the
    mask once for all heads (the default for a mask that does not depend on batch or head),
    and every wave looking at its own tiles (POLY_HIP_NO_MASK_TABLE=1)."""
    ctx, heads, hd, batch = 256, 2, 64, 1
    c = R.Ctx()
    bufs, sink = graphs.attention_bf16(c, batch=batch, heads=heads, ctx=ctx, hd=hd, mask_buffer=True)
    g = np.random.default_rng(5)
    ninf = np.float32(-np.inf)
    mask = np.where(np.arange(ctx)[:, None] < np.arange(ctx)[None, :], ninf, np.float32(0.0)).astype(np.float32)
    mask[128:, :64] = ninf
    mask[:, 96:128] = ninf
    mask[5, :] = ninf
    mask[200:, 200:] += g.normal(0, 1, (56, 56)).astype(np.float32)   # finite biases as well
    arrays = {bufs["mask"]: R.f32_to_bf16_bits(mask), bufs["out"]: np.zeros(batch * ctx * heads * hd, np.uint16)}
    for n in ("q", "k", "v"):
        arrays[bufs[n]] = R.f32_to_bf16_bits(g.uniform(-1, 1, batch * ctx * heads * hd).astype(np.float32) * (3.0 if n != "v" else 1.0))
    want = R.bf16_bits_to_f32(run_ref(c, sink, arrays)[bufs["out"]]).reshape(ctx, heads * hd)
    if form == "exact":
        os.environ["POLY_HIP_EXACT_ATTENTION"] = "1"
    if "every wave" in form:
        os.environ["POLY_HIP_NO_MASK_TABLE"] = "1"
    try:
        got, info = run_hip(c, sink, arrays)
    finally:
        os.environ.pop("POLY_HIP_EXACT_ATTENTION", None)
        os.environ.pop("POLY_HIP_NO_MASK_TABLE", None)
    c.close()
    assert any(k["klass"] == "attention-mfma" and ("one pass" if form.startswith("online") else "two passes") in k["desc"] for k in info), [k["desc"] for k in info]
    assert any("classified by a first kernel" in k["desc"] for k in info) == (form == "online"), [k["desc"] for k in info]
    have = R.bf16_bits_to_f32(got[bufs["out"]]).reshape(ctx, heads * hd)
    assert np.isnan(want[5]).all() and np.isnan(have[5]).all()
    assert np.isfinite(np.delete(want, 5, axis=0)).all() and np.isfinite(np.delete(have, 5, axis=0)).all()
    assert_close(have, want, rtol=2e-2, atol=8e-3 if form.startswith("online") else 2e-3, what=f"{form} attention with -inf mask entries")


@pytest.mark.parametrize("form", ["online", "exact"])
def test_attention_fp16(form):
    """The same kernel group in fp16.  The reference's mask constant -1e9 is -inf in fp16,
    so every masked score is -inf."""
    ctx, heads, hd, batch = 256, 2, 64, 2
    c = R.Ctx()
    bufs, sink = graphs.attention_bf16(c, batch=batch, heads=heads, ctx=ctx, hd=hd, dt=R.F16)
    g = np.random.default_rng(9)
    n = batch * ctx * heads * hd
    arrays = {bufs["arange"]: np.arange(ctx, dtype=np.float32), bufs["out"]: np.zeros(n, np.float16)}
    for name in ("q", "k", "v"):
        arrays[bufs[name]] = (g.uniform(-1, 1, n) * (2.0 if name != "v" else 1.0)).astype(np.float16)
    want = run_ref(c, sink, arrays)[bufs["out"]].astype(np.float32)
    if form == "exact":
        os.environ["POLY_HIP_EXACT_ATTENTION"] = "1"
    try:
        got, info = run_hip(c, sink, arrays)
    finally:
        os.environ.pop("POLY_HIP_EXACT_ATTENTION", None)
    c.close()
    assert any(k["klass"] == "attention-mfma" and "f16" in k["desc"] and ("one pass" if form == "online" else "two passes") in k["desc"]
               for k in info), [k["desc"] for k in info]
    assert np.isfinite(want).all()
    assert_close(got[bufs["out"]].astype(np.float32), want, rtol=2e-2, atol=2e-3, what=f"{form} attention in fp16")


@pytest.mark.parametrize("mask_value", ["-inf", "-1e9"])
def test_attention_with_more_than_64_key_tiles(mask_value):
    """2176 keys are 68 tiles of 32: a wave keeps the words of up to 64 mask tiles in its
    lanes and reads them one by one beyond that.  One head, causal; with -inf above the
    diagonal (tiles and key blocks passed over unseen) and with the reference's -1e9."""
    ctx, heads, hd, batch = 2176, 1, 64, 1
    c = R.Ctx()
    bufs, sink = graphs.attention_bf16(c, batch=batch, heads=heads, ctx=ctx, hd=hd, mask_buffer=True)
    g = np.random.default_rng(17)
    fill = np.float32(-np.inf) if mask_value == "-inf" else np.float32(-1e9)
    mask = np.where(np.arange(ctx)[:, None] < np.arange(ctx)[None, :], fill, np.float32(0.0)).astype(np.float32)
    arrays = {bufs["mask"]: R.f32_to_bf16_bits(mask), bufs["out"]: np.zeros(batch * ctx * heads * hd, np.uint16)}
    for n in ("q", "k", "v"):
        arrays[bufs[n]] = R.f32_to_bf16_bits(g.uniform(-1, 1, batch * ctx * heads * hd).astype(np.float32) * (2.0 if n != "v" else 1.0))
    want = R.bf16_bits_to_f32(run_ref(c, sink, arrays)[bufs["out"]]).reshape(ctx, heads * hd)
    got, info = run_hip(c, sink, arrays)
    c.close()
    assert any(k["klass"] == "attention-mfma" and "classified by a first kernel" in k["desc"] for k in info), [k["desc"] for k in info]
    have = R.bf16_bits_to_f32(got[bufs["out"]]).reshape(ctx, heads * hd)
    assert np.isfinite(want).all() and np.isfinite(have).all()
    assert_close(have, want, rtol=2e-2, atol=8e-3, what=f"attention over 2176 keys, mask {mask_value}")


def test_lookup_table_epilogue_is_bit_identical_to_the_arithmetic():
    """A pointwise kernel of one 16-bit input fused behind a matmul is evaluated through a
    65536-entry table filled by its own expression: results must not change by a bit.  The
    matmul keeps the table's entries for 2^-24 <= |x| < 256 in LDS and goes to the table in
    memory for a group of values with an input outside that range: rows of zeros, of huge,
    of undefined and of tiny products are among the inputs, and the result must be the same
    with the LDS copy switched off."""
    m, n, k = 512, 768, 256
    g = np.random.default_rng(21)
    c = R.Ctx()
    A = c.buffer((m, k), R.BF16, name="A")
    W = c.buffer((k, n), R.BF16, name="W")
    O = c.buffer((m, n), R.BF16, name="O")
    y = A.cast(R.F32).dot(W.cast(R.F32)).cast(R.BF16).contiguous()
    sink = c.sink((O, y.gelu()))
    a = g.normal(0, 1.0, (m, k)).astype(np.float32)
    a[3] = 0.0                 # products exactly 0
    a[40:44] *= 1e3            # |x| beyond 256
    a[77] = np.inf             # inf - inf: NaN in any order of summation
    a[130:133] *= 1e-9         # |x| below 2^-24
    a[200, ::2] = 0.0
    arrays = {A: R.f32_to_bf16_bits(a.reshape(-1)),
              W: R.f32_to_bf16_bits(g.normal(0, 0.2, k * n).astype(np.float32)), O: np.zeros(m * n, np.uint16)}
    with_table, info = run_hip(c, sink, arrays)
    assert any("lookup table" in kk["desc"] for kk in info), [kk["desc"] for kk in info]
    os.environ["POLY_HIP_NO_LUT_WINDOW"] = "1"
    try:
        from_memory, _ = run_hip(c, sink, arrays)
    finally:
        del os.environ["POLY_HIP_NO_LUT_WINDOW"]
    assert with_table[O].tobytes() == from_memory[O].tobytes()
    os.environ["POLY_HIP_NO_LUT"] = "1"
    try:
        plain, info2 = run_hip(c, sink, arrays)
    finally:
        del os.environ["POLY_HIP_NO_LUT"]
    assert not any("lookup table" in kk["desc"] for kk in info2) and len(info2) == len(info)
    assert with_table[O].tobytes() == plain[O].tobytes()
    got = R.bf16_bits_to_f32(with_table[O]).reshape(m, n)
    assert (got[3] == 0).all() and np.isnan(got[77]).all() and (np.abs(got[40:44]) > 256).any()
    want = run_ref(c, sink, arrays)
    c.close()
    assert_close(R.bf16_bits_to_f32(with_table[O]), R.bf16_bits_to_f32(want[O]), rtol=2e-2, atol=2e-2, what="matmul + GELU vs reference")


def test_table_epilogue_on_both_launches_of_a_product_with_leftover_columns():
    """8192 x 2296 with a GELU behind it (2304 columns would go out as 128 x 192 tiles, one
    launch): the columns from 2048 on are a launch of small tiles of their own, and both
    launches serve the table's middle from their LDS.  Every switch (one launch, table in
    memory only, no table) must give the same bits."""
    m, n, k = 8192, 2296, 64
    g = np.random.default_rng(77)
    c = R.Ctx()
    A = c.buffer((m, k), R.BF16, name="A")
    W = c.buffer((k, n), R.BF16, name="W")
    O = c.buffer((m, n), R.BF16, name="O")
    y = A.cast(R.F32).dot(W.cast(R.F32)).cast(R.BF16).contiguous()
    sink = c.sink((O, y.gelu()))
    a = g.normal(0, 1.0, (m, k)).astype(np.float32)
    a[5] = 0.0
    a[4000:4003] *= 1e3
    arrays = {A: R.f32_to_bf16_bits(a.reshape(-1)), W: R.f32_to_bf16_bits(g.normal(0, 0.2, k * n).astype(np.float32)),
              O: np.zeros(m * n, np.uint16)}
    got, info = run_hip(c, sink, arrays)
    assert any("lookup table" in kk["desc"] and "columns from 2048 on by a launch of" in kk["desc"] for kk in info), [kk["desc"] for kk in info]
    for switch in ("POLY_HIP_NO_TAIL_LAUNCH", "POLY_HIP_NO_LUT_WINDOW", "POLY_HIP_NO_LUT"):
        os.environ[switch] = "1"
        try:
            other, _ = run_hip(c, sink, arrays)
        finally:
            del os.environ[switch]
        assert got[O].tobytes() == other[O].tobytes(), switch
    c.close()


def test_small_independent_kernels_run_side_by_side_in_one_launch():
    """Casts of small fp32 parameters to bf16 that stand between larger kernels of a schedule
    (as in a training step, where every bias and LayerNorm parameter is cast before use) read
    nothing that the plan computes: they run as one launch at the place of the first, each
    on its own workgroups.  Against the reference, and bit for bit against the kernels
    launched one by one, where they stand."""
    import os
    c = R.Ctx()
    g = np.random.default_rng(12)
    rows, d = 512, 768
    x = c.buffer((rows, d), R.BF16, name="x")
    params = [c.buffer((n,), R.F32, name=f"p{i}") for i, n in enumerate((d, d, 3 * d, 1000))]
    out = c.buffer((rows, d), R.BF16, name="out")
    aux = c.buffer((1000,), R.BF16, name="aux")
    h = x
    for i, p in enumerate(params[:3]):
        pc = p.cast(R.BF16).contiguous()                       # one small kernel each
        pc = pc.shrink(((0, d),)) if pc.shape[0] != d else pc
        h = ((h.cast(R.F32) * c.const(0.5 + i)).cast(R.BF16) + pc.reshape((1, d)).expand((rows, d))).contiguous()
    sink = c.sink((out, h), (aux, (params[3] * c.const(3.0)).cast(R.BF16)))
    arrays = {x: R.f32_to_bf16_bits(g.normal(0, 1, rows * d).astype(np.float32)), out: np.zeros(rows * d, np.uint16), aux: np.zeros(1000, np.uint16)}
    for p in params:
        arrays[p] = g.normal(0, 1, p.shape[0]).astype(np.float32)
    want = run_ref(c, sink, arrays)
    got, info = run_hip(c, sink, arrays)
    assert any("small independent pointwise kernels side by side" in k["desc"] for k in info), [k["desc"] for k in info]
    os.environ["POLY_HIP_NO_SIDE_BY_SIDE"] = "1"
    try:
        apart, info1 = run_hip(c, sink, arrays)
    finally:
        del os.environ["POLY_HIP_NO_SIDE_BY_SIDE"]
    c.close()
    assert len(info1) > len(info) and not any("side by side" in k["desc"] for k in info1)
    for t in (out, aux):
        assert got[t].tobytes() == apart[t].tobytes()
        assert got[t].tobytes() == want[t].tobytes()
