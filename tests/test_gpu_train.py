"""Benchmark configuration 1 on the GPU: a 2-layer MLP (784 -> 512 -> 10, fp32, batch 4096),
forward, cross-entropy, reverse-mode gradients (the reference's poly_grad) and one SGD step
whose parameter updates are in-place ASSIGNs -- 22 scheduled kernels, among them the
optimizer kernels.  Logits, loss and the four updated parameters are compared with the
reference CPU backend."""
import numpy as np
import pytest

import graphs
import refpoly as R
from hipharness import assert_close, run_hip, run_ref

pytestmark = pytest.mark.gpu


def mlp_arrays(bufs, batch, seed=0):
    g = np.random.default_rng(seed)
    arr = {}
    for name, t in bufs.items():
        n = int(np.prod(t.shape))
        if name == "X":
            a = g.normal(0, 1, n)
        elif name.startswith("W"):       # Kaiming-uniform, U(+-sqrt(6 / fan_in)), stored (out, in)
            lim = (6.0 / t.shape[1]) ** 0.5
            a = g.uniform(-lim, lim, n)
        elif name == "Y":
            a = np.eye(10)[g.integers(0, 10, batch)].reshape(-1)
        else:
            a = np.zeros(n)
        arr[t] = a.astype(np.float32)
    return arr


@pytest.mark.parametrize("batch", [64, 4096])
def test_mlp_train_step_matches_reference(batch):
    c = R.Ctx()
    bufs, sink = graphs.mlp_train_step(c, batch=batch, lr=0.01)
    arrays = mlp_arrays(bufs, batch)
    want = run_ref(c, sink, arrays)
    got, info = run_hip(c, sink, arrays)
    c.close()
    assert len(info) >= 15
    for name in ("logits", "loss"):
        t = bufs[name]
        assert_close(got[t], want[t], rtol=1e-4, atol=1e-5, what=name)
    for name in ("W1", "b1", "W2", "b2"):
        t = bufs[name]
        step = want[t] - arrays[t]                      # -lr * gradient
        assert np.abs(step).max() > 0, f"{name} did not move"
        # the update is a sum over the batch: compare the step, relative to its own scale;
        # the step is read back as a difference of fp32 parameters, so it is only known to
        # a few ulps of the parameter itself
        ulp = 4 * np.finfo(np.float32).eps * float(np.abs(arrays[t]).max())
        assert_close(got[t] - arrays[t], step, rtol=1e-3, atol=1e-4 * float(np.abs(step).max()) + ulp, what=f"SGD step of {name}")
        assert_close(got[t], want[t], rtol=1e-5, atol=1e-6, what=f"updated {name}")
    # inputs that are only read stay untouched
    assert got[bufs["X"]].tobytes() == arrays[bufs["X"]].tobytes()


def test_adamw_update_matches_reference():
    """The optimizer kernels of the reference's training graph (src/instance.c:1162-1224):
    AdamW with decoupled decay, bias corrections from one-element buffers, three in-place
    updates per parameter -- seven fp32 streams per element once the four kernels are one
    launch, HBM-bound."""
    numel = 1 << 20
    c = R.Ctx()
    bufs, sink = graphs.adamw_step(c, numel)
    g = np.random.default_rng(8)
    arrays = {bufs["p"]: g.normal(0, 0.02, numel).astype(np.float32), bufs["g"]: g.normal(0, 1e-3, numel).astype(np.float32),
              bufs["m"]: g.normal(0, 1e-3, numel).astype(np.float32), bufs["v"]: (g.normal(0, 1e-3, numel) ** 2).astype(np.float32),
              bufs["bc1"]: np.array([1.0 / (1 - 0.9 ** 3)], np.float32), bufs["bc2"]: np.array([1.0 / (1 - 0.999 ** 3)], np.float32)}
    want = run_ref(c, sink, arrays)
    got, info = run_hip(c, sink, arrays)
    # the four kernels (new parameter into a temporary, copy back, two moments) walk the
    # same positions: one launch, the temporary never written, 7 streams instead of 13
    assert len(info) == 1 and "4 pointwise kernels over the same" in info[0]["desc"] and "1 buffers never written out" in info[0]["desc"], [k["desc"] for k in info]
    import os
    os.environ["POLY_HIP_NO_POINTWISE_GROUPS"] = "1"
    try:
        apart, info4 = run_hip(c, sink, arrays)
    finally:
        del os.environ["POLY_HIP_NO_POINTWISE_GROUPS"]
    c.close()
    assert len(info4) == 4 and all(k["klass"] == "elementwise" for k in info4)
    for name in ("p", "m", "v", "g"):
        assert got[bufs[name]].tobytes() == apart[bufs[name]].tobytes(), f"{name}: one launch against four"
    for name in ("p", "m", "v"):
        t = bufs[name]
        assert not np.array_equal(want[t], arrays[t]), f"{name} did not change"
        assert_close(got[t], want[t], rtol=1e-5, atol=1e-9, what=f"AdamW {name}")
    assert got[bufs["g"]].tobytes() == arrays[bufs["g"]].tobytes()


def check_train_step(c, bufs, sink, B, T, V, lr, names, n_kernels_at_least):
    """Runs one training step on the reference CPU backend and on the GPU and compares the
    loss, both moments and the updated value of every parameter in `names`."""
    arrays = graphs.gpt2_block_train_inputs(bufs, B, T, V)
    want = run_ref(c, sink, arrays)
    got, info = run_hip(c, sink, arrays)
    assert len(info) >= n_kernels_at_least
    assert_close(got[bufs["loss"]], want[bufs["loss"]], rtol=1e-4, what="loss")
    assert abs(float(want[bufs["loss"]][0]) - np.log(V)) < 0.05       # random init: loss is ln(vocab)
    for name in names:
        m_ref, m_got = want[bufs[name + ".m"]], got[bufs[name + ".m"]]
        scale = float(np.abs(m_ref).max())
        assert scale > 0, f"no gradient reached {name}"
        # gradients pass through bf16 activations: 2e-2 of the tensor's scale per element,
        # and far less on average (different accumulation orders, same roundings)
        assert_close(m_got, m_ref, rtol=2e-2, atol=2e-2 * scale, what=f"first moment of {name}")
        assert float(np.abs(m_got - m_ref).mean()) <= 2e-3 * scale, name
        v_ref, v_got = want[bufs[name + ".v"]], got[bufs[name + ".v"]]
        assert_close(v_got, v_ref, rtol=4e-2, atol=4e-2 * float(np.abs(v_ref).max()), what=f"second moment of {name}")
        # the first AdamW step moves every element by about lr * sign(g): where the
        # gradients agree in sign the parameters agree closely, and nowhere by more than 2 lr
        p0, p_ref, p_got = arrays[bufs[name]], want[bufs[name]], got[bufs[name]]
        assert np.abs(p_ref - p0).max() > 0.5 * lr * 0.9
        assert np.abs(p_got - p_ref).max() <= 2.2 * lr
        same = np.sign(m_ref) == np.sign(m_got)
        big = np.abs(m_ref) > 0.05 * scale
        assert same[big].all(), name
        assert_close(p_got[big], p_ref[big], rtol=0, atol=0.2 * lr, what=f"updated {name} where the gradient is not small")
    return info


@pytest.mark.parametrize("B,T,D,H,V", [(1, 32, 64, 2, 97), (2, 64, 128, 4, 301), (1, 128, 128, 2, 97)])
def test_gpt2_block_train_step_matches_reference(B, T, D, H, V):
    """Benchmark configuration 5 at a reduced size: one transformer block, final LayerNorm,
    vocabulary projection, next-token cross-entropy (sparse targets), reverse-mode
    gradients from the reference's poly_grad and AdamW on all 15 parameters -- about 150
    scheduled kernels with the backward forms of matmul, softmax, LayerNorm and GELU,
    bf16 activations with fp32 master parameters.  The first moments after one step from
    zero state are 0.1 x gradient, so they carry the gradient comparison."""
    lr = 3e-4
    c = R.Ctx()
    bufs, sink = graphs.gpt2_block_train_step(c, B, T, D, H, V, lr=lr)
    info = check_train_step(c, bufs, sink, B, T, V, lr, graphs.BLOCK_PARAMS, 60)     # launches (about 150 scheduled kernels; each parameter's four optimizer kernels are one)
    c.close()
    if D >= 128:      # large enough for the backward matmuls to leave the generic reductions
        assert sum("operands as expressions" in k["desc"] for k in info) >= 4, [k["desc"] for k in info if "reduce" in k["desc"]]
    if T >= 128:      # the derivative of the q | k | v concatenation: one batched matmul per slab of columns
        assert any("3 slabs of one output range" in k["desc"] for k in info)


def test_row_chains_store_the_row_values_that_the_backward_pass_reads():
    """In a training step the statistics of the forward pass (mean and variance of every
    LayerNorm, maximum and sum of the softmax) are read again by the backward pass, far
    down the schedule.  The forward kernels still run as one row chain each: the phase that
    makes such a value stores it as well.  Bit for bit against the same step with those
    kernels launched one by one."""
    import os
    B, T, D, H, V, lr = 1, 128, 128, 2, 97, 3e-4
    c = R.Ctx()
    bufs, sink = graphs.gpt2_block_train_step(c, B, T, D, H, V, lr=lr)
    arrays = graphs.gpt2_block_train_inputs(bufs, B, T, V)
    got, info = run_hip(c, sink, arrays)
    assert sum("row values stored for later kernels" in k["desc"] for k in info) >= 4, [k["desc"] for k in info if "row chain" in k["desc"]]
    os.environ["POLY_HIP_NO_ROW_CHAIN_EXPORTS"] = "1"
    try:
        apart, info1 = run_hip(c, sink, arrays)
    finally:
        del os.environ["POLY_HIP_NO_ROW_CHAIN_EXPORTS"]
    c.close()
    assert not any("row values stored" in k["desc"] for k in info1) and len(info1) > len(info)
    for name, t in bufs.items():
        assert got[t].tobytes() == apart[t].tobytes(), name


def test_epilogue_parts_of_one_16_bit_input_come_from_tables():
    """The backward product of the first MLP layer multiplies by the derivative of GELU at
    the saved bf16 pre-activation inside its epilogue; the parts of that expression that
    depend on the pre-activation alone are read from tables of 65 536 entries that the same
    expression filled -- the three parts in one table whose entries hold all three values,
    so that an element costs one gather.  Bit for bit against the arithmetic
    (POLY_HIP_NO_LUT) and against a table per part (POLY_HIP_NO_LUT_PACK)."""
    import os
    B, T, D, H, V, lr = 1, 128, 128, 2, 97, 3e-4
    c = R.Ctx()
    bufs, sink = graphs.gpt2_block_train_step(c, B, T, D, H, V, lr=lr)
    arrays = graphs.gpt2_block_train_inputs(bufs, B, T, V)
    got, info = run_hip(c, sink, arrays)
    assert any("3 parts of the epilogue as 16-bit lookup tables (1, one per load)" in k["desc"] for k in info), [k["desc"] for k in info if "matmul" in k["desc"]]
    os.environ["POLY_HIP_NO_LUT"] = "1"
    try:
        plain, info1 = run_hip(c, sink, arrays)
    finally:
        del os.environ["POLY_HIP_NO_LUT"]
    os.environ["POLY_HIP_NO_LUT_PACK"] = "1"
    try:
        apart, info2 = run_hip(c, sink, arrays)
    finally:
        del os.environ["POLY_HIP_NO_LUT_PACK"]
    c.close()
    assert not any("lookup table" in k["desc"] for k in info1)
    assert any("3 parts of the epilogue as 16-bit lookup tables (3, one per load)" in k["desc"] for k in info2)
    for name, t in bufs.items():
        assert got[t].tobytes() == plain[t].tobytes(), name
        assert got[t].tobytes() == apart[t].tobytes(), name


def test_pre_activation_read_by_the_backward_pass_is_stored_by_the_product():
    """The first MLP product's output (with its bias) feeds GELU and, much later, the backward
    pass.  The product takes GELU into its epilogue all the same and stores both tensors --
    the pre-activation where its own kernel would have, GELU's result where GELU's would --
    instead of leaving GELU to a launch of its own that reads the pre-activation back.  Bit
    for bit against the step with that launch (POLY_HIP_NO_STORED_MID)."""
    import os
    B, T, D, H, V, lr = 1, 128, 128, 2, 97, 3e-4
    c = R.Ctx()
    bufs, sink = graphs.gpt2_block_train_step(c, B, T, D, H, V, lr=lr)
    arrays = graphs.gpt2_block_train_inputs(bufs, B, T, V)
    got, info = run_hip(c, sink, arrays)
    assert sum("a value on the way stored as well" in k["desc"] for k in info) == 1, [k["desc"] for k in info if "matmul" in k["desc"]]
    os.environ["POLY_HIP_NO_STORED_MID"] = "1"
    try:
        apart, info1 = run_hip(c, sink, arrays)
    finally:
        del os.environ["POLY_HIP_NO_STORED_MID"]
    c.close()
    assert not any("stored as well" in k["desc"] for k in info1) and len(info1) == len(info) + 1
    for name, t in bufs.items():
        assert got[t].tobytes() == apart[t].tobytes(), name


def test_reduction_beside_the_softmax_derivative_chain_is_a_phase_of_it():
    """The derivative of the row maximum inside softmax counts, per row, the scores equal to
    the maximum: a reduction over the scores that the reference schedules as a kernel of its
    own, with a copy of its result feeding the last kernel of the softmax derivative.  The
    row chain of that derivative holds the scores' row anyway: the count becomes one more
    phase of it and the copy another name for its result (six scheduled kernels, one
    launch).  Bit for bit against the step with the count as a launch of its own
    (POLY_HIP_NO_SIDE_REDUCE)."""
    import os
    B, T, D, H, V, lr = 1, 128, 128, 2, 97, 3e-4
    c = R.Ctx()
    bufs, sink = graphs.gpt2_block_train_step(c, B, T, D, H, V, lr=lr)
    arrays = graphs.gpt2_block_train_inputs(bufs, B, T, V)
    got, info = run_hip(c, sink, arrays)
    assert sum("row chain of 6 kernels" in k["desc"] for k in info) == 1, [k["desc"] for k in info if "row chain" in k["desc"]]
    os.environ["POLY_HIP_NO_SIDE_REDUCE"] = "1"
    try:
        apart, info1 = run_hip(c, sink, arrays)
    finally:
        del os.environ["POLY_HIP_NO_SIDE_REDUCE"]
    c.close()
    assert not any("row chain of 6 kernels" in k["desc"] for k in info1) and len(info1) > len(info)
    for name, t in bufs.items():
        assert got[t].tobytes() == apart[t].tobytes(), name


def test_ordered_column_sums_of_a_step_run_side_by_side():
    """The order-preserving bf16 column sums of the backward pass (bias and LayerNorm-parameter
    gradients: a terms kernel and an in-order adder each) that depend on nothing between
    them run as one pair of launches, every member on its own workgroups and its own part
    of the scratch memory.  Bit for bit against the same step with every sum launched by
    itself."""
    import os
    B, T, D, H, V, lr = 2, 256, 128, 4, 301, 3e-4      # 512 rows: long enough for the ordered form
    c = R.Ctx()
    bufs, sink = graphs.gpt2_block_train_step(c, B, T, D, H, V, lr=lr)
    arrays = graphs.gpt2_block_train_inputs(bufs, B, T, V)
    got, info = run_hip(c, sink, arrays)
    merged = [k["desc"] for k in info if "ordered column sums side by side" in k["desc"]]
    assert merged, [k["desc"] for k in info if "ordered" in k["desc"]]
    os.environ["POLY_HIP_NO_MERGED_ADDERS"] = "1"
    try:
        apart, info1 = run_hip(c, sink, arrays)
    finally:
        del os.environ["POLY_HIP_NO_MERGED_ADDERS"]
    c.close()
    assert not any("side by side (terms" in k["desc"] for k in info1) and len(info1) > len(info)
    for name, t in bufs.items():
        assert got[t].tobytes() == apart[t].tobytes(), name


@pytest.mark.parametrize("T", [128, 1024])
def test_slabs_of_the_qkv_derivative_read_the_score_derivative_as_bf16(T):
    """Two slabs of the derivative of the q | k | v split multiply by the same tensor (the
    derivative of the scores dS: dq = dS K, dk = dS^T Q), an fp32 buffer in the schedule
    whose values are casts of bf16 products.  The row chain that makes dS stores the bf16
    values themselves and both products read them where they lie, on the bf16 MFMA.  Here
    at a size the reference CPU backend finishes quickly (one short sequence, and one of the
    full 1024 positions), with the size threshold of that path lowered: against the
    reference, and bit for bit against the same step with dS stored as fp32 and written
    as one bf16 plane first (which the second slab reads as the first one left it, rows
    along the depth, or writes again itself)."""
    import os
    B, D, H, V, lr = 1, 128, 2, 97, 3e-4
    os.environ["POLY_HIP_BF16_SPLIT_MIN"] = "1048576"
    try:
        c = R.Ctx()
        bufs, sink = graphs.gpt2_block_train_step(c, B, T, D, H, V, lr=lr)
        arrays = graphs.gpt2_block_train_inputs(bufs, B, T, V)
        if T <= 128:
            info = check_train_step(c, bufs, sink, B, T, V, lr, graphs.BLOCK_PARAMS, 60)
            got, _ = run_hip(c, sink, arrays)
        else:
            # (sums over 1024 positions that round to bf16 at every step: single elements of a
            # gradient move by more than the short-sequence bounds when one rounding upstream
            # falls the other way, so the loss and the mean error of every gradient are compared)
            want = run_ref(c, sink, arrays)
            got, info = run_hip(c, sink, arrays)
            assert_close(got[bufs["loss"]], want[bufs["loss"]], rtol=1e-4, what="loss")
            for name in graphs.BLOCK_PARAMS:
                m_ref, m_got = want[bufs[name + ".m"]], got[bufs[name + ".m"]]
                assert float(np.abs(m_got - m_ref).mean()) <= 2e-3 * float(np.abs(m_ref).max()), name
        slabs = [k["desc"] for k in info if "3 slabs of one output range" in k["desc"]]
        assert len(slabs) == 1 and slabs[0].count("read in place") == 3 and "rows and depth exchanged" not in slabs[0], slabs
        assert slabs[0].count("(1 + 1 planes") == 3, slabs
        assert sum("result stored as the bf16 values" in k["desc"] for k in info) == 1

        def again(*switches):
            for e in switches:
                os.environ[e] = "1"
            try:
                return run_hip(c, sink, arrays)
            finally:
                for e in switches:
                    del os.environ[e]

        wide, info1 = again("POLY_HIP_NO_NARROW_STORE")
        assert sum("rows and depth exchanged" in k["desc"] for k in info1) == 1
        assert not any("result stored as the bf16 values" in k["desc"] for k in info1)
        own, info2 = again("POLY_HIP_NO_NARROW_STORE", "POLY_HIP_NO_SHARED_PLANES")
        assert not any("rows and depth exchanged" in k["desc"] for k in info2)
        # every value of dS in three bf16 pieces, of which two are zero
        three, info3 = again("POLY_HIP_NO_EXACT16_BUFFERS", "POLY_HIP_SPLIT_THREE")
        assert any("(3 + 1 planes" in k["desc"] for k in info3)
        for name, t in bufs.items():
            assert got[t].tobytes() == wide[t].tobytes(), name
            assert got[t].tobytes() == own[t].tobytes(), name
        # (the pieces that are zero add nothing, but a product three times as deep may be dealt
        # to workgroups another way and add its terms in another order)
        assert_close(three[bufs["loss"]], got[bufs["loss"]], rtol=1e-5, what="loss")
        c.close()
    finally:
        del os.environ["POLY_HIP_BF16_SPLIT_MIN"]


@pytest.mark.parametrize("n_blocks", [2, 3])
def test_gpt2_multi_block_train_step_matches_reference(n_blocks):
    """The same with several blocks stacked (configuration 5 has 24): gradients flow through
    the residual stream of the blocks above, and the schedule outgrows the reference's stock
    limit of 256 buffers (src/frontend_internal.h:23), so it comes from the build with
    raised caps (oracle/_ref/libpolygrad_hip_ref.so), whose CPU backend is also the checker."""
    if not R.hip_ref_available():
        pytest.skip("oracle/_ref/libpolygrad_hip_ref.so is not built (make -C oracle ref_hip)")
    B, T, D, H, V, lr = 1, 128, 128, 2, 97, 3e-4
    c = R.Ctx(hip_ref=True)
    bufs, sink = graphs.gpt2_block_train_step(c, B, T, D, H, V, lr=lr, n_blocks=n_blocks)
    info = check_train_step(c, bufs, sink, B, T, V, lr, graphs.train_param_names(n_blocks), 55 * n_blocks)
    c.close()
    assert sum("3 slabs of one output range" in k["desc"] for k in info) == n_blocks


@pytest.mark.parametrize("streams", ["1", "2", "3"])
def test_launches_on_the_second_stream_change_nothing(streams):
    """The in-order adders of the bf16 column sums (one thread per output, a chain of 4096
    dependent additions each) run on side streams of the captured graph (dealt to them in
    turn), ordered against the main sequence and each other by the buffers they share.  Three
    replays of the graph must give what the single-stream graph gives, bit for bit (the
    optimizer state advances with every run, so a launch that ran too early or too late
    would show)."""
    import os
    # (large enough for most launches to fill more than a quarter of the chip: a plan of
    # small launches only is one chain and stays on one stream)
    B, T, D, H, V, lr = 4, 256, 256, 4, 1000, 3e-4
    outs = []
    for single in (False, True):
        c = R.Ctx()
        bufs, sink = graphs.gpt2_block_train_step(c, B, T, D, H, V, lr=lr)
        arrays = graphs.gpt2_block_train_inputs(bufs, B, T, V)
        os.environ["POLY_HIP_SIDE_STREAMS"] = streams
        if single:
            os.environ["POLY_HIP_NO_SIDE_STREAM"] = "1"
        try:
            got, info = run_hip(c, sink, arrays, repeats=3)
        finally:
            os.environ.pop("POLY_HIP_NO_SIDE_STREAM", None)
            os.environ.pop("POLY_HIP_SIDE_STREAMS", None)
        n_side = run_hip.side_launches
        assert (n_side == 0) if single else (n_side >= 4), n_side
        outs.append({name: got[t] for name, t in bufs.items()})
        c.close()
    for name in outs[0]:
        assert outs[0][name].tobytes() == outs[1][name].tobytes(), name
