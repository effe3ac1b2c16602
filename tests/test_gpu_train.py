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
    updates per parameter -- seven fp32 streams per element, HBM-bound."""
    numel = 1 << 20
    c = R.Ctx()
    bufs, sink = graphs.adamw_step(c, numel)
    g = np.random.default_rng(8)
    arrays = {bufs["p"]: g.normal(0, 0.02, numel).astype(np.float32), bufs["g"]: g.normal(0, 1e-3, numel).astype(np.float32),
              bufs["m"]: g.normal(0, 1e-3, numel).astype(np.float32), bufs["v"]: (g.normal(0, 1e-3, numel) ** 2).astype(np.float32),
              bufs["bc1"]: np.array([1.0 / (1 - 0.9 ** 3)], np.float32), bufs["bc2"]: np.array([1.0 / (1 - 0.999 ** 3)], np.float32)}
    want = run_ref(c, sink, arrays)
    got, info = run_hip(c, sink, arrays)
    c.close()
    assert all(k["klass"] == "elementwise" for k in info)
    for name in ("p", "m", "v"):
        t = bufs[name]
        assert not np.array_equal(want[t], arrays[t]), f"{name} did not change"
        assert_close(got[t], want[t], rtol=1e-5, atol=1e-9, what=f"AdamW {name}")
    assert got[bufs["g"]].tobytes() == arrays[bufs["g"]].tobytes()
