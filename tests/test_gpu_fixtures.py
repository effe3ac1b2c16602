"""GPU parity against the committed golden fixtures (outputs of the real
reference CPU backend): every fixture plan is compiled and run through the
plan-level C ABI on the GPU, with and without the hand-written templates."""
import numpy as np
import pytest

import fixtures as F
from hipharness import assert_close, from_device, to_device
from polygrad_amd import HipPlan

pytestmark = pytest.mark.gpu

# bit-exact: integer, index and movement work
BIT_EXACT = {"kat_threefry_u32", "kat_threefry_u64", "movement_i32", "int_alu", "assembled_partial_store",
             "reduce_singleton_axis"}
# tolerance per case: (rtol, atol)
TOL = {
    "kat_matmul_2x3x4": (1e-4, 0), "kat_xent_uniform": (1e-4, 1e-6),
    "rowops_sum": (1e-4, 1e-5), "rowops_max": (1e-5, 0), "rowops_softmax": (1e-4, 1e-7), "rowops_layernorm": (1e-4, 1e-5),
    "special_exp2": (1e-5, 1e-38), "special_log2": (1e-5, 1e-6), "special_sin": (1e-5, 1e-6),
    "bf16_gelu": (2e-2, 1e-3), "bf16_matmul": (2e-2, 1e-6), "bf16_matmul_bt_batch": (2e-2, 1e-6),
    "f16_cast_mul": (2e-2, 0), "gpt2_tiny_f32": (1e-4, 1e-5), "gpt2_tiny_bf16": (2e-2, 2e-3),
    # attention: the default single-pass kernel rounds exp-terms where the reference rounds
    # probabilities; for the first queries (a handful of keys, outputs up to 1) that is two
    # 16-bit steps of the output scale.  The exact two-pass form is held to 2e-3 below.
    "mlp_train_b32": (1e-4, 1e-5), "attention_bf16_t256": (2e-2, 8e-3), "attention_bf16_t1024": (2e-2, 8e-3), "bf16_matmul_gelu": (2e-2, 2e-3),
    "bf16_layernorm_rows": (2e-2, 2e-3),
}
# plans that update their inputs in place: a second run would start from other parameters
STATEFUL = {"mlp_train_b32"}
# fixtures whose plan must come out as one of the fused kernel groups
FUSED = {"attention_bf16_t256": "attention-mfma", "attention_bf16_t1024": "attention-mfma", "bf16_matmul_gelu": "lookup table", "bf16_layernorm_rows": "row chain of 3"}


def run_fixture_on_gpu(fx, env_flags=None):
    import torch
    plan = HipPlan(fx.plan.schedule, names=fx.plan.names, keepalive=fx.plan)
    dev = [None] * fx.n_slots
    for i in fx.external:
        dev[i] = to_device(fx.inputs[i])
    torch.cuda.synchronize()
    plan.run(dev)
    if fx.name not in STATEFUL:
        plan.run(dev)  # second run replays the captured graph
    out = {i: from_device(dev[i], fx.inputs[i].dtype) for i in fx.external}
    info = plan.kernel_info()
    plan.close()
    return out, info


@pytest.mark.parametrize("name", F.case_names())
def test_fixture_on_gpu(name):
    fx = F.Fixture(name)
    got, info = run_fixture_on_gpu(fx)
    if name in FUSED:
        assert any(FUSED[name] in k["desc"] for k in info), [k["desc"] for k in info]
    for slot in fx.external:
        want = fx.expected[slot]
        if name in BIT_EXACT:
            assert got[slot].tobytes() == want.tobytes(), f"{name}: slot {slot} not bit-exact"
        else:
            rtol, atol = TOL[name]
            assert_close(F.as_float(got[slot]), F.as_float(want), rtol=rtol, atol=atol, what=f"{name} slot {slot} ({fx.plan.names[slot]})")


@pytest.mark.parametrize("name", ["attention_bf16_t256", "attention_bf16_t1024"])
def test_attention_fixture_exact_form(monkeypatch, name):
    """The two-pass attention kernel keeps every rounding of the unfused kernels."""
    monkeypatch.setenv("POLY_HIP_EXACT_ATTENTION", "1")
    fx = F.Fixture(name)
    got, info = run_fixture_on_gpu(fx)
    assert any("two passes" in k["desc"] for k in info), [k["desc"] for k in info]
    for slot in fx.external:
        assert_close(F.as_float(got[slot]), F.as_float(fx.expected[slot]), rtol=2e-2, atol=2e-3, what=f"exact attention slot {slot}")


def test_oracle_agrees_with_gpu_on_fixture_inputs():
    """Same comparison with the CPU oracle as the checker (the form smoke() uses)."""
    fx = F.Fixture("gpt2_tiny_bf16")
    want = F.run_oracle_schedule(fx.plan.schedule, fx.n_slots, fx.inputs)
    got, info = run_fixture_on_gpu(fx)
    out = [i for i in fx.external if fx.plan.names[i] == "output"][0]
    assert_close(F.as_float(got[out]), F.as_float(want[out]), rtol=2e-2, atol=2e-3, what="gpt2 tiny bf16 logits")


def test_attention_with_a_non_finite_value_row(monkeypatch):
    """Where the single-pass attention kernel and the reference part ways on non-finite data,
    stated so that a change in either direction shows.  V of key 200 of head 0 is +inf.
    The reference multiplies every probability with every value, so the zero probabilities of
    the queries before key 200 meet the infinity (0 x inf = NaN) and every row of the head is
    non-finite; the CPU oracle and the two-pass kernel do the same.  The single-pass kernel
    never multiplies a key tile that the causal mask removes for a whole tile of queries: the
    queries before that key's tile of 32 (rows 0..191) come out finite and exactly as
    without the infinity; the rows from key 200 on are non-finite as in the reference (the
    rows 192..199 share the key's tile and see 0 x inf like the reference).  Head 1 is
    untouched in every form."""
    fx = F.Fixture("attention_bf16_t256")
    by = {fx.plan.names[i]: i for i in fx.external}
    T, J = 256, 200
    clean, _ = run_fixture_on_gpu(fx)
    clean = F.as_float(clean[by["out"]]).reshape(T, 2, 64)
    v = fx.inputs[by["v"]].copy().reshape(T, 2, 64)
    v[J, 0, :] = 0x7F80                      # +inf as a bf16 bit pattern
    fx.inputs[by["v"]] = v.reshape(-1)
    want = F.as_float(F.run_oracle_schedule(fx.plan.schedule, fx.n_slots, fx.inputs)[by["out"]]).reshape(T, 2, 64)
    assert not np.isfinite(want[:, 0, :]).any() and np.isfinite(want[:, 1, :]).all()
    online, info = run_fixture_on_gpu(fx)
    assert any("one pass" in k["desc"] for k in info), [k["desc"] for k in info]
    online = F.as_float(online[by["out"]]).reshape(T, 2, 64)
    assert np.isfinite(online[:, 1, :]).all() and (online[:, 1, :] == clean[:, 1, :]).all()
    assert not np.isfinite(online[J:, 0, :]).any(), "rows from the key on: non-finite, as in the reference"
    assert np.isfinite(online[:192, 0, :]).all() and (online[:192, 0, :] == clean[:192, 0, :]).all(), \
        "rows before the key's tile: the masked tile is never multiplied"
    monkeypatch.setenv("POLY_HIP_EXACT_ATTENTION", "1")
    exact, info = run_fixture_on_gpu(fx)
    assert any("two passes" in k["desc"] for k in info), [k["desc"] for k in info]
    exact = F.as_float(exact[by["out"]]).reshape(T, 2, 64)
    assert not np.isfinite(exact[:, 0, :]).any(), "the two-pass form propagates like the reference"
    assert np.isfinite(exact[:, 1, :]).all()
