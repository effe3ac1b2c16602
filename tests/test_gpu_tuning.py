"""On-device tuning (POLY_BEAM, as the reference's search is switched on,
src/render_c.c:839; its timing loop and disk cache are src/codegen.c:1012-1195).  The
candidates: tile shapes and pipelines of the 16-bit matmul templates, tile shapes of the
fp32 one, the register budget of the attention kernel, the access width of fused pointwise
kernels, the workgroup size of row chains, the streaming forms of large bandwidth-bound kernels.  A tuned plan must give bit-identical results -- no candidate changes the order
in which a value's terms are added -- and remember its decisions."""
import os

import pytest

from polygrad_amd import HipPlan
from polygrad_amd.inputs import gpt2_slot_tensors, random_slot_tensors

pytestmark = pytest.mark.gpu

PLANS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "polygrad_amd", "plans")


def run_plan(name, make_inputs, out_name):
    import torch
    plan = HipPlan.from_file(os.path.join(PLANS, name + ".polyplan"))
    data = make_inputs(plan)
    out = [s for s in plan.external_slots() if s.name == out_name][0]
    data[out.index].fill_(float("nan"))
    plan.run(data)
    plan.run(data)                      # second run replays the captured graph
    result = data[out.index].clone()
    descs = [k["desc"] for k in plan.kernel_info()]
    plan.close()
    torch.cuda.synchronize()
    return result, descs


def known_label(l):
    """A decision names the winner: "256x256w4x2p2" (16-bit template that stages through
    registers), "128x256x32w2x2s3g2" (the one that loads straight into LDS), "f32_128x64w2x2"
    (fp32 template), "attn_occ2" (attention, waves per SIMD), "pw_vec2" (fused pointwise
    kernels, elements per access), "rows_wg64" (row chains, threads per workgroup), "nt_loads"
    (a streaming kernel's accesses, alone or behind one of the two before), or keeps the
    default."""
    import re
    nt = r"nt_(none|loads|all)"      # a kernel that streams through a quarter of the memory-side cache and more: plain, nontemporal loads, loads and stores
    return bool(re.fullmatch(r"default|\d+x\d+w\dx\dp\d|\d+x\d+x\d+w\dx\ds\dg\d|f32_\d+x\d+w\dx\d|attn_occ\d|(pw_vec\d+|rows_wg\d+)(\+%s)?|%s" % (nt, nt), l))


@pytest.mark.parametrize("name,out_name", [("matmul_bf16_b16_1024x1024x1024", "C"), ("gpt2_small_bf16_b1_t1024", "output")])
def test_tuned_plan_is_bit_identical_and_remembered(name, out_name, tmp_path, monkeypatch):
    import torch
    if name.startswith("gpt2"):
        make = lambda plan: gpt2_slot_tensors(plan)[0]
    else:
        make = lambda plan: random_slot_tensors(plan, seed=2, scale=0.05)
    monkeypatch.setenv("POLY_HIP_CACHE_DIR", str(tmp_path / "cache"))
    want, plain_descs = run_plan(name, make, out_name)
    assert torch.isfinite(want.float()).all()
    monkeypatch.setenv("POLY_BEAM", "1")
    got, tuned_descs = run_plan(name, make, out_name)
    assert torch.equal(got.view(torch.uint8), want.view(torch.uint8)), "tuned result differs from the untuned one"
    decisions = [f for f in os.listdir(tmp_path / "cache") if f.endswith(".tune")]
    n_matmul_kinds = len({d.split(" ", 1)[1] for d in plain_descs if "matmul-mfma" in d})
    # (one decision per distinct set of candidates: every kind of matmul, and the attention
    # kernels, fused pointwise kernels and row chains, whose texts differ where their
    # descriptions do not)
    n_other = sum("attention" in d or "pointwise kernels over the same" in d or "row chain" in d for d in plain_descs)
    assert n_matmul_kinds <= len(decisions) <= n_matmul_kinds + n_other, (decisions, n_matmul_kinds, n_other)
    labels = {open(tmp_path / "cache" / f).read().strip() for f in decisions}
    assert all(known_label(l) for l in labels), labels
    # a later plan takes the recorded decisions: same kernels, nothing timed again
    again, again_descs = run_plan(name, make, out_name)
    assert torch.equal(again.view(torch.uint8), want.view(torch.uint8))
    assert [d.split(" ", 1)[1] for d in again_descs] == [d.split(" ", 1)[1] for d in tuned_descs]


def test_fp32_products_and_attention_are_tuned_too(tmp_path, monkeypatch):
    """The fp32 template (the 2-layer MLP's training step: forward, backward and SGD on fp32
    buffers) and the fused attention kernel carry candidates as well; what they decide
    changes no bit of any buffer of the plan."""
    import torch

    def all_buffers(name, make):
        plan = HipPlan.from_file(os.path.join(PLANS, name + ".polyplan"))
        data = make(plan)
        plan.run(data)
        plan.run(data)
        torch.cuda.synchronize()
        out = {s.name: data[s.index].clone() for s in plan.external_slots()}
        descs = [k["desc"] for k in plan.kernel_info()]
        plan.close()
        return out, descs

    cases = [("mlp_train_f32_b4096", lambda plan: random_slot_tensors(plan, seed=2), "mfma 32x32x2 f32", "f32_"),
             ("attention_bf16_b8_h12_t1024_d64", lambda plan: random_slot_tensors(plan, seed=2), "attention", "attn_occ")]
    for name, make, marker, prefix in cases:
        cache = tmp_path / name
        monkeypatch.setenv("POLY_HIP_CACHE_DIR", str(cache))
        monkeypatch.delenv("POLY_BEAM", raising=False)
        want, descs = all_buffers(name, make)
        assert any(marker in d for d in descs), descs
        monkeypatch.setenv("POLY_BEAM", "1")
        got, _ = all_buffers(name, make)
        for k in want:
            assert torch.equal(got[k].view(torch.uint8), want[k].view(torch.uint8)), (name, k)
        labels = [open(cache / f).read().strip() for f in os.listdir(cache) if f.endswith(".tune")]
        assert labels and all(known_label(l) for l in labels), labels
        assert any(l == "default" or l.startswith(prefix) for l in labels), labels


def test_streaming_forms_are_candidates_and_change_no_bit(tmp_path, monkeypatch):
    """The softmax over 8192 rows of 8192 (1 GiB moved) is timed with plain accesses, with
    nontemporal loads and with nontemporal loads and stores; whichever wins, the result is
    the untuned one bit for bit, and the decision is one of the three."""
    import torch
    name = "rowops_f32_8192_softmax"
    make = lambda plan: random_slot_tensors(plan, seed=1)
    monkeypatch.setenv("POLY_HIP_CACHE_DIR", str(tmp_path / "cache"))
    monkeypatch.delenv("POLY_BEAM", raising=False)
    want, descs = run_plan(name, make, "softmax")
    assert any("streaming loads" in d for d in descs), descs
    monkeypatch.setenv("POLY_BEAM", "1")
    got, tuned = run_plan(name, make, "softmax")
    assert torch.isfinite(want).all() and torch.equal(got.view(torch.uint8), want.view(torch.uint8))
    labels = [open(tmp_path / "cache" / f).read().strip() for f in os.listdir(tmp_path / "cache") if f.endswith(".tune")]
    assert len(labels) == 1 and (labels[0] == "default" or labels[0] in ("nt_none", "nt_all")), labels
    again, again_descs = run_plan(name, make, "softmax")
    assert torch.equal(again.view(torch.uint8), want.view(torch.uint8))
    assert [d.split(" ", 1)[1] for d in again_descs] == [d.split(" ", 1)[1] for d in tuned]
