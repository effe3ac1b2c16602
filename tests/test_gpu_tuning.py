"""On-device tuning of the matmul template's tile shape (POLY_BEAM, as the reference's
search is switched on, src/render_c.c:839; its timing loop and disk cache are
src/codegen.c:1012-1195): a tuned plan must give bit-identical results -- every tile
shape accumulates a dot product in the same order -- and remember its decisions."""
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
    assert len(decisions) == n_matmul_kinds, (decisions, n_matmul_kinds)
    labels = {open(tmp_path / "cache" / f).read().strip() for f in decisions}
    # a decision names the tile of the winner ("256x256w4x2p2": the template that stages through
    # registers; "128x256x32w2x2s3g2": the one that loads straight into LDS) or keeps the default
    assert all(l == "default" or (l.count("x") in (2, 3) and ("p" in l or "s" in l)) for l in labels), labels
    # a later plan takes the recorded decisions: same kernels, nothing timed again
    again, again_descs = run_plan(name, make, out_name)
    assert torch.equal(again.view(torch.uint8), want.view(torch.uint8))
    assert [d.split(" ", 1)[1] for d in again_descs] == [d.split(" ", 1)[1] for d in tuned_descs]
