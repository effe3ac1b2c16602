"""A plan's captured graph and the buffers it is run with.

The reference runs a plan kernel by kernel with the buffers of the call
(src/exec_plan.c:1000-1057), so any call may bring other buffers.  The HIP plan captures
its launch sequence once; a set of buffers it has not seen is served by a second
instantiation of that capture whose kernel nodes get the new arguments, and a set it has
seen (compared value by value) replays the graph made for it.  Every case here is checked
bit for bit against the same plan run launch by launch, without a graph."""
import os

import pytest

pytestmark = pytest.mark.gpu

from polygrad_amd import HipPlan
from polygrad_amd.inputs import block_train_slot_tensors, gpt2_slot_tensors

PLANS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "polygrad_amd", "plans")


def load(name):
    path = os.path.join(PLANS, name + ".polyplan")
    if not os.path.exists(path):
        pytest.skip(f"{name} is not generated (python tests/golden/make_plans.py)")
    return HipPlan.from_file(path)


def test_alternating_output_buffers_update_the_graph():
    """GPT-2 small, B=1: two output buffers in turn, then a third and a fourth input."""
    import torch
    plan = load("gpt2_small_bf16_b1_t1024")
    data, names = gpt2_slot_tensors(plan, seed=3)
    out_slot = next(s.index for s in plan.external_slots() if s.name == "output")
    x_slot = next(s.index for s in plan.external_slots() if s.name == "x")

    plan.set_graph(False)
    plan.run(data)
    want = names["output"].clone()
    x2 = torch.roll(names["x"], 7)
    d = list(data)
    d[x_slot] = x2
    plan.run(d)
    want2 = names["output"].clone()
    assert not torch.equal(want, want2)
    plan.set_graph(True)

    outs = [torch.zeros_like(want) for _ in range(2)]
    for i in range(6):
        d = list(data)
        d[out_slot] = outs[i % 2]
        outs[i % 2].zero_()
        plan.run(d)
        assert torch.equal(outs[i % 2], want), f"pass {i}"
    assert plan.graph_counts() == (1, 1)        # one capture, one update, four replays

    # another input tensor: the first kernels' arguments change, the rest stay
    d = list(data)
    d[out_slot] = outs[0]
    d[x_slot] = x2
    plan.run(d)
    assert torch.equal(outs[0], want2)
    assert plan.graph_counts() == (1, 2)
    # more bindings than graphs are kept (four): the oldest is dropped and made again
    more = [torch.zeros_like(want) for _ in range(4)]
    for i, o in enumerate(more):
        d = list(data)
        d[out_slot] = o
        plan.run(d)
        assert torch.equal(o, want), f"buffer {i}"
    d = list(data)
    d[out_slot] = outs[1]
    outs[1].zero_()
    plan.run(d)
    assert torch.equal(outs[1], want)
    captures, rebinds = plan.graph_counts()
    assert captures == 1 and rebinds == 7, (captures, rebinds)
    plan.close()


def test_graph_rebinding_can_be_switched_off():
    """POLY_HIP_NO_GRAPH_REBIND=1: every new set of buffers is captured afresh."""
    import torch
    plan = load("gpt2_small_bf16_b1_t1024")
    data, names = gpt2_slot_tensors(plan, seed=3)
    out_slot = next(s.index for s in plan.external_slots() if s.name == "output")
    plan.run(data)
    want = names["output"].clone()
    other = torch.zeros_like(want)
    d = list(data)
    d[out_slot] = other
    os.environ["POLY_HIP_NO_GRAPH_REBIND"] = "1"
    try:
        plan.run(d)
    finally:
        os.environ.pop("POLY_HIP_NO_GRAPH_REBIND", None)
    assert torch.equal(other, want)
    assert plan.graph_counts() == (2, 0)
    plan.close()


def test_24_layer_training_state_in_two_sets_of_buffers():
    """The 24-layer training plan (side streams inside its graph, fills in front of
    launches, an arena of shared intermediates) steps two copies of the same state in turn:
    every external pointer changes between calls.  After two steps each, both copies hold
    the same bits as a state stepped twice without a graph."""
    import torch
    plan = load("gpt2_medium_train_24l_b4_t1024")
    base, base_names = block_train_slot_tensors(plan)

    def copy_of():
        d = [None if t is None else t.clone() for t in base]
        return d, {s.name: d[s.index] for s in plan.external_slots()}

    d0, n0 = copy_of()
    plan.set_graph(False)
    plan.run(d0)
    plan.run(d0)
    plan.set_graph(True)
    d1, n1 = copy_of()
    d2, n2 = copy_of()
    for _ in range(2):
        plan.run(d1)
        plan.run(d2)
    torch.cuda.synchronize()
    captures, rebinds = plan.graph_counts()
    assert plan.side_launches() > 100
    assert (captures, rebinds) == (1, 1), (captures, rebinds)
    for got in (n1, n2):
        differing = [k for k in n0 if not torch.equal(got[k].view(torch.uint8), n0[k].view(torch.uint8))]
        assert not differing, differing[:10]
    assert bool(torch.isfinite(n0["loss"].float()).all())
    plan.close()


def test_per_launch_times_add_up_to_the_step():
    """poly_hip_plan_profile times every kernel with the events its own dispatch stamps at
    start and end.  On the GPT-2 plan (one sequence) every launch gets a positive time, the
    head product is the longest, and the sum of all of them lies a little under the time of
    a replayed step (which also holds the gaps between kernels) -- not above it, as it did
    when the time a launch waits in the queue was counted with it."""
    import time
    import torch
    plan = load("gpt2_small_bf16_b1_t1024")
    data, _ = gpt2_slot_tensors(plan, seed=3)
    for _ in range(3):
        plan.run(data)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    steps = 20
    for _ in range(steps):
        plan.run(data, sync=False)
    plan.sync()
    step_ms = (time.perf_counter() - t0) / steps * 1e3
    info = plan.kernel_info()
    acc = [0.0] * len(info)
    for _ in range(3):
        plan.run(data, sync=False)
        for i, ms in enumerate(plan.profile(data)):
            acc[i] += ms / 3
    plan.close()
    assert all(ms > 0 for ms in acc), [k["desc"][:60] for k, ms in zip(info, acc) if ms <= 0]
    longest = max(range(len(acc)), key=lambda i: acc[i])
    assert "N=50257" in info[longest]["desc"], info[longest]["desc"]
    total = sum(acc)
    assert 0.6 * step_ms <= total <= 1.05 * step_ms, (total, step_ms)
