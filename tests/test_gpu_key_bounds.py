"""Bounds on the keys of masked blocks.

The reference runs attention as separate kernels (gpt2.c:411-441): every score is computed,
the mask is added, and a key above the diagonal keeps a weight of zero only because
exp2(score - 1e9 - max) underflows.  The fused attention kernel may pass over such a key
block without computing its products only if it can prove that: the q | k | v product
leaves the largest |k| of every block of 64 keys, and the kernel bounds |q . k| by that times
sum |q|.  Every case here runs the GPT-2 plan with and without those bounds
(POLY_HIP_NO_KEY_BOUNDS=1 computes the products of every masked block and looks at them)
and wants the same bits, also where keys are so large that masked keys come back, or are
not finite."""
import os

import pytest

pytestmark = pytest.mark.gpu

from polygrad_amd import HipPlan
from polygrad_amd.inputs import gpt2_slot_tensors

PLANS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "polygrad_amd", "plans")


def logits(plan_name, tweak, bounds):
    import torch
    if not bounds:
        os.environ["POLY_HIP_NO_KEY_BOUNDS"] = "1"
    try:
        plan = HipPlan.from_file(os.path.join(PLANS, plan_name + ".polyplan"))
    finally:
        os.environ.pop("POLY_HIP_NO_KEY_BOUNDS", None)
    data, names = gpt2_slot_tensors(plan, seed=3)
    tweak(names)
    plan.run(data)
    plan.run(data)          # (the replayed graph)
    torch.cuda.synchronize()
    descs = [k["desc"] for k in plan.kernel_info()]
    out = names["output"].clone()
    plan.close()
    with_bounds = [d for d in descs if "bounded by the block maxima" in d]
    writers = [d for d in descs if "leaves the largest magnitude of every 64x64 block of columns [768, 1536)" in d]
    assert len(with_bounds) == len(writers) == (12 if bounds else 0), (len(with_bounds), len(writers))
    return out


def k_columns(names, layer, head):
    """The 64 key features of `head` in the q | k | v projection of `layer`: weight [768, 2304], bias [2304]."""
    w = names[f"h.{layer}.attn.c_attn.weight"].view(768, 2304)
    b = names[f"h.{layer}.attn.c_attn.bias"].view(2304)
    lo = 768 + 64 * head
    return w[:, lo:lo + 64], b[lo:lo + 64]


def nothing(names):
    pass


def huge_keys(names):
    """Keys of one head of two layers around 5e8: scores of the order of the mask's -1e9, so
    that keys above the diagonal come back with weight (a kernel that passed over them
    without looking gives other logits: tried with the bound scaled down); another head at
    5e7, where they do not but the bound cannot show it."""
    for layer, head, f in ((0, 3, 1e9), (5, 3, 1e9), (5, 9, 1e8)):
        w, _ = k_columns(names, layer, head)
        w.mul_(f)


def keys_not_finite(names):
    """NaN in one key feature of a head (every key of the head), +inf in another head's."""
    _, b = k_columns(names, 2, 5)
    b[7] = float("nan")
    _, b = k_columns(names, 4, 7)
    b[0] = float("inf")


def huge_queries(names):
    """Queries of a head around 1e10 (their sum |q| enters the bound)."""
    w = names["h.1.attn.c_attn.weight"].view(768, 2304)
    w[:, 64 * 2:64 * 3].mul_(2e10)


# The mask is data: the plan computes it as where(arange[i] < arange[j], -1e9, 0) from the
# `arange` input (reference builder: gpt2.c:344-358), so other contents of that buffer give
# other masks -- with the same plan, and the same inputs in both legs of the comparison.
def mask_the_other_way(names):
    """Keys BELOW the diagonal masked: the masked blocks of a query come before its live ones,
    when it has no maximum yet."""
    import torch
    a = names["arange"]
    a.copy_(torch.arange(a.numel() - 1, -1, -1, device=a.device).to(a.dtype))


def mask_in_bands(names):
    """arange in steps of 100 positions: a staircase whose tiles are mixed along every step,
    blocks of 64 keys that are masked for some waves of a workgroup and live for others."""
    import torch
    a = names["arange"]
    a.copy_((torch.arange(a.numel(), device=a.device) // 100).to(a.dtype))


def mask_at_random(names):
    """A random order of positions: hardly a tile with one value; with huge keys in one head."""
    import torch
    a = names["arange"]
    g = torch.Generator(device=a.device)
    g.manual_seed(5)
    a.copy_(torch.randperm(a.numel(), generator=g, device=a.device).to(a.dtype))
    w, _ = k_columns(names, 3, 1)
    w.mul_(1e9)


def no_mask(names):
    """All positions equal: nothing is masked, every tile holds zeros."""
    names["arange"].zero_()


@pytest.mark.parametrize("tweak", [nothing, huge_keys, keys_not_finite, huge_queries, mask_the_other_way, mask_in_bands, mask_at_random, no_mask],
                         ids=lambda f: f.__name__)
def test_one_sequence_same_bits_with_and_without_key_bounds(tweak):
    import torch
    got = logits("gpt2_small_bf16_b1_t1024", tweak, True)
    want = logits("gpt2_small_bf16_b1_t1024", tweak, False)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    if tweak in (nothing, huge_keys):
        assert bool(torch.isfinite(got.float()).all())
    if tweak in (mask_the_other_way, mask_in_bands, mask_at_random, no_mask):
        # (the buffer does feed the mask: other logits than with the causal one)
        assert not torch.equal(got.view(torch.int16), logits("gpt2_small_bf16_b1_t1024", nothing, True).view(torch.int16))
    if tweak is keys_not_finite:
        assert bool(torch.isnan(got.float()).any())


def test_eight_sequences_same_bits_with_and_without_key_bounds():
    """The plan the benchmark times: z counts the sequence fastest there."""
    import torch
    got = logits("gpt2_small_bf16_b8_t1024", huge_keys, True)
    want = logits("gpt2_small_bf16_b8_t1024", huge_keys, False)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    got = logits("gpt2_small_bf16_b8_t1024", nothing, True)
    want = logits("gpt2_small_bf16_b8_t1024", nothing, False)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_scores_of_1e10_stay_finite_in_the_single_pass_form():
    """Keys of a head around 1e10 give scores around 1e10, which the unfused kernels handle:
    they subtract the row's maximum before anything is multiplied.  The single-pass kernel
    forms its exponents as x c - m c while the reference m is small and as (x - m) c beyond
    4096 (the fused form would put the rounding of m c, here around 1e3, into the exponent:
    every term 0 or inf, rows of 0 / 0).  Wanted: finite logits, the same with and without
    the bounds on the keys, and as close to the two-pass form (which keeps every rounding of
    the unfused kernels) as on ordinary data."""
    import torch

    def tweak(names):
        w, _ = k_columns(names, 0, 3)
        w.mul_(2e10)

    got = logits("gpt2_small_bf16_b1_t1024", tweak, True)
    assert torch.equal(got.view(torch.int16), logits("gpt2_small_bf16_b1_t1024", tweak, False).view(torch.int16))
    os.environ["POLY_HIP_EXACT_ATTENTION"] = "1"
    try:
        plan = HipPlan.from_file(os.path.join(PLANS, "gpt2_small_bf16_b1_t1024.polyplan"))
    finally:
        os.environ.pop("POLY_HIP_EXACT_ATTENTION", None)
    data, names = gpt2_slot_tensors(plan, seed=3)
    tweak(names)
    plan.run(data)
    want = names["output"].clone().float()
    plan.close()
    assert bool(torch.isfinite(got.float()).all()) and bool(torch.isfinite(want).all())
    err = (got.float() - want).abs()
    scale = float(want.abs().max())
    assert float(err.mean()) <= 4e-3 * scale and float(err.max()) <= 4e-2 * scale, (float(err.mean()), float(err.max()), scale)
