"""Synthetic device-resident inputs for the benchmark plans, allocated with torch
(device memory only).  Follows the benchmark configuration: random-init weights
~ N(0, 0.02), LayerNorm weights 1, biases 0, token ids uniform in [0, vocab)
stored as floats (as the reference's GPT-2 builder stores them,
src/modelzoo/models/gpt2.c:294-318), aranges 0..n-1."""
import torch

_TORCH = {"bool": torch.bool, "int8": torch.int8, "uint8": torch.uint8, "int16": torch.int16, "uint16": torch.int16,
          "int32": torch.int32, "uint32": torch.int32, "int64": torch.int64, "uint64": torch.int64,
          "float16": torch.float16, "bfloat16": torch.bfloat16, "float32": torch.float32, "float64": torch.float64}


def torch_dtype(name):
    return _TORCH[name]


def gpt2_slot_tensors(plan, vocab=50257, seed=3, device="cuda"):
    """One tensor per external slot of a GPT-2 forward plan, keyed by the slot names
    the plan file carries.  Returns (list indexed by slot, dict by name)."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    data = [None] * len(plan.slots)
    by_name = {}
    for s in plan.slots:
        if s.is_intermediate:
            continue
        dt = torch_dtype(s.dtype)
        n = s.numel
        name = s.name
        if name == "x":
            t = torch.randint(0, vocab, (n,), generator=g, device=device).to(dt)
        elif name in ("positions", "arange", "vocab_arange"):
            t = torch.arange(n, device=device).to(dt)
        elif name == "output":
            t = torch.zeros(n, dtype=dt, device=device)
        elif name.endswith("ln_1.weight") or name.endswith("ln_2.weight") or name == "ln_f.weight":
            t = torch.ones(n, dtype=dt, device=device)
        elif name.endswith(".bias"):
            t = torch.zeros(n, dtype=dt, device=device)
        else:
            t = (torch.randn(n, generator=g, device=device, dtype=torch.float32) * 0.02).to(dt)
        data[s.index] = t
        by_name[name] = t
    return data, by_name


def random_slot_tensors(plan, seed=0, device="cuda", scale=1.0, outputs=()):
    """Uniform(-scale, scale) floats (or small ints) for every external slot; slots named
    like the reference's index helpers (arange, positions, vocab_arange) hold 0..n-1."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    data = [None] * len(plan.slots)
    for s in plan.slots:
        if s.is_intermediate:
            continue
        dt = torch_dtype(s.dtype)
        if s.name in outputs:
            t = torch.zeros(s.numel, dtype=dt, device=device)
        elif s.name in ("positions", "arange", "vocab_arange") or s.name.startswith("__arange_"):
            t = torch.arange(s.numel, device=device).to(dt)
        elif dt.is_floating_point:
            t = ((torch.rand(s.numel, generator=g, device=device, dtype=torch.float32) * 2 - 1) * scale).to(dt)
        else:
            t = torch.randint(0, 100, (s.numel,), generator=g, device=device).to(dt)
        data[s.index] = t
    return data


def block_train_slot_tensors(plan, vocab=50257, seed=4, device="cuda"):
    """Inputs of the one-block training plan (benchmark configuration 5): fp32 master
    weights ~ N(0, 0.02), LayerNorm weights 1, biases and optimizer state 0, bf16
    activations ~ N(0, 1), uniform random targets stored as floats, bias corrections of
    the first AdamW step.  Returns (list indexed by slot, dict by name)."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    data = [None] * len(plan.slots)
    by_name = {}
    for s in plan.slots:
        if s.is_intermediate:
            continue
        dt = torch_dtype(s.dtype)
        n, name = s.numel, s.name
        if name == "h0":
            t = torch.randn(n, generator=g, device=device, dtype=torch.float32).to(dt)
        elif name == "target":
            t = torch.randint(0, vocab, (n,), generator=g, device=device).to(dt)
        elif name == "arange" or name.startswith("__arange_"):
            t = torch.arange(n, device=device).to(dt)
        elif name == "bc1":
            t = torch.full((n,), 1.0 / (1.0 - 0.9), dtype=dt, device=device)
        elif name == "bc2":
            t = torch.full((n,), 1.0 / (1.0 - 0.999), dtype=dt, device=device)
        elif name.endswith(".m") or name.endswith(".v") or name == "loss" or name.endswith("_b"):
            t = torch.zeros(n, dtype=dt, device=device)
        elif name.split(".")[-1] in ("ln1_w", "ln2_w", "lnf_w"):     # (blocks of a deeper stack are named h<i>.<parameter>)
            t = torch.ones(n, dtype=dt, device=device)
        else:
            t = (torch.randn(n, generator=g, device=device, dtype=torch.float32) * 0.02).to(dt)
        data[s.index] = t
        by_name[name] = t
    return data, by_name
