"""Seeded synthetic GPT-2 inputs by buffer name, numpy only (no reference library), so the
build container that writes the full-size golden vectors and the GPU box that checks them
draw identical weights and tokens.  Follows the benchmark configuration: weights
~ N(0, 0.02), LayerNorm weights 1, biases 0, token ids uniform in [0, vocab) stored as
floats (src/modelzoo/models/gpt2.c:294-318), aranges 0..n-1."""
import numpy as np


def f32_to_bf16_bits(a):
    """Round-to-nearest-even conversion of float32 to bfloat16 bit patterns (uint16)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    u = a.view(np.uint32).astype(np.uint64)
    nan = np.isnan(a)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    r[nan] = 0x7FC0
    return r


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def gpt2_buffer_shapes(n_layer, d_model, vocab, ctx, batch):
    """(name, shape, is_float_index_buffer) of every buffer of the forward graph, in the
    order tests/graphs.py::gpt2_forward declares them (the order the generator draws in)."""
    V, D, T, B = vocab, d_model, ctx, batch
    out = [("wte.weight", (V, D), False), ("wpe.weight", (T, D), False)]
    for i in range(n_layer):
        p = f"h.{i}."
        out += [(p + "ln_1.weight", (D,), False), (p + "ln_1.bias", (D,), False),
                (p + "attn.c_attn.weight", (D, 3 * D), False), (p + "attn.c_attn.bias", (3 * D,), False),
                (p + "attn.c_proj.weight", (D, D), False), (p + "attn.c_proj.bias", (D,), False),
                (p + "ln_2.weight", (D,), False), (p + "ln_2.bias", (D,), False),
                (p + "mlp.c_fc.weight", (D, 4 * D), False), (p + "mlp.c_fc.bias", (4 * D,), False),
                (p + "mlp.c_proj.weight", (4 * D, D), False), (p + "mlp.c_proj.bias", (D,), False)]
    out += [("ln_f.weight", (D,), False), ("ln_f.bias", (D,), False),
            ("x", (B, T), True), ("output", (B, T, V), False),
            ("positions", (1, T), True), ("arange", (T,), True), ("vocab_arange", (V,), True)]
    return out


def gpt2_named_arrays(n_layer, d_model, vocab, ctx, batch, seed=3, bf16=True, skip=("output",)):
    """name -> flat array (uint16 bf16 bit patterns or float32; index buffers float32).
    Buffers named in `skip` consume no random numbers in the generator either way and are
    left out (the logits buffer is 100 MB per sequence)."""
    g = np.random.default_rng(seed)
    arrays = {}
    for name, shape, is_index in gpt2_buffer_shapes(n_layer, d_model, vocab, ctx, batch):
        n = int(np.prod(shape))
        if name == "x":
            a = g.integers(0, vocab, n).astype(np.float32)
        elif name in ("positions", "arange"):
            a = np.arange(ctx, dtype=np.float32)
        elif name == "vocab_arange":
            a = np.arange(vocab, dtype=np.float32)
        elif name == "output":
            if name in skip:
                continue
            a = np.zeros(n, np.float32)
        elif name.endswith("ln_1.weight") or name.endswith("ln_2.weight") or name == "ln_f.weight":
            a = np.ones(n, np.float32)
        elif name.endswith(".bias"):
            a = np.zeros(n, np.float32)
        else:
            a = g.normal(0.0, 0.02, n).astype(np.float32)
        if name in skip:
            continue
        arrays[name] = f32_to_bf16_bits(a) if (bf16 and not is_index) else a
    return arrays
