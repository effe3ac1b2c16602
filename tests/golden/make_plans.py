"""Writes the serialized schedules (plan files) that bench.py and smoke() load on
the GPU box, where the reference frontend is not part of the product path:

    polygrad_amd/plans/gpt2_small_bf16_b8_t1024.polyplan   GPT-2 small forward, B=8, T=1024, bf16
    polygrad_amd/plans/gpt2_small_bf16_b1_t1024.polyplan   the same graph for one sequence (parity slice)
    polygrad_amd/plans/rowops_f32_8192.polyplan            config 2 (fused chain + row ops), 8192x8192 fp32
    polygrad_amd/plans/matmul_bf16_<m>x<n>x<k>[_bt].polyplan   config 3 shapes
    polygrad_amd/plans/attention_bf16_b8_h12_t1024_d64.polyplan   the attention block of config 4 alone
    polygrad_amd/plans/mlp_train_f32_b4096.polyplan        config 1: MLP forward + backward + SGD step
    polygrad_amd/plans/adamw_f32_355m.polyplan             config 5: AdamW update of 355 M fp32 parameters
    polygrad_amd/plans/gpt2_medium_block_train_b4_t1024.polyplan   config 5: one block + head, backward, AdamW
    polygrad_amd/plans/gpt2_small_layer_matmuls_b8_t1024.polyplan  the four weight matmuls of a GPT-2 small layer with their tails
    polygrad_amd/plans/gpt2_medium_train_24l_b4_t1024.polyplan     config 5 whole: 24 blocks, head, loss, backward, AdamW
                                                                   (`python tests/golden/make_plans.py train24`)

The graphs are built with the REAL reference frontend and scheduler
(oracle/_ref/libpolygrad.so through tests/refpoly.py); only the scheduled kernel
graphs are stored, no reference code.  Run from the repository root:
    python tests/golden/make_plans.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import graphs  # noqa: E402
import refpoly as R  # noqa: E402
from hipharness import constant_name, constant_slots, schedule_slots  # noqa: E402
from polygrad_amd import save_schedule  # noqa: E402

OUT = os.path.join(ROOT, "polygrad_amd", "plans")


def save(c, sink, name):
    sched = c.schedule(sink)
    slots, n = schedule_slots(c, sched)
    names = [None] * n
    consts = constant_slots(c, sched)
    for i, tn in slots.items():
        names[i] = tn[1] if tn is not None else constant_name(consts[i])
    path = os.path.join(OUT, name + ".polyplan")
    save_schedule(sched, names, path)
    c.L.poly_schedule_free(sched)
    print(f"{name}: {os.path.getsize(path)} bytes")


def main():
    os.makedirs(OUT, exist_ok=True)
    for batch in (8, 1):
        c = R.Ctx()
        cfg = graphs.GPT2Config(batch=batch)
        sink, _ = graphs.gpt2_forward(c, cfg, R.BF16)
        save(c, sink, f"gpt2_small_bf16_b{batch}_t1024")
        c.close()
    c = R.Ctx()
    _, outs, sinks = graphs.fused_rowops(c, 8192, 8192)
    for k, s in sinks.items():
        save(c, s, f"rowops_f32_8192_{k}")
    c.close()
    for m, n, k, tb in ((4096, 4096, 4096, False), (8192, 8192, 8192, False), (16384, 3072, 768, False),
                        (8192, 768, 3072, False), (4096, 4096, 4096, True)):
        c = R.Ctx()
        _, _, _, sink = graphs.matmul_bf16(c, m, n, k, transposed_b=tb)
        save(c, sink, f"matmul_bf16_{m}x{n}x{k}" + ("_bt" if tb else ""))
        c.close()
    c = R.Ctx()
    _, sink = graphs.mlp_train_step(c, batch=4096)
    save(c, sink, "mlp_train_f32_b4096")
    c.close()
    c = R.Ctx()
    _, sink = graphs.adamw_step(c, 354_823_168)      # GPT-2 medium parameter count
    save(c, sink, "adamw_f32_355m")
    c.close()
    c = R.Ctx()
    _, sink = graphs.attention_bf16(c, batch=8, heads=12, ctx=1024, hd=64)
    save(c, sink, "attention_bf16_b8_h12_t1024_d64")
    c.close()
    c = R.Ctx()
    _, _, _, sink = graphs.matmul_bf16(c, 1024, 1024, 1024, batch=16)
    save(c, sink, "matmul_bf16_b16_1024x1024x1024")
    c.close()
    # the four weight matmuls of one GPT-2 small layer with their pointwise tails (bias, residual,
    # GELU), as gpt2_forward schedules them, without LayerNorm and attention: for timing them alone
    c = R.Ctx()
    BT, D = 8192, 768
    P = lambda name, shape: c.buffer(shape, R.BF16, name=name)
    x, o_qkv, o_h = P("x", (BT, D)), P("qkv", (BT, 3 * D)), P("h", (BT, D))
    qkv = graphs._linear(x, P("attn_w", (D, 3 * D)), P("attn_b", (3 * D,)), R.BF16).contiguous()
    a = graphs._linear(x, P("proj_w", (D, D)), P("proj_b", (D,)), R.BF16).contiguous()
    h = (x + a).contiguous()
    ff = graphs._linear(h, P("fc_w", (D, 4 * D)), P("fc_b", (4 * D,)), R.BF16).contiguous()
    ff = ff.gelu().contiguous()
    ff = graphs._linear(ff, P("fc2_w", (4 * D, D)), P("fc2_b", (D,)), R.BF16).contiguous()
    save(c, c.sink((o_qkv, qkv), (o_h, (h + ff).contiguous())), "gpt2_small_layer_matmuls_b8_t1024")
    c.close()
    c = R.Ctx()
    _, sink = graphs.gpt2_block_train_step(c, batch=4, ctx=1024, d_model=1024, heads=16, vocab=50257)
    save(c, sink, "gpt2_medium_block_train_b4_t1024")
    c.close()


def train_24_layers():
    """Config 5 whole: 24 blocks of GPT-2 medium above the embedding, head, loss, backward,
    AdamW.  Needs the build of the reference with raised buffer caps
    (oracle/_ref/libpolygrad_hip_ref.so, `make -C oracle ref_hip`): the stock limits stop at
    256 buffers (src/frontend_internal.h:23).  Scheduling takes about six minutes."""
    c = R.Ctx(hip_ref=True)
    _, sink = graphs.gpt2_block_train_step(c, batch=4, ctx=1024, d_model=1024, heads=16, vocab=50257, n_blocks=24)
    save(c, sink, "gpt2_medium_train_24l_b4_t1024")
    c.close()


if __name__ == "__main__":
    if sys.argv[1:] == ["train24"]:
        train_24_layers()
    else:
        main()
