"""Golden vectors at the benchmark's sequence length (T = 1024), computed by the REAL
reference CPU backend (oracle/_ref/libpolygrad.so, built from /root/reference).  Takes
10-20 minutes on one core, so it is separate from make_golden.py.

Run from the repository root in the build container:
    python tests/golden/make_golden_fullsize.py [attention] [block0] [logits] [truth]

Writes
  tests/golden/attention_bf16_t1024.{polyplan,npz}
      an ordinary fixture (inputs + reference outputs): one sequence, two heads of 64
      features, 1024 positions, causal.
  tests/golden/fullsize/gpt2_small_bf16_b1_t1024_block0.{polyplan,npz}
      GPT-2 small (d_model 768, 12 heads, vocab 50257), embedding + block 0 for one
      sequence of 1024 tokens; npz: `hidden` = the residual stream after block 0,
      [1024, 768] bf16 bit patterns.
  tests/golden/fullsize/gpt2_small_bf16_b1_t1024_logits.npz
      the full 12-layer forward for the same sequence; `rows` = sampled positions,
      `logits_rows` = their full logit rows [len(rows), 50257], `cols` = sampled vocabulary
      columns, `logits_cols` = those columns at every position [1024, len(cols)]; bf16 bit
      patterns.  The plan is polygrad_amd/plans/gpt2_small_bf16_b1_t1024.polyplan.
  tests/golden/fullsize/gpt2_small_f32_b1_t1024_logits.npz
      the same network and sequence evaluated in fp32 by the reference (fp32 graph, the
      same bf16-valued weights), same rows and columns, float32.
Inputs are not stored: tests/gpt2_data.py regenerates them from seed 3.
"""
import os
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import gpt2_data  # noqa: E402
import graphs  # noqa: E402
import refpoly as R  # noqa: E402
from hipharness import schedule_slots  # noqa: E402
import make_golden  # noqa: E402
from make_golden import emit  # noqa: E402
from polygrad_amd import save_schedule  # noqa: E402

make_golden.ONLY = set()     # its case filter reads this script's arguments otherwise
FULL = os.path.join(HERE, "fullsize")
ROWS = np.array([0, 1, 31, 127, 128, 511, 1022, 1023])
COLS = np.arange(5, 50257, 787)      # 64 columns


def bind(bufs, named, extra):
    arrays = {}
    for name, t in bufs.items():
        if name in named:
            arrays[t] = named[name]
        elif name in extra:
            arrays[t] = extra[name]
    return arrays


def attention():
    g = np.random.default_rng(1024)
    c = R.Ctx()
    bufs, sink = graphs.attention_bf16(c, batch=1, heads=2, ctx=1024, hd=64)
    arrays = {bufs[n]: R.f32_to_bf16_bits(g.normal(0, 1.0, 1024 * 128).astype(np.float32)) for n in ("q", "k", "v")}
    arrays[bufs["arange"]] = np.arange(1024, dtype=np.float32)
    arrays[bufs["out"]] = np.zeros(1024 * 128, np.uint16)
    emit("attention_bf16_t1024", c, sink, arrays)
    c.close()


def block0():
    cfg = graphs.GPT2Config(n_layer=1, batch=1)
    # weights and tokens of the 12-layer model: the generator draws layer 0 before the rest
    named = gpt2_data.gpt2_named_arrays(12, cfg.d_model, cfg.vocab, cfg.ctx, 1, seed=3)
    c = R.Ctx()
    sink, bufs = graphs.gpt2_forward(c, cfg, R.BF16, hidden_only=True)
    hidden = np.zeros(cfg.ctx * cfg.d_model, np.uint16)
    arrays = bind(bufs, named, {"hidden": hidden})
    sched = c.schedule(sink)
    slots, n = schedule_slots(c, sched)
    names = [tn[1] if tn is not None else None for tn in (slots.get(i) for i in range(n))]
    save_schedule(sched, names, os.path.join(FULL, "gpt2_small_bf16_b1_t1024_block0.polyplan"))
    c.L.poly_schedule_free(sched)
    used = {tn[0] for tn in slots.values() if tn is not None}
    t0 = time.time()
    c.realize_cpu(sink, {t: a for t, a in arrays.items() if t in used})
    print(f"block0: reference ran in {time.time() - t0:.0f} s")
    np.savez_compressed(os.path.join(FULL, "gpt2_small_bf16_b1_t1024_block0.npz"), hidden=hidden)
    c.close()


def block0_truth():
    """Block 0 evaluated in fp32 by the reference (fp32 graph, same bf16-valued weights).
    Stored as float16: an 11-bit mantissa, eight times finer than the bf16 values that are
    compared against it, on values below 2."""
    cfg = graphs.GPT2Config(n_layer=1, batch=1)
    named = gpt2_data.gpt2_named_arrays(12, cfg.d_model, cfg.vocab, cfg.ctx, 1, seed=3)
    named = {k: (gpt2_data.bf16_bits_to_f32(a) if a.dtype == np.uint16 else a) for k, a in named.items()}
    c = R.Ctx()
    sink, bufs = graphs.gpt2_forward(c, cfg, R.F32, hidden_only=True)
    hidden = np.zeros(cfg.ctx * cfg.d_model, np.float32)
    arrays = bind(bufs, named, {"hidden": hidden})
    sched = c.schedule(sink)
    slots, _ = schedule_slots(c, sched)
    c.L.poly_schedule_free(sched)
    used = {tn[0] for tn in slots.values() if tn is not None}
    t0 = time.time()
    c.realize_cpu(sink, {t: a for t, a in arrays.items() if t in used})
    print(f"block0_truth: reference ran in {time.time() - t0:.0f} s")
    np.savez_compressed(os.path.join(FULL, "gpt2_small_f32_b1_t1024_block0.npz"), hidden=hidden.astype(np.float16))
    c.close()


def logits():
    cfg = graphs.GPT2Config(batch=1)
    named = gpt2_data.gpt2_named_arrays(12, cfg.d_model, cfg.vocab, cfg.ctx, 1, seed=3)
    c = R.Ctx()
    sink, bufs = graphs.gpt2_forward(c, cfg, R.BF16)
    out = np.zeros(cfg.ctx * cfg.vocab, np.uint16)
    arrays = bind(bufs, named, {"output": out})
    t0 = time.time()
    c.realize_cpu(sink, arrays)
    print(f"logits: reference ran in {time.time() - t0:.0f} s")
    lg = out.reshape(cfg.ctx, cfg.vocab)
    np.savez_compressed(os.path.join(FULL, "gpt2_small_bf16_b1_t1024_logits.npz"), rows=ROWS, logits_rows=lg[ROWS],
                        cols=COLS, logits_cols=np.ascontiguousarray(lg[:, COLS]))
    c.close()


def truth():
    """The same network evaluated in fp32 by the reference (same bf16-valued weights): what
    both bf16 evaluations approximate.  Stored at the same rows and columns."""
    cfg = graphs.GPT2Config(batch=1)
    named = gpt2_data.gpt2_named_arrays(12, cfg.d_model, cfg.vocab, cfg.ctx, 1, seed=3)
    named = {k: (gpt2_data.bf16_bits_to_f32(a) if a.dtype == np.uint16 else a) for k, a in named.items()}
    c = R.Ctx()
    sink, bufs = graphs.gpt2_forward(c, cfg, R.F32)
    out = np.zeros(cfg.ctx * cfg.vocab, np.float32)
    arrays = bind(bufs, named, {"output": out})
    t0 = time.time()
    c.realize_cpu(sink, arrays)
    print(f"truth: reference ran in {time.time() - t0:.0f} s")
    lg = out.reshape(cfg.ctx, cfg.vocab)
    np.savez_compressed(os.path.join(FULL, "gpt2_small_f32_b1_t1024_logits.npz"), rows=ROWS, logits_rows=lg[ROWS],
                        cols=COLS, logits_cols=np.ascontiguousarray(lg[:, COLS]))
    c.close()


if __name__ == "__main__":
    os.makedirs(FULL, exist_ok=True)
    which = sys.argv[1:] or ["attention", "block0", "block0_truth", "logits", "truth"]
    for w in which:
        {"attention": attention, "block0": block0, "block0_truth": block0_truth, "logits": logits, "truth": truth}[w]()
