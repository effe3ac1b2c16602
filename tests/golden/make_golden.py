"""Generates the committed golden fixtures: for each small case, the scheduled
plan (as a plan file) and the inputs plus the outputs computed by the REAL
reference CPU backend (oracle/_ref/libpolygrad.so, built from /root/reference).

Run from the repository root in the build container:
    python tests/golden/make_golden.py [case ...]
Writes tests/golden/<case>.polyplan and tests/golden/<case>.npz
(npz keys: in<slot> = initial contents of external slot, out<slot> = contents
after the reference ran).  bf16 data is stored as uint16 bit patterns.
"""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import graphs  # noqa: E402
import refpoly as R  # noqa: E402
from hipharness import schedule_slots  # noqa: E402
from polygrad_amd import save_schedule  # noqa: E402


ONLY = set(sys.argv[1:])     # optional: regenerate only the named cases


def emit(name, c, sink, arrays):
    if ONLY and name not in ONLY:
        return
    want = {t: np.array(a, copy=True) for t, a in arrays.items()}
    c.realize_cpu(sink, want)
    sched = c.schedule(sink)
    slots, n = schedule_slots(c, sched)
    names = [None] * n
    data = {}
    for i, tn in slots.items():
        t, nm = tn
        names[i] = nm
        data[f"in{i}"] = np.ascontiguousarray(arrays[t]).reshape(-1)
        data[f"out{i}"] = np.ascontiguousarray(want[t]).reshape(-1)
    save_schedule(sched, names, os.path.join(HERE, name + ".polyplan"))
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **data)
    c.L.poly_schedule_free(sched)
    print(f"{name}: {n} slots, {sum(v.nbytes for v in data.values())} bytes of vectors")


def emit_assembled(name):
    """A schedule put together by hand from kernels the reference scheduled, run through the
    reference's own poly_compile_schedule / poly_compiled_plan_run: an intermediate twice
    as large as what its producer writes.  The reference clears every intermediate at the
    start of every run (src/exec_plan.c:946-963), so the half nobody writes reads as zero.
    The reference frontend itself never builds such a schedule (poly_assign always targets
    a whole buffer, src/frontend.c:98-120); the case pins the rule for callers that do.

        J[0:2N]  = x2 * 3         (k0; J dies after k1, so I may take its bytes)
        out2     = J + 1          (k1)
        I[0:N]   = x * 2          (k2: writes the first half of I only)
        out      = I + 1          (k3: reads all 2N elements of I)
    """
    if ONLY and name not in ONLY:
        return
    from polygrad_amd import _ffi
    N = 1536
    c = R.Ctx()
    x, o1 = c.buffer((N,), name="x"), c.buffer((N,), name="o1")
    x2, o2 = c.buffer((2 * N,), name="x2"), c.buffer((2 * N,), name="o2")
    y, o3 = c.buffer((2 * N,), name="y"), c.buffer((2 * N,), name="o3")
    scheds = [c.schedule(c.sink((o2, x2 * c.const(3.0)))), c.schedule(c.sink((o3, y + c.const(1.0)))),
              c.schedule(c.sink((o1, x * c.const(2.0))))]
    parts = [C.cast(p, C.POINTER(_ffi.PolySchedule)).contents for p in scheds]
    for p, sp, out_t in zip(parts, scheds, (o2, o3, o1)):
        assert p.n_items == 1 and p.items[0].n_buf_slots == 2 and p.n_buf_slots == 2
        by_slot, _ = schedule_slots(c, sp)
        assert by_slot[p.items[0].buf_slot_indices[0]][0] == out_t, "PARAM 0 is expected to be the output"
    mul3, add1, mul2 = (p.items[0] for p in parts)
    f32_2n = parts[0].buf_slots[0]          # a float32 slot of 2N elements to copy dtype and sizes from
    # slots: 0 x2 (ext), 1 x (ext), 2 out2 (ext), 3 out (ext), 4 J (tmp), 5 I (tmp)
    slots = (_ffi.PolyScheduleBufSlot * 6)()
    for i, (numel, tmp) in enumerate(((2 * N, False), (N, False), (2 * N, False), (2 * N, False), (2 * N, True), (2 * N, True))):
        slots[i].dtype = f32_2n.dtype
        slots[i].numel, slots[i].nbytes = numel, 4 * numel
        slots[i].buf_uop = None
        slots[i].is_intermediate = tmp
        slots[i].external_buf_idx = -1
    items = (_ffi.PolyExecItem * 4)()
    keep = []
    for i, (src, (dst_slot, src_slot)) in enumerate(((mul3, (4, 0)), (add1, (2, 4)), (mul2, (5, 1)), (add1, (3, 5)))):
        idx = (C.c_int * 2)(dst_slot, src_slot)       # PARAM 0 is the output (checked above)
        keep.append(idx)
        items[i].kind = src.kind
        items[i].root = src.root
        items[i].buf_slot_indices = idx
        items[i].n_buf_slots = 2
    order = (C.c_int * 4)(0, 1, 2, 3)
    sched = _ffi.PolySchedule()
    sched.entrypoint_name = b"assembled"
    sched.buf_slots, sched.n_buf_slots = slots, 6
    sched.items, sched.n_items = items, 4
    sched.exec_order = order
    sched.loss_buf_slot = -1
    names = ["x2", "x", "out2", "out", None, None]
    g = np.random.default_rng(77)
    ins = [g.uniform(-1, 1, 2 * N).astype(np.float32), g.uniform(-1, 1, N).astype(np.float32),
           np.zeros(2 * N, np.float32), np.zeros(2 * N, np.float32)]
    outs = [a.copy() for a in ins]
    for _ in range(2):       # twice: the second run must find the holes cleared again
        c.run_schedule_ref(C.addressof(sched), outs + [None, None])
    assert np.array_equal(outs[3][:N], ins[1] * np.float32(2) + np.float32(1)) and np.all(outs[3][N:] == 1.0)
    data = {}
    for i in range(4):
        data[f"in{i}"], data[f"out{i}"] = ins[i], outs[i]
    save_schedule(C.addressof(sched), names, os.path.join(HERE, name + ".polyplan"))
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **data)
    for p in scheds:
        c.L.poly_schedule_free(p)
    c.close()
    print(f"{name}: hand-assembled, 6 slots")


def main():
    g = np.random.default_rng(1234)
    emit_assembled("assembled_partial_store")

    # reference KAT: (2,3)@(3,4) = [[38,44,50,56],[83,98,113,128]]  (test/test_nn.c:417-439)
    c = R.Ctx()
    A, B, O = c.buffer((2, 3), name="A"), c.buffer((3, 4), name="B"), c.buffer((2, 4), name="O")
    emit("kat_matmul_2x3x4", c, c.sink((O, A.dot(B))),
         {A: np.arange(1, 7, dtype=np.float32), B: np.arange(1, 13, dtype=np.float32), O: np.zeros(8, np.float32)})
    c.close()

    # reference KAT: threefry2x32, key 1337, counters 0..19 (test/test_nn.c:1122-1197)
    for dt, npdt, nm in ((R.U32, np.uint32, "u32"), (R.U64, np.uint64, "u64")):
        c = R.Ctx()
        ctr, key, out = c.buffer((20,), dt, name="counter"), c.buffer((20,), dt, name="key"), c.buffer((20,), dt, name="out")
        thr = ctr._bin("THREEFRY", key)
        emit(f"kat_threefry_{nm}", c, c.sink((out, thr)),
             {ctr: np.arange(20, dtype=npdt), key: np.full(20, 1337, npdt), out: np.zeros(20, npdt)})
        c.close()

    # cross-entropy of uniform logits over 3 classes = log 3 (test/test_nn.c:518-624)
    c = R.Ctx()
    lg, tg, o = c.buffer((4, 3), name="logits"), c.buffer((4, 3), name="target"), c.buffer((1,), name="loss")
    onehot = np.zeros((4, 3), np.float32)
    onehot[np.arange(4), [0, 1, 2, 1]] = 1
    emit("kat_xent_uniform", c, c.sink((o, lg.cross_entropy(tg))),
         {lg: np.full((4, 3), 0.7, np.float32), tg: onehot, o: np.zeros(1, np.float32)})
    c.close()

    # reductions over an axis of extent 1 (a batch of one): no loop, the value itself passes
    # through -- -0.0 stays -0.0, NaN stays NaN (src/codegen.c:1444-1450)
    c = R.Ctx()
    x, o1, o2 = c.buffer((8, 1), name="x"), c.buffer((8,), name="sum"), c.buffer((8,), name="max")
    xs = np.array([0.0, -0.0, 1.5, -2.25, np.nan, np.inf, -np.inf, 1e-40], np.float32)
    emit("reduce_singleton_axis", c, c.sink((o1, x.sum(1)), (o2, x.max(1))), {x: xs, o1: np.ones(8, np.float32), o2: np.ones(8, np.float32)})
    c.close()

    # fused chain + row ops (config 2 at a reduced shape)
    c = R.Ctx()
    (a, b, d), outs, sinks = graphs.fused_rowops(c, 24, 160)
    base = {a: g.uniform(-1, 1, (24, 160)).astype(np.float32), b: g.uniform(-1, 1, (24, 160)).astype(np.float32),
            d: g.uniform(-1, 1, (24, 160)).astype(np.float32)}
    for k in ("sum", "max", "softmax", "layernorm"):
        arr = dict(base)
        arr[outs[k]] = np.zeros(int(np.prod(outs[k].shape)), np.float32)
        emit(f"rowops_{k}", c, sinks[k], arr)
    c.close()

    # special values through exp2 / log2 / sqrt / reciprocal
    c = R.Ctx()
    x, o1, o2 = c.buffer((32,), name="x"), c.buffer((32,), name="exp2"), c.buffer((32,), name="log2")
    xs = np.array([0, -0.0, 1, -1, 0.5, 10, -10, 127, 128, 129, -126, -149, -150, -151, 1e-40, 3.14159,
                   np.inf, -np.inf, np.nan, 1e-4, 1e-5, 2.0**-127, 88.7, -88.7, 1e30, 1e-30, 7, 0.1, 0.9999999, 1.0000001,
                   1024, 3], np.float32)
    emit("special_exp2", c, c.sink((o1, x.exp2())), {x: xs, o1: np.zeros(32, np.float32)})
    emit("special_log2", c, c.sink((o2, x.log2())), {x: xs, o2: np.zeros(32, np.float32)})
    c.close()

    # movement ops on integers: permute / shrink / pad / flip, bit exact
    c = R.Ctx()
    x = c.buffer((6, 10, 8), R.I32, name="x")
    o = c.buffer((8, 5, 8), R.I32, name="o")
    y = x.permute((2, 1, 0)).shrink(((0, 8), (2, 7), (1, 5))).pad(((0, 0), (0, 0), (2, 2))).flip((1,))
    emit("movement_i32", c, c.sink((o, y)), {x: g.integers(-1000, 1000, 480).astype(np.int32), o: np.zeros(320, np.int32)})
    c.close()

    # integer ALU: div / mod / shifts / bit ops, bit exact
    c = R.Ctx()
    p, q, o = c.buffer((64,), R.I32, name="p"), c.buffer((64,), R.I32, name="q"), c.buffer((64,), R.I32, name="o")
    y = (p.idiv(q) + p.mod(q)).bxor(p.shl(c.const(3, R.I32))).band(q.bor(c.const(255, R.I32))) + p.shr(c.const(2, R.I32)) * q
    emit("int_alu", c, c.sink((o, y)),
         {p: g.integers(-5000, 5000, 64).astype(np.int32), q: g.integers(1, 50, 64).astype(np.int32), o: np.zeros(64, np.int32)})
    c.close()

    # bf16: elementwise GELU and matmul with f32 accumulate
    c = R.Ctx()
    x, o = c.buffer((8, 32), R.BF16, name="x"), c.buffer((8, 32), R.BF16, name="o")
    emit("bf16_gelu", c, c.sink((o, x.gelu())),
         {x: R.f32_to_bf16_bits(g.normal(0, 1.5, 256)), o: np.zeros(256, np.uint16)})
    c.close()
    c = R.Ctx()
    A, Bm, O, sink = graphs.matmul_bf16(c, 24, 40, 48)
    emit("bf16_matmul", c, sink, {A: R.f32_to_bf16_bits(g.normal(0, 0.02, 24 * 48)), Bm: R.f32_to_bf16_bits(g.normal(0, 0.02, 48 * 40)),
                                  O: np.zeros(24 * 40, np.float32)})
    c.close()
    c = R.Ctx()
    A, Bm, O, sink = graphs.matmul_bf16(c, 16, 24, 32, transposed_b=True, batch=3)
    emit("bf16_matmul_bt_batch", c, sink, {A: R.f32_to_bf16_bits(g.normal(0, 0.02, 3 * 16 * 32)), Bm: R.f32_to_bf16_bits(g.normal(0, 0.02, 24 * 32)),
                                           O: np.zeros(3 * 16 * 24, np.float32)})
    c.close()

    # fp16 casts and arithmetic (test/test_f16.c)
    c = R.Ctx()
    x, o = c.buffer((64,), R.F32, name="x"), c.buffer((64,), R.F16, name="o")
    xs = np.concatenate([g.normal(0, 100, 56).astype(np.float32),
                         np.array([0, -0.0, 65504, 65520, 1e-8, 6e-8, 6.1e-5, np.inf], np.float32)])
    emit("f16_cast_mul", c, c.sink((o, x.cast(R.F16) * x.cast(R.F16))), {x: xs, o: np.zeros(64, np.float16)})
    c.close()

    # tiny GPT-2, fp32 and bf16 (2 layers, d_model 32, vocab 97, T=16, B=2)
    for wdt, nm in ((R.F32, "f32"), (R.BF16, "bf16")):
        c = R.Ctx()
        sink, bufs = graphs.gpt2_forward(c, graphs.GPT2_TINY, wdt)
        arrays = graphs.gpt2_inputs(graphs.GPT2_TINY, bufs, seed=3, wdt=wdt)
        emit(f"gpt2_tiny_{nm}", c, sink, arrays)
        c.close()

    # sin over the ranges its decomposition distinguishes (src/codegen.c:2338-2660: small
    # arguments, Cody-Waite reduction, Payne-Hanek for huge ones) and its special values
    c = R.Ctx()
    x, o = c.buffer((64,), name="x"), c.buffer((64,), name="o")
    xs = np.concatenate([np.array([0, -0.0, 1e-8, -1e-8, 0.5, -0.5, 1, 2, 3, np.pi, -np.pi, np.pi / 2, 3 * np.pi / 2, 2 * np.pi, 10, 100, 1e3,
                                   1e4, 1e5, 3e5, 1e6, 1e8, 1e12, 1e20, 1e30, 3e38, np.inf, -np.inf, np.nan, 7.7, -123.456, 0.1], np.float32),
                         g.uniform(-30, 30, 32).astype(np.float32)])
    emit("special_sin", c, c.sink((o, x.sin())), {x: xs, o: np.zeros(64, np.float32)})
    c.close()

    # benchmark configuration 1 in small: MLP forward, cross-entropy, gradients, SGD step
    # with in-place parameter updates (22 kernels; src/instance.c:1152-1224 builds the same
    # p - lr * g ASSIGNs)
    c = R.Ctx()
    bufs, sink = graphs.mlp_train_step(c, batch=32, d_in=48, d_hid=40, d_out=10, lr=0.05)
    arrays = {}
    for name, t in bufs.items():
        n = int(np.prod(t.shape))
        if name == "X":
            a = g.normal(0, 1, n)
        elif name.startswith("W"):
            lim = (6.0 / t.shape[1]) ** 0.5
            a = g.uniform(-lim, lim, n)
        elif name == "Y":
            a = np.eye(10)[g.integers(0, 10, 32)].reshape(-1)
        else:
            a = np.zeros(n)
        arrays[t] = a.astype(np.float32)
    emit("mlp_train_b32", c, sink, arrays)
    c.close()

    # the kernel groups the plan compiler fuses, at the smallest shapes it takes them:
    # attention (128-query blocks, 64 features per head), matmul + GELU, LayerNorm rows
    c = R.Ctx()
    bufs, sink = graphs.attention_bf16(c, batch=1, heads=2, ctx=256, hd=64)
    arrays = {bufs[n]: R.f32_to_bf16_bits(g.normal(0, 1.0, 256 * 128).astype(np.float32)) for n in ("q", "k", "v")}
    arrays[bufs["arange"]] = np.arange(256, dtype=np.float32)
    arrays[bufs["out"]] = np.zeros(256 * 128, np.uint16)
    emit("attention_bf16_t256", c, sink, arrays)
    c.close()
    c = R.Ctx()
    A = c.buffer((128, 64), R.BF16, name="A")
    W = c.buffer((64, 256), R.BF16, name="W")
    bias = c.buffer((256,), R.BF16, name="bias")
    O = c.buffer((128, 256), R.BF16, name="O")
    y = (A.cast(R.F32).dot(W.cast(R.F32)).cast(R.BF16) + bias.reshape((1, 256)).expand((128, 256))).contiguous()
    emit("bf16_matmul_gelu", c, c.sink((O, y.gelu())),
         {A: R.f32_to_bf16_bits(g.normal(0, 1.0, 128 * 64).astype(np.float32)), W: R.f32_to_bf16_bits(g.normal(0, 0.3, 64 * 256).astype(np.float32)),
          bias: R.f32_to_bf16_bits(g.normal(0, 0.1, 256).astype(np.float32)), O: np.zeros(128 * 256, np.uint16)})
    c.close()
    c = R.Ctx()
    x = c.buffer((24, 256), R.BF16, name="x")
    w = c.buffer((256,), R.BF16, name="w")
    b = c.buffer((256,), R.BF16, name="b")
    o = c.buffer((24, 256), R.BF16, name="o")
    emit("bf16_layernorm_rows", c, c.sink((o, graphs._layernorm(x, w, b, 1e-5, R.BF16).contiguous())),
         {x: R.f32_to_bf16_bits(g.normal(0.3, 2.0, 24 * 256).astype(np.float32)), w: R.f32_to_bf16_bits(g.normal(1, 0.1, 256).astype(np.float32)),
          b: R.f32_to_bf16_bits(g.normal(0, 0.1, 256).astype(np.float32)), o: np.zeros(24 * 256, np.uint16)})
    c.close()


if __name__ == "__main__":
    main()
