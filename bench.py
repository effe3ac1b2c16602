#!/usr/bin/env python3
"""Benchmark of the HIP backend on one MI355X.

Default workload: GPT-2 small forward, random-init, B=8, T=1024, bf16 weights and
activations with fp32 reductions (BASELINE.json configs[3], the configuration the
headline metric is quoted on).  One step = one pass of the compiled plan over one
batch resident in HBM: poly_hip_plan_run() replaying the captured hipGraph.

Prints ONE JSON line: whole-job tokens/s, the roofline figures of the dominant
kernel (algorithmic flops or bytes / its average launch duration, measured with
HIP events on the backend's stream), a per-class breakdown, and the reference CPU
backend timed on a bounded sample of the same workload on this box's host cores.

    python bench.py --gpus 1 --steps 20 --warmup 3
    python bench.py --workload matmul_bf16_8192x8192x8192     (any plan in polygrad_amd/plans)
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0          # MI355X HBM3E
PEAK_MFMA_TFLOPS = 2500.0      # MI355X dense bf16/fp16 MFMA
PEAK_MFMA_F32_TFLOPS = 157.3   # MI355X dense fp32 MFMA
GPT2_PLAN = "gpt2_small_bf16_b8_t1024"

# HBM bytes per launch measured with `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE`
# (two runs of this script, counters scaled by what a plain copy of known size reads:
# FETCH_SIZE x 2.0 KiB, WRITE_SIZE x 1.0 KiB).  A counter run cannot be made from inside
# this script, so the figures are a table; each key is the start of a kernel description
# INCLUDING its tile shape or form, so that a kernel built differently from the one that
# was measured finds no entry and reports null.  The summaries with the commands are
# under profiles/ (…hbm_traffic_pmc.md).
MEASURED_TRAFFIC = {
    # FETCH_SIZE x 2.0 KiB + WRITE_SIZE x 1.0 KiB per launch (factors from `bench.py --copy-calibration`
    # under the same counters), rocprofv3 --pmc runs of `bench.py --steps 2 --warmup 1 --no-cpu-baseline`
    "attention-mfma: fused attention (9 kernels): mfma 32x32x16 bf16 Z=96 M=1024 N=1024 D=64, one pass, online softmax, mask tiles classified by a first kernel": 39.0e6 + 12.8e6 + 2.1e6,
    "matmul-mfma: mfma 32x32x16 bf16 M=8192 N=3072 K=768 Z=1 tile 128x256x32 A:k-major B:n-major, operands straight into LDS: 4 waves, 3 stages, 2 per CU, 64 workgroups read B ahead": 65.7e6 + 51.1e6,
    "matmul-mfma: mfma 32x32x16 bf16 M=8192 N=2304 K=768 Z=1 tile 128x192x32 A:k-major B:n-major, operands straight into LDS: 4 waves, 3 stages, 2 per CU, 64 workgroups read B ahead": 53.8e6 + 38.6e6,
    "matmul-mfma: mfma 32x32x16 bf16 M=8192 N=768 K=3072 Z=1 tile 128x128x64 A:k-major B:n-major, operands straight into LDS: 4 waves, 2 stages, 2 per CU, 64 workgroups read B ahead": 103.8e6 + 12.8e6,
    "matmul-mfma: mfma 32x32x16 bf16 M=8192 N=768 K=768 Z=1 tile 128x128x64 A:k-major B:n-major, operands straight into LDS: 4 waves, 2 stages, 2 per CU, 32 workgroups read B ahead": 34.8e6 + 12.7e6,
    "matmul-mfma: mfma 32x32x16 bf16 M=8192 N=50257 K=768 Z=1 tile 192x128x64 A:k-major B:k-major, operands straight into LDS: 4 waves, 2 stages, 2 per CU, 64 workgroups read B ahead": 1106.5e6 + 849.1e6,
    # the same two counters for `--workload rowops_f32_8192_{softmax,layernorm,sum,max} --steps 2 --warmup 1` and `--workload adamw_f32_355m`
    # (sum and max are the same kernel but for the combining operation)
    "row-reduce: row chain of 4 kernels (reduce vec4, map vec4, reduce vec4, map vec4) G=256 R=8192 rows=8192, 3 row loads kept in registers, intermediate rows kept in registers, streaming loads": 393310 * 2048.0 + 262144 * 1024.0,
    "row-reduce: row-reduce G=256 vec4 R=8192 rows=8192, streaming loads": 393230 * 2048.0 + 257 * 1024.0,
    "elementwise: 4 pointwise kernels over the same 354823168 positions as one, vec1, 1 buffers never written out, streaming loads and stores": 2772070 * 2048.0 + 4158090 * 1024.0,
    # the same two counters for `--workload gpt2_medium_train_24l_b4_t1024 --steps 1 --warmup 1`
    "row-reduce: row chain of 4 kernels (reduce vec4, map vec4, reduce vec4, map vec4) G=64 R=1024 rows=65536, 3 row loads kept in registers, intermediate rows kept in registers, result stored as the bf16 values that its fp32 values are casts of": 411.2e6 + 134.2e6,
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def kernel_key(desc):
    # "hip0_k12 row-reduce: ..." -> drop the per-plan kernel name
    return desc.split(" ", 1)[1] if " " in desc else desc


def run_gpu(workload, steps, warmup):
    import torch
    from polygrad_amd import HipPlan
    from polygrad_amd.inputs import block_train_slot_tensors, gpt2_slot_tensors, random_slot_tensors

    path = os.path.join(ROOT, "polygrad_amd", "plans", workload + ".polyplan")
    t0 = time.perf_counter()
    plan = HipPlan.from_file(path)
    compile_s = time.perf_counter() - t0
    if workload.startswith("gpt2_medium_block_train") or workload.startswith("gpt2_medium_train"):
        data, _ = block_train_slot_tensors(plan)
        tokens = None
    elif workload.startswith("gpt2_small_bf16"):
        data, _ = gpt2_slot_tensors(plan)
        tokens = [s for s in plan.slots if s.name == "x"][0].numel
    else:
        data = random_slot_tensors(plan, seed=2, scale=0.05 if "matmul" in workload else 1.0)
        tokens = None
    torch.cuda.synchronize()
    for _ in range(max(warmup, 1)):
        plan.run(data, sync=False)
    plan.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        plan.run(data, sync=False)
    plan.sync()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / steps * 1e3

    # per-kernel durations: every launch of a pass carries the pair of HIP events that its own
    # dispatch stamps at the kernel's start and end (poly_hip_plan_profile), on the backend's
    # stream; a replay of the graph goes ahead of each timed pass without a wait in between,
    # so that the timed launches find the chip busy, as they do inside the timed steps
    info = plan.kernel_info()
    passes = 5
    acc = [0.0] * len(info)
    for _ in range(passes):
        plan.run(data, sync=False)
        for i, ms in enumerate(plan.profile(data)):
            acc[i] += ms
    per_kernel_ms = [a / passes for a in acc]
    groups = {}
    for k, ms in zip(info, per_kernel_ms):
        g = groups.setdefault(kernel_key(k["desc"]), dict(klass=k["klass"], launches=0, ms=0.0, bytes=k["bytes"], flops=k["flops"]))
        g["launches"] += 1
        g["ms"] += ms
    dominant_key = max(groups, key=lambda k: groups[k]["ms"])
    d = groups[dominant_key]
    avg_ms = d["ms"] / d["launches"]
    if d["flops"] > 0:
        achieved = d["flops"] / (avg_ms * 1e-3) / 1e12
        # (the fp32 template multiplies on v_mfma_f32_32x32x2_f32, whose published peak is 157.3)
        peak = PEAK_MFMA_F32_TFLOPS if "mfma 32x32x2 f32" in dominant_key else PEAK_MFMA_TFLOPS
        roofline = dict(bound="mfma", achieved=round(achieved, 2), peak=peak, unit="TFLOP/s",
                        frac=round(achieved / peak, 4), traffic=None)
    else:
        achieved = d["bytes"] / (avg_ms * 1e-3) / 1e9
        roofline = dict(bound="hbm", achieved=round(achieved, 1), peak=PEAK_HBM_GBS, unit="GB/s",
                        frac=round(achieved / PEAK_HBM_GBS, 4), traffic=None)
    for prefix, traffic in MEASURED_TRAFFIC.items():
        if dominant_key.startswith(prefix):
            roofline["traffic"] = traffic
            roofline["traffic_source"] = ("rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE runs of this script, per launch, scaled by "
                                          "the same counters over bench.py --copy-calibration (x 2.0 KiB, x 1.0 KiB); summaries under profiles/")
    if roofline["traffic"] is None:
        roofline["traffic_source"] = "no counter run for this kernel in this form"
    roofline.update(kernel=dominant_key, launches_per_step=d["launches"], avg_launch_ms=round(avg_ms, 4),
                    algorithmic_bytes=d["bytes"], algorithmic_flops=d["flops"])
    if d["klass"] == "attention-mfma":
        # neither of the two rooflines binds this kernel: say what does
        roofline["note"] = ("bound by neither roofline: per score two roundings to bf16 (as the unfused kernels store "
                            "it), the mask, running maximum, exp2 and the sum on the VALU, in a dependent chain between "
                            "the two MFMAs of a tile at 3 waves per SIMD; SQ counters under profiles/")

    classes = {}
    for k, ms in zip(info, per_kernel_ms):
        c = classes.setdefault(k["klass"], dict(launches=0, ms=0.0, bytes=0.0, flops=0.0))
        c["launches"] += 1
        c["ms"] += ms
        c["bytes"] += k["bytes"]
        c["flops"] += k["flops"]
    for c in classes.values():
        c["GBps"] = round(c["bytes"] / (c["ms"] * 1e-3) / 1e9, 1) if c["ms"] > 0 else 0.0
        c["TFLOPs"] = round(c["flops"] / (c["ms"] * 1e-3) / 1e12, 1) if c["ms"] > 0 else 0.0
        c["hbm_frac"] = round(c["GBps"] / PEAK_HBM_GBS, 4)
        c["mfma_frac"] = round(c["TFLOPs"] / PEAK_MFMA_TFLOPS, 4)
        c["ms"] = round(c["ms"], 4)
        c["bytes"] = int(c["bytes"])
        c["flops"] = int(c["flops"])
    total_flops = sum(k["flops"] for k in info)
    total_bytes = sum(k["bytes"] for k in info)
    extra = dict(classes=classes, n_kernels=len(info), eager_sum_ms=round(sum(per_kernel_ms), 3),
                 plan_flops=int(total_flops), plan_bytes=int(total_bytes),
                 flop_time_ms=round(total_flops / (PEAK_MFMA_TFLOPS * 1e12) * 1e3, 3),
                 byte_time_ms=round(total_bytes / (PEAK_HBM_GBS * 1e9) * 1e3, 3),
                 workspace_MiB=round(plan.workspace_bytes() / 2**20, 1), compile_s=round(compile_s, 1))
    forms = sorted({("one pass, online softmax" if "one pass" in k["desc"] else "two passes, exact roundings") +
                    (", masked key blocks bounded by the keys' block maxima" if "bounded by the block maxima" in k["desc"] else "")
                    for k in info if k["klass"] == "attention-mfma"})
    if forms:
        extra["attention_form"] = "; ".join(forms)
    if tokens is not None:
        ctx = [s for s in plan.slots if s.name == "positions"]
        extra["seq_len"] = ctx[0].numel if ctx else None
    top = sorted(groups.items(), key=lambda kv: -kv[1]["ms"])[:int(os.environ.get("POLY_BENCH_GROUPS", "8"))]
    for key, g in top:
        log(f"  {g['ms']:8.3f} ms  x{g['launches']:3d}  {key[:int(os.environ.get('POLY_BENCH_DESC_CHARS', '150'))]}")
    plan.close()
    return ms_per_step, tokens, roofline, extra


def run_vtable(workload, steps, warmup):
    """The same schedule through the PolyBackendDesc row alone, the way the reference's own
    poly_compile_schedule / poly_compiled_plan_run drive a backend (src/exec_plan.c:801-1060):
    one lower_item per scheduled kernel, every intermediate its own allocation, one execute
    per kernel in execution order -- no fusion, no buffer sharing, no hipGraph.  Returns
    (ms per step, number of launches, MiB of intermediates)."""
    import ctypes as C
    import torch
    from polygrad_amd import PlanFile, _ffi
    from polygrad_amd.inputs import gpt2_slot_tensors, random_slot_tensors

    lib = _ffi.load()
    desc = lib.poly_hip_backend_desc().contents
    alloc = desc.get_allocator().contents
    pf = PlanFile(os.path.join(ROOT, "polygrad_amd", "plans", workload + ".polyplan"))
    sched = C.cast(pf.schedule, C.POINTER(_ffi.PolySchedule)).contents

    from polygrad_amd.plan import Slot

    class _Slots:          # what the input helpers need of a plan: its slots, with names
        pass
    shim = _Slots()
    shim.slots = [Slot(i, sched.buf_slots[i], pf.names[i] or "") for i in range(sched.n_buf_slots)]
    data = gpt2_slot_tensors(shim)[0] if workload.startswith("gpt2_small_bf16") else random_slot_tensors(shim, seed=2)
    runners = []
    for k in range(sched.n_items):
        r = _ffi.PolyRunner()
        if desc.lower_item(None, sched.items[k].root, f"lower0_k{k}".encode(), C.byref(r)) != 0:
            raise RuntimeError(f"lower_item failed for kernel {k}")
        runners.append(r)
    ptr, inter_bytes = [None] * sched.n_buf_slots, 0
    for i in range(sched.n_buf_slots):
        sl = sched.buf_slots[i]
        if sl.is_intermediate:
            ptr[i] = alloc.alloc(max(int(sl.nbytes), 4), alloc.dev_ctx)
            if not ptr[i]:
                raise RuntimeError("allocator returned NULL")
            inter_bytes += int(sl.nbytes)
        else:
            ptr[i] = data[i].data_ptr()
    args = []
    for k in range(sched.n_items):
        it = sched.items[k]
        args.append((C.c_void_p * it.n_buf_slots)(*[ptr[it.buf_slot_indices[j]] for j in range(it.n_buf_slots)]))
    order = [sched.exec_order[e] for e in range(sched.n_items)]
    torch.cuda.synchronize()

    def step():
        for k in order:
            if desc.execute(C.byref(runners[k]), args[k], len(args[k])) != 0:
                raise RuntimeError(f"execute failed for kernel {k}")

    for _ in range(max(warmup, 1)):
        step()
    lib.poly_hip_sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    lib.poly_hip_sync()
    ms = (time.perf_counter() - t0) / steps * 1e3
    for r in runners:
        desc.free_runner(C.byref(r))
    for i in range(sched.n_buf_slots):
        if sched.buf_slots[i].is_intermediate:
            alloc.free(ptr[i], alloc.dev_ctx)
    tokens = [sl for sl in shim.slots if sl.name == "x"][0].numel if workload.startswith("gpt2_small_bf16") else None
    return ms, sched.n_items, inter_bytes / 2**20, tokens


def cpu_baseline_reference(seconds_hint=20):
    """Times the REAL reference CPU backend (oracle/_ref/libpolygrad.so, built from the
    reference sources) on a bounded sample: GPT-2 small, 12 layers, bf16, one sequence
    of 32 tokens, single core (the reference has no threads)."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import graphs
    import refpoly as R
    if not R.available():
        return None
    cfg = graphs.GPT2Config(batch=1, ctx=32)
    c = R.Ctx()
    sink, bufs = graphs.gpt2_forward(c, cfg, R.BF16)
    arrays = graphs.gpt2_inputs(cfg, bufs, seed=3, wdt=R.BF16)
    t0 = time.perf_counter()
    c.realize_cpu(sink, arrays)          # first call: JIT (fork + clang per kernel), not timed as throughput
    jit_s = time.perf_counter() - t0
    t0 = time.perf_counter()
    c.realize_cpu(sink, arrays)          # warm call
    warm_s = time.perf_counter() - t0
    c.close()
    toks = cfg.batch * cfg.ctx
    return dict(value=round(toks / warm_s, 3), unit="tokens/s", cores=1, kind="reference",
                sample=f"GPT-2 small forward bf16, 12 layers, B=1, T=32 ({toks} tokens), warm poly_realize "
                       f"{warm_s:.2f} s (first call incl. clang JIT {jit_s:.1f} s); 1 of {os.cpu_count()} cores",
                warm_s=round(warm_s, 3))


def cpu_baseline_port():
    """Fallback when the reference library is not present: the CPU oracle on the tiny fixture."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import fixtures as F
    fx = F.Fixture("gpt2_tiny_bf16")
    t0 = time.perf_counter()
    F.run_oracle_schedule(fx.plan.schedule, fx.n_slots, fx.inputs)
    dt = time.perf_counter() - t0
    return dict(value=round(32 / dt, 3), unit="tokens/s", cores=1, kind="port",
                sample=f"CPU oracle on the tiny GPT-2 fixture (2 layers, d_model 32, vocab 97, 32 tokens) in {dt:.2f} s")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default=GPT2_PLAN)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--path", choices=["plan", "vtable"], default="plan",
                    help="plan: poly_hip_compile_schedule + poly_hip_plan_run (default, what the metric is quoted on); "
                         "vtable: the descriptor row alone, one launch per scheduled kernel")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="instead of a benchmark: three device-to-device copies of 1 GiB, the kernel of known traffic "
                         "that the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run are scaled by")
    args = ap.parse_args()
    if args.copy_calibration:
        import torch
        x = torch.empty(1 << 28, dtype=torch.float32, device="cuda").fill_(1.0)
        y = torch.empty_like(x)
        for _ in range(3):
            y.copy_(x)
        torch.cuda.synchronize()
        print(json.dumps({"copied_bytes_per_launch": x.numel() * 4, "launches": 3}), flush=True)
        return
    if args.gpus != 1:
        sys.exit("bench.py: this backend runs on one GPU; --gpus must be 1 (nothing here shards across devices)")
    # The CPU baseline first, before anything touches the GPU: the reference's CPU backend
    # forks and executes clang for every kernel (src/runtime_cpu.c:115-137), which a process
    # that has initialised the GPU should not do.
    cpu = None
    if not args.no_cpu_baseline and args.workload == GPT2_PLAN and args.path == "plan":
        try:
            cpu = cpu_baseline_reference() or cpu_baseline_port()
        except Exception as e:  # the baseline is reported, never required
            log(f"cpu baseline failed: {e}")
    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU available (there is no CPU path to benchmark)")

    if args.path == "vtable":
        ms, n, mib, tokens = run_vtable(args.workload, args.steps, args.warmup)
        value, unit = (tokens / (ms * 1e-3), "tokens/s") if tokens else (1e3 / ms, "passes/s")
        print(json.dumps({
            "metric": ("GPT-2-small fwd tokens/s on 1 MI355X" if tokens else "plan passes/s on 1 MI355X"), "value": round(value, 1), "unit": unit,
            "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "f32" if "_f32" in args.workload else "bf16", "data": "synthetic",
            "config": {"workload": args.workload, "plan": args.workload, "parallelism": "single GPU",
                       "execution": f"PolyBackendDesc row alone: {n} launches per step, one per scheduled kernel, "
                                    f"{mib:.0f} MiB of intermediates, no fusion, no hipGraph"},
            "roofline": None, "cpu_baseline": None}), flush=True)
        return
    ms, tokens, roofline, extra = run_gpu(args.workload, args.steps, args.warmup)
    if args.workload == GPT2_PLAN:
        # the drop-in path next to it: the descriptor row alone, a few steps
        try:
            vms, vn, vmib, vtok = run_vtable(args.workload, 3, 1)
            extra["vtable_path"] = {"ms_per_step": round(vms, 3), "tokens_per_s": round(vtok / (vms * 1e-3), 1), "launches": vn,
                                    "intermediates_MiB": round(vmib, 1),
                                    "note": "the PolyBackendDesc row driven kernel by kernel as src/exec_plan.c:1000-1057 does: "
                                            "no fusion, no buffer sharing, no hipGraph (bench.py --path vtable)"}
        except Exception as e:
            log(f"vtable path failed: {e}")
    if tokens is not None:
        metric, value, unit = "GPT-2-small fwd tokens/s on 1 MI355X", tokens / (ms * 1e-3), "tokens/s"
        T = extra.get("seq_len") or 1024
        workload = (f"GPT-2 small forward, random-init, B={tokens // T} T={T}, bf16 weights/activations, fp32 reductions"
                    + (" (BASELINE.json configs[3])" if (tokens // T, T) == (8, 1024) else ""))
    else:
        metric, value, unit = "plan passes/s on 1 MI355X", 1e3 / ms, "passes/s"
        workload = args.workload
    line = {
        "metric": metric, "value": round(value, 1), "unit": unit, "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32" if "_f32" in args.workload else "bf16", "data": "synthetic",
        "config": {"workload": workload, "plan": args.workload, "global_batch": (tokens // (extra.get("seq_len") or 1024)) if tokens else None,
                   "seq_len": extra.get("seq_len") if tokens else None, "parallelism": "single GPU",
                   "execution": "hipGraph replay of the compiled plan, inputs resident in HBM",
                   "parity": "against the reference CPU backend on the same seeded inputs (tests/, -m gpu): bit-exact for integer, "
                             "index and movement kernels; rtol 1e-5 fp32 elementwise, 1e-4 fp32 reductions and matmul, 2e-2 bf16/fp16, with an "
                             "absolute floor of 2e-2 of the tensor's scale on the T=1024 logits and residual stream (99.9 % of entries within "
                             "2.5e-3 of it) and of 8e-3 on the one-pass attention form's output (2e-3 for the two-pass form)"},
        "roofline": roofline, "cpu_baseline": cpu, "detail": extra,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
