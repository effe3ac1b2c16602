"""CPU-only checks of the product library: it loads and exports the whole C ABI,
every fixture kernel lowers to HIP C that hiprtc compiles for gfx950 (no device
needed), the index simplifier agrees with the raw index arithmetic, the plan
file round-trips, and error paths return errors instead of crashing."""
import ctypes as C
import os
import re
import subprocess
import tempfile

import numpy as np
import pytest

import fixtures as F
from polygrad_amd import PlanFile, _ffi, save_schedule

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def items_of(schedule_ptr):
    s = C.cast(schedule_ptr, C.POINTER(_ffi.PolySchedule)).contents
    return [s.items[s.exec_order[k]] for k in range(s.n_items)]


def test_library_exports_every_declared_symbol(hiplib):
    header = open(os.path.join(ROOT, "include", "polygrad_hip.h")).read()
    declared = set(re.findall(r"\b(poly_hip_\w+)\s*\(", header))
    assert len(declared) >= 35
    for name in sorted(declared):
        assert hasattr(hiplib, name), f"{name} is declared but not exported"
        assert name in _ffi.SYMBOLS, f"{name} has no ctypes signature"


def test_backend_descriptor_is_wired(hiplib):
    d = hiplib.poly_hip_backend_desc().contents
    assert d.name == b"hip" and d.id == 7 and not d.host_executed
    assert C.cast(d.lower_item, C.c_void_p).value == C.cast(hiplib.poly_hip_lower_item, C.c_void_p).value
    assert C.cast(d.execute, C.c_void_p).value == C.cast(hiplib.poly_hip_execute, C.c_void_p).value
    alloc = d.get_allocator().contents
    assert alloc.alloc and alloc.free and alloc.copy_in and alloc.copy_out and alloc.copy_between


@pytest.mark.parametrize("name", F.case_names())
def test_fixture_kernels_render_and_compile(name, hiplib):
    fx = F.Fixture(name)
    seen = set()
    for k, it in enumerate(items_of(fx.plan.schedule)):
        assert hiplib.poly_hip_check_index_simplification(it.root, 4096) == 0, f"{name} kernel {k}"
        for flags in (0, 1 | 2 | 4):
            src = _ffi.take_string(hiplib.poly_hip_render(it.root, b"k", flags, None))
            assert src, f"{name} kernel {k} did not render (flags {flags})"
            if src in seen:
                continue
            seen.add(src)
            assert hiplib.poly_hip_compile_check(src.encode()) == 0, f"{name} kernel {k} did not compile"


def test_planfile_round_trip(tmp_path):
    fx = F.Fixture("gpt2_tiny_bf16")
    out = tmp_path / "copy.polyplan"
    save_schedule(fx.plan.schedule, fx.plan.names, out)
    assert open(out, "rb").read() == open(os.path.join(F.GOLDEN, "gpt2_tiny_bf16.polyplan"), "rb").read()
    again = PlanFile(out)
    assert again.names == fx.plan.names and again.n_items == fx.plan.n_items
    # the reloaded schedule evaluates to the same outputs
    got = F.run_oracle_schedule(again.schedule, fx.n_slots, fx.inputs)
    for slot in fx.external:
        assert got[slot].tobytes() == fx.expected[slot].tobytes()


def test_planfile_rejects_garbage(tmp_path, hiplib):
    bad = tmp_path / "bad.polyplan"
    bad.write_bytes(b"not a plan file at all")
    assert not hiplib.poly_hip_planfile_load(str(bad).encode())
    good = open(os.path.join(F.GOLDEN, "kat_matmul_2x3x4.polyplan"), "rb").read()
    trunc = tmp_path / "trunc.polyplan"
    trunc.write_bytes(good[: len(good) // 2])
    assert not hiplib.poly_hip_planfile_load(str(trunc).encode())
    assert not hiplib.poly_hip_planfile_load(b"/nonexistent/file")


def test_error_paths_return_errors(hiplib):
    assert hiplib.poly_hip_render(None, b"k", 0, None) is None
    assert hiplib.poly_hip_compile_check(b"this is not HIP C") != 0
    assert hiplib.poly_hip_lower_item(None, None, b"k", None) < 0
    assert hiplib.poly_hip_execute(None, None, 0) < 0
    assert hiplib.poly_hip_plan_run(None, None, 0, None, 0) < 0
    assert not hiplib.poly_hip_compile_schedule(None, None)


def test_no_device_means_failure_not_fallback(hiplib):
    """Without a GPU every compute entry point must fail loudly."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    assert hiplib.poly_hip_available() == 0
    assert hiplib.poly_hip_init() != 0
    assert not hiplib.poly_hip_alloc(1024)
    fx = F.Fixture("kat_matmul_2x3x4")
    assert not hiplib.poly_hip_compile_schedule(None, fx.plan.schedule)
    it = items_of(fx.plan.schedule)[0]
    runner = _ffi.PolyRunner()
    assert hiplib.poly_hip_lower_item(None, it.root, b"k", C.byref(runner)) < 0


@pytest.mark.skipif(not os.path.exists("/root/reference/src/exec_plan.h"), reason="reference headers not present")
def test_abi_layout_matches_reference_headers(tmp_path):
    """sizeof/offsetof of every mirrored struct, from both sets of headers."""
    probe = r'''
#include <stdio.h>
#include <stddef.h>
#define P(T) printf(#T " %zu\n", sizeof(T))
#define O(T, f) printf(#T "." #f " %zu\n", offsetof(T, f))
int main(void) {
  P(PolyDType); O(PolyDType, bitsize); O(PolyDType, name); O(PolyDType, fmt); O(PolyDType, count); O(PolyDType, is_ptr);
  O(PolyDType, addrspace); O(PolyDType, vcount); O(PolyDType, ptr_size);
  P(PolyArg); O(PolyArg, i); O(PolyArg, range.axis_type); O(PolyArg, range.extra); O(PolyArg, define_var.max_val);
  P(PolyUOp); O(PolyUOp, dtype); O(PolyUOp, src); O(PolyUOp, n_src); O(PolyUOp, arg); O(PolyUOp, tag); O(PolyUOp, hash);
  P(PolyBufferHandle); O(PolyBufferHandle, nbytes); O(PolyBufferHandle, domain); O(PolyBufferHandle, owned);
  P(PolyAllocator); O(PolyAllocator, copy_between); O(PolyAllocator, dev_ctx);
  P(PolyVarBinding); O(PolyVarBinding, value);
  P(PolyScheduleBufSlot); O(PolyScheduleBufSlot, numel); O(PolyScheduleBufSlot, buf_uop); O(PolyScheduleBufSlot, is_intermediate); O(PolyScheduleBufSlot, external_buf_idx);
  P(PolyExecItem); O(PolyExecItem, root); O(PolyExecItem, buf_slot_indices); O(PolyExecItem, fixedvars); O(PolyExecItem, var_uops); O(PolyExecItem, n_var_uops);
  P(PolySchedule); O(PolySchedule, buf_slots); O(PolySchedule, items); O(PolySchedule, exec_order); O(PolySchedule, default_vars); O(PolySchedule, loss_buf_slot); O(PolySchedule, grad_buf_slots);
  P(PolyRunner); O(PolyRunner, handle); O(PolyRunner, execute); O(PolyRunner, grid); O(PolyRunner, block); O(PolyRunner, param_to_slot); O(PolyRunner, var_indices); O(PolyRunner, n_vars);
  P(PolyBackendDesc); O(PolyBackendDesc, id); O(PolyBackendDesc, host_executed); O(PolyBackendDesc, lower_item); O(PolyBackendDesc, get_allocator);
  printf("ops %d %d %d %d %d %d\n", (int)POLY_OP_PARAM, (int)POLY_OP_INDEX, (int)POLY_OP_ADD, (int)POLY_OP_WHERE, (int)POLY_OP_RANGE, (int)POLY_OP_REDUCE);
  printf("enums %d %d %d\n", (int)POLY_ARG_DEFINE_VAR, (int)POLY_AXIS_REDUCE, (int)POLY_DEVICE_X64_JIT);
  return 0;
}
'''
    outs = []
    for label, pre, inc in (("ours", '#include "polygrad_abi.h"\n', os.path.join(ROOT, "include")),
                            ("ref", '#include "frontend.h"\n#include "exec_plan.h"\n', "/root/reference/src")):
        src = tmp_path / f"{label}.c"
        src.write_text(pre + probe)
        exe = tmp_path / label
        subprocess.run(["gcc", "-std=c11", "-I", inc, str(src), "-o", str(exe)], check=True)
        outs.append(subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout)
    assert outs[0] == outs[1]


def test_kernel_groups_of_the_gpt2_plan_fuse_and_compile(hiplib):
    """Needs no device: in the benchmark schedule the plan compiler recognises, per layer,
    one attention group (six scheduled kernels plus the three q/k/v copies), three matmuls followed by a pointwise
    kernel (residual add, GELU, residual add) and two LayerNorms of three kernels each
    (plus the final LayerNorm); the generated sources compile.  The q | k | v product of a
    layer is a launch of its own that leaves the largest magnitude of every block of keys
    for the attention kernel behind it, which bounds the products of masked key blocks by
    them (POLY_HIP_NO_KEY_BOUNDS=1: neither)."""
    from polygrad_amd import PlanFile
    pf = PlanFile(os.path.join(ROOT, "polygrad_amd", "plans", "gpt2_small_bf16_b8_t1024.polyplan"))
    count = hiplib.poly_hip_fused_groups(pf.schedule, -1, None, None)
    assert count == 12 + 36 + 25 + 12
    seen = {}
    for i in range(count):
        src, n = C.c_void_p(), C.c_int()
        hiplib.poly_hip_fused_groups(pf.schedule, i, C.byref(src), C.byref(n))
        text = _ffi.take_string(src.value)
        kind = ("attention" if "POLY_FA_M" in text else "rows" if "poly_row_p0" in text else
                "keys" if "#define POLY_EP_BLOCKMAX_LO 768" in text else "tail")
        assert n.value == {"attention": 9, "tail": 2, "rows": 3, "keys": 1}[kind]
        seen.setdefault(kind, []).append(text)
    assert len(seen["attention"]) == 12 and len(seen["tail"]) == 36 and len(seen["rows"]) == 25 and len(seen["keys"]) == 12
    keys = seen["keys"][0]
    # 8 sequences x 12 heads x 16 blocks of 64 keys, z counting the sequence fastest
    assert "#define POLY_EP_BLOCKMAX_HI 1536" in keys and "(((n) - 768) / 64) * 8 + (m) / 1024) * 16 + ((m) % 1024) / 64" in keys
    assert "unsigned int* poly_scratch" in keys and "\n// ---- scratch ---- bytes=6144\n" in keys
    assert hiplib.poly_hip_compile_check(keys.split("\n// ---- ")[0].encode()) == 0
    assert all("#define POLY_FA_KMAX_TABLE ((const unsigned int*)poly_scratch + " in a for a in seen["attention"])
    os.environ["POLY_HIP_NO_KEY_BOUNDS"] = "1"
    try:
        assert hiplib.poly_hip_fused_groups(pf.schedule, -1, None, None) == 12 + 36 + 25
        src = C.c_void_p()
        hiplib.poly_hip_fused_groups(pf.schedule, 1, C.byref(src), None)
        assert "POLY_FA_KMAX_TABLE ((" not in _ffi.take_string(src.value)
    finally:
        del os.environ["POLY_HIP_NO_KEY_BOUNDS"]
    assert hiplib.poly_hip_compile_check(seen["rows"][0].encode()) == 0
    att = seen["attention"][0]
    assert "poly_fa_term" in att and "__builtin_amdgcn_mfma_f32_32x32x16_bf16" in att
    assert hiplib.poly_hip_compile_check(att.encode()) == 0
    for text in seen["tail"][:3]:      # one layer: attention residual, GELU, MLP residual
        assert "poly_ep_e1" in text
        assert hiplib.poly_hip_compile_check(text.encode()) == 0
    os.environ["POLY_HIP_NO_FUSION"] = "1"
    try:
        assert hiplib.poly_hip_fused_groups(pf.schedule, -1, None, None) == 0
    finally:
        del os.environ["POLY_HIP_NO_FUSION"]
    # softmax and LayerNorm on their own (scheduled as reduce, pointwise, reduce, pointwise over
    # rows of 8192): one row chain of all four kernels each, the inputs and the row in between
    # kept in registers; a single reduction: nothing
    for name, want in (("softmax", 1), ("layernorm", 1), ("sum", 0)):
        pf2 = PlanFile(os.path.join(ROOT, "polygrad_amd", "plans", f"rowops_f32_8192_{name}.polyplan"))
        src, n = C.c_void_p(), C.c_int()
        assert hiplib.poly_hip_fused_groups(pf2.schedule, 0, C.byref(src), C.byref(n)) == want
        if want:
            text = _ffi.take_string(src.value)
            assert n.value == 4 and "poly_row_p3" in text and "c0[it] = poly_vload" in text and "t2[it].v[u] =" in text
            assert hiplib.poly_hip_compile_check(text.encode()) == 0


def test_attention_forms_and_fp32_matmul_render(hiplib):
    """The attention group renders in its single-pass form by default and in the two-pass
    form on request; fp32 matmuls of the MLP train step take the fp32 MFMA template."""
    from polygrad_amd import PlanFile
    pf = PlanFile(os.path.join(ROOT, "polygrad_amd", "plans", "attention_bf16_b8_h12_t1024_d64.polyplan"))
    def attention_source():
        for i in range(hiplib.poly_hip_fused_groups(pf.schedule, -1, None, None)):
            src = C.c_void_p()
            hiplib.poly_hip_fused_groups(pf.schedule, i, C.byref(src), None)
            text = _ffi.take_string(src.value)
            if "POLY_FA_M" in text:
                return text
        raise AssertionError("no attention group")
    assert "#define POLY_FA_ONLINE 1" in attention_source()
    os.environ["POLY_HIP_EXACT_ATTENTION"] = "1"
    try:
        exact = attention_source()
    finally:
        del os.environ["POLY_HIP_EXACT_ATTENTION"]
    assert "#define POLY_FA_ONLINE 0" in exact and hiplib.poly_hip_compile_check(exact.encode()) == 0
    mlp = PlanFile(os.path.join(ROOT, "polygrad_amd", "plans", "mlp_train_f32_b4096.polyplan"))
    s = C.cast(mlp.schedule, C.POINTER(_ffi.PolySchedule)).contents
    descs = [_ffi.take_string(hiplib.poly_hip_describe(s.items[k].root, 0)) for k in range(s.n_items)]
    f32 = [d for d in descs if "mfma 32x32x2 f32" in d]
    assert len(f32) == 2 and any("M=4096 N=512 K=784" in d for d in f32) and any("M=512 N=784 K=4096" in d for d in f32), descs
    for k in range(s.n_items):
        if "mfma 32x32x2 f32" in descs[k]:
            src = _ffi.take_string(hiplib.poly_hip_render(s.items[k].root, b"k", 0, None))
            assert "__builtin_amdgcn_mfma_f32_32x32x2f32" in src and hiplib.poly_hip_compile_check(src.encode()) == 0


def test_tuning_candidates_render_and_compile(hiplib):
    """With POLY_BEAM set (the switch of the reference's own search, src/render_c.c:839) a
    16-bit matmul comes with its other tile shapes as candidates, and every one compiles;
    without it there are none."""
    from polygrad_amd import PlanFile
    pf = PlanFile(os.path.join(ROOT, "polygrad_amd", "plans", "matmul_bf16_8192x768x3072.polyplan"))
    s = C.cast(pf.schedule, C.POINTER(_ffi.PolySchedule)).contents
    plain = _ffi.take_string(hiplib.poly_hip_render(s.items[0].root, b"k", 0, None))
    assert "// ---- variant" not in plain
    os.environ["POLY_BEAM"] = "2"
    try:
        tuned = _ffi.take_string(hiplib.poly_hip_render(s.items[0].root, b"k", 0, None))
    finally:
        del os.environ["POLY_BEAM"]
    labels = re.findall(r"// ---- variant (\S+)", tuned)
    assert len(labels) >= 6 and len(set(labels)) == len(labels), labels
    # tile shapes of the register-staged template, and of the one that loads straight into LDS
    # (its labels carry the depth of a stage, the number of stages and the workgroups per CU)
    assert any(re.fullmatch(r"\d+x\d+w\dx\dp\d", l) for l in labels), labels
    assert any(re.fullmatch(r"\d+x\d+x\d+w\dx\ds\dg\d", l) for l in labels), labels
    assert tuned.startswith(plain)          # the default choice stays the kernel itself
    shapes = set(re.findall(r"#define POLY_BM (\d+)\n#define POLY_BN (\d+)", tuned))
    assert shapes >= {("256", "256"), ("256", "128"), ("128", "256"), ("128", "128")}, shapes
    assert hiplib.poly_hip_compile_check(tuned.encode()) == 0
    # a row chain (the LayerNorm of the GPT-2 plan) comes in smaller workgroups as well
    gpt2 = PlanFile(os.path.join(ROOT, "polygrad_amd", "plans", "gpt2_small_bf16_b1_t1024.polyplan"))
    os.environ["POLY_BEAM"] = "2"
    try:
        chains = []
        for i in range(hiplib.poly_hip_fused_groups(gpt2.schedule, -1, None, None)):
            src = C.c_void_p()
            hiplib.poly_hip_fused_groups(gpt2.schedule, i, C.byref(src), None)
            text = _ffi.take_string(src.value)
            if "poly_row_p0" in text:
                chains.append(text)
    finally:
        del os.environ["POLY_BEAM"]
    assert chains and all(re.findall(r"// ---- variant (\S+)", t) == ["rows_wg128", "rows_wg64"] for t in chains)
    units = chains[0].split("\n// ---- variant ")
    assert "__launch_bounds__(256) poly_k" in units[0] and "__launch_bounds__(128) poly_k" in units[1] and "__launch_bounds__(64) poly_k" in units[2]
    for u in units[1:]:
        assert hiplib.poly_hip_compile_check(u[u.index("\n") + 1:].encode()) == 0
