"""poly_hip_execute_static -- the entry point that allocates nothing -- against
poly_hip_execute, through the C ABI: two-stage kernels of the MLP training step (config 1)
run once with scratch memory the runner allocates and once with the library's static
device array, on the same inputs; results must be bit-identical (same kernels, same
arithmetic, only the scratch address differs).  Two calls in a row share the array, the
second with a smaller kernel, so what the first left behind is still in it."""
import ctypes as C
import os

import numpy as np
import pytest

import gpt2_data
from polygrad_amd import PlanFile, _ffi

pytestmark = pytest.mark.gpu

PLANS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "polygrad_amd", "plans")
STATIC_BYTES = 32 << 20      # POLY_HIP_STATIC_SCRATCH_BYTES in include/polygrad_hip.h


class Kernel:
    """One scheduled kernel lowered through the descriptor row, with device buffers of its own."""

    def __init__(self, plan, k, seed):
        self.lib = _ffi.load()
        self.desc = self.lib.poly_hip_backend_desc().contents
        self.alloc = self.desc.get_allocator().contents
        sched = C.cast(plan.schedule, C.POINTER(_ffi.PolySchedule)).contents
        item = sched.items[k]
        self.runner = _ffi.PolyRunner()
        assert self.desc.lower_item(None, item.root, f"noalloc_k{k}".encode(), C.byref(self.runner)) == 0
        assert item.n_var_uops == 0
        g = np.random.default_rng(seed)
        self.host, self.dev = [], []
        for j in range(item.n_buf_slots):
            slot = sched.buf_slots[item.buf_slot_indices[j]]
            a = g.uniform(-1, 1, int(slot.numel)).astype(np.float32)
            if slot.dtype.name == b"__bf16":
                a = gpt2_data.f32_to_bf16_bits(a)
            else:
                assert slot.dtype.name == b"float", slot.dtype.name
            self.host.append(a)
            p = self.alloc.alloc(int(slot.nbytes), self.alloc.dev_ctx)
            assert p
            self.dev.append(p)
        self.args = (C.c_void_p * len(self.dev))(*self.dev)

    def upload(self):
        for a, p in zip(self.host, self.dev):
            assert self.alloc.copy_in(p, a.ctypes.data, a.nbytes, self.alloc.dev_ctx) == 0

    def download(self):
        out = []
        for a, p in zip(self.host, self.dev):
            b = np.empty_like(a)
            assert self.alloc.copy_out(b.ctypes.data, p, b.nbytes, self.alloc.dev_ctx) == 0
            out.append(b)
        return out

    def run(self, static):
        self.upload()
        fn = self.lib.poly_hip_execute_static if static else self.lib.poly_hip_execute
        rc = fn(C.byref(self.runner), self.args, len(self.dev))
        return rc, (self.download() if rc == 0 else None)

    def close(self):
        self.desc.free_runner(C.byref(self.runner))
        for p in self.dev:
            self.alloc.free(p, self.alloc.dev_ctx)


def two_stage_kernels(plan):
    """Kernel index -> bytes of scratch memory, for the kernels that run in two stages."""
    import re
    lib = _ffi.load()
    sched = C.cast(plan.schedule, C.POINTER(_ffi.PolySchedule)).contents
    out = {}
    for k in range(sched.n_items):
        src = _ffi.take_string(lib.poly_hip_render(sched.items[k].root, b"k", 0, None))
        m = re.search(r"// ---- first stage ---- .* scratch=(\d+)", src or "")
        if m:
            out[k] = int(m.group(1))
    return out


def test_static_scratch_matches_allocated_scratch_two_calls_in_a_row():
    assert _ffi.load().poly_hip_init() == 0
    plan = PlanFile(os.path.join(PLANS, "mlp_train_f32_b4096.polyplan"))
    staged = two_stage_kernels(plan)
    fits = sorted((b, k) for k, b in staged.items() if b <= STATIC_BYTES)
    assert len(fits) >= 2, staged
    big, small = fits[-1][1], fits[0][1]          # the largest scratch user first, then the smallest
    assert staged[big] > staged[small]
    kernels = [Kernel(plan, big, seed=11), Kernel(plan, small, seed=12)]
    try:
        import torch
        # the static path first, on runners that have never run and so own no scratch memory:
        # the calls must leave the device's free memory where it was (the runner's own scratch
        # of this size would show: hipMalloc takes whole 2 MiB pieces for it)
        for kn in kernels:
            kn.upload()
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        got = []
        for kn in kernels:                           # back to back on the shared array
            rc = kn.lib.poly_hip_execute_static(C.byref(kn.runner), kn.args, len(kn.dev))
            assert rc == 0
        assert kn.lib.poly_hip_sync() == 0
        free_after = torch.cuda.mem_get_info()[0]
        # (the runtime may take a little memory of its own at a kernel's first launch; the
        # runner's scratch for the larger kernel is 12 MiB)
        assert staged[big] >= (8 << 20), "the larger kernel's scratch would be too small to show in the free memory"
        assert free_before - free_after < staged[big] // 2, f"poly_hip_execute_static took {free_before - free_after} bytes of device memory"
        for kn in kernels:
            got.append(kn.download())
        want = []
        for kn in kernels:
            rc, out = kn.run(static=False)
            assert rc == 0
            want.append(out)
        for w, g_, kn, k in zip(want, got, kernels, (big, small)):
            assert (g_[0] != kn.host[0]).any(), "the static path wrote nothing"
            assert (w[0] != kn.host[0]).any(), "the kernel wrote nothing"
            for a, b in zip(w, g_):
                assert a.tobytes() == b.tobytes(), f"kernel {k}: static-scratch result differs"
        # and once more in the other order
        for kn, w in zip(reversed(kernels), reversed(want)):
            rc, out = kn.run(static=True)
            assert rc == 0
            for a, b in zip(w, out):
                assert a.tobytes() == b.tobytes()
    finally:
        for kn in kernels:
            kn.close()


def test_static_scratch_rejects_kernels_that_need_more():
    # the training step of one GPT-2 medium block: its in-order column sums over 3072 x 4096
    # terms keep 48 MiB of terms in scratch memory
    plan = PlanFile(os.path.join(PLANS, "gpt2_medium_block_train_b4_t1024.polyplan"))
    staged = two_stage_kernels(plan)
    too_big = sorted((b, k) for k, b in staged.items() if STATIC_BYTES < b <= (64 << 20))
    assert too_big, staged
    kn = Kernel(plan, too_big[0][1], seed=13)
    try:
        rc, _ = kn.run(static=True)
        assert rc == -1
        rc, out = kn.run(static=False)               # the ordinary entry point still takes it
        assert rc == 0
    finally:
        kn.close()
