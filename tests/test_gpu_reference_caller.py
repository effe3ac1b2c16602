"""The backend under the REFERENCE'S OWN CALLER.  oracle/_ref/libpolygrad_hip_ref.so is the
reference library compiled from its sources with the integration edits applied
(oracle/hip_integration.py: POLY_DEVICE_HIP = 7, the BACKENDS[] row, the whole-plan hook,
staging of host-resident bindings, device-resident training state) and linked against
libpolygrad_hip.so.  The tests follow the reference's own pattern for a device backend:
test/test_cuda.c:438-516 (poly_realize with device-domain bindings next to the same graph
with host bindings) and :533-652 (poly_instance_set_device, forward parity, CPU <-> device
round trips), plus what is broken in the reference on any device today: training steps whose
loss and bias-correction slots are host addresses (src/instance.c:1299-1311), value_and_grad
with host-resident outputs (src/instance.c:1027-1043), constants of the frontend's registry
(src/frontend.c:2231-2232).  Each test runs the whole-plan hook and, with
POLY_HIP_PER_KERNEL=1, the kernel-by-kernel path through the table row."""
import ctypes as C
import json

import numpy as np
import pytest

import graphs
import refpoly as R
from hipharness import assert_close
from polygrad_amd import _ffi

pytestmark = pytest.mark.gpu

if not R.hip_ref_available():
    pytest.skip("oracle/_ref/libpolygrad_hip_ref.so is not built (make -C oracle ref_hip)", allow_module_level=True)


@pytest.fixture(params=["whole-plan", "per-kernel"])
def path(request, monkeypatch):
    if request.param == "per-kernel":
        monkeypatch.setenv("POLY_HIP_PER_KERNEL", "1")
    else:
        monkeypatch.delenv("POLY_HIP_PER_KERNEL", raising=False)
    return request.param


class DeviceBuffers:
    """Device copies made through the backend's PolyAllocator, as build_cuda_bindings does
    with the CUDA runtime (test/test_cuda.c:405-432)."""

    def __init__(self):
        self.alloc = _ffi.load().poly_hip_get_allocator().contents
        self.ptrs = []

    def upload(self, a):
        p = self.alloc.alloc(max(a.nbytes, 4), self.alloc.dev_ctx)
        assert p
        assert self.alloc.copy_in(p, a.ctypes.data, a.nbytes, self.alloc.dev_ctx) == 0
        self.ptrs.append(p)
        return p

    def download(self, p, like):
        out = np.empty_like(like)
        assert self.alloc.copy_out(out.ctypes.data, p, out.nbytes, self.alloc.dev_ctx) == 0
        return out

    def close(self):
        for p in self.ptrs:
            self.alloc.free(p, self.alloc.dev_ctx)
        self.ptrs = []


def realize_both(c, sink, arrays, host_resident=()):
    """Runs `sink` with host bindings (CPU backend) and with HIP-domain bindings (device
    inferred from the bindings, src/frontend.c:2195-2215); buffers in `host_resident` stay
    CPU-domain handles in the device run.  Returns ({T: cpu result}, {T: device result})."""
    cpu = {t: np.array(a, copy=True) for t, a in arrays.items()}
    assert c.realize_bound(sink, {t: (a.ctypes.data, a.nbytes, R.DEVICE_CPU) for t, a in cpu.items()}) == 0
    dev = DeviceBuffers()
    host_side = {t: np.array(arrays[t], copy=True) for t in host_resident}
    handles, ptr = {}, {}
    for t, a in arrays.items():
        if t in host_side:
            handles[t] = (host_side[t].ctypes.data, a.nbytes, R.DEVICE_CPU)
        else:
            ptr[t] = dev.upload(np.ascontiguousarray(a))
            handles[t] = (ptr[t], a.nbytes, R.DEVICE_HIP)
    assert c.realize_bound(sink, handles) == 0
    got = {t: dev.download(p, arrays[t]) for t, p in ptr.items()}
    got.update(host_side)
    dev.close()
    return cpu, got


def test_realize_unified_vecadd(path):
    """test/test_cuda.c:438-474."""
    n = 1024
    c = R.Ctx(hip_ref=True)
    a, b, o = c.buffer((n,), name="a"), c.buffer((n,), name="b"), c.buffer((n,), name="c")
    av = (np.arange(n) * 0.1).astype(np.float32)
    bv = ((n - np.arange(n)) * 0.05).astype(np.float32)
    cpu, got = realize_both(c, c.sink((o, a + b)), {o: np.zeros(n, np.float32), a: av, b: bv})
    assert np.array_equal(cpu[o], av + bv)
    assert_close(got[o], cpu[o], rtol=1e-5, what="vecadd through poly_realize")
    c.close()


def test_realize_unified_reduce(path):
    """test/test_cuda.c:476-516."""
    n = 256
    c = R.Ctx(hip_ref=True)
    a, o = c.buffer((n,), name="a"), c.buffer((1,), name="c")
    av = np.arange(1, n + 1, dtype=np.float32)
    cpu, got = realize_both(c, c.sink((o, a.sum(0))), {o: np.zeros(1, np.float32), a: av})
    assert abs(float(cpu[o][0]) - av.sum()) < 1e-2
    assert_close(got[o], cpu[o], rtol=1e-4, what="full reduce through poly_realize")
    c.close()


def test_realize_matmul_softmax_layernorm_chain(path):
    """The row kernels and the matmul under poly_realize (device bindings)."""
    g = np.random.default_rng(21)
    c = R.Ctx(hip_ref=True)
    x, w, o = c.buffer((64, 96), name="x"), c.buffer((96, 128), name="w"), c.buffer((64, 128), name="o")
    y = x.dot(w).contiguous().softmax(-1).contiguous().layernorm(1e-5)
    arrays = {x: g.normal(0, 1, 64 * 96).astype(np.float32), w: g.normal(0, 0.2, 96 * 128).astype(np.float32),
              o: np.zeros(64 * 128, np.float32)}
    cpu, got = realize_both(c, c.sink((o, y)), arrays)
    assert_close(got[o], cpu[o], rtol=1e-4, atol=1e-4, what="matmul -> softmax -> layernorm through poly_realize")
    c.close()


def test_realize_gpt2_tiny_bf16_forward(path):
    """A whole (tiny) GPT-2 forward through poly_realize on the device: 51 kernels, bf16."""
    cfg = graphs.GPT2_TINY
    c = R.Ctx(hip_ref=True)
    sink, bufs = graphs.gpt2_forward(c, cfg, R.BF16)
    arrays = graphs.gpt2_inputs(cfg, bufs, seed=3, wdt=R.BF16)
    cpu, got = realize_both(c, sink, arrays)
    out = bufs["output"]
    assert_close(R.bf16_bits_to_f32(got[out]), R.bf16_bits_to_f32(cpu[out]), rtol=2e-2, atol=2e-3, what="tiny GPT-2 logits through poly_realize")
    c.close()


def test_realize_with_registry_constant_and_host_resident_output(path):
    """Sparse cross-entropy creates its class arange itself (src/frontend.c:1213, a registry
    constant nobody binds), and the loss stays a CPU-domain handle as
    poly_instance_value_and_grad binds it (src/instance.c:1027-1043): both are staged."""
    g = np.random.default_rng(22)
    B, K = 32, 10
    c = R.Ctx(hip_ref=True)
    lg, tg, o = c.buffer((B, K), name="logits"), c.buffer((B,), name="target"), c.buffer((1,), name="loss")
    arrays = {lg: g.normal(0, 2, B * K).astype(np.float32), tg: g.integers(0, K, B).astype(np.float32), o: np.zeros(1, np.float32)}
    cpu, got = realize_both(c, c.sink((o, lg.cross_entropy(tg))), arrays, host_resident=(o,))
    assert cpu[o][0] > 0
    assert_close(got[o], cpu[o], rtol=1e-4, what="sparse cross-entropy loss, host-resident output")
    c.close()


def make_mlp(L, n_in, n_hidden, n_out, batch=1):
    spec = json.dumps({"layers": [n_in, n_hidden, n_out], "activation": "relu", "bias": True, "loss": "mse",
                       "batch_size": batch, "seed": 42}).encode()
    inst = L.poly_mlp_instance(spec, len(spec))
    assert inst
    return inst


def seed_params(L, inst, mod, scale):
    for p in range(L.poly_instance_param_count(inst)):
        n = C.c_int64()
        data = L.poly_instance_param_data(inst, p, C.byref(n))
        assert data
        a = np.ctypeslib.as_array(C.cast(data, C.POINTER(C.c_float)), shape=(n.value,))
        a[:] = ((np.arange(n.value) % mod) - mod // 2) * scale


def output_index(L, inst):
    for i in range(L.poly_instance_buf_count(inst)):
        if L.poly_instance_buf_role(inst, i) == 3:      # POLY_ROLE_OUTPUT
            return i
    raise AssertionError("no output buffer")


def host_output(L, inst, idx, n):
    cnt = C.c_int64()
    p = L.poly_instance_buf_data(inst, idx, C.byref(cnt))
    assert p
    return np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_float)), shape=(n,)).copy()


def forward(L, inst, x):
    io = (R.PolyIOBinding * 1)(R.PolyIOBinding(b"x", x.ctypes.data))
    assert L.poly_instance_forward(inst, io, 1) == 0


def test_instance_set_device(path):
    """test/test_cuda.c:533-553."""
    L = R.lib(R.HIP_REF_LIB)
    inst = make_mlp(L, 2, 4, 3)
    assert L.poly_instance_set_device(inst, R.DEVICE_HIP) == 0
    n = C.c_int64()
    assert not L.poly_instance_buf_data(inst, 0, C.byref(n)), "device-resident buffers have no host data pointer"
    assert not L.poly_instance_param_data(inst, 0, C.byref(n))
    assert L.poly_instance_set_device(inst, R.DEVICE_CPU) == 0
    assert L.poly_instance_buf_data(inst, 0, C.byref(n))
    L.poly_instance_free(inst)


def test_instance_forward_parity(path):
    """test/test_cuda.c:555-604."""
    L = R.lib(R.HIP_REF_LIB)
    inst = make_mlp(L, 2, 4, 3)
    seed_params(L, inst, 7, 0.1)
    x = np.array([1.0, 2.0], np.float32)
    forward(L, inst, x)
    oi = output_index(L, inst)
    cpu = host_output(L, inst, oi, 3)
    assert L.poly_instance_set_device(inst, R.DEVICE_HIP) == 0
    forward(L, inst, x)
    got = np.zeros(3, np.float32)
    assert L.poly_instance_readback_buf(inst, oi, got.ctypes.data, got.nbytes) == 0
    assert np.abs(cpu).max() > 0
    assert_close(got, cpu, rtol=1e-4, atol=1e-6, what="MLP instance forward, HIP vs CPU")
    L.poly_instance_free(inst)


def test_instance_round_trip(path):
    """test/test_cuda.c:606-652: CPU -> HIP -> CPU -> HIP, the same output four times."""
    L = R.lib(R.HIP_REF_LIB)
    inst = make_mlp(L, 2, 4, 1)
    seed_params(L, inst, 5, 0.2)
    x = np.array([1.0, -1.0], np.float32)
    oi = output_index(L, inst)
    results = []
    for device in (R.DEVICE_CPU, R.DEVICE_HIP, R.DEVICE_CPU, R.DEVICE_HIP):
        assert L.poly_instance_set_device(inst, device) == 0
        forward(L, inst, x)
        if device == R.DEVICE_CPU:
            results.append(float(host_output(L, inst, oi, 1)[0]))
        else:
            r = np.zeros(1, np.float32)
            assert L.poly_instance_readback_buf(inst, oi, r.ctypes.data, 4) == 0
            results.append(float(r[0]))
    assert results[0] != 0
    for r in results[1:]:
        assert abs(r - results[0]) <= 1e-4 * abs(results[0]) + 1e-6, results
    L.poly_instance_free(inst)


@pytest.mark.parametrize("optim", ["sgd", "adamw"])
def test_instance_train_steps_on_device_match_cpu(path, optim):
    """Three training steps of the same MLP on the CPU and on the device: the losses and
    the updated parameters agree.  On the device the loss slot, the moments and the bias
    corrections must live in device memory (src/instance.c:1264-1311 binds host addresses)."""
    L = R.lib(R.HIP_REF_LIB)
    kind = {"sgd": 1, "adamw": 3}[optim]
    x = np.array([0.5, -1.5, 2.0], np.float32)
    y = np.array([1.0, -0.5], np.float32)
    runs = {}
    for device in (R.DEVICE_CPU, R.DEVICE_HIP):
        inst = make_mlp(L, 3, 8, 2)
        seed_params(L, inst, 11, 0.07)
        assert L.poly_instance_set_optimizer(inst, kind, 0.05, 0.9, 0.999, 1e-8, 0.01) == 0
        if device != R.DEVICE_CPU:
            assert L.poly_instance_set_device(inst, device) == 0
        io = (R.PolyIOBinding * 2)(R.PolyIOBinding(b"x", x.ctypes.data), R.PolyIOBinding(b"y", y.ctypes.data))
        losses = []
        for _ in range(3):
            loss = C.c_float(-1.0)
            assert L.poly_instance_train_step(inst, io, 2, C.byref(loss)) == 0
            losses.append(loss.value)
        if device != R.DEVICE_CPU:
            assert L.poly_instance_set_device(inst, R.DEVICE_CPU) == 0      # reads the parameters back
        params = []
        for p in range(L.poly_instance_param_count(inst)):
            n = C.c_int64()
            d = L.poly_instance_param_data(inst, p, C.byref(n))
            assert d
            params.append(np.ctypeslib.as_array(C.cast(d, C.POINTER(C.c_float)), shape=(n.value,)).copy())
        runs[device] = (losses, params)
        L.poly_instance_free(inst)
    (l_cpu, p_cpu), (l_hip, p_hip) = runs[R.DEVICE_CPU], runs[R.DEVICE_HIP]
    assert l_cpu[0] > 0 and l_cpu[2] < l_cpu[0], l_cpu
    assert_close(np.array(l_hip), np.array(l_cpu), rtol=1e-4, what=f"{optim}: losses of three steps")
    for a, b in zip(p_hip, p_cpu):
        assert_close(a, b, rtol=1e-4, atol=1e-6, what=f"{optim}: parameters after three steps")


def test_unknown_device_and_missing_binding_fail_cleanly(path):
    """Error conventions of the seam (src/exec_plan.c:805-809, :1018-1022): NULL / -1 and a
    message, no abort."""
    c = R.Ctx(hip_ref=True)
    a, o = c.buffer((16,), name="a"), c.buffer((16,), name="o")
    sink = c.sink((o, a + a))
    sched = c.schedule(sink)
    assert not c.L.poly_compile_schedule(c.ctx, sched, 9), "device 9 does not exist"
    dev = DeviceBuffers()
    po = dev.upload(np.zeros(16, np.float32))
    assert c.realize_bound(sink, {o: (po, 64, R.DEVICE_HIP)}) != 0, "the input is not bound"
    dev.close()
    c.L.poly_schedule_free(sched)
    c.close()
