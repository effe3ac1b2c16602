"""Host-side wrapper of the plan-level C ABI (poly_hip_compile_schedule /
poly_hip_plan_run), the device counterpart of the reference's
poly_compile_schedule / poly_compiled_plan_run (src/exec_plan.c:801-1060).

torch is used for device memory only: callers hand in CUDA tensors (or raw
device pointers) for the external slots; all compute happens in the HIP
kernels the library generates.  There is no CPU path here.
"""
import ctypes as C

from . import _ffi

DT_NAMES = ["void", "bool", "int8", "uint8", "int16", "uint16", "int32", "uint32", "int64", "uint64",
            "float16", "bfloat16", "float32", "float64", "index"]
KERNEL_CLASSES = ["elementwise", "row-reduce", "thread-reduce", "matmul-mfma", "gather", "copy", "attention-mfma"]


def _dt_code(d):
    """Scalar dtype code (index into DT_NAMES) of a PolyDType struct."""
    table = {-1: 0, 0: 1, 1: 2, 2: 3, 3: 4, 4: 5, 5: 6, 6: 7, 7: 8, 8: 9, 11: 10, 12: 11, 13: 12, 14: 13}
    if d.priority == -1 and d.bitsize != 0:
        return 14
    return table[d.priority]


class Slot:
    def __init__(self, index, raw, name):
        self.index = index
        self.is_intermediate = bool(raw.is_intermediate)
        self.numel = int(raw.numel)
        self.nbytes = int(raw.nbytes)
        self.dtype = DT_NAMES[_dt_code(raw.dtype)]
        self.name = name

    def __repr__(self):
        kind = "tmp" if self.is_intermediate else "ext"
        return f"Slot({self.index} {kind} {self.name!r} {self.dtype}[{self.numel}])"


class HipPlan:
    """A schedule compiled for the GPU.  `schedule` is a PolySchedule* (an int /
    c_void_p) that must outlive the plan, e.g. one returned by the reference's
    poly_schedule_for or by PlanFile."""

    def __init__(self, schedule, ctx=None, names=None, keepalive=None):
        self.lib = _ffi.load()
        self._keep = keepalive
        self.schedule = schedule if isinstance(schedule, int) else C.cast(schedule, C.c_void_p).value
        self.handle = self.lib.poly_hip_compile_schedule(ctx, self.schedule)
        if not self.handle:
            raise RuntimeError("poly_hip_compile_schedule failed (see stderr)")
        s = C.cast(self.schedule, C.POINTER(_ffi.PolySchedule)).contents
        self.slots = [Slot(i, s.buf_slots[i], (names[i] if names and i < len(names) else "") or "")
                      for i in range(s.n_buf_slots)]
        self.n_kernels = self.lib.poly_hip_plan_n_kernels(self.handle)
        self._ext_stream = None

    @classmethod
    def from_file(cls, path):
        pf = PlanFile(path)
        return cls(pf.schedule, names=pf.names, keepalive=pf)

    def close(self):
        if getattr(self, "handle", None):
            self.lib.poly_hip_plan_free(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def external_slots(self):
        return [s for s in self.slots if not s.is_intermediate]

    def _order_after_torch(self):
        """The backend launches on its own non-blocking stream: make that stream wait
        for whatever torch has queued so far (fills, copies, random init of the tensors
        handed in), without blocking the host."""
        import torch
        if self._ext_stream is None:
            self._ext_stream = torch.cuda.ExternalStream(self.lib.poly_hip_stream())
        self._ext_stream.wait_stream(torch.cuda.current_stream())

    def _ptr_array(self, slot_data):
        n = len(self.slots)
        arr = (C.c_void_p * n)()
        if any(v is not None and not isinstance(v, int) for v in slot_data):
            self._order_after_torch()
        for i in range(n):
            v = slot_data[i] if i < len(slot_data) else None
            if v is None:
                arr[i] = None
            elif isinstance(v, int):
                arr[i] = v
            else:  # torch tensor
                if not v.is_cuda or not v.is_contiguous():
                    raise ValueError(f"slot {i}: need a contiguous CUDA tensor")
                if v.numel() * v.element_size() < self.slots[i].nbytes:
                    raise ValueError(f"slot {i}: tensor has {v.numel() * v.element_size()} bytes, "
                                     f"slot needs {self.slots[i].nbytes}")
                arr[i] = v.data_ptr()
        return arr

    def run(self, slot_data, sync=True, var_bindings=None):
        """Enqueues one pass of the plan.  slot_data[i]: tensor / device pointer for
        every external slot i (None for intermediates).  var_bindings: [(DEFINE_VAR UOp
        pointer, int value)] overriding the schedule's defaults."""
        arr = self._ptr_array(slot_data)
        vb, nvb = None, 0
        if var_bindings:
            nvb = len(var_bindings)
            vb = (_ffi.PolyVarBinding * nvb)(*[_ffi.PolyVarBinding(v, val) for v, val in var_bindings])
        rc = self.lib.poly_hip_plan_run(self.handle, arr, len(self.slots), vb, nvb)
        if rc != 0:
            raise RuntimeError("poly_hip_plan_run failed (see stderr)")
        if sync:
            self.sync()

    def sync(self):
        if self.lib.poly_hip_sync() != 0:
            raise RuntimeError("poly_hip_sync failed")

    def set_graph(self, enabled):
        self.lib.poly_hip_plan_set_graph(self.handle, 1 if enabled else 0)

    def kernel_info(self):
        n = self.n_kernels
        k = (C.c_int * n)()
        b = (C.c_double * n)()
        f = (C.c_double * n)()
        self.lib.poly_hip_plan_kernel_info(self.handle, n, k, b, f)
        return [dict(klass=KERNEL_CLASSES[k[i]], bytes=b[i], flops=f[i],
                     desc=_ffi.take_string(self.lib.poly_hip_plan_kernel_desc(self.handle, i)))
                for i in range(n)]

    def profile(self, slot_data):
        """Per-launch milliseconds of one eager pass: the durations of each launch's kernels,
        from the HIP events that their dispatches stamp at start and end."""
        arr = self._ptr_array(slot_data)
        ms = (C.c_float * self.n_kernels)()
        rc = self.lib.poly_hip_plan_profile(self.handle, arr, len(self.slots), ms, self.n_kernels)
        if rc < 0:
            raise RuntimeError("poly_hip_plan_profile failed")
        return list(ms)

    def workspace_bytes(self):
        return int(self.lib.poly_hip_plan_workspace_bytes(self.handle))

    def side_launches(self):
        """Launches that the plan's captured graph runs on a second stream."""
        return int(self.lib.poly_hip_plan_side_launches(self.handle))

    def graph_counts(self):
        """(captures, rebinds): how often the launch sequence was captured, and how often a
        new set of buffers was served by updating the captured graph's kernel nodes."""
        import ctypes as C
        c, r = C.c_longlong(0), C.c_longlong(0)
        self.lib.poly_hip_plan_graph_counts(self.handle, C.byref(c), C.byref(r))
        return int(c.value), int(r.value)

    def slot_ptr(self, slot):
        return self.lib.poly_hip_plan_slot_ptr(self.handle, slot)


class PlanFile:
    """A serialized schedule (see csrc/planfile.cc for the layout)."""

    def __init__(self, path):
        self.lib = _ffi.load()
        self.handle = self.lib.poly_hip_planfile_load(str(path).encode())
        if not self.handle:
            raise RuntimeError(f"cannot load plan file {path}")
        sp = self.lib.poly_hip_planfile_schedule(self.handle)
        self.schedule = C.cast(sp, C.c_void_p).value
        s = sp.contents
        self.names = [self.lib.poly_hip_planfile_slot_name(self.handle, i).decode() for i in range(s.n_buf_slots)]
        self.n_items = s.n_items

    def close(self):
        if getattr(self, "handle", None):
            self.lib.poly_hip_planfile_free(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def save_schedule(schedule, names, path):
    lib = _ffi.load()
    arr = None
    if names is not None:
        arr = (C.c_char_p * len(names))(*[(n or "").encode() for n in names])
    rc = lib.poly_hip_planfile_save(schedule, arr, str(path).encode())
    if rc != 0:
        raise RuntimeError(f"poly_hip_planfile_save failed for {path}")
