"""Loading of the committed golden fixtures (tests/golden/*.polyplan + *.npz) and
running them through the CPU oracle."""
import ctypes as C
import glob
import os

import numpy as np

from polygrad_amd import PlanFile, _ffi

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden")
ORACLE_LIB = os.path.join(HERE, "..", "oracle", "liboracle.so")

_oracle = None


def oracle():
    global _oracle
    if _oracle is None:
        L = C.CDLL(os.path.abspath(ORACLE_LIB))
        L.oracle_run_schedule.restype = C.c_int
        L.oracle_run_schedule.argtypes = [C.c_void_p, C.POINTER(C.c_void_p), C.c_int]
        L.oracle_run_kernel.restype = C.c_int
        L.oracle_run_kernel.argtypes = [C.c_void_p, C.POINTER(C.c_void_p), C.c_int]
        for name, res, args in (("oracle_exp2f", C.c_float, [C.c_float]), ("oracle_log2f", C.c_float, [C.c_float]),
                                ("oracle_exp2", C.c_double, [C.c_double]), ("oracle_log2", C.c_double, [C.c_double]),
                                ("oracle_threefry", C.c_uint64, [C.c_uint64, C.c_uint64]),
                                ("oracle_f32_to_bf16", C.c_uint16, [C.c_float]), ("oracle_bf16_to_f32", C.c_float, [C.c_uint16]),
                                ("oracle_f32_to_f16", C.c_uint16, [C.c_float]), ("oracle_f16_to_f32", C.c_float, [C.c_uint16])):
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _oracle = L
    return _oracle


def case_names():
    return sorted(os.path.basename(p)[:-len(".polyplan")] for p in glob.glob(os.path.join(GOLDEN, "*.polyplan")))


class Fixture:
    def __init__(self, name):
        self.name = name
        self.plan = PlanFile(os.path.join(GOLDEN, name + ".polyplan"))
        z = np.load(os.path.join(GOLDEN, name + ".npz"))
        self.inputs = {int(k[2:]): z[k] for k in z.files if k.startswith("in")}
        self.expected = {int(k[3:]): z[k] for k in z.files if k.startswith("out")}
        s = C.cast(self.plan.schedule, C.POINTER(_ffi.PolySchedule)).contents
        self.n_slots = s.n_buf_slots
        self.external = [i for i in range(s.n_buf_slots) if not s.buf_slots[i].is_intermediate]

    def outputs(self):
        """Slots whose contents the reference changed."""
        return [i for i in self.external
                if self.inputs[i].tobytes() != self.expected[i].tobytes() or self.plan.names[i] in ("output", "o", "O", "C", "out", "loss")]


def run_oracle_schedule(schedule_ptr, n_slots, arrays):
    """arrays: {slot: ndarray}; run in place on copies, returns the copies."""
    out = {i: np.array(a, copy=True) for i, a in arrays.items()}
    data = (C.c_void_p * n_slots)()
    for i, a in out.items():
        data[i] = a.ctypes.data
    rc = oracle().oracle_run_schedule(schedule_ptr, data, n_slots)
    if rc != 0:
        raise RuntimeError("oracle_run_schedule failed")
    return out


def as_float(a):
    """float view of fixture data (uint16 arrays hold bf16 bit patterns)."""
    if a.dtype == np.uint16:
        return (a.astype(np.uint32) << 16).view(np.float32)
    return a
