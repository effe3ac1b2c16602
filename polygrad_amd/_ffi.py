"""ctypes binding of libpolygrad_hip.so (the C ABI in include/polygrad_hip.h).

Mirrors how the reference's Python package binds its own C library
(py/polygrad/_ffi.py): plain ctypes, pointers and sizes only.  The library is
built in-tree by ``make -C polygrad_amd/csrc``; importing this module never
builds it and never substitutes a host implementation when it is missing.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libpolygrad_hip.so")


class PolyDType(C.Structure):
    _fields_ = [("priority", C.c_int8), ("bitsize", C.c_uint16), ("name", C.c_char_p),
                ("fmt", C.c_char), ("count", C.c_uint16), ("is_ptr", C.c_bool),
                ("addrspace", C.c_int), ("vcount", C.c_uint16), ("ptr_size", C.c_int64)]


class PolyScheduleBufSlot(C.Structure):
    _fields_ = [("dtype", PolyDType), ("numel", C.c_int64), ("nbytes", C.c_int64),
                ("buf_uop", C.c_void_p), ("is_intermediate", C.c_bool), ("external_buf_idx", C.c_int)]


class PolyVarBinding(C.Structure):
    _fields_ = [("var", C.c_void_p), ("value", C.c_int32)]


class PolyExecItem(C.Structure):
    _fields_ = [("kind", C.c_int), ("root", C.c_void_p), ("buf_slot_indices", C.POINTER(C.c_int)),
                ("n_buf_slots", C.c_int), ("fixedvars", C.c_void_p), ("n_fixedvars", C.c_int),
                ("var_uops", C.POINTER(C.c_void_p)), ("n_var_uops", C.c_int)]


class PolySchedule(C.Structure):
    _fields_ = [("entrypoint_name", C.c_char_p), ("mode", C.c_int), ("graph_hash", C.c_uint32),
                ("buf_slots", C.POINTER(PolyScheduleBufSlot)), ("n_buf_slots", C.c_int),
                ("items", C.POINTER(PolyExecItem)), ("n_items", C.c_int),
                ("exec_order", C.POINTER(C.c_int)), ("default_vars", C.c_void_p),
                ("n_default_vars", C.c_int), ("loss_buf_slot", C.c_int),
                ("grad_buf_slots", C.POINTER(C.c_int))]


class PolyRunner(C.Structure):
    _fields_ = [("kind", C.c_int), ("handle", C.c_void_p), ("handle_size", C.c_int),
                ("execute", C.c_void_p), ("free_handle", C.c_void_p),
                ("grid", C.c_int * 3), ("block", C.c_int * 3),
                ("param_to_slot", C.POINTER(C.c_int)), ("n_params", C.c_int),
                ("var_indices", C.POINTER(C.c_int)), ("n_vars", C.c_int)]


class PolyAllocator(C.Structure):
    _fields_ = [("alloc", C.CFUNCTYPE(C.c_void_p, C.c_size_t, C.c_void_p)),
                ("free", C.CFUNCTYPE(None, C.c_void_p, C.c_void_p)),
                ("copy_in", C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p)),
                ("copy_out", C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p)),
                ("copy_between", C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p)),
                ("dev_ctx", C.c_void_p)]


class PolyBackendDesc(C.Structure):
    _fields_ = [("name", C.c_char_p), ("id", C.c_int), ("host_executed", C.c_bool),
                ("lower_item", C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_void_p, C.c_char_p, C.POINTER(PolyRunner))),
                ("execute", C.CFUNCTYPE(C.c_int, C.POINTER(PolyRunner), C.POINTER(C.c_void_p), C.c_int)),
                ("free_runner", C.CFUNCTYPE(None, C.POINTER(PolyRunner))),
                ("get_allocator", C.CFUNCTYPE(C.POINTER(PolyAllocator)))]


# name -> (restype, argtypes); every symbol include/polygrad_hip.h declares.
SYMBOLS = {
    "poly_hip_backend_desc": (C.POINTER(PolyBackendDesc), []),
    "poly_hip_lower_item": (C.c_int, [C.c_void_p, C.c_void_p, C.c_char_p, C.POINTER(PolyRunner)]),
    "poly_hip_execute": (C.c_int, [C.POINTER(PolyRunner), C.POINTER(C.c_void_p), C.c_int]),
    "poly_hip_execute_static": (C.c_int, [C.POINTER(PolyRunner), C.POINTER(C.c_void_p), C.c_int]),
    "poly_hip_free_runner": (None, [C.POINTER(PolyRunner)]),
    "poly_hip_get_allocator": (C.POINTER(PolyAllocator), []),
    "poly_hip_init": (C.c_int, []),
    "poly_hip_available": (C.c_int, []),
    "poly_hip_alloc": (C.c_void_p, [C.c_size_t]),
    "poly_hip_free": (None, [C.c_void_p]),
    "poly_hip_copy_htod": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "poly_hip_copy_dtoh": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "poly_hip_copy_dtod": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "poly_hip_memset": (C.c_int, [C.c_void_p, C.c_int, C.c_size_t]),
    "poly_hip_sync": (C.c_int, []),
    "poly_hip_stream": (C.c_void_p, []),
    "poly_hip_compile": (C.c_void_p, [C.c_char_p, C.c_char_p]),
    "poly_hip_launch": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p), C.c_int] + [C.c_uint] * 7),
    "poly_hip_program_destroy": (None, [C.c_void_p]),
    "poly_hip_render": (C.c_void_p, [C.c_void_p, C.c_char_p, C.c_int, C.POINTER(C.c_int)]),
    "poly_hip_describe": (C.c_void_p, [C.c_void_p, C.c_int]),
    "poly_hip_compile_check": (C.c_int, [C.c_char_p]),
    "poly_hip_free_string": (None, [C.c_void_p]),
    "poly_hip_check_index_simplification": (C.c_int, [C.c_void_p, C.c_int]),
    "poly_hip_compile_schedule": (C.c_void_p, [C.c_void_p, C.c_void_p]),
    "poly_hip_plan_run": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p), C.c_int, C.POINTER(PolyVarBinding), C.c_int]),
    "poly_hip_plan_free": (None, [C.c_void_p]),
    "poly_hip_fused_groups": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(C.c_void_p), C.POINTER(C.c_int)]),
    "poly_hip_fused_group_launch": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(C.c_int), C.c_int, C.POINTER(C.c_int)]),
    "poly_hip_unwritten_slots": (C.c_int, [C.c_void_p, C.POINTER(C.c_int), C.c_int]),
    "poly_hip_plan_n_kernels": (C.c_int, [C.c_void_p]),
    "poly_hip_plan_kernel_info": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "poly_hip_plan_profile": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p), C.c_int, C.POINTER(C.c_float), C.c_int]),
    "poly_hip_plan_kernel_desc": (C.c_void_p, [C.c_void_p, C.c_int]),
    "poly_hip_plan_slot_ptr": (C.c_void_p, [C.c_void_p, C.c_int]),
    "poly_hip_plan_set_graph": (None, [C.c_void_p, C.c_int]),
    "poly_hip_plan_workspace_bytes": (C.c_size_t, [C.c_void_p]),
    "poly_hip_plan_side_launches": (C.c_int, [C.c_void_p]),
    "poly_hip_plan_graph_counts": (None, [C.c_void_p, C.POINTER(C.c_longlong), C.POINTER(C.c_longlong)]),
    "poly_hip_planfile_save": (C.c_int, [C.c_void_p, C.POINTER(C.c_char_p), C.c_char_p]),
    "poly_hip_planfile_load": (C.c_void_p, [C.c_char_p]),
    "poly_hip_planfile_schedule": (C.POINTER(PolySchedule), [C.c_void_p]),
    "poly_hip_planfile_slot_name": (C.c_char_p, [C.c_void_p, C.c_int]),
    "poly_hip_planfile_free": (None, [C.c_void_p]),
}

_lib = None


def load():
    """Loads the in-tree library.  Raises (never falls back) when it is absent."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is not built; run `make -C polygrad_amd/csrc` (there is no host fallback)")
    lib = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def take_string(ptr):
    """Copies and frees a malloc'd C string returned by the library."""
    if not ptr:
        return None
    s = C.string_at(ptr).decode()
    load().poly_hip_free_string(ptr)
    return s
