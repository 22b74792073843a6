"""ctypes binding of libsgnn_hip.so (the C ABI declared in include/sgnn.h).

There is no CPU fallback: if the HIP library is missing or fails to load, importing this module
raises, and every operator built on it is unusable -- by design.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsgnn_hip.so")

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int

# name -> (restype, argtypes); mirrors include/sgnn.h one to one.
SIGNATURES = {
    "sgnn_last_error": (ctypes.c_char_p, []),
    "sgnn_version": (_int, []),
    "sgnn_spmm_plan_create": (_int, [_vp, _vp, _int, _i64, _i64, _i64, _int, _int, _vp, ctypes.POINTER(_vp)]),
    "sgnn_spmm_plan_destroy": (_int, [_vp]),
    "sgnn_spmm_plan_info": (_int, [_vp, ctypes.POINTER(_i64)]),
    "sgnn_spmm_plan_schedule": (_int, [_vp, _i64, ctypes.POINTER(_i64)]),
    "sgnn_spmm_csr_f32": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp, _vp]),
    "sgnn_spmm_csr_f32_noalloc": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp, _vp]),
    "sgnn_spmm_reference_overwrites": (_int, [_i64, _i64, _i64, _i64]),
    "sgnn_quant_segment_offsets": (_i64, [ctypes.POINTER(ctypes.c_int32), _int, _int, ctypes.POINTER(ctypes.c_int32)]),
    "sgnn_quant_pack_rows_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _int, _vp]),
    "sgnn_unpack_dequant_rows_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _int, _vp]),
    "sgnn_quant_row_slots": (_int, [_vp, _vp, _int, _int, _i64, _vp, _vp]),
    "sgnn_spmm_plan_bind_values": (_int, [_vp, _vp, _vp]),
    "sgnn_spmm_plan_bind_row_slots": (_int, [_vp, _vp, _vp]),
    "sgnn_spmm_csr_dq_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _vp, _i64, _i64, _int, _vp, _vp]),
    "sgnn_quant_pack_rows_wire_f32": (_int, [_vp, _i64, _vp, _i64, _vp, _vp, _int, _vp, _vp, _int, _i64, _i64, _i64, _int, _vp]),
    "sgnn_unpack_dequant_rows_wire_f32": (_int, [_vp, _vp, _vp, _int, _vp, _vp, _int, _i64, _i64, _i64, _int, _vp]),
    "sgnn_spmm_csr_dq_wire_f32": (_int, [_vp, _vp, _vp, _vp, _int, _vp, _int, _vp, _i64, _i64, _int, _vp, _vp]),
    "sgnn_quant_v1_f32": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _vp]),
    "sgnn_dequant_v1_f32": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _vp]),
    "sgnn_profile_enable": (_int, [_int]),
    "sgnn_profile_read": (_int, [_int, ctypes.POINTER(_i64), ctypes.POINTER(ctypes.c_double)]),
    "sgnn_profile_kernel_name": (ctypes.c_char_p, [_int]),
    "sgnn_profile_kernel_count": (_int, []),
    "sgnn_stream_copy_f32": (_int, [_vp, _vp, _i64, _vp]),
}


class SgnnError(RuntimeError):
    """An entry point of libsgnn_hip.so returned a negative status."""


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `make -C super_gnn_amd/csrc` "
            "(hipcc --offload-arch=gfx950). There is no CPU fallback."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here = header and library out of sync
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


def check(status):
    if status < 0:
        msg = lib.sgnn_last_error().decode("utf-8", "replace")
        if status == -1:
            raise ValueError(f"libsgnn_hip: {msg}")
        if status == -3:
            raise IndexError(f"libsgnn_hip: {msg}")
        raise SgnnError(f"libsgnn_hip (status {status}): {msg}")
    return status


def profile_start():
    """Start recording a HIP event pair around every kernel launch of the library."""
    check(lib.sgnn_profile_enable(1))


def profile_stop():
    """Stop recording and return {kernel name: (launches, total_ms)} for kernels that ran."""
    check(lib.sgnn_profile_enable(0))
    out = {}
    for k in range(lib.sgnn_profile_kernel_count()):
        n, ms = _i64(0), ctypes.c_double(0.0)
        check(lib.sgnn_profile_read(k, ctypes.byref(n), ctypes.byref(ms)))
        if n.value:
            out[lib.sgnn_profile_kernel_name(k).decode()] = (n.value, ms.value)
    return out
