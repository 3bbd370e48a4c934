"""ctypes binding of libtandem_hip.so (include/tandem_hip.h).

There is no fallback: if the library has not been built, or a call fails, the
caller gets an exception. Nothing here computes on the CPU.
"""

import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libtandem_hip.so")

TDM_MAX_PAIRS = 16
TDM_MAX_WORLD = 8
ABI_VERSION = 1

DTYPES = {torch.float32: 0, torch.float64: 1, torch.float16: 2, torch.bfloat16: 3, torch.int64: 4, torch.int32: 5,
          torch.int16: 7, torch.int8: 8, torch.uint8: 9}  # 6 is TDM_BYTES: any dtype, copied only

ALLREDUCE_RING = 0
ALLREDUCE_FOLD = 1
ADAMW_HOST_ORDER = 0
ADAMW_DEVICE_ORDER = 1


class HipLibraryMissing(RuntimeError):
    pass


class Pair(ctypes.Structure):
    _fields_ = [("dst", ctypes.c_void_p), ("src", ctypes.c_void_p), ("count", ctypes.c_int64)]


class FoldSeg(ctypes.Structure):
    _fields_ = [("src", ctypes.c_void_p * TDM_MAX_WORLD), ("dst", ctypes.c_void_p * TDM_MAX_WORLD),
                ("count", ctypes.c_int64), ("chunk", ctypes.c_int32), ("reserved", ctypes.c_int32)]


class StepSeg(ctypes.Structure):
    _fields_ = [("grad", ctypes.c_void_p * TDM_MAX_WORLD), ("param", ctypes.c_void_p * TDM_MAX_WORLD),
                ("exp_avg", ctypes.c_void_p), ("exp_avg_sq", ctypes.c_void_p), ("count", ctypes.c_int64),
                ("chunk", ctypes.c_int32), ("dtype", ctypes.c_int32)]


class AdamwScalars(ctypes.Structure):
    _fields_ = [("use_decay", ctypes.c_int32), ("decay", ctypes.c_float), ("w1", ctypes.c_float),
                ("beta2", ctypes.c_float), ("one_m_b2", ctypes.c_float), ("bc2_sqrt", ctypes.c_float),
                ("eps", ctypes.c_float), ("neg_step", ctypes.c_float), ("inv_bc2_sqrt", ctypes.c_float)]


class AdamwHyper(ctypes.Structure):
    _fields_ = [("use_decay", ctypes.c_int32), ("reserved", ctypes.c_int32), ("decay", ctypes.c_double), ("w1", ctypes.c_double),
                ("beta2", ctypes.c_double), ("one_m_b2", ctypes.c_double), ("bc2_sqrt", ctypes.c_double),
                ("eps", ctypes.c_double), ("neg_step", ctypes.c_double)]


_SIGNATURES = {
    "tdm_last_error": (ctypes.c_char_p, []),
    "tdm_abi_version": (ctypes.c_int, []),
    "tdm_device_info": (ctypes.c_int, [ctypes.c_int, ctypes.c_char_p, ctypes.c_int, ctypes.POINTER(ctypes.c_int),
                                       ctypes.POINTER(ctypes.c_int64)]),
    "tdm_set_blocks_per_cu": (ctypes.c_int, [ctypes.c_int]),
    "tdm_set_xcd_group": (ctypes.c_int, [ctypes.c_int, ctypes.c_int]),
    "tdm_set_occupancy_pad": (ctypes.c_int, [ctypes.c_int, ctypes.c_int]),
    "tdm_set_ring_form": (ctypes.c_int, [ctypes.c_int]),
    "tdm_tile_of": (ctypes.c_int64, [ctypes.c_int64, ctypes.c_int64, ctypes.c_int]),
    "tdm_table_tile_bytes": (ctypes.c_int, []),
    "tdm_build_geometry": (ctypes.c_int, [ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)]),
    "tdm_engine_set_timing": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int]),
    "tdm_k1_reduce_step": (ctypes.c_int, [ctypes.POINTER(Pair), ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                          ctypes.c_int, ctypes.c_int, ctypes.c_void_p]),
    "tdm_k1_copy_step": (ctypes.c_int, [ctypes.POINTER(Pair), ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]),
    "tdm_local_reduce_scatter": (ctypes.c_int, [ctypes.POINTER(ctypes.c_void_p), ctypes.c_int, ctypes.c_int64, ctypes.c_int,
                                                ctypes.POINTER(ctypes.c_int64), ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                ctypes.c_void_p]),
    "tdm_local_all_gather": (ctypes.c_int, [ctypes.POINTER(ctypes.c_void_p), ctypes.c_int, ctypes.c_int64, ctypes.c_int,
                                            ctypes.POINTER(ctypes.c_int64), ctypes.c_int, ctypes.c_void_p]),
    "tdm_local_all_reduce": (ctypes.c_int, [ctypes.POINTER(ctypes.c_void_p), ctypes.c_int, ctypes.c_int64, ctypes.c_int,
                                            ctypes.c_int, ctypes.c_int, ctypes.c_void_p]),
    "tdm_k2_table_bytes": (ctypes.c_int64, [ctypes.POINTER(FoldSeg), ctypes.c_int, ctypes.c_int]),
    "tdm_k2_table_build": (ctypes.c_int, [ctypes.POINTER(FoldSeg), ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]),
    "tdm_k2_table_tiles": (ctypes.c_int64, [ctypes.POINTER(FoldSeg), ctypes.c_int, ctypes.c_int]),
    "tdm_k2_bucket_fold": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                          ctypes.c_int, ctypes.c_void_p]),
    "tdm_k2_static_max_tiles": (ctypes.c_int64, []),
    "tdm_k2_bucket_fold_static": (ctypes.c_int, [ctypes.POINTER(FoldSeg), ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                 ctypes.c_int, ctypes.c_void_p]),
    "tdm_k3_adamw": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64,
                                    ctypes.POINTER(AdamwScalars), ctypes.c_int, ctypes.c_void_p]),
    "tdm_k3_adamw_gather": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64,
                                           ctypes.POINTER(AdamwScalars), ctypes.c_int, ctypes.POINTER(ctypes.c_void_p),
                                           ctypes.c_int, ctypes.c_void_p]),
    "tdm_k3_adamw_typed": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64,
                                          ctypes.c_int, ctypes.POINTER(AdamwHyper), ctypes.c_int, ctypes.POINTER(ctypes.c_void_p),
                                          ctypes.c_int, ctypes.c_void_p]),
    "tdm_k23_table_tiles": (ctypes.c_int64, [ctypes.POINTER(StepSeg), ctypes.c_int]),
    "tdm_k23_table_bytes": (ctypes.c_int64, [ctypes.POINTER(StepSeg), ctypes.c_int]),
    "tdm_k23_table_build": (ctypes.c_int, [ctypes.POINTER(StepSeg), ctypes.c_int, ctypes.c_int, ctypes.c_void_p]),
    "tdm_k23_zero2_step": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                          ctypes.POINTER(AdamwScalars), ctypes.c_int, ctypes.c_void_p]),
    "tdm_k23_zero2_step_typed": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                ctypes.POINTER(AdamwHyper), ctypes.c_int, ctypes.c_void_p]),
    "tdm_k23_zero2_step_segment": (ctypes.c_int, [ctypes.POINTER(StepSeg), ctypes.c_int, ctypes.c_int,
                                                  ctypes.POINTER(AdamwScalars), ctypes.c_int, ctypes.c_void_p]),
    "tdm_k23_zero2_step_segment_typed": (ctypes.c_int, [ctypes.POINTER(StepSeg), ctypes.c_int, ctypes.c_int,
                                                        ctypes.POINTER(AdamwHyper), ctypes.c_int, ctypes.c_void_p]),
    "tdm_k4_unit_gather_all": (ctypes.c_int, [ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_void_p),
                                              ctypes.POINTER(ctypes.c_int64), ctypes.c_int, ctypes.c_int, ctypes.c_void_p]),
    "tdm_k4_unit_gather": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_int64),
                                          ctypes.c_int, ctypes.c_int, ctypes.c_void_p]),
}

_lib = None


_VP = ctypes.c_void_p
_PVP = ctypes.POINTER(ctypes.c_void_p)
_PI64 = ctypes.POINTER(ctypes.c_int64)
_ENGINE_SIGNATURES = {
    "tdm_engine_create": (ctypes.c_int, [ctypes.c_char_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int64,
                                         ctypes.c_double, ctypes.c_int, _PVP]),
    "tdm_engine_connect": (ctypes.c_int, [_VP]),
    "tdm_engine_close": (ctypes.c_int, [_VP]),
    "tdm_engine_destroy": (ctypes.c_int, [_VP]),
    "tdm_all_reduce": (ctypes.c_int, [_VP, _VP, ctypes.c_int64, ctypes.c_int, ctypes.c_int, _VP, _PVP]),
    "tdm_reduce_scatter": (ctypes.c_int, [_VP, _VP, ctypes.c_int64, ctypes.c_int, _PI64, ctypes.c_int, ctypes.c_int, _VP, _PVP]),
    "tdm_all_gather": (ctypes.c_int, [_VP, _VP, ctypes.c_int64, ctypes.c_int, _PI64, ctypes.c_int, _VP, _PVP]),
    "tdm_reduce_scatter_owner": (ctypes.c_int, [_VP, _VP, ctypes.c_int64, ctypes.c_int, _PI64, ctypes.c_int, ctypes.c_int, _VP, _PVP]),
    "tdm_broadcast": (ctypes.c_int, [_VP, _VP, ctypes.c_int64, ctypes.c_int, ctypes.c_int, _VP, _PVP]),
    "tdm_unit_gather": (ctypes.c_int, [_VP, _VP, ctypes.c_int64, ctypes.c_int, _VP, _PI64, ctypes.c_int, _VP, _PVP]),
    "tdm_sendrecv": (ctypes.c_int, [_VP, _VP, ctypes.c_int64, ctypes.c_int, _VP, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                    _VP, _PVP]),
    "tdm_barrier": (ctypes.c_int, [_VP, _PVP]),
    "tdm_fence": (ctypes.c_int, [_VP, _VP, _PVP]),
    "tdm_direct_all_reduce": (ctypes.c_int, [_VP, _VP, ctypes.c_int64, ctypes.c_int, ctypes.c_int, _PI64, ctypes.c_int, _VP,
                                             _PVP]),
    "tdm_direct_reduce_scatter": (ctypes.c_int, [_VP, _VP, ctypes.c_int64, ctypes.c_int, _PI64, ctypes.c_int, ctypes.c_int,
                                                 _PI64, ctypes.c_int, _VP, _PVP]),
    "tdm_direct_all_gather": (ctypes.c_int, [_VP, _VP, ctypes.c_int64, ctypes.c_int, _PI64, ctypes.c_int, _PI64, ctypes.c_int,
                                             _VP, _PVP]),
    "tdm_direct_zero2_step": (ctypes.c_int, [_VP, _VP, _PI64, _VP, _PI64, ctypes.c_int, _VP, _VP, ctypes.c_int64, ctypes.c_int64,
                                             ctypes.c_int, ctypes.POINTER(AdamwScalars), ctypes.c_int, _VP, _PVP]),
    "tdm_direct_zero2_step_typed": (ctypes.c_int, [_VP, _VP, _PI64, _VP, _PI64, ctypes.c_int, _VP, _VP, ctypes.c_int64, ctypes.c_int64,
                                                   ctypes.c_int, ctypes.c_int, ctypes.POINTER(AdamwHyper), ctypes.c_int, _VP, _PVP]),
    "tdm_engine_share": (ctypes.c_int, [_VP, ctypes.c_int64, _PVP]),
    "tdm_engine_arena_offset": (ctypes.c_int, [_VP, _VP, ctypes.c_int64, ctypes.POINTER(ctypes.c_int64)]),
    "tdm_unit_gather_direct": (ctypes.c_int, [_VP, _VP, ctypes.c_int64, ctypes.c_int, _VP, _PI64, ctypes.c_int, _PI64,
                                              ctypes.c_int, _VP, _PVP]),
    "tdm_work_wait": (ctypes.c_int, [_VP, _VP]),
    "tdm_work_wait_stream": (ctypes.c_int, [_VP, _VP]),
    "tdm_work_done": (ctypes.c_int, [_VP]),
    "tdm_work_times": (ctypes.c_int, [_VP, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]),
    "tdm_work_free": (ctypes.c_int, [_VP]),
}
TDM_BYTES = 6


def exported_symbols():
    """Every entry point include/tandem_hip.h declares."""
    return sorted(list(_SIGNATURES) + list(_ENGINE_SIGNATURES))


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise HipLibraryMissing(
                f"{LIB_PATH} has not been built; run `python -m tandem_amd.build` (hipcc, gfx950). "
                "tandem_amd has no CPU or PyTorch fallback for its kernels.")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in {**_SIGNATURES, **_ENGINE_SIGNATURES}.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        if L.tdm_abi_version() != ABI_VERSION:
            raise HipLibraryMissing(f"{LIB_PATH} has ABI version {L.tdm_abi_version()}, this package needs {ABI_VERSION}; rebuild it")
        _lib = L
    return _lib


def check(status):
    """0, or the exception the reference's binding would raise for that failure
    (tandem/csrc/engine.cpp:54-55 in the reference: invalid_argument -> ValueError,
    Timeout -> TimeoutError, anything else -> RuntimeError)."""
    if status == 0:
        return
    msg = lib().tdm_last_error().decode(errors="replace")
    if status == 1:
        raise ValueError(msg)
    if status == 3:
        raise TimeoutError(msg)
    raise RuntimeError(msg)


def dtype_code(dtype):
    try:
        return DTYPES[dtype]
    except KeyError:
        raise ValueError(f"tandem_amd's kernels do not handle {dtype}") from None


def stream_ptr(device=None):
    """torch's current HIP stream on `device`, as the hipStream_t the C ABI takes."""
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def require_device_tensor(t, what):
    if not isinstance(t, torch.Tensor) or t.device.type != "cuda":
        raise ValueError(f"{what}: needs a tensor in GPU memory (got {getattr(t, 'device', type(t))}); "
                         "tandem_amd has no CPU path")
    if not t.is_contiguous():
        raise ValueError(f"{what}: needs a contiguous tensor")
