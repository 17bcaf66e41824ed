"""ctypes binding of libwcn_hip.so (the C ABI declared in include/wcn_hip.h)."""
import ctypes
import os

import torch  # noqa: F401  (loads the HIP runtime the library links against)

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libwcn_hip.so")

OK = 0
ERR_TABLE_OVERFLOW = -3

DTYPE_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}

_vp, _i32, _i64, _sz = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_size_t
_i32p, _i64p = ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int64)

# name -> (restype, argtypes); must list every symbol include/wcn_hip.h declares
SIGNATURES = {
    "wcn_version": (ctypes.c_int, []),
    "wcn_status_string": (ctypes.c_char_p, [ctypes.c_int]),
    "wcn_thread_release": (ctypes.c_int, []),
    "wcn_table_default_capacity": (_i64, [_i64]),
    "wcn_table_bytes": (_sz, [_i64, _i64]),
    "wcn_table_build": (ctypes.c_int, [_vp, _i64, _vp, _i64, _vp]),
    "wcn_table_query": (ctypes.c_int, [_vp, _i64, _i64, _vp, _i64, _vp, _vp]),
    "wcn_table_read_status": (ctypes.c_int, [_vp, _i32p, _vp]),
    "wcn_kmap_workspace_bytes": (_sz, [_i64, _i32]),
    "wcn_kmap_count": (ctypes.c_int, [_vp, _i64, _i64, _vp, _i64, _i32p, _i32p, _vp, _vp]),
    "wcn_kmap_count_dilated": (ctypes.c_int, [_vp, _i64, _i64, _vp, _i64, _i32p, _i32p, _i32p, _i32p, _vp, _vp]),
    "wcn_kmap_read_result": (ctypes.c_int, [_vp, _i64, _i32, _i64p, _vp]),
    "wcn_kmap_fill": (ctypes.c_int, [_vp, _i64, _i64, _vp, _i64, _i32p, _i32p, _vp, _i64, _vp, _vp,
                                     _vp]),
    "wcn_kmap_self_supported": (ctypes.c_int, [_i32p, _i64]),
    "wcn_kmap_count_self": (ctypes.c_int, [_vp, _i64, _i64, _i32p, _vp, _vp]),
    "wcn_kmap_fill_self": (ctypes.c_int, [_i64, _i32p, _vp, _i64, _vp, _vp, _vp]),
    "wcn_kmap_group_start": (_vp, [_vp, _i64, _i32]),
    "wcn_kmap_last_table_flags": (_i32, []),
    "wcn_stride_unique_workspace_bytes": (_sz, [_i64, _i64]),
    "wcn_stride_unique": (ctypes.c_int, [_vp, _i64, _i32p, _vp, _i64, _vp, _vp, _vp]),
    "wcn_stride_unique_cells_workspace_bytes": (_sz, [_i64]),
    "wcn_stride_unique_cells": (ctypes.c_int, [_vp, _i64, _i64, _vp, _i32p, _vp, _vp, _vp, _vp]),
    "wcn_stride_unique_read_count": (ctypes.c_int, [_vp, _i64, _i64, _i64p, _vp]),
    "wcn_stride_unique_read_bounds": (ctypes.c_int, [_vp, _i64, _i64, _i64p, _i64p, _vp]),
    "wcn_conv_workspace_bytes": (_sz, [_i64, _i32, _i32, _i32, _i32, _i64, _i32]),
    "wcn_conv_last_kernel": (ctypes.c_char_p, []),
    "wcn_conv_set_timing_events": (ctypes.c_int, [_vp, _vp]),
    "wcn_sparse_conv_fwd": (ctypes.c_int, [_vp, _i64, _i32, _i32, _vp, _i32, _i32, _i32, _vp, _vp,
                                           _vp, _i64p, _i32, _i32, _vp, _vp, _i64, _vp, _sz, _vp]),
    "wcn_sparse_conv_fwd_fused": (ctypes.c_int, [_vp, _i64, _i32, _i32, _vp, _i32, _i32, _i32, _vp, _vp,
                                                 _vp, _i64p, _i32, _i32, _vp, _vp, _i32, _vp, _i64, _vp, _sz, _vp]),
    "wcn_conv_prepared_weight_bytes": (_sz, [_i32, _i32, _i32, _i32]),
    "wcn_conv_prepared_workspace_bytes": (_sz, [_i64, _i32, _i32, _i32, _i32]),
    "wcn_conv_prepare_weight": (ctypes.c_int, [_vp, _i32, _i32, _i32, _i32, _i32, _vp, _sz, _vp]),
    "wcn_sparse_conv_fwd_prepared": (ctypes.c_int, [_vp, _i64, _i32, _i32, _vp, _sz, _i32, _i32, _vp, _vp,
                                                    _vp, _i64p, _vp, _i32, _vp, _vp, _i32, _vp, _i64,
                                                    _vp, _sz, _vp]),
    "wcn_conv_single_supported": (ctypes.c_int, [_i32, _i32, _i32, _i32]),
    "wcn_sparse_conv_fwd_single": (ctypes.c_int, [_vp, _i64, _i32, _i32, _vp, _i32, _i32, _i32, _i32, _vp, _vp,
                                                  _vp, _i64p, _vp, _i32, _vp, _i64, _vp, _sz, _vp]),
    "wcn_sparse_conv_fwd_static": (ctypes.c_int, [_vp, _i64, _i32, _i32, _vp, _i32, _i32, _i32, _vp, _vp,
                                                  _vp, _i64p, _i32, _i32, _vp, _vp, _i64, _vp]),
    "wcn_pairs_sort_workspace_bytes": (_sz, [_i64, _i32, _i64]),
    "wcn_pairs_sort_by_out": (ctypes.c_int, [_vp, _vp, _i64p, _i32, _i64, _vp, _vp, _vp, _vp, _sz, _vp]),
    "wcn_sparse_conv_dgrad": (ctypes.c_int, [_vp, _i64, _i32, _i32, _vp, _i32, _i32, _i32, _vp, _vp,
                                             _i64p, _i32, _i32, _i32, _vp, _vp, _i64, _vp, _sz, _vp]),
    "wcn_map_rows_workspace_bytes": (_sz, [_i64, _i32, _i64]),
    "wcn_map_rows_build": (ctypes.c_int, [_vp, _vp, _i64p, _i32, _i64, _vp, _sz, _vp]),
    "wcn_sparse_pool_fwd": (ctypes.c_int, [_vp, _i64, _i32, _i32, _vp, _i64, _i32, _i64, _i32, _vp,
                                           _vp, _vp]),
    "wcn_sparse_pool_bwd": (ctypes.c_int, [_vp, _i64, _i32, _i32, _vp, _vp, _i64, _i32, _i64, _i32,
                                           _vp, _vp, _vp]),
    "wcn_sparse_depthwise_fwd": (ctypes.c_int, [_vp, _i64, _i32, _i32, _vp, _i32, _vp, _i64, _i32, _i64,
                                                _i32, _vp, _vp]),
    "wcn_depthwise_wgrad_workspace_bytes": (_sz, [_i32, _i32, _i64, _i64]),
    "wcn_sparse_depthwise_wgrad": (ctypes.c_int, [_vp, _i64, _vp, _i64, _i32, _i32, _vp, _vp, _i64p, _i32,
                                                  _i32, _vp, _i32, _vp, _sz, _vp]),
    "wcn_morton_codes": (ctypes.c_int, [_vp, _i64, _i32, _i32, _vp, _i32p, _vp, _vp]),
    "wcn_conv_wgrad_workspace_bytes": (_sz, [_i32, _i32, _i32, _i64, _i64]),
    "wcn_sparse_conv_wgrad": (ctypes.c_int, [_vp, _i64, _i32, _vp, _i64, _i32, _i32, _vp, _vp, _i64p,
                                             _i32, _i32, _vp, _i32, _vp, _sz, _vp]),
    "wcn_probe_gather_rows": (ctypes.c_int, [_vp, _i64, _i32, _vp, _i64, _vp, _vp]),
    "wcn_voxel_rows": (ctypes.c_int, [_vp, _i64, _i64p, _vp, _i32, ctypes.c_double, _vp, _vp]),
    "wcn_batch_indexed_rows": (ctypes.c_int, [_vp, _i64, _i32, _i64p, _i32, _vp, _vp]),
    "wcn_unique_rows_workspace_bytes": (_sz, [_i64]),
    "wcn_unique_rows_csr": (ctypes.c_int, [_vp, _i64, _i32, _vp, _sz, _vp, _vp, _vp, _vp, _vp, _i64p, _vp]),
    "wcn_voxelize_points_csr": (ctypes.c_int, [_vp, _i64, _i64p, _vp, _i32, ctypes.c_double, _vp, _sz, _vp, _vp,
                                               _vp, _vp, _vp, _i64p, _vp]),
    "wcn_segment_reduce": (ctypes.c_int, [_vp, _i64, _i32, _i32, _vp, _vp, _i64, _i64, _i32, _vp, _vp, _vp]),
    "wcn_segment_reduce_bwd": (ctypes.c_int, [_vp, _i64, _i32, _i32, _vp, _vp, _i64, _i32, _vp, _vp, _vp]),
}

_lib = None


def lib():
    """The loaded library; raises (never falls back) when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m warpconvnet_amd._build` "
                "(hipcc, gfx950). There is no CPU or PyTorch fallback for this path.")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


class WcnError(RuntimeError):
    def __init__(self, status: int, where: str):
        self.status = status
        text = lib().wcn_status_string(status).decode()
        super().__init__(f"{where}: {text} (status {status})")


def check(status: int, where: str) -> None:
    if status != OK:
        raise WcnError(status, where)


# The current stream's handle without the Stream object torch.cuda.current_stream builds around it
# (a few microseconds, several times per layer of a network).
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(device) -> ctypes.c_void_p:
    if _raw_stream is not None and isinstance(device, torch.device) and device.type == "cuda":
        index = device.index if device.index is not None else torch.cuda.current_device()
        return ctypes.c_void_p(_raw_stream(index))
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def ptr(t):
    """A tensor's address as the void* argument of a library call (None: a null pointer); ctypes
    converts the plain int itself."""
    return None if t is None else t.data_ptr()


def int3(values):
    return (ctypes.c_int32 * 3)(*[int(v) for v in values])


def require_device(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise ValueError(f"{what} must be on a GPU device, got {t.device}")


def workspace(nbytes: int, device) -> torch.Tensor:
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)
