"""ctypes front end of the C oracle (oracle/wcn_oracle.c).  TEST INFRASTRUCTURE ONLY.

Only tests/, the smoke check and the benchmark's cpu_baseline leg may import this module; the
product package never does.  All inputs and outputs are numpy arrays on the host.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libwcn_oracle.so")

HASH_FNV1A, HASH_CITY, HASH_MURMUR = 0, 1, 2


def build(force: bool = False) -> str:
    """Compile the oracle with the Makefile next to it."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        i32p = ctypes.POINTER(ctypes.c_int32)
        i64p = ctypes.POINTER(ctypes.c_int64)
        f64p = ctypes.POINTER(ctypes.c_double)
        L.wcn_oracle_hash32.restype = ctypes.c_uint32
        L.wcn_oracle_hash32.argtypes = [i32p, ctypes.c_int, ctypes.c_int]
        L.wcn_oracle_hash_slot.restype = ctypes.c_int
        L.wcn_oracle_hash_slot.argtypes = [i32p, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        L.wcn_oracle_table_init.restype = None
        L.wcn_oracle_table_init.argtypes = [i32p, ctypes.c_int]
        L.wcn_oracle_table_insert.restype = ctypes.c_int
        L.wcn_oracle_table_insert.argtypes = [i32p, ctypes.c_int, i32p, ctypes.c_int, ctypes.c_int,
                                              ctypes.c_int]
        L.wcn_oracle_table_search.restype = None
        L.wcn_oracle_table_search.argtypes = [i32p, ctypes.c_int, i32p, ctypes.c_int, i32p,
                                              ctypes.c_int64, ctypes.c_int, i32p]
        L.wcn_oracle_kernel_offsets.restype = None
        L.wcn_oracle_kernel_offsets.argtypes = [i32p, i32p, i32p]
        L.wcn_oracle_kernel_map_found.restype = ctypes.c_int
        L.wcn_oracle_kernel_map_found.argtypes = [i32p, ctypes.c_int, i32p, ctypes.c_int64, i32p,
                                                  i32p, ctypes.c_int, i32p]
        L.wcn_oracle_kernel_map_offsets.restype = ctypes.c_int
        L.wcn_oracle_kernel_map_offsets.argtypes = [i32p, ctypes.c_int, i32p, ctypes.c_int64, i32p,
                                                    ctypes.c_int, i32p, ctypes.c_int, i32p]
        L.wcn_oracle_compact_found.restype = ctypes.c_int64
        L.wcn_oracle_compact_found.argtypes = [i32p, ctypes.c_int, ctypes.c_int64, i64p, i32p, i32p]
        L.wcn_oracle_stride_coords.restype = ctypes.c_int64
        L.wcn_oracle_stride_coords.argtypes = [i32p, ctypes.c_int, i32p, ctypes.c_int, i32p, i32p,
                                               i64p]
        L.wcn_oracle_explicit_conv_f64.restype = None
        L.wcn_oracle_explicit_conv_f64.argtypes = [f64p, ctypes.c_int64, f64p, ctypes.c_int,
                                                   ctypes.c_int, ctypes.c_int, i32p, i32p, i64p,
                                                   ctypes.c_int, ctypes.c_int64, f64p]
        _lib = L
    return _lib


def _i32(a):
    a = np.ascontiguousarray(a, dtype=np.int32)
    return a, a.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))


def _ptr(a, ct):
    return a.ctypes.data_as(ctypes.POINTER(ct))


def hash32(key, method=HASH_CITY) -> int:
    k, kp = _i32(key)
    return int(lib().wcn_oracle_hash32(kp, k.size, method))


class HashTable:
    """The reference's (capacity, 2) int32 open-addressing table, built serially."""

    def __init__(self, keys, capacity=None, method=HASH_CITY):
        self.keys, kp = _i32(keys)
        assert self.keys.ndim == 2
        n, self.key_dim = self.keys.shape
        self.capacity = int(capacity) if capacity is not None else max(16, 2 * n)
        self.method = method
        self.kvs = np.empty((self.capacity, 2), dtype=np.int32)
        L = lib()
        L.wcn_oracle_table_init(_ptr(self.kvs, ctypes.c_int32), self.capacity)
        self.dropped = L.wcn_oracle_table_insert(_ptr(self.kvs, ctypes.c_int32), self.capacity, kp,
                                                 n, self.key_dim, method)

    def search(self, queries) -> np.ndarray:
        q, qp = _i32(queries)
        assert q.ndim == 2 and q.shape[1] == self.key_dim
        out = np.empty(q.shape[0], dtype=np.int32)
        lib().wcn_oracle_table_search(_ptr(self.kvs, ctypes.c_int32), self.capacity,
                                      _ptr(self.keys, ctypes.c_int32), self.key_dim, qp,
                                      q.shape[0], self.method, _ptr(out, ctypes.c_int32))
        return out


def kernel_map_found(in_coords, out_coords, kernel_size, stride=(1, 1, 1), method=HASH_CITY):
    """Dense (K, M) table of found input indices (-1 where absent)."""
    ic, icp = _i32(in_coords)
    oc, ocp = _i32(out_coords)
    ks, ksp = _i32(kernel_size)
    st, stp = _i32(stride)
    K = int(np.prod(ks))
    found = np.empty((K, oc.shape[0]), dtype=np.int32)
    rc = lib().wcn_oracle_kernel_map_found(icp, ic.shape[0], ocp, oc.shape[0], ksp, stp, method,
                                           _ptr(found, ctypes.c_int32))
    if rc != 0:
        raise MemoryError("oracle allocation failed")
    return found


def compact_found(found):
    """(in_maps[L], out_maps[L], offsets[K+1]) from a dense found table, reference pair order."""
    f, fp = _i32(found)
    K, M = f.shape
    offsets = np.empty(K + 1, dtype=np.int64)
    L = lib().wcn_oracle_compact_found(fp, K, M, _ptr(offsets, ctypes.c_int64), None, None)
    in_maps = np.empty(L, dtype=np.int32)
    out_maps = np.empty(L, dtype=np.int32)
    lib().wcn_oracle_compact_found(fp, K, M, _ptr(offsets, ctypes.c_int64),
                                   _ptr(in_maps, ctypes.c_int32), _ptr(out_maps, ctypes.c_int32))
    return in_maps, out_maps, offsets


def kernel_offsets(kernel_size, dilation=(1, 1, 1), center_offset=None):
    """(K, 4) offsets of kernel_offsets_from_size (torch_discrete.py:44-77): last dimension fastest,
    (index - centre) * dilation, centre (s - 1) // 2 for odd sizes and 0 for even ones unless given."""
    ks, ksp = _i32(kernel_size)
    dl, dlp = _i32(dilation)
    K = int(np.prod(ks))
    out = np.empty((K, 4), dtype=np.int32)
    lib().wcn_oracle_kernel_offsets(ksp, dlp, _ptr(out, ctypes.c_int32))
    if center_offset is not None:  # the default centre is replaced, not shifted (:64-67)
        default = np.array([(int(s) - 1) // 2 if int(s) % 2 == 1 else 0 for s in ks], dtype=np.int32)
        out[:, 1:] += (default - np.asarray(center_offset, dtype=np.int32)) * dl
    return out


def kernel_map_found_offsets(in_coords, out_coords, offsets, stride=(1, 1, 1), method=HASH_CITY):
    """Dense (K, M) table of found input indices for an explicit offset table (method="offset")."""
    ic, icp = _i32(in_coords)
    oc, ocp = _i32(out_coords)
    of, ofp = _i32(offsets)
    st, stp = _i32(stride)
    found = np.empty((of.shape[0], oc.shape[0]), dtype=np.int32)
    rc = lib().wcn_oracle_kernel_map_offsets(icp, ic.shape[0], ocp, oc.shape[0], ofp, of.shape[0], stp,
                                             method, _ptr(found, ctypes.c_int32))
    if rc != 0:
        raise MemoryError("oracle allocation failed")
    return found


def kernel_map(in_coords, out_coords, kernel_size, stride=(1, 1, 1), method=HASH_CITY, dilation=None,
               center_offset=None):
    """Reference-ordered kernel map plus the identity index rule of torch_discrete.py:418-425.
    With `dilation` / `center_offset` the offsets are those of method="offset"."""
    if dilation is None and center_offset is None:
        found = kernel_map_found(in_coords, out_coords, kernel_size, stride, method)
    else:
        offs = kernel_offsets(kernel_size, dilation or (1, 1, 1), center_offset)
        found = kernel_map_found_offsets(in_coords, out_coords, offs, stride, method)
    in_maps, out_maps, offsets = compact_found(found)
    odd = all(int(k) % 2 == 1 for k in kernel_size)
    iden = int(np.prod(kernel_size)) // 2 if odd and len(in_coords) == len(out_coords) else None
    return in_maps, out_maps, offsets, iden


def stride_coords(coords, stride, num_batches):
    c, cp = _i32(coords)
    st, stp = _i32(stride)
    n = c.shape[0]
    out = np.empty((max(n, 1), 4), dtype=np.int32)
    first = np.empty(max(n, 1), dtype=np.int32)
    offsets = np.empty(num_batches + 1, dtype=np.int64)
    M = lib().wcn_oracle_stride_coords(cp, n, stp, num_batches, _ptr(out, ctypes.c_int32),
                                       _ptr(first, ctypes.c_int32), _ptr(offsets, ctypes.c_int64))
    if M < 0:
        raise MemoryError("oracle allocation failed")
    return out[:M].copy(), first[:M].copy(), offsets


def explicit_conv_f64(x, w, in_maps, out_maps, offsets, iden, num_out):
    """Double-precision explicit gather-GEMM-scatter forward (the accuracy yardstick)."""
    X = np.ascontiguousarray(x, dtype=np.float64)
    W = np.ascontiguousarray(w, dtype=np.float64)
    im, imp = _i32(in_maps)
    om, omp = _i32(out_maps)
    off = np.ascontiguousarray(offsets, dtype=np.int64)
    K, Cin, Cout = W.shape
    out = np.empty((num_out, Cout), dtype=np.float64)
    lib().wcn_oracle_explicit_conv_f64(_ptr(X, ctypes.c_double), X.shape[0],
                                       _ptr(W, ctypes.c_double), K, Cin, Cout, imp, omp,
                                       _ptr(off, ctypes.c_int64), -1 if iden is None else int(iden),
                                       num_out, _ptr(out, ctypes.c_double))
    return out
