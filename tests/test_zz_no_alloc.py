"""wcn_sparse_conv_fwd_static (the contraction for callers that cannot allocate) against
wcn_sparse_conv_fwd on the same inputs, both called through the C ABI, and both against the fp64
oracle; that the call leaves the allocators alone; and that it can be captured into a HIP graph.

Two calls in a row on the same GPU, the second with a smaller input: the library's one scratch
array keeps the first call's contents, and the second result must not depend on them.
Tolerance (max|a-b| / max|b|): 1e-2 for fp16, the bar of the feature parity tests.
"""
import ctypes

import numpy as np
import pytest
import torch

from helpers import kaiming_weight, normal_features, rel_err
from warpconvnet_amd.utils import synthetic

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
STATIC_SCRATCH_BYTES = 4 << 20  # WCN_CONV_STATIC_SCRATCH_BYTES of include/wcn_hip.h


def _both_entry_points(oracle, n_voxels, seed, ascend=True):
    from warpconvnet_amd._lib import DTYPE_CODE, check, lib, ptr, stream_ptr, workspace
    L = lib()
    dtype, c_in, c_out, K = torch.float16, 64, 64, 27
    bc = synthetic.random_cloud(seed, n_voxels, 30, batch_size=2)
    n = len(bc)
    im, om, off, iden = oracle.kernel_map(bc, bc, (3, 3, 3))
    if not ascend:  # the exchanged lists of a transposed convolution: re-ordered inside the scratch
        im, om = om, im
    x = normal_features(n, c_in, seed=seed, dtype=dtype).to(DEV)
    w = kaiming_weight(K, c_in, c_out, seed=seed + 1, dtype=dtype).to(DEV)
    bias = (torch.randn(c_out, generator=torch.Generator().manual_seed(seed)) * 0.1).to(dtype).to(DEV)
    imd = torch.as_tensor(im, dtype=torch.int32, device=DEV)
    omd = torch.as_tensor(om, dtype=torch.int32, device=DEV)
    offs = (ctypes.c_int64 * (K + 1))(*[int(v) for v in off])
    code = DTYPE_CODE[dtype]
    stream = stream_ptr(torch.device(DEV))
    need = L.wcn_conv_workspace_bytes(n, K, c_in, c_out, code, len(im), 1 if ascend else 0)
    assert 0 < need <= STATIC_SCRATCH_BYTES
    ws = workspace(need, DEV)
    want = torch.empty(n, c_out, dtype=dtype, device=DEV)
    check(L.wcn_sparse_conv_fwd(ptr(x), n, c_in, code, ptr(w), code, K, c_out, ptr(bias), ptr(imd),
                                ptr(omd), offs, -1, 1 if ascend else 0, None, ptr(want), n, ptr(ws),
                                ws.numel(), stream), "wcn_sparse_conv_fwd")
    got = torch.full((n, c_out), float("nan"), dtype=dtype, device=DEV)
    check(L.wcn_sparse_conv_fwd_static(ptr(x), n, c_in, code, ptr(w), code, K, c_out, ptr(bias),
                                       ptr(imd), ptr(omd), offs, -1, 1 if ascend else 0, None,
                                       ptr(got), n, stream), "wcn_sparse_conv_fwd_static")
    torch.cuda.synchronize()
    exact = oracle.explicit_conv_f64(x.double().cpu().numpy(), w.double().cpu().numpy(), im, om, off, None, n)
    exact = exact + bias.double().cpu().numpy()
    return got.float().cpu().numpy(), want.float().cpu().numpy(), exact


def test_static_scratch_entry_point_matches_the_workspace_one(oracle):
    got, want, exact = _both_entry_points(oracle, 9000, seed=5)
    assert np.isfinite(got).all() and rel_err(got, want) <= 1e-2 and rel_err(got, exact) <= 1e-2
    got, want, exact = _both_entry_points(oracle, 2500, seed=6)  # smaller: stale scratch contents behind it
    assert np.isfinite(got).all() and rel_err(got, want) <= 1e-2 and rel_err(got, exact) <= 1e-2
    got, want, exact = _both_entry_points(oracle, 1500, seed=7, ascend=False)  # lists re-ordered in the scratch
    assert np.isfinite(got).all() and rel_err(got, want) <= 1e-2 and rel_err(got, exact) <= 1e-2


def test_static_scratch_entry_point_allocates_nothing_and_can_be_captured(oracle):
    """What the entry point promises: no allocation (the allocators' figures do not move across a
    call) and kernels only (a call records into a HIP graph; every replay, with eager work and
    synchronisations in between, gives the eager result)."""
    from warpconvnet_amd._lib import DTYPE_CODE, check, lib, ptr
    L = lib()
    dtype, c_in, c_out, K = torch.float16, 64, 64, 27
    bc = synthetic.random_cloud(11, 6000, 30, batch_size=2)
    n = len(bc)
    im, om, off, _ = oracle.kernel_map(bc, bc, (3, 3, 3))
    x = normal_features(n, c_in, seed=11, dtype=dtype).to(DEV)
    w = kaiming_weight(K, c_in, c_out, seed=12, dtype=dtype).to(DEV)
    imd = torch.as_tensor(im, dtype=torch.int32, device=DEV)
    omd = torch.as_tensor(om, dtype=torch.int32, device=DEV)
    offs = (ctypes.c_int64 * (K + 1))(*[int(v) for v in off])
    code = DTYPE_CODE[dtype]
    eager = torch.empty(n, c_out, dtype=dtype, device=DEV)
    replayed = torch.empty(n, c_out, dtype=dtype, device=DEV)

    def call(out, stream):
        check(L.wcn_sparse_conv_fwd_static(ptr(x), n, c_in, code, ptr(w), code, K, c_out, None, ptr(imd),
                                           ptr(omd), offs, -1, 1, None, ptr(out), n,
                                           ctypes.c_void_p(stream.cuda_stream)), "wcn_sparse_conv_fwd_static")

    call(eager, torch.cuda.current_stream())  # first call on the device: the scratch array's address is looked up
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    held0, reserved0 = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    call(eager, torch.cuda.current_stream())
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0
    assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved()) == (held0, reserved0)
    exact = oracle.explicit_conv_f64(x.double().cpu().numpy(), w.double().cpu().numpy(), im, om, off, None, n)
    assert rel_err(eager.float().cpu().numpy(), exact) <= 1e-2

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.graph(graph, stream=side):  # an allocation or a copy command would fail the capture
        call(replayed, torch.cuda.current_stream())
    for turn in range(3):
        replayed.fill_(float("nan"))
        x2 = torch.randn(1000, 64, device=DEV) @ torch.randn(64, 64, device=DEV)  # eager work in between
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(replayed, eager), turn
        del x2


def test_static_scratch_entry_point_rejects_what_does_not_fit():
    from warpconvnet_amd._lib import lib
    L = lib()
    K = 27
    offs = (ctypes.c_int64 * (K + 1))(*([0] * (K + 1)))
    one = ctypes.c_void_p(256)  # never dereferenced: the size check comes first
    n = 50_000_000  # group starts alone exceed the scratch array
    st = L.wcn_sparse_conv_fwd_static(one, n, 64, 1, one, 1, K, 64, None, None, None, offs, -1, 1,
                                      None, one, n, None)
    assert st == -6 and b"workspace" in L.wcn_status_string(st).lower()
    many = (ctypes.c_int64 * 201)(*([0] * 201))
    st = L.wcn_sparse_conv_fwd_static(one, 10, 64, 1, one, 1, 200, 64, None, None, None, many, -1, 1,
                                      None, one, 10, None)
    assert st == -1
