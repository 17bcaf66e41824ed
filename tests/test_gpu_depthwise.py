"""GPU parity of the depthwise convolution over a kernel map (wcn_sparse_depthwise_fwd / _wgrad)
against the torch restatement of the reference's explicit depthwise path
(oracle/explicit_conv.py::explicit_depthwise_forward, float64) and its gradients as torch
differentiates them.  Tolerances: 1e-5 (fp32), 1e-2 (fp16 / bf16) relative."""
import numpy as np
import pytest
import torch

from helpers import normal_features, rel_err
from warpconvnet_amd.utils import synthetic

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {torch.float32: 1e-5, torch.float16: 1e-2, torch.bfloat16: 1e-2}


def _voxels(items, feats):
    from warpconvnet_amd.geometry.types.voxels import Voxels
    offsets = np.zeros(len(items) + 1, dtype=np.int64)
    offsets[1:] = np.cumsum([len(i) for i in items])
    coords = torch.as_tensor(np.concatenate(items, axis=0), dtype=torch.int32, device=DEV)
    return Voxels(coords, feats, offsets=torch.as_tensor(offsets))


@pytest.mark.parametrize("dtype,channels,ksize,stride", [
    (torch.float32, 32, 3, 1), (torch.float16, 64, 3, 1), (torch.bfloat16, 40, 3, 2),
    (torch.float32, 7, 2, 2), (torch.float16, 300, 3, 1)])
def test_depthwise_forward_and_gradients(oracle, dtype, channels, ksize, stride):
    from oracle.explicit_conv import explicit_depthwise_forward
    from warpconvnet_amd.nn.modules.sparse_conv_depth import SparseDepthwiseConv3d
    items = [synthetic.indoor_scene(seed=90 + b, n_target=4000, voxel_size=0.05) for b in range(2)]
    bc = synthetic.batch_indexed(items)
    x = normal_features(len(bc), channels, seed=2, dtype=dtype)
    torch.manual_seed(3)
    conv = SparseDepthwiseConv3d(channels, ksize, stride=stride, bias=False).to(DEV).to(dtype)
    xd = x.to(DEV).requires_grad_(True)
    out = conv(_voxels(items, xd))
    out_bc = out.batch_indexed_coordinates.cpu().numpy()
    im, om, off, iden = oracle.kernel_map(bc, out_bc, (ksize,) * 3, (stride,) * 3)
    x64 = x.double().requires_grad_(True)
    w64 = conv.weight.detach().double().cpu().requires_grad_(True)
    want = explicit_depthwise_forward(x64, w64, torch.as_tensor(im), torch.as_tensor(om), off, iden,
                                      len(out_bc))
    assert out.feature_tensor.dtype == dtype
    assert rel_err(out.feature_tensor.detach().double().cpu().numpy(), want.detach().numpy()) <= TOL[dtype]
    gy = normal_features(len(out_bc), channels, seed=4, dtype=dtype)
    out.feature_tensor.backward(gy.to(DEV))
    want_gx, want_gw = torch.autograd.grad(want, (x64, w64), gy.double())
    assert xd.grad.dtype == dtype and conv.weight.grad.dtype == dtype
    assert rel_err(xd.grad.double().cpu().numpy(), want_gx.numpy()) <= TOL[dtype]
    assert rel_err(conv.weight.grad.double().cpu().numpy(), want_gw.numpy()) <= TOL[dtype]


def test_depthwise_fp32_weights_with_fp16_features(oracle):
    from oracle.explicit_conv import explicit_depthwise_forward
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    from warpconvnet_amd.nn.functional.sparse_conv_depth import spatially_sparse_depthwise_conv
    bc = synthetic.random_cloud(95, 5000, 22, batch_size=2)
    c = torch.as_tensor(bc, device=DEV)
    km = generate_kernel_map(c, c, (1, 1, 1), (3, 3, 3))
    x = normal_features(len(bc), 48, seed=5, dtype=torch.float16)
    w = (torch.randn(27, 48, generator=torch.Generator().manual_seed(6)) * 0.2)
    wd = w.to(DEV).requires_grad_(True)
    out = spatially_sparse_depthwise_conv(x.to(DEV), wd, km, len(bc))
    im, om, off, iden = oracle.kernel_map(bc, bc, (3, 3, 3))
    want = explicit_depthwise_forward(x.double(), w.double(), torch.as_tensor(im), torch.as_tensor(om),
                                      off, iden, len(bc))
    assert rel_err(out.detach().double().cpu().numpy(), want.numpy()) <= 1e-2
    out.float().sum().backward()
    assert wd.grad.dtype == torch.float32
    want_gw = torch.stack([x.double()[im[off[k]:off[k + 1]]].sum(0) for k in range(27)])
    assert rel_err(wd.grad.double().cpu().numpy(), want_gw.numpy()) <= 1e-2


def test_depthwise_at_benchmark_size():
    """4 x 250k voxels, 64 channels fp16, 3x3x3: with all-ones weights the result is the sum of the
    neighbours' features (torch index_add over the map); with the centre tap alone it is a copy."""
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    from warpconvnet_amd.nn.functional.sparse_conv_depth import spatially_sparse_depthwise_conv
    items, _ = synthetic.indoor_batch(4, 250_000)
    c = torch.as_tensor(synthetic.batch_indexed(items), device=DEV)
    n = c.shape[0]
    km = generate_kernel_map(c, c, (1, 1, 1), (3, 3, 3))
    x = torch.randn(n, 64, generator=torch.Generator().manual_seed(7)).half().to(DEV)
    w = torch.zeros(27, 64, dtype=torch.float16, device=DEV)
    w[13] = 1
    assert torch.equal(spatially_sparse_depthwise_conv(x, w, km, n), x)
    w[:] = 1
    want = torch.zeros(n, 64, dtype=torch.float32, device=DEV)
    want.index_add_(0, km.out_maps.long(), x.float()[km.in_maps.long()])
    got = spatially_sparse_depthwise_conv(x, w, km, n)
    assert rel_err(got.float().cpu().numpy(), want.cpu().numpy()) <= 1e-2
