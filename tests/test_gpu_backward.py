"""GPU parity of the gradients of the feature contraction (wcn_sparse_conv_dgrad / _wgrad).

Yardstick: the torch-CPU restatement of the reference's explicit backward
(oracle/explicit_conv.py, pinned by autograd of the pinned forward) evaluated in float64 on the
same (already rounded) inputs.  Tolerances (max|a-b| / max|b| per tensor): 1e-5 for fp32,
1e-2 for fp16 / bf16.  At benchmark size the gradients are checked through properties that need
no oracle: they are the adjoints of the forward product in its two arguments.
"""
import numpy as np
import pytest
import torch

from helpers import kaiming_weight, normal_features, rel_err
from warpconvnet_amd.utils import synthetic

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {torch.float32: 1e-5, torch.float16: 1e-2, torch.bfloat16: 1e-2}


def _voxels(items, feats, **kw):
    from warpconvnet_amd.geometry.types.voxels import Voxels
    offsets = np.zeros(len(items) + 1, dtype=np.int64)
    offsets[1:] = np.cumsum([len(i) for i in items])
    coords = torch.as_tensor(np.concatenate(items, axis=0), dtype=torch.int32, device=DEV)
    return Voxels(coords, feats.to(DEV), offsets=torch.as_tensor(offsets), **kw)


def _oracle_grads(gy, x, w, im, om, off, iden):
    from oracle.explicit_conv import explicit_gemm_backward
    return explicit_gemm_backward(gy.double(), x.double(), w.double(), torch.as_tensor(im),
                                  torch.as_tensor(om), off, iden)


CASES = [
    # name, dtype, c_in, c_out, voxels per item, batch, kernel
    ("f32_32_32", torch.float32, 32, 32, 5000, 2, (3, 3, 3)),
    ("f16_64_64", torch.float16, 64, 64, 5000, 2, (3, 3, 3)),
    ("bf16_96_128", torch.bfloat16, 96, 128, 3000, 1, (3, 3, 3)),
    ("f32_7_13", torch.float32, 7, 13, 2500, 2, (3, 3, 3)),
    ("f16_3_32", torch.float16, 3, 32, 2500, 1, (3, 3, 3)),
    ("f16_16_16_k5", torch.float16, 16, 16, 2500, 1, (5, 5, 5)),
    ("bf16_40_72_k2", torch.bfloat16, 40, 72, 2500, 1, (2, 2, 2)),
    # wide rows and enough of them for the output-stationary kernel: forward 128 -> 256 and, for the
    # input gradient, the same kernel over 256 -> 128 (odd kernel: symmetric map; even: re-ordered map)
    ("f16_128_256_rows", torch.float16, 128, 256, 13000, 2, (3, 3, 3)),
    ("bf16_128_128_rows_k2", torch.bfloat16, 128, 128, 13000, 2, (2, 2, 2)),
]


@pytest.mark.parametrize("name,dtype,c_in,c_out,n,batch,ksize", CASES, ids=[c[0] for c in CASES])
def test_gradients_stride1_match_oracle(oracle, name, dtype, c_in, c_out, n, batch, ksize):
    """Through autograd of the public functional: same coordinates in and out (for odd kernels the
    map is symmetric and carries the identity offset)."""
    from warpconvnet_amd.nn.functional.sparse_conv import spatially_sparse_conv
    items = [synthetic.random_cloud(30 + b, n, 24)[:, 1:] for b in range(batch)]
    bc = synthetic.batch_indexed(items)
    K = int(np.prod(ksize))
    x = normal_features(len(bc), c_in, seed=6, dtype=dtype)
    w = kaiming_weight(K, c_in, c_out, seed=7, dtype=dtype)
    gy = normal_features(len(bc), c_out, seed=8, dtype=dtype)
    xd = x.to(DEV).requires_grad_(True)
    wd = w.to(DEV).requires_grad_(True)
    out = spatially_sparse_conv(_voxels(items, xd), wd, ksize)
    out.feature_tensor.backward(gy.to(DEV))
    im, om, off, iden = oracle.kernel_map(bc, bc, ksize)
    want_x, want_w = _oracle_grads(gy, x, w, im, om, off, iden)
    assert xd.grad.dtype == dtype and wd.grad.dtype == dtype
    assert rel_err(xd.grad.float().cpu().numpy(), want_x.numpy()) <= TOL[dtype], name
    assert rel_err(wd.grad.float().cpu().numpy(), want_w.numpy()) <= TOL[dtype], name


def test_gradients_with_duplicate_voxels_use_the_general_path(oracle):
    """Duplicate voxels break the symmetry of the map; the table reports them and the library
    exchanges the lists instead.  Two duplicate output rows find the same input row, so the
    reference's `grad_in[in_map] += ...` (sparse_conv.py:350) keeps one of the two contributions,
    whichever is written last: those input rows have no defined gradient and are left out of the
    comparison.  The weight gradient sums over pairs and is defined everywhere."""
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    from warpconvnet_amd.nn.functional.sparse_conv import sparse_conv_backward
    bc = synthetic.random_cloud(40, 3000, 20)
    bc = np.ascontiguousarray(np.concatenate([bc, bc[100:400]], axis=0))
    c = torch.as_tensor(bc, device=DEV)
    km = generate_kernel_map(c, c, (1, 1, 1), (3, 3, 3))
    assert km._symmetric is False
    n = len(bc)
    x, w, gy = (normal_features(n, 32, 1), kaiming_weight(27, 32, 48, 2), normal_features(n, 48, 3))
    with pytest.warns(RuntimeWarning, match="repeat an"):  # says how many pairs the gradient leaves out
        gx, gw = sparse_conv_backward(gy.to(DEV), x.to(DEV), w.to(DEV), km)
    im, om, off, iden = oracle.kernel_map(bc, bc, (3, 3, 3))
    want_x, want_w = _oracle_grads(gy, x, w, im, om, off, iden)
    assert rel_err(gw.cpu().numpy(), want_w.numpy()) <= 1e-5
    defined = np.ones(n, dtype=bool)
    for k in range(27):
        if k == iden:
            continue
        rows, counts = np.unique(im[off[k]:off[k + 1]], return_counts=True)
        defined[rows[counts > 1]] = False
    assert 0.3 < defined.mean() < 1.0
    assert rel_err(gx.cpu().numpy()[defined], want_x.numpy()[defined]) <= 1e-5


@pytest.mark.parametrize("dtype,c1,c2", [(torch.float32, 24, 40), (torch.bfloat16, 24, 40), (torch.bfloat16, 32, 64)],
                         ids=["f32_24_40", "bf16_24_40", "bf16_32_64_one_pair_per_row"])
def test_gradients_of_strided_and_transposed_pair(oracle, dtype, c1, c2):
    """2x2x2 stride-2 convolution followed by its transposed convolution back onto the fine
    voxels: the gradient of the first exchanges an unsorted map (re-ordered by the library, or, for
    16-bit rows of whole 32-channel steps, taken as it is: every fine row is in one pair, so its
    gradient is one product), the gradient of the second a map whose input list ascends."""
    from warpconvnet_amd._lib import lib
    from warpconvnet_amd.nn.functional.sparse_conv import spatially_sparse_conv
    from oracle.explicit_conv import explicit_gemm_forward
    items = [synthetic.indoor_scene(seed=50 + b, n_target=6000, voxel_size=0.05) for b in range(2)]
    bc = synthetic.batch_indexed(items)
    x = normal_features(len(bc), c1, seed=9, dtype=dtype)
    w_down = kaiming_weight(8, c1, c2, seed=10, dtype=dtype)
    w_up = kaiming_weight(8, c2, c1, seed=11, dtype=dtype)
    gy = normal_features(len(bc), c1, seed=12, dtype=dtype)
    xd = x.to(DEV).requires_grad_(True)
    wd, wu = w_down.to(DEV).requires_grad_(True), w_up.to(DEV).requires_grad_(True)
    fine = _voxels(items, xd)
    coarse = spatially_sparse_conv(fine, wd, (2, 2, 2), stride=(2, 2, 2))
    back = spatially_sparse_conv(coarse, wu, (2, 2, 2), stride=(2, 2, 2), transposed=True,
                                 output_spatially_sparse_tensor=fine)
    back.feature_tensor.backward(gy.to(DEV))
    took_single = lib().wcn_conv_last_kernel().decode().startswith("conv_fwd_single<")
    assert took_single == (c1 % 32 == 0 and dtype != torch.float32), lib().wcn_conv_last_kernel()

    # float64 chain on the CPU over the library's own coarse coordinates (their order is free)
    coarse_bc = coarse.batch_indexed_coordinates.cpu().numpy()
    im, om, off, iden = oracle.kernel_map(bc, coarse_bc, (2, 2, 2), (2, 2, 2))
    im_t, om_t = torch.as_tensor(im), torch.as_tensor(om)
    x64 = x.double().requires_grad_(True)
    wd64, wu64 = w_down.double().requires_grad_(True), w_up.double().requires_grad_(True)
    mid = explicit_gemm_forward(x64, wd64, im_t, om_t, off, iden, len(coarse_bc))
    if dtype != torch.float32:
        mid = mid + (mid.detach().to(dtype).double() - mid.detach())  # the rounding between the layers
    out = explicit_gemm_forward(mid, wu64, om_t, im_t, off, None, len(bc))
    want_x, want_wd, want_wu = torch.autograd.grad(out, (x64, wd64, wu64), gy.double())
    tol = TOL[dtype] * (1 if dtype == torch.float32 else 2)  # two rounded layers in the chain
    assert rel_err(xd.grad.float().cpu().numpy(), want_x.numpy()) <= tol
    assert rel_err(wd.grad.float().cpu().numpy(), want_wd.numpy()) <= tol
    assert rel_err(wu.grad.float().cpu().numpy(), want_wu.numpy()) <= tol


def test_module_trains_one_step(oracle):
    """SparseConv3d with fp32 parameters and fp16 features: the weight gradient comes back in the
    parameter's dtype and an SGD step changes the output."""
    from warpconvnet_amd.nn.modules.sparse_conv import SparseConv3d
    items = [synthetic.random_cloud(60, 3000, 20)[:, 1:]]
    x = normal_features(len(items[0]), 16, seed=13, dtype=torch.float16)
    torch.manual_seed(0)
    conv = SparseConv3d(16, 32, kernel_size=3, bias=True).to(DEV)
    vox = _voxels(items, x)
    out = conv(vox).feature_tensor
    loss = out.float().square().mean()
    loss.backward()
    assert conv.weight.grad is not None and conv.weight.grad.dtype == conv.weight.dtype
    assert torch.isfinite(conv.weight.grad).all() and conv.weight.grad.abs().max() > 0
    with torch.no_grad():
        conv.weight -= 0.1 * conv.weight.grad
    loss2 = conv(vox).feature_tensor.float().square().mean()
    assert loss2 < loss


def test_gradients_are_adjoints_at_benchmark_size():
    """4 x 250k voxels, 3x3x3, 64 -> 64 fp16.  For the forward product F(x, W):
    <F(x, W), y> = <x, dgrad(y)>  and  <F(x, V), y> = <V, wgrad(x, y)> for any V (F is linear in
    both).  Evaluated in float64 on the GPU from the fp16 results; the tolerance is the feature
    tolerance relative to the size of the inner product's terms."""
    import bench
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    from warpconvnet_amd.nn.functional.sparse_conv import sparse_conv_backward, sparse_conv_forward
    bcoords, _, feats, weight = bench.make_workload()
    n = len(bcoords)
    c = torch.as_tensor(bcoords, device=DEV)
    # fp32 parameters, as a module holds them: a sum over 10^6 pairs does not fit fp16
    x, w = feats.to(DEV), weight.float().to(DEV)
    km = generate_kernel_map(c, c, (1, 1, 1), (3, 3, 3))
    assert km._symmetric
    f_w = sparse_conv_forward(x, w, km, n)
    # y and V are correlated with F(x, W) and W, so that both inner products are far from zero
    g = torch.Generator().manual_seed(17)
    y = (f_w.float().cpu() + 0.5 * torch.randn(n, 64, generator=g)).to(torch.float16).to(DEV)
    v = (0.7 * weight.float() + 0.02 * torch.randn(27, 64, 64, generator=g)).to(DEV)
    gx, gw = sparse_conv_backward(y, x, w, km)
    assert gw.dtype == torch.float32 and torch.isfinite(gw).all()
    f_v = sparse_conv_forward(x, v, km, n)

    def dot(a, b):
        return float((a.double() * b.double()).sum())

    lhs, rhs = dot(f_w, y), dot(x, gx)
    assert abs(lhs) > 1e5 and abs(lhs - rhs) <= 1e-3 * abs(lhs), (lhs, rhs)
    lhs, rhs = dot(f_v, y), dot(v, gw)
    assert abs(lhs) > 1e5 and abs(lhs - rhs) <= 1e-3 * abs(lhs), (lhs, rhs)
    # the general path (lists exchanged and re-ordered) gives the same input gradient up to the
    # order of the fp32 additions
    km._symmetric = False
    gx2, _ = sparse_conv_backward(y, x, w, km, need_weight_grad=False)
    km._symmetric = True
    assert rel_err(gx2.float().cpu().numpy(), gx.float().cpu().numpy()) <= 2e-3


def test_every_device_result_is_bitwise_reproducible():
    """No result depends on the order in which waves happen to run: maps, the contraction, both
    gradients, pooling, the depthwise weight gradient and the point -> voxel grouping come out
    bit for bit the same from two runs (the reductions run in a fixed order, nothing is summed
    with floating-point atomics)."""
    from warpconvnet_amd.geometry.coords.ops.voxel import voxel_downsample_csr_mapping
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    from warpconvnet_amd.nn.functional.sparse_conv import sparse_conv_backward, sparse_conv_forward
    from warpconvnet_amd.nn.functional.sparse_conv_depth import spatially_sparse_depthwise_conv
    from warpconvnet_amd.nn.functional.sparse_pool import sparse_reduce
    from warpconvnet_amd.ops.reductions import segment_reduction
    items = [synthetic.indoor_scene(seed=300 + b, n_target=30_000, voxel_size=0.04) for b in range(2)]
    bc = torch.as_tensor(synthetic.batch_indexed(items), device=DEV)
    n = len(bc)
    x = normal_features(n, 64, seed=1, dtype=torch.float16).to(DEV)
    w = kaiming_weight(27, 64, 64, seed=2, dtype=torch.float16).to(DEV)
    gy = normal_features(n, 64, seed=3, dtype=torch.float16).to(DEV)
    wd = normal_features(27, 64, seed=4, dtype=torch.float16).to(DEV)
    pts = torch.rand((200_000, 3), device=DEV, generator=torch.Generator(device=DEV).manual_seed(5)) * 4
    pf = normal_features(200_000, 16, seed=6).to(DEV)

    def run():
        km = generate_kernel_map(bc.clone(), bc.clone(), (1, 1, 1), (3, 3, 3))
        y = sparse_conv_forward(x, w, km, n)
        gx, gw = sparse_conv_backward(gy, x, w, km)
        xd = x.clone().requires_grad_(True)
        wdp = wd.clone().requires_grad_(True)
        spatially_sparse_depthwise_conv(xd, wdp, km, n).backward(gy)
        pooled = sparse_reduce(_voxels(items, x.cpu()), 2, 2, "mean").feature_tensor
        _, _, ci, co, tu = voxel_downsample_csr_mapping(pts, torch.tensor([0, 90_000, 200_000]), 0.05)
        vf = segment_reduction(pf, co, "mean", indices=ci)
        return [km.in_maps, km.out_maps, km.offsets, y, gx, gw, xd.grad, wdp.grad, pooled, ci, co,
                tu.to_unique_indices, vf]

    first, second = run(), run()
    for i, (a, b) in enumerate(zip(first, second)):
        assert torch.equal(a, b), i
