"""MinkUNet-style encoder-decoder inference (stem, strided down stages with residual blocks,
transposed up stages with skip concatenation, BN folded into conv bias, ReLU) built from the
sparse-convolution modules, bf16 and fp32.

Every convolution of the network is checked on its own: its output must match the fp64 oracle
applied to the features the GPU actually fed it (<= 1e-2 relative in bf16, <= 1e-5 in fp32), and
its coordinates / kernel map must be the oracle's.  End to end, the bf16 network must stay close
to the same network run in fp32."""
import numpy as np
import pytest
import torch

from helpers import rel_err
from warpconvnet_amd.utils import synthetic

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {torch.float32: 1e-5, torch.bfloat16: 1e-2}


class CheckedNet:
    """Tiny functional U-Net whose every sparse convolution is verified against the oracle."""

    def __init__(self, oracle, dtype, seed=0):
        from warpconvnet_amd.nn.modules.sparse_conv import SparseConv3d
        torch.manual_seed(seed)
        self.oracle, self.dtype, self.errors = oracle, dtype, []
        mk = lambda *a, **k: SparseConv3d(*a, **k).to(DEV)  # noqa: E731
        c0, c1, c2 = 16, 32, 64
        self.stem = mk(3, c0, 3)
        self.down1, self.enc1a, self.enc1b = mk(c0, c1, 2, stride=2), mk(c1, c1, 3), mk(c1, c1, 3)
        self.down2, self.enc2a, self.enc2b = mk(c1, c2, 2, stride=2), mk(c2, c2, 3), mk(c2, c2, 3)
        self.up2 = mk(c2, c1, 2, stride=2, transposed=True)
        self.dec2a, self.dec2b, self.dec2s = mk(2 * c1, c1, 3), mk(c1, c1, 3), mk(2 * c1, c1, 1)
        self.up1 = mk(c1, c0, 2, stride=2, transposed=True)
        self.dec1a, self.dec1b, self.dec1s = mk(2 * c0, c0, 3), mk(c0, c0, 3), mk(2 * c0, c0, 1)

    def conv(self, module, x, out_like=None):
        with torch.no_grad():
            y = module(x, out_like) if out_like is not None else module(x)
        if int(np.prod(module.kernel_size)) == 1:
            return y  # plain matmul shortcut, no sparse machinery
        in_bc = x.batch_indexed_coordinates.cpu().numpy()
        out_bc = y.batch_indexed_coordinates.cpu().numpy()
        ks, st = module.kernel_size, module.stride
        if module.transposed:  # forward map of the matching strided conv, in/out exchanged
            om, im, off, _ = self.oracle.kernel_map(out_bc, in_bc, ks, st)
            iden = None
        else:
            im, om, off, iden = self.oracle.kernel_map(in_bc, out_bc, ks, st)
        w = module.weight.detach().to(self.dtype).double().cpu().numpy()
        want = self.oracle.explicit_conv_f64(x.feature_tensor.double().cpu().numpy(), w, im, om, off,
                                             iden, len(out_bc))
        want = want + module.bias.detach().to(self.dtype).double().cpu().numpy()
        self.errors.append(rel_err(y.feature_tensor.double().cpu().numpy(), want))
        return y

    @staticmethod
    def relu(x):
        return x.replace(batched_features=torch.relu(x.feature_tensor))

    def block(self, x, a, b, shortcut=None):
        y = self.relu(self.conv(a, x))
        y = self.conv(b, y)
        skip = x if shortcut is None else self.conv(shortcut, x)
        return self.relu(y.replace(batched_features=y.feature_tensor + skip.feature_tensor))

    @staticmethod
    def cat(a, b):
        return a.replace(batched_features=torch.cat([a.feature_tensor, b.feature_tensor], dim=1))

    def forward(self, x):
        s0 = self.relu(self.conv(self.stem, x))
        s1 = self.block(self.relu(self.conv(self.down1, s0)), self.enc1a, self.enc1b)
        s2 = self.block(self.relu(self.conv(self.down2, s1)), self.enc2a, self.enc2b)
        u1 = self.relu(self.conv(self.up2, s2, s1))
        u1 = self.block(self.cat(u1, s1), self.dec2a, self.dec2b, self.dec2s)
        u0 = self.relu(self.conv(self.up1, u1, s0))
        return self.block(self.cat(u0, s0), self.dec1a, self.dec1b, self.dec1s)


def _input(dtype):
    from warpconvnet_amd.geometry.types.voxels import Voxels
    items = [synthetic.indoor_scene(40 + b, 12_000, 0.05) for b in range(2)]
    offsets = np.zeros(3, dtype=np.int64)
    offsets[1:] = np.cumsum([len(i) for i in items])
    n = int(offsets[-1])
    feats = torch.randn(n, 3, generator=torch.Generator().manual_seed(9)).to(dtype)
    coords = torch.as_tensor(np.concatenate(items), dtype=torch.int32, device=DEV)
    return Voxels(coords, feats.to(DEV), offsets=torch.as_tensor(offsets))


def test_unet_every_layer_matches_oracle(oracle):
    outs = {}
    for dtype in (torch.float32, torch.bfloat16):
        net = CheckedNet(oracle, dtype, seed=3)
        if dtype != torch.float32:
            for m in vars(net).values():
                if isinstance(m, torch.nn.Module):
                    m.to(dtype)
        x = _input(dtype)
        y = net.forward(x)
        assert len(net.errors) == 13  # sparse convolutions checked (the two 1x1 shortcuts are dense)
        assert max(net.errors) <= TOL[dtype], (dtype, net.errors)
        assert y.feature_tensor.shape == (len(x), 16) and y.feature_tensor.dtype == dtype
        assert torch.equal(y.coordinate_tensor, x.coordinate_tensor)
        assert y.tensor_stride in (None, (1, 1, 1))
        # one map per resolution and kind: 3^3 at three levels, two strided, two transposed
        assert len(x.cache) == 7
        outs[dtype] = y.feature_tensor.double().cpu().numpy()
    assert rel_err(outs[torch.bfloat16], outs[torch.float32]) <= 6e-2


# ------------------------------------------------------------------------------------------------
# The benchmark's network (configs[3]): stem 3x3x3 C = 32, four down stages (32, 64, 128, 256) with
# two residual blocks each, four up stages with skip concatenation and 1x1 shortcuts, bf16.
# ------------------------------------------------------------------------------------------------

def _baseline_net(dtype):
    from bench import _UNet
    return _UNet(torch.device(DEV), dtype, seed=5)


def _conv_modules(net):
    mods = [net.stem] + list(net.down) + list(net.up)
    for stage in net.enc_blocks + net.dec_blocks:
        for blk in stage:
            mods.extend(m for m in blk if m is not None)
    return mods


def _wrap_every_conv(net, check):
    """Every convolution module of the network reports (module, input, output) to `check`."""
    for m in _conv_modules(net):
        plain = m.forward

        def checked(x, *rest, _m=m, _plain=plain, **extras):
            y = _plain(x, *rest, **extras)
            check(_m, x, y, extras)
            return y

        m.forward = checked


def _voxels_of(items, channels, dtype, seed):
    from warpconvnet_amd.geometry.types.voxels import Voxels
    offsets = np.zeros(len(items) + 1, dtype=np.int64)
    offsets[1:] = np.cumsum([len(i) for i in items])
    feats = torch.randn(int(offsets[-1]), channels, generator=torch.Generator().manual_seed(seed)).to(dtype)
    coords = torch.as_tensor(np.concatenate(items), dtype=torch.int32, device=DEV)
    return Voxels(coords, feats.to(DEV), offsets=torch.as_tensor(offsets))


def _map_of(x, module, num_out):
    """The cached kernel map this layer used (kept on its input tensor)."""
    hits = [km for key, km in x.cache.items()
            if key.kernel_size == tuple(module.kernel_size) and key.transposed == bool(module.transposed)
            and int(key.out_offsets[-1]) == num_out]
    assert len(hits) == 1, (module, len(hits))
    return hits[0]


def test_baseline_unet_every_layer_matches_oracle(oracle):
    """configs[3] at a size the CPU oracle finishes: every sparse convolution's kernel map is the
    oracle's bit for bit (native order) and its output matches the fp64 oracle applied to the
    features the GPU fed it (<= 1e-2 relative, bf16)."""
    dtype = torch.bfloat16
    net = _baseline_net(dtype)
    errors, maps = [], []

    def check(m, x, y, extras):
        if int(np.prod(m.kernel_size)) == 1:
            return
        in_bc = x.batch_indexed_coordinates.cpu().numpy()
        out_bc = y.batch_indexed_coordinates.cpu().numpy()
        if m.transposed:
            om, im, off, iden = oracle.kernel_map(out_bc, in_bc, m.kernel_size, m.stride)
            iden = None
        else:
            im, om, off, iden = oracle.kernel_map(in_bc, out_bc, m.kernel_size, m.stride)
        km = _map_of(x, m, len(out_bc))
        assert np.array_equal(km.in_maps.cpu().numpy(), im) and np.array_equal(km.out_maps.cpu().numpy(), om)
        assert np.array_equal(km.offsets.numpy().astype(np.int64), off)
        maps.append(id(km))
        w = m.weight.detach().to(dtype).double().cpu().numpy()
        want = oracle.explicit_conv_f64(x.feature_tensor.double().cpu().numpy(), w, im, om, off, iden, len(out_bc))
        want = want + m.bias.detach().to(dtype).double().cpu().numpy()
        # the block's shortcut and the ReLU ride in the convolution's epilogue
        if extras.get("residual") is not None:
            want = want + extras["residual"].feature_tensor.double().cpu().numpy()
            fused.append("residual")
        if extras.get("relu"):
            want = np.maximum(want, 0.0)
            fused.append("relu")
        errors.append(rel_err(y.feature_tensor.double().cpu().numpy(), want))

    fused = []
    _wrap_every_conv(net, check)
    x = _voxels_of([synthetic.indoor_scene(60 + b, 15_000, 0.05) for b in range(4)], 3, dtype, seed=12)
    y = net(x)
    assert len(errors) == 41  # sparse convolutions; the four 1x1 shortcuts are dense products
    assert max(errors) <= 1e-2, errors
    assert fused.count("relu") == 41 and fused.count("residual") == 16  # every block's second convolution
    assert len(set(maps)) == 13  # 3^3 maps at five resolutions, four strided, four transposed
    assert y.feature_tensor.shape == (len(x), 32) and y.feature_tensor.dtype == dtype
    assert torch.equal(y.coordinate_tensor, x.coordinate_tensor)
    assert bool(torch.isfinite(y.feature_tensor).all())


def test_fused_epilogues_give_the_network_of_separate_elementwise_kernels():
    """The same network with ReLU and the blocks' shortcuts as torch operations after every
    convolution (one more rounding each): the outputs agree to bf16 accuracy over the depth of
    the network."""
    from bench import _UNet
    dtype = torch.bfloat16
    x = _voxels_of([synthetic.indoor_scene(70 + b, 12_000, 0.05) for b in range(2)], 3, dtype, seed=13)
    fused = _UNet(torch.device(DEV), dtype, seed=5, fused=True)(x).feature_tensor.float()
    plain = _UNet(torch.device(DEV), dtype, seed=5, fused=False)(x).feature_tensor.float()
    assert float((fused - plain).abs().max()) <= 3e-2 * float(plain.abs().max())
    assert bool((fused >= 0).all())


def test_baseline_unet_full_size_every_layer_matches_plain_torch():
    """configs[3] at its full size (4 x 250k voxels, bf16): every sparse convolution against the
    per-offset gather-GEMM-scatter written with plain torch fp32 operations on the same GPU, over
    the layer's own kernel map (<= 1e-2 relative), plus the maps' invariants."""
    from test_gpu_fullsize import torch_explicit_fp32
    dtype = torch.bfloat16
    net = _baseline_net(dtype)
    errors, seen = [], {}

    def check(m, x, y, extras):
        if int(np.prod(m.kernel_size)) == 1:
            return
        n_in, n_out = len(x), len(y)
        km = _map_of(x, m, n_out)
        if id(km) not in seen:
            seen[id(km)] = True
            K = len(km)
            assert int(km.in_maps.max()) < n_in and int(km.out_maps.max()) < n_out
            assert int(km.in_maps.min()) >= 0 and int(km.out_maps.min()) >= 0
            counts = torch.diff(km.offsets)
            if K == 27:  # a stride-1 map of a coordinate set onto itself: centre = identity, mirror symmetry
                ar = torch.arange(n_in, dtype=torch.int32, device=DEV)
                assert km.identity_map_index == 13
                assert torch.equal(km[13][0], ar) and torch.equal(km[13][1], ar)
                assert torch.equal(counts, counts.flip(0))
            elif not m.transposed:  # 2x2x2 stride 2: every fine voxel has exactly one coarse parent
                assert int(km.offsets[-1]) == n_in
                assert torch.equal(torch.sort(km.in_maps).values, torch.arange(n_in, dtype=torch.int32, device=DEV))
            else:                   # its exchange: every fine output row appears exactly once
                assert int(km.offsets[-1]) == n_out
                assert torch.equal(torch.sort(km.out_maps).values, torch.arange(n_out, dtype=torch.int32, device=DEV))
        w = m.weight.detach().to(dtype)
        want = torch_explicit_fp32(x.feature_tensor, w, km, n_out) + m.bias.detach().to(dtype).float()
        if extras.get("residual") is not None:
            want = want + extras["residual"].feature_tensor.float()
        if extras.get("relu"):
            want = torch.relu(want)
        scale = float(want.abs().max())
        errors.append(float((y.feature_tensor.float() - want).abs().max()) / max(scale, 1e-30))

    _wrap_every_conv(net, check)
    items, _ = synthetic.indoor_batch(4, 250_000, 0.02, seed=0)
    x = _voxels_of(items, 3, dtype, seed=11)
    y = net(x)
    assert len(errors) == 41 and len(seen) == 13
    assert max(errors) <= 1e-2, errors
    assert y.feature_tensor.shape == (len(x), 32) and bool(torch.isfinite(y.feature_tensor).all())
