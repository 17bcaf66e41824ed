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
