#!/usr/bin/env python3
"""Benchmark of the sparse-convolution forward hot path on one MI355X.

One step = one cold pass of the path over the resident synthetic batch: kernel-map build
(coordinate table + count + fill) followed by the feature contraction of a 3x3x3, 64 -> 64 fp16
convolution on 4 indoor scenes x 250k voxels.  Inputs (coordinates, features, weights) are in
HBM before the timed region starts.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline]
"""
import argparse
import gc
import ctypes
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X published HBM3E bandwidth
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X published dense fp16 MFMA rate

# Bytes the contraction kernel moves between L2 and the memory fabric per launch on this workload
# come from the committed counter summary (two `rocprofv3 --pmc` runs of this script: FETCH_SIZE,
# then WRITE_SIZE, each scaled by what the same counter reads for the 1 GiB device copy of
# --calibrate-copy).  The summary names the kernel it was taken from; a line for another kernel
# than the one this run launches is reported as stale (traffic: null).
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "conv_fwd_cfg2_hbm_traffic.txt")
MAP_TRAFFIC_FILE = os.path.join(ROOT, "profiles", "kernel_map_cfg2_hbm_traffic.txt")


def measured_traffic(path, kernel):
    """(bytes per launch or None, note) from the line `TRAFFIC_JSON: {...}` of a counter summary;
    `kernel` is what this run launched (the library says), and a summary taken from another kernel
    is reported as stale."""
    try:
        with open(path) as f:
            for line in f:
                if line.startswith("TRAFFIC_JSON:"):
                    rec = json.loads(line[len("TRAFFIC_JSON:"):])
                    if rec.get("kernel") != kernel:
                        return None, f"stale: {os.path.basename(path)} holds {rec.get('kernel')}, this run launched {kernel}"
                    total = (rec["fetch_kib"] * rec["fetch_factor"] + rec["write_kib"] * rec["write_factor"]) * 1024
                    return float(total), f"{os.path.basename(path)} (tree {rec.get('tree', '?')})"
    except (OSError, ValueError, KeyError):
        pass
    return None, "no counter summary found"


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def measured_peaks(dev):
    """What this GPU reaches on two plain library operations, beside the published peaks: a 1 GiB
    device copy (bytes read + written per second) and an 8192^3 fp16 GEMM."""
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    a = torch.randn(8192, 8192, device=dev, dtype=torch.float16)
    b = torch.randn(8192, 8192, device=dev, dtype=torch.float16)
    out = {}
    for name, fn, work in (("stream_copy_GBps", lambda: dst.copy_(src), 2.0 * (1 << 30) / 1e9),
                           ("fp16_gemm_8192_TFLOPs", lambda: torch.matmul(a, b), 2.0 * 8192 ** 3 / 1e12)):
        for _ in range(3):
            fn()
        times = []
        for _ in range(10):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            torch.cuda.synchronize()
            times.append(e0.elapsed_time(e1) * 1e-3)
        out[name] = work / float(np.median(times))
    del src, dst, a, b
    return out


METRIC = "voxels/sec, 3x3x3 C64->64 fp16 conv @1M voxels; kernel-map build ms"


def make_workload(batch=4, per_item=250_000, c_in=64, c_out=64, seed=0):
    from warpconvnet_amd.utils import synthetic
    items, offsets = synthetic.indoor_batch(batch, per_item, 0.02, seed=seed)
    bcoords = synthetic.batch_indexed(items)
    n = len(bcoords)
    g = torch.Generator().manual_seed(seed)
    feats = torch.randn(n, c_in, generator=g).to(torch.float16)
    weight = (torch.randn(27, c_in, c_out, generator=g) * (2.0 / (c_in * 27)) ** 0.5).to(torch.float16)
    return bcoords, offsets, feats, weight


def _cpu_kernel_map_by_item(bcoords, threads):
    """The scalar C oracle's kernel map, one batch item per host thread (the items are independent:
    a pair never crosses items), merged into one map."""
    from concurrent.futures import ThreadPoolExecutor
    from oracle import cpu_oracle
    batch = bcoords[:, 0]
    bounds = np.flatnonzero(np.diff(batch)) + 1
    starts = np.concatenate([[0], bounds, [len(bcoords)]])
    parts = [np.ascontiguousarray(bcoords[a:b]) for a, b in zip(starts[:-1], starts[1:])]
    with ThreadPoolExecutor(max_workers=max(1, min(threads, len(parts)))) as pool:
        maps = list(pool.map(lambda c: cpu_oracle.kernel_map(c, c, (3, 3, 3)), parts))
    K = len(maps[0][2]) - 1
    ins, outs, off = [], [], [0]
    for k in range(K):
        for (im, om, o, _), base in zip(maps, starts[:-1]):
            ins.append(im[o[k]:o[k + 1]] + base)
            outs.append(om[o[k]:o[k + 1]] + base)
        off.append(off[-1] + sum(int(m[2][k + 1] - m[2][k]) for m in maps))
    return (np.concatenate(ins).astype(np.int32), np.concatenate(outs).astype(np.int32),
            np.asarray(off, dtype=np.int64), maps[0][3])


def cpu_baseline(bcoords, feats, weight):
    """The reference's explicit gather-GEMM-scatter algorithm (torch-CPU restatement, computed in
    fp32 through the reference's own compute_dtype knob) on the host cores, with the kernel map
    from the scalar C oracle.  Full workload, one pass each, twice: on all host threads (the map
    one batch item per thread) and on a single thread."""
    from oracle import cpu_oracle
    from oracle.explicit_conv import explicit_gemm_forward
    threads = os.cpu_count() or 1
    threads = min(threads, int(os.environ.get("OMP_NUM_THREADS", threads)))
    n = len(bcoords)
    # single thread
    torch.set_num_threads(1)
    t0 = time.perf_counter()
    im, om, off, iden = cpu_oracle.kernel_map(bcoords, bcoords, (3, 3, 3))
    t_map1 = time.perf_counter() - t0
    im_t, om_t = torch.as_tensor(im), torch.as_tensor(om)
    t0 = time.perf_counter()
    explicit_gemm_forward(feats, weight, im_t, om_t, off, iden, n, compute_dtype=torch.float32)
    t_conv1 = time.perf_counter() - t0
    # all threads
    torch.set_num_threads(threads)
    t0 = time.perf_counter()
    im_p, om_p, off_p, iden_p = _cpu_kernel_map_by_item(bcoords, threads)
    t_map = time.perf_counter() - t0
    assert iden_p == iden and np.array_equal(off_p, off) and np.array_equal(im_p, im) and np.array_equal(om_p, om)
    explicit_gemm_forward(feats[:1000], weight, im_t[:0], om_t[:0], [0] * 28, None, 1000,
                          compute_dtype=torch.float32)  # warm the thread pool
    t0 = time.perf_counter()
    out = explicit_gemm_forward(feats, weight, im_t, om_t, off, iden, n, compute_dtype=torch.float32)
    t_conv = time.perf_counter() - t0
    return {
        "value": n / (t_map + t_conv),
        "unit": "voxels/s",
        "cores": threads,
        "kind": "port",
        "cpu": cpu_model(),
        "sample": (f"full workload once: {n} voxels, {int(off[-1])} pairs; kernel map by the scalar "
                   f"C oracle, one batch item per thread ({t_map * 1e3:.0f} ms) + explicit "
                   f"gather-GEMM-scatter in torch fp32 on {threads} threads ({t_conv * 1e3:.0f} ms)"),
        "map_ms": t_map * 1e3,
        "conv_ms": t_conv * 1e3,
        "single_thread": {"value": n / (t_map1 + t_conv1), "unit": "voxels/s", "cores": 1,
                          "map_ms": t_map1 * 1e3, "conv_ms": t_conv1 * 1e3},
    }, out, (im, om, off)


def secondary_configs(dev, steps, warmup):
    """The other single-layer configurations (parity-test cases; reported under config.other_configs
    with --all-configs, never as the headline value): cold map build + contraction per step."""
    from warpconvnet_amd._lib import lib
    from warpconvnet_amd.geometry.coords.ops.stride import stride_coords
    from warpconvnet_amd.geometry.coords.search.search_results import IntSearchResult
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    from warpconvnet_amd.nn.functional.sparse_conv import sparse_conv_forward
    from warpconvnet_amd.utils import synthetic

    def timed(fn):
        for _ in range(warmup):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(steps):
            r = fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps, r

    def weights(K, ci, co, dtype, seed):
        g = torch.Generator().manual_seed(seed)
        return (torch.randn(K, ci, co, generator=g) * (2.0 / (ci * K)) ** 0.5).to(dtype).to(dev)

    def single(name, bc, ksize, ci, co, dtype, out):
        c = torch.as_tensor(bc, device=dev)
        n = len(bc)
        K = int(np.prod(ksize))
        x = torch.randn(n, ci, generator=torch.Generator().manual_seed(1)).to(dtype).to(dev)
        w = weights(K, ci, co, dtype, 2)
        def cold_map():
            cold = c.view(-1, 4)  # a new tensor object: the coordinate table is built again
            return generate_kernel_map(cold, cold, (1, 1, 1), ksize)

        t_map, km = timed(cold_map)
        t_conv, _ = timed(lambda: sparse_conv_forward(x, w, km, n))
        L = int(km.offsets[-1])
        out[name] = {"num_voxels": n, "num_pairs": L, "kernel_map_build_ms": t_map,
                     "contraction_call_ms": t_conv, "voxels_per_s": n / ((t_map + t_conv) * 1e-3),
                     "contraction_TFLOPs": 2.0 * L * ci * co / (t_conv * 1e-3) / 1e12}

    out = {}
    single("configs[0]: 3x3x3 32->32 fp32, 100k voxels on 3 spheres",
           synthetic.batch_indexed([synthetic.spheres_scene(0, 100_000, 0.01)]), (3, 3, 3), 32, 32,
           torch.float32, out)
    items, _ = synthetic.indoor_batch(4, 250_000, 0.02, seed=0)
    bc = synthetic.batch_indexed(items)
    single("configs[4a]: 5x5x5 16->16 fp16, 1M voxels", bc, (5, 5, 5), 16, 16, torch.float16, out)
    coarse_items = [synthetic.indoor_scene(b, None, 0.16) for b in range(4)]
    single("configs[4b]: 3x3x3 256->256 fp16, 16 cm voxels", synthetic.batch_indexed(coarse_items),
           (3, 3, 3), 256, 256, torch.float16, out)
    # configs[2]: 2x2x2 stride-2 96 -> 128 and its transposed 128 -> 96, bf16, 1M fine voxels
    c = torch.as_tensor(bc, device=dev)
    n = len(bc)
    x = torch.randn(n, 96, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16).to(dev)
    wd, wu = weights(8, 96, 128, torch.bfloat16, 4), weights(8, 128, 96, torch.bfloat16, 5)

    def build():
        cold = c.view(-1, 4)
        coarse, _ = stride_coords(cold, (2, 2, 2))
        return coarse, generate_kernel_map(cold, coarse, (2, 2, 2), (2, 2, 2))

    t_map, (coarse, km) = timed(build)
    m = len(coarse)
    t_down, y = timed(lambda: sparse_conv_forward(x, wd, km, m))
    # the transposed convolution's map as spatially_sparse_conv makes it: the forward map with its lists
    # exchanged; kernel = stride over voxels without repeats, so every fine voxel has exactly one pair
    up = IntSearchResult(km.out_maps, km.in_maps, km.offsets)
    up._in_ascend, up._in_group_start = km._out_ascend, km._group_start
    up._keys_unique, up._from_builder = km._keys_unique, True
    up._single_out = bool(km._keys_unique and int(km.offsets[-1]) == n)
    t_up, y_up = timed(lambda: sparse_conv_forward(y, wu, up, n))
    # the same product by the general path (lists re-ordered once, sums in LDS), for comparison
    up_general = IntSearchResult(km.out_maps, km.in_maps, km.offsets)
    up_general._keys_unique, up_general._from_builder = km._keys_unique, True
    t_up_general, y_general = timed(lambda: sparse_conv_forward(y, wu, up_general, n))
    assert float((y_up.float() - y_general.float()).abs().max()) <= 2e-2 * float(y_general.float().abs().max())
    # the same two paths over the same map for other channel counts (whole calls, warm map)
    up_shapes = {}
    for c_coarse, c_fine in ((32, 32), (64, 32), (256, 128)):
        ys = torch.randn(m, c_coarse, generator=torch.Generator().manual_seed(9)).to(torch.bfloat16).to(dev)
        ws = weights(8, c_coarse, c_fine, torch.bfloat16, 10)
        t_single, _ = timed(lambda: sparse_conv_forward(ys, ws, up, n))
        kernel_single = lib().wcn_conv_last_kernel().decode()
        t_general, _ = timed(lambda: sparse_conv_forward(ys, ws, up_general, n))
        up_shapes[f"{c_coarse}->{c_fine}"] = {"one_pair_per_row_call_ms": t_single, "kernel": kernel_single,
                                              "general_path_call_ms": t_general,
                                              "general_path_kernel": lib().wcn_conv_last_kernel().decode()}
    # consumers of the same maps: depthwise 3x3x3 over the 1M-voxel map, 2x2x2 stride-2 max pooling
    from warpconvnet_amd.nn.functional.sparse_conv_depth import spatially_sparse_depthwise_conv
    km3 = generate_kernel_map(c, c, (1, 1, 1), (3, 3, 3))
    xdw = torch.randn(n, 64, generator=torch.Generator().manual_seed(7)).to(torch.float16).to(dev)
    wdw = (torch.randn(27, 64, generator=torch.Generator().manual_seed(8)) * 0.2).to(torch.float16).to(dev)
    with torch.no_grad():
        t_dw, _ = timed(lambda: spatially_sparse_depthwise_conv(xdw, wdw, km3, n))
    L3 = int(km3.offsets[-1])
    out["depthwise 3x3x3 over the configs[1] map, 64 channels fp16 (warm map)"] = {
        "num_voxels": n, "num_pairs": L3, "call_ms": t_dw,
        "gathered_GBps": 2 * 64 * (L3 + n) / (t_dw * 1e-3) / 1e9}
    del km3
    # a consumer of the same strided map: 2x2x2 stride-2 max pooling of 64 fp16 channels
    from warpconvnet_amd.nn.functional.sparse_pool import _SparsePoolFunction
    xp = torch.randn(n, 64, generator=torch.Generator().manual_seed(6)).to(torch.float16).to(dev)
    t_pool, _ = timed(lambda: _SparsePoolFunction.apply(xp, km, m, 2))
    pool_bytes = 2 * 64 * (n + m) + 4 * (n + m)
    out["max pooling 2x2x2 s2 over the configs[2] map, 64 channels fp16 (warm map)"] = {
        "num_voxels": n, "num_coarse": m, "call_ms": t_pool,
        "algorithmic_GBps": pool_bytes / (t_pool * 1e-3) / 1e9}
    # the step before the path: 4 x 1M points -> voxels of 2 cm with the mean of 32 fp16 channels,
    # beside the torch ops the reference composes for it (voxel.py:92-100, unique.py:84-100)
    from warpconvnet_amd.geometry.coords.ops.voxel import voxel_downsample_csr_mapping
    from warpconvnet_amd.ops.reductions import segment_reduction
    gp = torch.Generator(device=dev).manual_seed(7)
    npts = 4_000_000
    pts = torch.rand((npts, 3), device=dev, generator=gp) * torch.tensor([8.0, 8.0, 0.1], device=dev)
    poffsets = torch.tensor([0, 1_000_000, 2_000_000, 3_000_000, npts])
    pfeat = torch.randn((npts, 32), device=dev, generator=gp).to(torch.float16)

    def voxelize():
        _, _, ci, co, _ = voxel_downsample_csr_mapping(pts, poffsets, 0.02)
        return segment_reduction(pfeat, co, "mean", indices=ci)

    def voxelize_torch_ops():
        rows = torch.cat([torch.searchsorted(poffsets[1:].to(dev), torch.arange(npts, device=dev),
                                             right=True).int().unsqueeze(1),
                          torch.floor(pts / 0.02).int()], dim=1)
        u, inv, cnt = torch.unique(rows, dim=0, sorted=True, return_inverse=True, return_counts=True)
        order = inv.argsort(stable=True)
        sums = torch.zeros((len(u), 32), device=dev).index_add_(0, inv, pfeat.float())
        return (sums / cnt[:, None]).half(), order

    t_vox, vox = timed(voxelize)
    t_vox_torch, _ = timed(voxelize_torch_ops)
    mvox = len(vox)
    # points read, (key, index) pairs written and read, grouping and distinct rows written, features gathered
    vox_bytes = 12 * npts + 2 * 8 * npts + 8 * npts + (8 + 8 + 16) * mvox + 2 * 32 * (npts + mvox) + 8 * npts
    out["points -> voxels: 4 x 1M points, 2 cm voxels, mean of 32 fp16 channels"] = {
        "num_points": npts, "num_voxels": mvox, "call_ms": t_vox, "points_per_s": npts / (t_vox * 1e-3),
        "algorithmic_GBps": vox_bytes / (t_vox * 1e-3) / 1e9, "same_result_with_torch_ops_ms": t_vox_torch}
    del pts, pfeat, vox
    # the reference's own standard fixture (tests/nn/test_sparse_conv.py:35-47): three clouds of
    # randint(1e5, 1e6) points in [0, 100)^3 made unique, 16 channels; cold map + contraction of
    # the two convolutions its tests run (3x3x3 stride 2 16 -> 13 fp32, 3x3x3 stride 1 16 -> 16 fp16)
    from warpconvnet_amd.geometry.types.voxels import Voxels
    torch.manual_seed(0)
    Ns = torch.randint(100000, 1000000, (3,))
    fix = Voxels([(torch.rand((int(N), 3)) / 0.01).int() for N in Ns],
                 [torch.rand((int(N), 16)) for N in Ns], device=dev).unique()
    fc = fix.batch_indexed_coordinates.contiguous()
    nf = fc.shape[0]
    w13 = weights(27, 16, 13, torch.float32, 9)
    w16 = weights(27, 16, 16, torch.float16, 10)
    xf32, xf16 = fix.feature_tensor.float().contiguous(), fix.feature_tensor.half().contiguous()

    def fixture_s2():
        cold = fc.view(-1, 4)
        coarse, _ = stride_coords(cold, (2, 2, 2))
        return coarse, generate_kernel_map(cold, coarse, (2, 2, 2), (3, 3, 3))

    def fixture_s1():
        cold = fc.view(-1, 4)
        return generate_kernel_map(cold, cold, (1, 1, 1), (3, 3, 3))

    t_map2, (fcoarse, fkm2) = timed(fixture_s2)
    t_conv2, _ = timed(lambda: sparse_conv_forward(xf32, w13, fkm2, len(fcoarse)))
    t_map1, fkm1 = timed(fixture_s1)
    t_conv1, _ = timed(lambda: sparse_conv_forward(xf16, w16, fkm1, nf))
    out["reference fixture (tests/nn/test_sparse_conv.py:35-47): 3 clouds in [0,100)^3, 16 channels"] = {
        "num_voxels": nf, "occupancy_of_cells": nf / 3e6,
        "3x3x3 s2 16->13 fp32": {"num_out": len(fcoarse), "num_pairs": int(fkm2.offsets[-1]),
                                 "pairs_per_out_voxel": int(fkm2.offsets[-1]) / len(fcoarse),
                                 "coords_and_kernel_map_build_ms": t_map2, "contraction_call_ms": t_conv2},
        "3x3x3 s1 16->16 fp16": {"num_pairs": int(fkm1.offsets[-1]), "pairs_per_voxel": int(fkm1.offsets[-1]) / nf,
                                 "kernel_map_build_ms": t_map1, "contraction_call_ms": t_conv1}}
    del fix, fkm1, fkm2
    out["configs[2]: 2x2x2 s2 96->128 + transposed 128->96 bf16, 1M fine voxels"] = {
        "num_voxels": n, "num_coarse": m, "num_pairs": int(km.offsets[-1]),
        "coords_and_kernel_map_build_ms": t_map, "down_contraction_call_ms": t_down,
        "up_contraction_call_ms": t_up, "up_contraction_call_general_path_ms": t_up_general,
        "up_other_channel_counts_bf16": up_shapes, "voxels_per_s": n / ((t_map + t_down + t_up) * 1e-3)}
    return out


class _UNet:
    """configs[3]: MinkUNet18-style encoder-decoder for inference: 3x3x3 stem (C = 32), four down
    stages (32, 64, 128, 256: 2x2x2 stride-2 convolution + two residual blocks of two 3x3x3
    convolutions) and four up stages (transposed 2x2x2 stride-2 convolution, skip concatenation,
    two residual blocks, 1x1 shortcut where the channel count changes).  Batch norm is folded into
    the convolutions' weight and bias; ReLU and the residual adds ride in the convolutions'
    epilogues (`fused=False`: as torch elementwise ops after every convolution).  The weights do
    not change between passes, so the layers keep the kernels' tiles of their weight
    (`keep_tiles=False`: made again by one more kernel in every call)."""

    def __init__(self, dev, dtype, seed=0, fused=True, keep_tiles=True):
        from warpconvnet_amd.nn.modules.sparse_conv import SparseConv3d
        self.fused = fused
        torch.manual_seed(seed)

        def mk(*a, **k):
            conv = SparseConv3d(*a, bias=True, **k).to(dev).to(dtype)
            conv.keep_prepared_weight = keep_tiles
            return conv

        enc = (32, 64, 128, 256)
        self.stem = mk(3, 32, 3)
        self.down, self.enc_blocks = [], []
        prev = 32
        for ch in enc:
            self.down.append(mk(prev, ch, 2, stride=2))
            self.enc_blocks.append([(mk(ch, ch, 3), mk(ch, ch, 3), None) for _ in range(2)])
            prev = ch
        skips = (128, 64, 32, 32)  # channels of the encoder level each up stage lands on
        self.up, self.dec_blocks = [], []
        for ch in skips:
            self.up.append(mk(prev, ch, 2, stride=2, transposed=True))
            self.dec_blocks.append([(mk(2 * ch, ch, 3), mk(ch, ch, 3), mk(2 * ch, ch, 1)),
                                    (mk(ch, ch, 3), mk(ch, ch, 3), None)])
            prev = ch

    @staticmethod
    def _relu(x):
        return x.replace(batched_features=torch.relu(x.feature_tensor))

    def _conv_relu(self, conv, x, out=None, residual=None):
        if self.fused:
            return conv(x, out, residual=residual, relu=True)
        y = conv(x, out)
        if residual is not None:
            y = y.replace(batched_features=y.feature_tensor + residual.feature_tensor)
        return self._relu(y)

    def _block(self, x, blk):
        a, b, shortcut = blk
        skip = x if shortcut is None else shortcut(x)
        return self._conv_relu(b, self._conv_relu(a, x), residual=skip)

    @torch.no_grad()
    def __call__(self, x):
        levels = [self._conv_relu(self.stem, x)]
        for down, blocks in zip(self.down, self.enc_blocks):
            y = self._conv_relu(down, levels[-1])
            for blk in blocks:
                y = self._block(y, blk)
            levels.append(y)
        y = levels.pop()
        for up, blocks in zip(self.up, self.dec_blocks):
            skip = levels.pop()
            y = self._conv_relu(up, y, skip)
            y = y.replace(batched_features=torch.cat([y.feature_tensor, skip.feature_tensor], dim=1))
            for blk in blocks:
                y = self._block(y, blk)
        return y


def unet_config(dev, steps, warmup, compare=True):
    """One inference pass per step over a fresh Voxels (every kernel map is rebuilt, as for a new
    input): 4 x 250k voxels, 3-channel features, bf16, random-init weights.  `compare`: the same
    network timed again with the weights' tiles made in every call, and the outputs compared."""
    from warpconvnet_amd.geometry.types.voxels import Voxels
    from warpconvnet_amd.utils import synthetic
    items, offsets = synthetic.indoor_batch(4, 250_000, 0.02, seed=0)
    coords = torch.as_tensor(np.concatenate(items), dtype=torch.int32, device=dev)
    n = coords.shape[0]
    feats = torch.randn(n, 3, generator=torch.Generator().manual_seed(11)).to(torch.bfloat16).to(dev)
    def timed(net):
        def run():
            return net(Voxels(coords, feats, offsets=torch.as_tensor(np.asarray(offsets))))

        for _ in range(warmup):
            out = run()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            out = run()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps, out

    net = _UNet(dev, torch.bfloat16)
    ms, out = timed(net)
    assert out.feature_tensor.shape == (n, 32) and bool(torch.isfinite(out.feature_tensor).all())
    extra = {}
    if compare:
        ms_every_call, out_every_call = timed(_UNet(dev, torch.bfloat16, keep_tiles=False))
        assert torch.equal(out.feature_tensor, out_every_call.feature_tensor)
        extra["ms_per_pass_weight_tiles_made_in_every_call"] = ms_every_call
    convs = [net.stem] + net.down + net.up + [m for stage in net.enc_blocks + net.dec_blocks
                                             for blk in stage for m in blk if m is not None]
    sparse = sum(1 for m in convs if int(np.prod(m.kernel_size)) > 1)
    return {"num_voxels": n, "sparse_convolutions": sparse, "pointwise_convolutions": len(convs) - sparse,
            "ms_per_pass": ms, **extra,
            "voxels_per_s": n / (ms * 1e-3)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # the GPU's clocks settle over the first few dozen steps of a fresh process (the same kernels
    # run ~8 % slower in steps 5..25 than in steps 45..65), hence the generous default warm-up
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--backward", action="store_true",
                    help="also time the gradients of the same convolution (reported under config.backward; "
                         "the headline value stays the forward path)")
    ap.add_argument("--all-configs", action="store_true",
                    help="also time the other single-layer configurations (config.other_configs)")
    ap.add_argument("--network-only", action="store_true",
                    help="run nothing but passes of configs[3]'s network (--steps of them after --warmup) and "
                         "print their timing: the command to put under a profiler for a pass's kernels")
    ap.add_argument("--gather-floor", action="store_true",
                    help="also time a kernel that only gathers the map's rows (roofline.gather_floor)")
    ap.add_argument("--sorted-voxels", action="store_true",
                    help="also time the same step on the voxels sorted along a Morton curve, and the sort "
                         "(config.morton_sorted)")
    ap.add_argument("--sizes", action="store_true",
                    help="also time the same layer on 16 and 64 scenes (4 M and 16 M voxels)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 1 GiB device copy (reference point for rocprofv3 byte counters)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this path is built and measured on a single MI355X; "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    from warpconvnet_amd._lib import lib, stream_ptr
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    from warpconvnet_amd.nn.functional.sparse_conv import sparse_conv_forward

    dev = torch.device("cuda:0")
    if args.network_only:
        print(json.dumps({"configs[3]: MinkUNet18-style encoder-decoder, bf16, 1M voxels":
                          unet_config(dev, args.steps, args.warmup, compare=False)}))
        return
    bcoords, offsets, feats, weight = make_workload()
    n = len(bcoords)
    coords_d = torch.as_tensor(bcoords, device=dev)
    feats_d = feats.to(dev)
    weight_d = weight.to(dev)
    L = lib()

    def step(time_kernel=None, probes=True):
        cold = coords_d.view(-1, 4)  # a new tensor object: no coordinate table is kept on it yet
        km = generate_kernel_map(cold, cold, (1, 1, 1), (3, 3, 3))
        mid = None
        if probes:
            mid = torch.cuda.Event(enable_timing=True)
            mid.record()
        if time_kernel is not None:
            L.wcn_conv_set_timing_events(ctypes.c_void_p(time_kernel[0].cuda_event),
                                         ctypes.c_void_p(time_kernel[1].cuda_event))
        out = sparse_conv_forward(feats_d, weight_d, km, n)
        return km, out, mid

    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    def run_steps(count, probes):
        """`count` steps back to back between two synchronisations; wall time and the events.
        The contraction kernel is bracketed by events in every step; with `probes` every step also
        records where it starts, where the map is done and where it ends (three more event
        commands per step on the stream)."""
        kernel_events = []
        for _ in range(count):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()  # creates the underlying hipEvent_t; re-recorded by the library
            b.record()
            kernel_events.append((a, b))
        starts = [torch.cuda.Event(enable_timing=True) for _ in range(count)]
        ends = [torch.cuda.Event(enable_timing=True) for _ in range(count)]
        mids = []
        last = None
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(count):
            if probes:
                starts[i].record()
            km, out, mid = step(kernel_events[i], probes)
            if probes:
                ends[i].record()
            mids.append(mid)
            last = (km, out)
        torch.cuda.synchronize()
        return time.perf_counter() - t0, starts, mids, ends, kernel_events, last

    # The warm-up steps go through the very code of the timed ones (events included): the first
    # pass through it in a process has cost a single stall of tens of milliseconds on a fresh machine.
    if args.warmup > 0:
        run_steps(args.warmup, False)
    # As timeit does: no collection of the interpreter's garbage inside the timed region (a full
    # collection of a heap with torch loaded takes tens of milliseconds, dozens of steps).
    gc.collect()
    gc.disable()
    try:
        elapsed, _, _, _, kernel_events, (km, out) = run_steps(args.steps, False)
        # the split into map build and contraction call comes from a second pass of the same
        # steps with the three extra events per step
        _, starts, mids, ends, _, _ = run_steps(args.steps, True)
    finally:
        gc.enable()

    ms_per_step = elapsed * 1e3 / args.steps
    # medians over the steps (the wall-clock figure above is the mean of the same K steps)
    map_ms = float(np.median([s.elapsed_time(m) for s, m in zip(starts, mids)]))
    conv_call_ms = float(np.median([m.elapsed_time(e) for m, e in zip(mids, ends)]))
    conv_kernel_ms = float(np.median([a.elapsed_time(b) for a, b in kernel_events]))
    step_device_ms = float(np.median([s.elapsed_time(e) for s, e in zip(starts, ends)]))

    # The same cold step through the module interface: SpatiallySparseConv.forward on a Voxels
    # object made anew in every step (no cached table or map), as a caller of the reference does.
    from warpconvnet_amd.geometry.types.voxels import Voxels
    from warpconvnet_amd.nn.modules.sparse_conv import SparseConv3d
    module = SparseConv3d(64, 64, 3, bias=False).to(dev).half()
    with torch.no_grad():
        module.weight.copy_(weight_d)
    offsets_t = torch.as_tensor(np.asarray(offsets, dtype=np.int64))
    coords3 = coords_d[:, 1:].contiguous()

    def module_step():
        vox = Voxels(coords3.view(-1, 3), feats_d, offsets=offsets_t)
        with torch.no_grad():
            return module(vox)

    for _ in range(min(args.warmup, 20)):
        module_step()
    torch.cuda.synchronize()
    gc.collect()
    gc.disable()
    try:
        t0 = time.perf_counter()
        for _ in range(args.steps):
            mod_out = module_step()
        torch.cuda.synchronize()
        module_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    finally:
        gc.enable()
    module_max_diff = float((mod_out.feature_tensor.float() - out.float()).abs().max())
    # the same with the weight's tiles kept on the parameter (an option for weights that stay put:
    # the call then enqueues the contraction alone); reported beside, never as the headline value
    module.keep_prepared_weight = True
    for _ in range(5):
        module_step()
    torch.cuda.synchronize()
    gc.collect()
    gc.disable()
    try:
        t0 = time.perf_counter()
        for _ in range(args.steps):
            kept_out = module_step()
        torch.cuda.synchronize()
        module_kept_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    finally:
        gc.enable()
    assert torch.equal(kept_out.feature_tensor, mod_out.feature_tensor)
    # The same steps from several host threads, each with a stream of its own (a server that has
    # more than one batch in hand): one thread's map build overlaps another's contraction.  Reported
    # beside the headline, which stays one step after the other on one stream.
    import threading

    def steps_on(stream, count, outs):
        with torch.cuda.stream(stream):
            for _ in range(count):
                _, o, _ = step(probes=False)
            outs.append(o)
            stream.synchronize()
        L.wcn_thread_release()  # this thread's pinned mailbox and events

    concurrent = {}
    for threads in (2, 4):
        streams = [torch.cuda.Stream() for _ in range(threads)]
        for timed in (False, True):
            outs = []
            workers = [threading.Thread(target=steps_on, args=(st, args.steps if timed else 10, outs))
                       for st in streams]
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for w in workers:
                w.start()
            for w in workers:
                w.join()
            torch.cuda.synchronize()
            elapsed_c = time.perf_counter() - t0
        assert len(outs) == threads and all(torch.equal(o, out) for o in outs)  # no thread gave up
        concurrent[f"{threads} streams"] = {
            "ms_per_step": elapsed_c * 1e3 / (threads * args.steps),
            "voxels_per_s": n * threads * args.steps / elapsed_c}
    if os.environ.get("WCN_BENCH_TRACE"):  # per-step device times, for looking into an odd average
        for i in range(args.steps):
            print(f"step {i}: map {starts[i].elapsed_time(mids[i]):.3f} ms, contraction call "
                  f"{mids[i].elapsed_time(ends[i]):.3f} ms, kernel "
                  f"{kernel_events[i][0].elapsed_time(kernel_events[i][1]):.3f} ms", file=sys.stderr)

    conv_kernel = L.wcn_conv_last_kernel().decode()  # this thread's last contraction: the timed one
    num_pairs = int(km.offsets[-1])
    c_in, c_out, K, s = 64, 64, 27, 2
    conv_bytes = s * (n * c_in + n * c_out + K * c_in * c_out) + 8 * num_pairs
    conv_flops = 2.0 * num_pairs * c_in * c_out
    cap = 2 * n
    map_bytes = 24 * n + 8 * cap + 16 * n + 8 * K * n + 8 * num_pairs
    achieved = conv_bytes / (conv_kernel_ms * 1e-3) / 1e9
    traffic_bytes, traffic_note = measured_traffic(TRAFFIC_FILE, conv_kernel)
    map_kernels = ("kmap_pass_fixed<3, 3, 3>" if os.environ.get("WCN_KMAP_PROBE") != "blocks" else "self_probe<1>")
    map_traffic_bytes, map_traffic_note = measured_traffic(MAP_TRAFFIC_FILE, map_kernels)

    result = {
        "metric": METRIC,
        "value": n / (ms_per_step * 1e-3),
        "unit": "voxels/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": ("configs[1]: SpatiallySparseConv 3x3x3 stride 1, C 64->64, fp16, batch 4 x "
                         "250k voxels of seeded indoor scenes at 2 cm; each step builds the kernel "
                         "map from scratch and runs the contraction"),
            "num_voxels": n,
            "num_pairs": num_pairs,
            "timing": "ms_per_step: wall clock over the K steps / K; the *_ms fields below: medians over the steps of device-event intervals",
            "step_device_ms": step_device_ms,
            "kernel_map_build_ms": map_ms,
            "contraction_call_ms": conv_call_ms,
            "contraction_kernel_ms": conv_kernel_ms,
            "module_forward_ms": module_ms,
            "module_forward_kept_weight_tiles_ms": module_kept_ms,
            "module_forward_note": ("SparseConv3d.forward on a Voxels object made anew per step (cold table and "
                                    "map, cache lookups, output Voxels); wall clock / K; max |difference| to the "
                                    f"direct path's output: {module_max_diff:.3g}"),
            "steps_from_concurrent_host_threads": concurrent,
            "steps_from_concurrent_host_threads_note": (
                "K steps from each of 2 / 4 host threads, each thread on a stream of its own: one thread's map "
                "build overlaps another's contraction; wall clock over all the steps; outputs equal to the "
                "headline's.  The headline value is one step after the other on one stream"),
            "kernel_map_algorithmic_GBps": map_bytes / (map_ms * 1e-3) / 1e9,
            "kernel_map_frac_of_hbm_peak": map_bytes / (map_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "contraction_TFLOPs": conv_flops / (conv_kernel_ms * 1e-3) / 1e12,
            "contraction_frac_of_mfma_peak": conv_flops / (conv_kernel_ms * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS,
        },
        "roofline": {
            "kernel": conv_kernel,
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": traffic_bytes,
            "traffic_source": traffic_note,
            "algorithmic_bytes": conv_bytes,
            "measured_peaks": measured_peaks(dev),
            # the second half of the metric as a roofline line of its own: all kernels of the map
            # build together (table: hist, colscan, scatter, bins; map: probe, scan, emit) against
            # the bytes the survey's formula prices for it
            "map_build": {
                "kernel": "table_hist + table_colscan + table_scatter + table_bins + " + map_kernels
                          + " + kmap_scan_rows + " + ("kmap_emit_flat" if "kmap_pass" in map_kernels else "self_count + self_emit"),
                "probe_kernel": map_kernels,
                "bound": "hbm",
                "achieved": map_bytes / (map_ms * 1e-3) / 1e9,
                "peak": HBM_PEAK_GBS,
                "unit": "GB/s",
                "frac": map_bytes / (map_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                "ms": map_ms,
                "traffic": map_traffic_bytes,
                "traffic_source": map_traffic_note,
                "algorithmic_bytes": map_bytes,
            },
        },
    }

    if args.gather_floor:
        sink = torch.zeros(64, dtype=torch.int32, device=dev)
        from warpconvnet_amd._lib import check, ptr
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(30)]
        for a, b in ev:
            a.record()
            check(L.wcn_probe_gather_rows(ptr(feats_d), n, 128, ptr(km.in_maps), num_pairs, ptr(sink),
                                          stream_ptr(dev)), "wcn_probe_gather_rows")
            b.record()
        torch.cuda.synchronize()
        floor_ms = float(np.median([a.elapsed_time(b) for a, b in ev[10:]]))
        result["roofline"]["gather_floor"] = {
            "kernel": "gather_rows_probe<8>", "ms": floor_ms,
            "gathered_GBps": num_pairs * 128 / (floor_ms * 1e-3) / 1e9,
            "note": ("a kernel that only fetches features[in_maps[p]] for every pair (128-byte rows, 16 rows per "
                     "wave and request, four requests in flight): no contraction that gathers every pair's row "
                     "from beyond the L2 runs faster than this plus the output's write")}

    if args.sorted_voxels:
        from warpconvnet_amd.geometry.coords.ops.serialization import encode
        a0, a1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        offsets_i = torch.as_tensor(np.asarray(offsets, dtype=np.int64))
        sort_ms = []
        for _ in range(5):
            a0.record()
            res = encode(coords_d[:, 1:].contiguous(), batch_offsets=offsets_i, return_perm=True)
            order = res.perm
            sorted_coords = coords_d[order.long()].contiguous()
            sorted_feats = feats_d[order.long()].contiguous()
            a1.record()
            torch.cuda.synchronize()
            sort_ms.append(a0.elapsed_time(a1))
        maps, kernels = [], []
        for _ in range(30):
            cold = sorted_coords.view(-1, 4)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            k0, k1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            k0.record(); k1.record()
            e0.record()
            km_s = generate_kernel_map(cold, cold, (1, 1, 1), (3, 3, 3))
            e1.record()
            L.wcn_conv_set_timing_events(ctypes.c_void_p(k0.cuda_event), ctypes.c_void_p(k1.cuda_event))
            sparse_conv_forward(sorted_feats, weight_d, km_s, n)
            torch.cuda.synchronize()
            maps.append(e0.elapsed_time(e1))
            kernels.append(k0.elapsed_time(k1))
        result["config"]["morton_sorted"] = {
            "sort_ms": float(np.median(sort_ms)),
            "sort_note": "Morton codes + torch sorts + the permuted copies of coordinates (16 MB) and features (128 MB)",
            "kernel_map_build_ms": float(np.median(maps[10:])),
            "contraction_kernel_ms": float(np.median(kernels[10:])),
            "unsorted_kernel_map_build_ms": map_ms, "unsorted_contraction_kernel_ms": conv_kernel_ms}

    if args.sizes:
        larger = {}
        for batch in (16, 64):
            bc, _, f, _ = make_workload(batch=batch, seed=1)
            big_coords = torch.as_tensor(bc, device=dev)
            big_feats = f.to(dev)
            m = len(bc)
            maps, kernels = [], []
            for _ in range(12):
                cold = big_coords.view(-1, 4)
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                k0, k1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                k0.record(); k1.record()
                e0.record()
                km_b = generate_kernel_map(cold, cold, (1, 1, 1), (3, 3, 3))
                e1.record()
                L.wcn_conv_set_timing_events(ctypes.c_void_p(k0.cuda_event), ctypes.c_void_p(k1.cuda_event))
                sparse_conv_forward(big_feats, weight_d, km_b, m)
                torch.cuda.synchronize()
                maps.append(e0.elapsed_time(e1))
                kernels.append(k0.elapsed_time(k1))
            map_b, conv_b = float(np.median(maps[4:])), float(np.median(kernels[4:]))
            larger[f"{batch} scenes"] = {
                "num_voxels": m, "num_pairs": int(km_b.offsets[-1]),
                "kernel_map_build_ms": map_b, "contraction_kernel_ms": conv_b,
                "voxels_per_s_map_plus_kernel": m / ((map_b + conv_b) * 1e-3),
                "kernel": L.wcn_conv_last_kernel().decode()}
            del big_coords, big_feats, km_b
        result["config"]["larger_batches"] = larger

    if args.backward:
        from warpconvnet_amd.nn.functional.sparse_conv import sparse_conv_backward
        gy = torch.randn(n, c_out, device=dev).to(torch.float16)
        w32 = weight_d.float()  # parameters are fp32 in training; the weight gradient comes back in fp32
        times = {}
        for name, kw in (("dgrad", dict(need_weight_grad=False)), ("wgrad", dict(need_input_grad=False))):
            for _ in range(args.warmup):
                sparse_conv_backward(gy, feats_d, w32, km, **kw)
            a0, a1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            a0.record()
            for _ in range(args.steps):
                sparse_conv_backward(gy, feats_d, w32, km, **kw)
            a1.record()
            torch.cuda.synchronize()
            times[name] = a0.elapsed_time(a1) / args.steps
        wgrad_bytes = s * (n * c_in + n * c_out) + 8 * num_pairs + 4 * K * c_in * c_out
        wgrad_flops = 2.0 * (num_pairs + n) * c_in * c_out  # the identity offset runs over all rows
        result["config"]["backward"] = {
            "dgrad_call_ms": times["dgrad"],
            "wgrad_call_ms": times["wgrad"],
            "dgrad_algorithmic_GBps": conv_bytes / (times["dgrad"] * 1e-3) / 1e9,
            "wgrad_algorithmic_GBps": wgrad_bytes / (times["wgrad"] * 1e-3) / 1e9,
            "wgrad_TFLOPs": wgrad_flops / (times["wgrad"] * 1e-3) / 1e12,
            "note": "warm kernel map (the forward's), fp32 weights, whole calls incl. weight preparation",
        }

    if args.all_configs:
        result["config"]["other_configs"] = secondary_configs(dev, max(3, args.steps // 2), 2)
        result["config"]["other_configs"]["configs[3]: MinkUNet18-style encoder-decoder, bf16, 1M voxels"] = \
            unet_config(dev, max(3, args.steps // 4), 2)

    if not args.no_cpu_baseline:
        base, ref_out, _ = cpu_baseline(bcoords, feats, weight)
        result["cpu_baseline"] = base
        got = out.float().cpu()
        err = float((got - ref_out.float()).abs().max() / ref_out.float().abs().max())
        result["config"]["max_rel_err_vs_cpu_baseline"] = err
        # entry by entry, the form the reference's native GEMM tests print (tests/csrc/test_cutlass_gemm.py:24-26),
        # over the entries above a thousandth of the largest
        ref64 = ref_out.double()
        keep = ref64.abs() > 1e-3 * ref64.abs().max()
        result["config"]["elementwise_rel_err_vs_cpu_baseline"] = float(
            ((got.double() - ref64).abs()[keep] / (ref64.abs()[keep] + 1e-6)).max())
    print(json.dumps(result))


if __name__ == "__main__":
    main()
