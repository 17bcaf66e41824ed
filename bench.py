#!/usr/bin/env python3
"""Benchmark of the sparse-convolution forward hot path on one MI355X.

One step = one cold pass of the path over the resident synthetic batch: kernel-map build
(coordinate table + count + fill) followed by the feature contraction of a 3x3x3, 64 -> 64 fp16
convolution on 4 indoor scenes x 250k voxels.  Inputs (coordinates, features, weights) are in
HBM before the timed region starts.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline]
"""
import argparse
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

# Bytes the contraction kernel moves between L2 and the memory fabric per launch on this workload,
# from two `rocprofv3 --pmc` runs of this script (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch),
# each scaled by what the same counter reads for the 1 GiB device copy of --calibrate-copy
# (FETCH_SIZE reads 0.5 GiB for it -> x2.0; WRITE_SIZE reads 1 GiB -> x1.0).  Summary kept in
# profiles/conv_fwd_cfg2_hbm_traffic.txt; to be re-measured whenever the kernel changes.
CONV_FWD_TRAFFIC_BYTES = (282586 * 2.0 + 160172 * 1.0) * 1024

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


def cpu_baseline(bcoords, feats, weight):
    """The reference's explicit gather-GEMM-scatter algorithm (torch-CPU restatement, computed in
    fp32 through the reference's own compute_dtype knob) on the host cores, with the kernel map
    from the scalar C oracle.  Full workload, one pass each."""
    from oracle import cpu_oracle
    from oracle.explicit_conv import explicit_gemm_forward
    threads = os.cpu_count() or 1
    threads = min(threads, int(os.environ.get("OMP_NUM_THREADS", threads)))
    torch.set_num_threads(threads)
    t0 = time.perf_counter()
    im, om, off, iden = cpu_oracle.kernel_map(bcoords, bcoords, (3, 3, 3))
    t_map = time.perf_counter() - t0
    im_t, om_t = torch.as_tensor(im), torch.as_tensor(om)
    n = len(bcoords)
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
        "sample": (f"full workload once: {n} voxels, {int(off[-1])} pairs; kernel map by the scalar "
                   f"C oracle on 1 thread ({t_map * 1e3:.0f} ms) + explicit gather-GEMM-scatter in "
                   f"torch fp32 on {threads} threads ({t_conv * 1e3:.0f} ms)"),
        "map_ms": t_map * 1e3,
        "conv_ms": t_conv * 1e3,
    }, out, (im, om, off)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--backward", action="store_true",
                    help="also time the gradients of the same convolution (reported under config.backward; "
                         "the headline value stays the forward path)")
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
    bcoords, offsets, feats, weight = make_workload()
    n = len(bcoords)
    coords_d = torch.as_tensor(bcoords, device=dev)
    feats_d = feats.to(dev)
    weight_d = weight.to(dev)
    L = lib()

    def step(time_kernel=None):
        km = generate_kernel_map(coords_d, coords_d, (1, 1, 1), (3, 3, 3))
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

    for _ in range(args.warmup):
        km, out, _ = step()
    torch.cuda.synchronize()

    kernel_events = []
    for _ in range(args.steps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()  # creates the underlying hipEvent_t; re-recorded by the library
        b.record()
        kernel_events.append((a, b))
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    mids = []
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        starts[i].record()
        km, out, mid = step(kernel_events[i])
        ends[i].record()
        mids.append(mid)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0

    ms_per_step = elapsed * 1e3 / args.steps
    map_ms = float(np.mean([s.elapsed_time(m) for s, m in zip(starts, mids)]))
    conv_call_ms = float(np.mean([m.elapsed_time(e) for m, e in zip(mids, ends)]))
    conv_kernel_ms = float(np.mean([a.elapsed_time(b) for a, b in kernel_events]))

    num_pairs = int(km.offsets[-1])
    c_in, c_out, K, s = 64, 64, 27, 2
    conv_bytes = s * (n * c_in + n * c_out + K * c_in * c_out) + 8 * num_pairs
    conv_flops = 2.0 * num_pairs * c_in * c_out
    cap = 2 * n
    map_bytes = 24 * n + 8 * cap + 16 * n + 8 * K * n + 8 * num_pairs
    achieved = conv_bytes / (conv_kernel_ms * 1e-3) / 1e9

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
            "kernel_map_build_ms": map_ms,
            "contraction_call_ms": conv_call_ms,
            "contraction_kernel_ms": conv_kernel_ms,
            "kernel_map_algorithmic_GBps": map_bytes / (map_ms * 1e-3) / 1e9,
            "kernel_map_frac_of_hbm_peak": map_bytes / (map_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "contraction_TFLOPs": conv_flops / (conv_kernel_ms * 1e-3) / 1e12,
            "contraction_frac_of_mfma_peak": conv_flops / (conv_kernel_ms * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS,
        },
        "roofline": {
            "kernel": "conv_fwd_ring<f16, 6>",
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": CONV_FWD_TRAFFIC_BYTES,
            "algorithmic_bytes": conv_bytes,
        },
    }

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

    if not args.no_cpu_baseline:
        base, ref_out, _ = cpu_baseline(bcoords, feats, weight)
        result["cpu_baseline"] = base
        got = out.float().cpu()
        err = float((got - ref_out.float()).abs().max() / ref_out.float().abs().max())
        result["config"]["max_rel_err_vs_cpu_baseline"] = err
    print(json.dumps(result))


if __name__ == "__main__":
    main()
