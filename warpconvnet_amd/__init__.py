"""MI355X-native sparse-convolution forward path with WarpConvNet's Python interface.

The device work (coordinate table, kernel map, strided coordinates, MFMA feature contraction) is
done by hand-written HIP kernels for gfx950 in libwcn_hip.so, called through a C ABI with ctypes;
this package is the host-side mirror of the reference's modules for that path:

    warpconvnet_amd.geometry.types.voxels.Voxels
    warpconvnet_amd.geometry.coords.search.torch_hashmap.TorchHashTable
    warpconvnet_amd.geometry.coords.search.torch_discrete.generate_kernel_map
    warpconvnet_amd.geometry.coords.ops.stride.stride_coords
    warpconvnet_amd.nn.functional.sparse_conv.spatially_sparse_conv
    warpconvnet_amd.nn.modules.sparse_conv.SpatiallySparseConv / SparseConv3d

There is no CPU fallback: every device entry point raises if the HIP library is missing.
"""
__version__ = "0.1.0"
