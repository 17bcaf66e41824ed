// Space-filling-curve codes of voxel coordinates (gfx950).  Replaces the CuPy launches of
// warpconvnet/csrc/morton_code.cu (assign_order_discrete_20bit_kernel_4points) behind
// warpconvnet/geometry/coords/ops/serialization.py:234-254.
//
//   code = spread(c[a2] - origin[a2]) << 2 | spread(c[a1] - origin[a1]) << 1 | spread(c[a0] - origin[a0])
//
// where spread() puts two zero bits between consecutive bits of its argument (21 bits kept) and
// (a0, a1, a2) is the axis permutation of the ordering (x, y, z for MORTON_XYZ).  One thread per
// row, 12 bytes read and 8 written: a pure streaming pass.
#include "wcn_common.h"

namespace {

__device__ __forceinline__ unsigned long long spread_by_3(unsigned long long n) {
  n &= 0x1FFFFFull;
  n = (n | (n << 32)) & 0x001F00000000FFFFull;
  n = (n | (n << 16)) & 0x001F0000FF0000FFull;
  n = (n | (n << 8)) & 0x100F00F00F00F00Full;
  n = (n | (n << 4)) & 0x10C30C30C30C30C3ull;
  n = (n | (n << 2)) & 0x1249249249249249ull;
  return n;
}

__global__ void __launch_bounds__(256) morton_codes(const int32_t* __restrict__ coords, int64_t n,
                                                    int columns, int first_spatial,
                                                    const int32_t* __restrict__ origin, int a0, int a1,
                                                    int a2, int64_t* __restrict__ codes) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int32_t* row = coords + i * columns + first_spatial;
  const unsigned long long x = (unsigned long long)(uint32_t)(row[a0] - origin[a0]);
  const unsigned long long y = (unsigned long long)(uint32_t)(row[a1] - origin[a1]);
  const unsigned long long z = (unsigned long long)(uint32_t)(row[a2] - origin[a2]);
  codes[i] = (int64_t)((spread_by_3(z) << 2) | (spread_by_3(y) << 1) | spread_by_3(x));
}

}  // namespace

extern "C" {

int wcn_morton_codes(const int32_t* coords, int64_t n, int32_t columns, int32_t first_spatial,
                     const int32_t* device_origin, const int32_t host_axes[3], int64_t* codes,
                     void* stream) {
  if (n < 0 || columns < 3 || first_spatial < 0 || first_spatial + 3 > columns || !host_axes)
    return WCN_ERR_INVALID_ARGUMENT;
  bool seen[3] = {false, false, false};
  for (int d = 0; d < 3; ++d) {
    if (host_axes[d] < 0 || host_axes[d] > 2 || seen[host_axes[d]]) return WCN_ERR_INVALID_ARGUMENT;
    seen[host_axes[d]] = true;
  }
  if (n == 0) return WCN_OK;
  if (!coords || !device_origin || !codes) return WCN_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(morton_codes, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     coords, n, columns, first_spatial, device_origin, host_axes[0], host_axes[1],
                     host_axes[2], codes);
  WCN_LAUNCH_CHECK();
  return WCN_OK;
}

}  // extern "C"
