// Measurement probe: what the memory system delivers when the rows of a kernel map are gathered and
// nothing else is done.  Not on the product path; the benchmark uses it to put a floor under the
// contraction's run time (a kernel that gathers every pair's row cannot be faster than this).
#include "wcn_common.h"

namespace {

// A wave fetches 16 rows per request: lane = (row of the request, 16-byte piece of the row), as the
// contraction's multiplying waves do.  REQUESTS requests are in flight per wave; what arrives is
// folded into one word per lane so that the loads cannot be dropped.
template <int PIECES>  // 16-byte pieces per row: 8 for rows of 128 bytes
__global__ void __launch_bounds__(256) gather_rows_probe(const uint4* __restrict__ rows,
                                                         const int32_t* __restrict__ in_maps,
                                                         int64_t num_pairs, uint32_t* __restrict__ sink) {
  constexpr int ROWS = 64 / PIECES, REQUESTS = 4;
  const int lane = wcn_lane();
  const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const int64_t waves = ((int64_t)gridDim.x * blockDim.x) >> 6;
  const int piece = lane % PIECES, row_of_lane = lane / PIECES;
  uint32_t acc = 0;
  for (int64_t p0 = wave * ROWS * REQUESTS; p0 < num_pairs; p0 += waves * ROWS * REQUESTS) {
    int32_t r[REQUESTS];
#pragma unroll
    for (int q = 0; q < REQUESTS; ++q) {
      const int64_t p = p0 + q * ROWS + row_of_lane;
      r[q] = in_maps[p < num_pairs ? p : num_pairs - 1];
    }
    uint4 v[REQUESTS];
#pragma unroll
    for (int q = 0; q < REQUESTS; ++q) v[q] = rows[(int64_t)r[q] * PIECES + piece];
#pragma unroll
    for (int q = 0; q < REQUESTS; ++q) acc ^= v[q].x ^ v[q].y ^ v[q].z ^ v[q].w;
  }
  if (acc == 0x9e3779b9u) sink[0] = acc;  // practically never: keeps the loads alive
}

}  // namespace

extern "C" int wcn_probe_gather_rows(const void* features, int64_t num_rows, int32_t row_bytes,
                                     const int32_t* in_maps, int64_t num_pairs, void* sink,
                                     void* stream) {
  if (!features || !in_maps || !sink || num_rows <= 0 || num_pairs <= 0) return WCN_ERR_INVALID_ARGUMENT;
  if (row_bytes != 128 && row_bytes != 64 && row_bytes != 32) return WCN_ERR_INVALID_ARGUMENT;
  const int grid = 256 * 8;  // eight workgroups of four waves per CU
  hipStream_t s = (hipStream_t)stream;
  if (row_bytes == 128)
    hipLaunchKernelGGL(gather_rows_probe<8>, dim3(grid), dim3(256), 0, s, (const uint4*)features, in_maps, num_pairs, (uint32_t*)sink);
  else if (row_bytes == 64)
    hipLaunchKernelGGL(gather_rows_probe<4>, dim3(grid), dim3(256), 0, s, (const uint4*)features, in_maps, num_pairs, (uint32_t*)sink);
  else
    hipLaunchKernelGGL(gather_rows_probe<2>, dim3(grid), dim3(256), 0, s, (const uint4*)features, in_maps, num_pairs, (uint32_t*)sink);
  WCN_LAUNCH_CHECK();
  return WCN_OK;
}
