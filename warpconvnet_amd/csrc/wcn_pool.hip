// Pooling over a kernel map (gfx950): every output row is the sum / mean / maximum of the input
// rows its pairs name (reference: warpconvnet/nn/functional/sparse_pool.py:25-120, which sorts
// the pairs by output row with torch and reduces the segments with torch_scatter.segment_csr).
//
// The pairs are first put in output-row form (wcn_rows_build: row_ptr / row_in, the kernels the
// contraction uses to re-order lists), then one thread per (output row, 16 bytes of channels)
// walks the row's input rows with fp32 accumulators and writes its piece once: no atomics, every
// feature row read in whole 16-byte pieces, the output written once.  HBM-bound:
// s * C * (L + M) + 4 (L + M) bytes.
//
// The gradient runs the same walk over the map with in and out exchanged: the gradient of an
// input row is the sum over its pairs of the output row's gradient (divided by the output row's
// pair count for the mean; only where the input row was the maximum for max).
#include <algorithm>

#include "wcn_common.h"
#include "wcn_mma.h"

namespace {

using namespace wcn_mma;

enum { POOL_SUM = 0, POOL_MEAN = 1, POOL_MAX = 2, POOL_MIN = 3 };

template <typename T>
struct Piece {  // 16 bytes of channels
  static constexpr int N = 16 / sizeof(T);
  T v[N];
};

// One 16-byte piece of row `row`, channels c0 .. c0 + N - 1 (zeros past the last channel; rows
// whose byte length is not a multiple of 16 are read element by element).
template <typename T>
__device__ __forceinline__ void load_piece(const T* __restrict__ base, int64_t row, int channels, int c0,
                                           bool vec, float* out) {
  constexpr int N = Piece<T>::N;
  const T* src = base + row * channels + c0;
  if (vec) {
    const u32x4 raw = *reinterpret_cast<const u32x4*>(src);
    const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
    for (int j = 0; j < N; ++j) out[j] = to_float(e[j]);
  } else {
#pragma unroll
    for (int j = 0; j < N; ++j) out[j] = c0 + j < channels ? to_float(src[j]) : 0.f;
  }
}

template <typename T>
__device__ __forceinline__ void store_piece(T* __restrict__ base, int64_t row, int channels, int c0,
                                            bool vec, const float* val) {
  constexpr int N = Piece<T>::N;
  T* dst = base + row * channels + c0;
  if (vec) {
    Piece<T> p;
#pragma unroll
    for (int j = 0; j < N; ++j) p.v[j] = from_float<T>(val[j]);
    *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(&p);
  } else {
#pragma unroll
    for (int j = 0; j < N; ++j)
      if (c0 + j < channels) dst[j] = from_float<T>(val[j]);
  }
}

// out[m] = reduce over row_in[row_ptr[m] .. row_ptr[m+1]) of X[.]; rows without pairs become 0
// (sparse_pool.py:92-104).  For the maximum / minimum, arg[m][c] is the input row that supplied it
// (the first one in the row's order among equals), -1 for rows without pairs.
template <typename T>
__global__ void __launch_bounds__(256) pool_fwd(const T* __restrict__ X, int64_t num_in, int channels,
                                                const int32_t* __restrict__ row_ptr,
                                                const int32_t* __restrict__ row_in, int64_t num_out,
                                                int mode, bool vec, T* __restrict__ out,
                                                int32_t* __restrict__ arg) {
  constexpr int N = Piece<T>::N;
  const int pieces = (channels + N - 1) / N;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= num_out * pieces) return;
  const int64_t m = i / pieces;
  const int c0 = (int)(i % pieces) * N;
  const int begin = row_ptr[m], end = row_ptr[m + 1];
  float acc[N];
  int32_t who[N];
#pragma unroll
  for (int j = 0; j < N; ++j) {
    acc[j] = 0.f;
    who[j] = -1;
  }
  for (int e = begin; e < end; ++e) {
    const int32_t r = row_in[e];
    if ((uint32_t)r >= (uint64_t)num_in) continue;
    float x[N];
    load_piece<T>(X, r, channels, c0, vec, x);
    if (mode >= POOL_MAX) {
      const float sign = mode == POOL_MAX ? 1.f : -1.f;  // the minimum is the maximum of -x
#pragma unroll
      for (int j = 0; j < N; ++j) {
        const bool better = who[j] < 0 || sign * x[j] > sign * acc[j];
        acc[j] = better ? x[j] : acc[j];
        who[j] = better ? r : who[j];
      }
    } else {
#pragma unroll
      for (int j = 0; j < N; ++j) acc[j] += x[j];
    }
  }
  if (mode == POOL_MEAN && end > begin) {
    const float inv = 1.f / (float)(end - begin);
#pragma unroll
    for (int j = 0; j < N; ++j) acc[j] *= inv;
  }
  store_piece<T>(out, m, channels, c0, vec, acc);
  if (mode >= POOL_MAX && arg) {
#pragma unroll
    for (int j = 0; j < N; ++j)
      if (c0 + j < channels) arg[m * channels + c0 + j] = who[j];
  }
}

// dX[n] = sum over the pairs (n, m) of input row n of dY[m] (sum), dY[m] / count[m] (mean), or
// dY[m] where arg[m][c] == n (max).  `row_ptr` / `row_in` are the rows form of the exchanged map
// (rows = input rows, entries = output rows); out_ptr is the row_ptr of the forward rows form
// (pair count of every output row), used by the mean.
template <typename T>
__global__ void __launch_bounds__(256) pool_bwd(const T* __restrict__ dY, int64_t num_out, int channels,
                                                const int32_t* __restrict__ row_ptr,
                                                const int32_t* __restrict__ row_in, int64_t num_in,
                                                int mode, bool vec, const int32_t* __restrict__ out_ptr,
                                                const int32_t* __restrict__ arg, T* __restrict__ dX) {
  constexpr int N = Piece<T>::N;
  const int pieces = (channels + N - 1) / N;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= num_in * pieces) return;
  const int64_t n = i / pieces;
  const int c0 = (int)(i % pieces) * N;
  float acc[N];
#pragma unroll
  for (int j = 0; j < N; ++j) acc[j] = 0.f;
  for (int e = row_ptr[n]; e < row_ptr[n + 1]; ++e) {
    const int32_t m = row_in[e];
    if ((uint32_t)m >= (uint64_t)num_out) continue;
    float g[N];
    load_piece<T>(dY, m, channels, c0, vec, g);
    if (mode == POOL_MEAN) {
      const int cnt = out_ptr[m + 1] - out_ptr[m];
      const float inv = cnt > 0 ? 1.f / (float)cnt : 0.f;
#pragma unroll
      for (int j = 0; j < N; ++j) acc[j] += g[j] * inv;
    } else if (mode >= POOL_MAX) {
#pragma unroll
      for (int j = 0; j < N; ++j)
        if (c0 + j < channels && arg[(int64_t)m * channels + c0 + j] == (int32_t)n) acc[j] += g[j];
    } else {
#pragma unroll
      for (int j = 0; j < N; ++j) acc[j] += g[j];
    }
  }
  store_piece<T>(dX, n, channels, c0, vec, acc);
}

// ---- reduction over CSR segments (the point -> voxel pooling) -----------------------------------
//
//   out[u] = reduce over e in [offsets[u], offsets[u+1]) of X[indices ? indices[e] : e]
//
// (reference: warpconvnet/ops/reductions.py:36-72, torch_scatter.segment_csr over features that
// were gathered with features[to_csr_indices] first; here the gather is part of the walk, so the
// gathered copy is never written).  Offsets and indices are 64-bit, as torch.unique and argsort
// return them.  arg[u][c] = the input row that supplied the extremum.
template <typename T>
__global__ void __launch_bounds__(256) segment_reduce(const T* __restrict__ X, int64_t num_in, int channels,
                                                      const int64_t* __restrict__ offsets,
                                                      const int64_t* __restrict__ indices,
                                                      int64_t num_entries, int64_t num_out, int mode,
                                                      bool vec, T* __restrict__ out,
                                                      int64_t* __restrict__ arg) {
  constexpr int N = Piece<T>::N;
  const int pieces = (channels + N - 1) / N;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= num_out * pieces) return;
  const int64_t u = i / pieces;
  const int c0 = (int)(i % pieces) * N;
  // offsets that do not fit the entry list are cut to it: nothing is read past its end
  int64_t begin = offsets[u], end = offsets[u + 1];
  begin = begin < 0 ? 0 : begin;
  end = end > num_entries ? num_entries : end;
  float acc[N];
  int64_t who[N];
#pragma unroll
  for (int j = 0; j < N; ++j) {
    acc[j] = 0.f;
    who[j] = -1;
  }
  for (int64_t e = begin; e < end; ++e) {
    const int64_t r = indices ? indices[e] : e;
    if ((uint64_t)r >= (uint64_t)num_in) continue;
    float x[N];
    load_piece<T>(X, r, channels, c0, vec, x);
    if (mode >= POOL_MAX) {
      const float sign = mode == POOL_MAX ? 1.f : -1.f;
#pragma unroll
      for (int j = 0; j < N; ++j) {
        const bool better = who[j] < 0 || sign * x[j] > sign * acc[j];
        acc[j] = better ? x[j] : acc[j];
        who[j] = better ? r : who[j];
      }
    } else {
#pragma unroll
      for (int j = 0; j < N; ++j) acc[j] += x[j];
    }
  }
  if (mode == POOL_MEAN && end > begin) {
    const float inv = 1.f / (float)(end - begin);
#pragma unroll
    for (int j = 0; j < N; ++j) acc[j] *= inv;
  }
  store_piece<T>(out, u, channels, c0, vec, acc);
  if (mode >= POOL_MAX && arg) {
#pragma unroll
    for (int j = 0; j < N; ++j)
      if (c0 + j < channels) arg[u * channels + c0 + j] = who[j];
  }
}

// Every input row lies in at most one segment: dX[n] = dY[u] (sum), dY[u] / count[u] (mean),
// dY[u] where arg[u][c] == n (max, min), with u = segment_of[n]; 0 for rows outside every segment.
template <typename T>
__global__ void __launch_bounds__(256) segment_reduce_bwd(const T* __restrict__ dY, int64_t num_out,
                                                          int channels, const int64_t* __restrict__ offsets,
                                                          const int64_t* __restrict__ segment_of,
                                                          int64_t num_in, int mode, bool vec,
                                                          const int64_t* __restrict__ arg,
                                                          T* __restrict__ dX) {
  constexpr int N = Piece<T>::N;
  const int pieces = (channels + N - 1) / N;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= num_in * pieces) return;
  const int64_t n = i / pieces;
  const int c0 = (int)(i % pieces) * N;
  float acc[N];
#pragma unroll
  for (int j = 0; j < N; ++j) acc[j] = 0.f;
  const int64_t u = segment_of[n];
  if ((uint64_t)u < (uint64_t)num_out) {
    float g[N];
    load_piece<T>(dY, u, channels, c0, vec, g);
    if (mode == POOL_MEAN) {
      const int64_t cnt = offsets[u + 1] - offsets[u];
      const float inv = cnt > 0 ? 1.f / (float)cnt : 0.f;
#pragma unroll
      for (int j = 0; j < N; ++j) acc[j] = g[j] * inv;
    } else if (mode >= POOL_MAX) {
#pragma unroll
      for (int j = 0; j < N; ++j)
        if (c0 + j < channels && arg[u * channels + c0 + j] == n) acc[j] = g[j];
    } else {
#pragma unroll
      for (int j = 0; j < N; ++j) acc[j] = g[j];
    }
  }
  store_piece<T>(dX, n, channels, c0, vec, acc);
}

// ---- depthwise convolution over the same rows form ---------------------------------------------
//
//   out[m][c] = sum over the pairs (n, m) of offset k of X[n][c] * W[k][c]
//
// (reference: warpconvnet/nn/functional/sparse_conv_depth.py:151-182).  The set bits of
// row_mask[m] name the offsets of the row's entries in order, which selects the weight row.  With
// an identity offset that offset is X[m] * W[identity] for every m < rows_in and its pairs are
// ignored (sparse_conv_depth.py:163-165).  The input gradient is the same walk over the exchanged
// map with dY in place of X.
template <typename T, typename WT>
__global__ void __launch_bounds__(256) depthwise_fwd(const T* __restrict__ X, int64_t num_in, int channels,
                                                     const WT* __restrict__ W, int K, int identity,
                                                     const uint32_t* __restrict__ row_mask, int words,
                                                     const int32_t* __restrict__ row_ptr,
                                                     const int32_t* __restrict__ row_in, int64_t num_out,
                                                     bool vec, T* __restrict__ out) {
  constexpr int N = Piece<T>::N;
  const int pieces = (channels + N - 1) / N;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= num_out * pieces) return;
  const int64_t m = i / pieces;
  const int c0 = (int)(i % pieces) * N;
  float acc[N];
#pragma unroll
  for (int j = 0; j < N; ++j) acc[j] = 0.f;
  auto add = [&](int64_t r, int k) {
    float x[N];
    load_piece<T>(X, r, channels, c0, vec, x);
#pragma unroll
    for (int j = 0; j < N; ++j)
      if (c0 + j < channels) acc[j] += x[j] * to_float(W[(int64_t)k * channels + c0 + j]);
  };
  if (identity >= 0 && m < num_in) add(m, identity);
  int e = row_ptr[m];
  for (int w = 0; w < words; ++w) {
    uint32_t bits = row_mask[m * words + w];
    while (bits) {
      const int k = w * 32 + __builtin_ctz(bits);
      bits &= bits - 1u;
      const int32_t r = row_in[e++];
      if (k == identity || (uint32_t)r >= (uint64_t)num_in) continue;
      add(r, k);
    }
  }
  store_piece<T>(out, m, channels, c0, vec, acc);
}

// dW[k][c] = sum over the pairs of offset k of X[in][c] * dY[out][c]; a workgroup owns a chunk of
// the pairs of one offset and writes one partial row; the chunks of an offset are added in order.
constexpr int DW_CHUNK = 2048;  // pairs per workgroup

__global__ void __launch_bounds__(64) depthwise_plan(const int64_t* __restrict__ offsets, int K, int identity,
                                                     int64_t identity_rows, int32_t* __restrict__ chunk_first) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  int32_t run = 0;
  for (int k = 0; k < K; ++k) {
    chunk_first[k] = run;
    const int64_t n = k == identity ? identity_rows : offsets[k + 1] - offsets[k];
    run += (int32_t)((n + DW_CHUNK - 1) / DW_CHUNK);
  }
  chunk_first[K] = run;
}

template <typename T>
__global__ void __launch_bounds__(256) depthwise_wgrad(const T* __restrict__ X, int64_t num_in,
                                                       const T* __restrict__ dY, int64_t num_out,
                                                       int channels, const int32_t* __restrict__ in_maps,
                                                       const int32_t* __restrict__ out_maps,
                                                       const int64_t* __restrict__ offsets,
                                                       const int32_t* __restrict__ chunk_first, int K,
                                                       int identity, int64_t identity_rows, bool vec,
                                                       float* __restrict__ partial) {
  constexpr int N = Piece<T>::N;
  __shared__ float s_sum[256][N + 1];
  const int chunk = blockIdx.x;
  int lo = 0, hi = K;  // the last k with chunk_first[k] <= chunk
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (chunk_first[mid] <= chunk) lo = mid; else hi = mid;
  }
  const int k = lo;
  const bool ident = k == identity;
  const int64_t n_k = ident ? identity_rows : offsets[k + 1] - offsets[k];
  const int64_t first = (int64_t)(chunk - chunk_first[k]) * DW_CHUNK;
  const int count = (int)(n_k - first < DW_CHUNK ? n_k - first : DW_CHUNK);
  const int64_t pbase = offsets[k] + first;
  const int pieces = (channels + N - 1) / N;
  // the 256 threads are `lanes` pairs wide and `pieces` channel pieces deep, piece by piece
  for (int p0 = 0; p0 < pieces; p0 += 256) {
    const int width = pieces - p0 < 256 ? pieces - p0 : 256;  // pieces handled in this pass
    const int lanes = 256 / width;
    const int piece = p0 + (int)threadIdx.x % width, lane = (int)threadIdx.x / width;
    const int c0 = piece * N;
    float acc[N];
#pragma unroll
    for (int j = 0; j < N; ++j) acc[j] = 0.f;
    if (lane < lanes) {
      for (int p = lane; p < count; p += lanes) {
        const int64_t rin = ident ? first + p : (int64_t)in_maps[pbase + p];
        const int64_t rout = ident ? first + p : (int64_t)out_maps[pbase + p];
        if ((uint64_t)rin >= (uint64_t)num_in || (uint64_t)rout >= (uint64_t)num_out) continue;
        float x[N], g[N];
        load_piece<T>(X, rin, channels, c0, vec, x);
        load_piece<T>(dY, rout, channels, c0, vec, g);
#pragma unroll
        for (int j = 0; j < N; ++j) acc[j] += x[j] * g[j];
      }
    }
#pragma unroll
    for (int j = 0; j < N; ++j) s_sum[threadIdx.x][j] = acc[j];
    __syncthreads();
    if (lane == 0) {  // one thread per piece adds the lanes in order
      for (int l = 1; l < lanes; ++l)
#pragma unroll
        for (int j = 0; j < N; ++j) acc[j] += s_sum[l * width + (int)threadIdx.x % width][j];
#pragma unroll
      for (int j = 0; j < N; ++j)
        if (c0 + j < channels) partial[(int64_t)chunk * channels + c0 + j] = acc[j];
    }
    __syncthreads();
  }
}

template <typename WT>
__global__ void __launch_bounds__(256) depthwise_wgrad_reduce(const float* __restrict__ partial,
                                                              const int32_t* __restrict__ chunk_first,
                                                              int K, int channels, WT* __restrict__ dW) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)K * channels) return;
  const int k = (int)(i / channels), c = (int)(i % channels);
  float sum = 0.f;
  for (int ch = chunk_first[k]; ch < chunk_first[k + 1]; ++ch) sum += partial[(int64_t)ch * channels + c];
  dW[i] = from_float<WT>(sum);
}

inline bool rows_are_vectors(const void* p, int channels, int dtype) {
  const size_t es = dtype == WCN_DTYPE_F32 ? 4 : 2;
  return ((size_t)channels * es) % 16 == 0 && ((uintptr_t)p % 16) == 0;
}

template <typename T>
void launch_pool_fwd(const void* X, int64_t num_in, int channels, const WcnRowsView& v, int64_t num_out,
                     int mode, bool vec, void* out, int32_t* arg, hipStream_t s) {
  const int pieces = (channels + Piece<T>::N - 1) / Piece<T>::N;
  const int64_t items = num_out * pieces;
  hipLaunchKernelGGL(pool_fwd<T>, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, s, (const T*)X,
                     num_in, channels, (const int32_t*)v.row_ptr, (const int32_t*)v.row_in, num_out, mode,
                     vec, (T*)out, arg);
}

template <typename T>
void launch_pool_bwd(const void* dY, int64_t num_out, int channels, const WcnRowsView& v, int64_t num_in,
                     int mode, bool vec, const int32_t* out_ptr, const int32_t* arg, void* dX,
                     hipStream_t s) {
  const int pieces = (channels + Piece<T>::N - 1) / Piece<T>::N;
  const int64_t items = num_in * pieces;
  hipLaunchKernelGGL(pool_bwd<T>, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, s, (const T*)dY,
                     num_out, channels, (const int32_t*)v.row_ptr, (const int32_t*)v.row_in, num_in, mode,
                     vec, out_ptr, arg, (T*)dX);
}

template <typename T>
void launch_segment_reduce(const void* X, int64_t num_in, int channels, const int64_t* offsets,
                           const int64_t* indices, int64_t num_entries, int64_t num_out, int mode,
                           bool vec, void* out, int64_t* arg, hipStream_t s) {
  const int pieces = (channels + Piece<T>::N - 1) / Piece<T>::N;
  const int64_t items = num_out * pieces;
  hipLaunchKernelGGL(segment_reduce<T>, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, s,
                     (const T*)X, num_in, channels, offsets, indices, num_entries, num_out, mode, vec, (T*)out,
                     arg);
}

template <typename T>
void launch_segment_reduce_bwd(const void* dY, int64_t num_out, int channels, const int64_t* offsets,
                               const int64_t* segment_of, int64_t num_in, int mode, bool vec,
                               const int64_t* arg, void* dX, hipStream_t s) {
  const int pieces = (channels + Piece<T>::N - 1) / Piece<T>::N;
  const int64_t items = num_in * pieces;
  hipLaunchKernelGGL(segment_reduce_bwd<T>, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, s,
                     (const T*)dY, num_out, channels, offsets, segment_of, num_in, mode, vec, arg, (T*)dX);
}

bool map_args_ok(const int64_t* host_offsets, int K, const int32_t* in_maps, const int32_t* out_maps,
                 int64_t* pairs) {
  if (!host_offsets || K < 1 || K > WCN_MAX_OFFSETS || host_offsets[0] != 0) return false;
  for (int k = 0; k < K; ++k)
    if (host_offsets[k + 1] < host_offsets[k]) return false;
  *pairs = host_offsets[K];
  if (*pairs > INT32_MAX) return false;
  return *pairs == 0 || (in_maps && out_maps);
}

}  // namespace

extern "C" {

size_t wcn_map_rows_workspace_bytes(int64_t num_rows, int32_t num_offsets, int64_t num_pairs) {
  if (num_rows < 0 || num_offsets < 1 || num_offsets > WCN_MAX_OFFSETS || num_pairs < 0) return 0;
  return wcn_rows_layout(nullptr, num_rows, num_offsets, num_pairs, nullptr);
}

int wcn_map_rows_build(const int32_t* gathered_rows, const int32_t* grouping_rows,
                       const int64_t* host_offsets, int32_t num_offsets, int64_t num_rows,
                       void* workspace, size_t workspace_bytes, void* stream) {
  int64_t pairs = 0;
  if (!map_args_ok(host_offsets, num_offsets, gathered_rows, grouping_rows, &pairs) || num_rows < 0 ||
      num_rows >= (1ll << 31) || !workspace)
    return WCN_ERR_INVALID_ARGUMENT;
  if (workspace_bytes < wcn_map_rows_workspace_bytes(num_rows, num_offsets, pairs))
    return WCN_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  WcnRowsView v;
  wcn_rows_layout(workspace, num_rows, num_offsets, pairs, &v);
  if (hipMemcpyAsync(v.offsets, host_offsets, sizeof(int64_t) * (size_t)(num_offsets + 1),
                     hipMemcpyHostToDevice, s) != hipSuccess)
    return WCN_ERR_LAUNCH;
  if (num_rows == 0) return WCN_OK;
  return wcn_rows_build(gathered_rows, grouping_rows, num_offsets, num_rows, pairs, v, s);
}

int wcn_sparse_pool_fwd(const void* features, int64_t num_in, int32_t channels, int32_t dtype,
                        const void* rows_by_out, int64_t num_out, int32_t num_offsets,
                        int64_t num_pairs, int32_t mode, void* out, int32_t* argmax_or_null,
                        void* stream) {
  if (dtype < 0 || dtype > 2 || mode < POOL_SUM || mode > POOL_MIN || channels < 1 || num_in < 0 ||
      num_out < 0 || num_pairs < 0 || !rows_by_out || num_offsets < 1 || num_offsets > WCN_MAX_OFFSETS)
    return WCN_ERR_INVALID_ARGUMENT;
  if (num_out == 0) return WCN_OK;
  if (!out || (num_in > 0 && !features)) return WCN_ERR_INVALID_ARGUMENT;
  WcnRowsView v;
  wcn_rows_layout(const_cast<void*>(rows_by_out), num_out, num_offsets, num_pairs, &v);
  const bool vec = rows_are_vectors(features, channels, dtype) && rows_are_vectors(out, channels, dtype);
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case WCN_DTYPE_F32:
      launch_pool_fwd<float>(features, num_in, channels, v, num_out, mode, vec, out, argmax_or_null, s);
      break;
    case WCN_DTYPE_F16:
      launch_pool_fwd<_Float16>(features, num_in, channels, v, num_out, mode, vec, out, argmax_or_null, s);
      break;
    default:
      launch_pool_fwd<__bf16>(features, num_in, channels, v, num_out, mode, vec, out, argmax_or_null, s);
      break;
  }
  WCN_LAUNCH_CHECK();
  return WCN_OK;
}

int wcn_sparse_pool_bwd(const void* grad_out, int64_t num_out, int32_t channels, int32_t dtype,
                        const void* rows_by_in, const void* rows_by_out, int64_t num_in,
                        int32_t num_offsets, int64_t num_pairs, int32_t mode,
                        const int32_t* argmax_or_null, void* grad_in, void* stream) {
  if (dtype < 0 || dtype > 2 || mode < POOL_SUM || mode > POOL_MIN || channels < 1 || num_in < 0 ||
      num_out < 0 || num_pairs < 0 || !rows_by_in || num_offsets < 1 || num_offsets > WCN_MAX_OFFSETS)
    return WCN_ERR_INVALID_ARGUMENT;
  if ((mode >= POOL_MAX && !argmax_or_null) || (mode == POOL_MEAN && !rows_by_out))
    return WCN_ERR_INVALID_ARGUMENT;
  if (num_in == 0) return WCN_OK;
  if (!grad_in || (num_out > 0 && !grad_out)) return WCN_ERR_INVALID_ARGUMENT;
  WcnRowsView v, vo;
  wcn_rows_layout(const_cast<void*>(rows_by_in), num_in, num_offsets, num_pairs, &v);
  const int32_t* out_ptr = nullptr;
  if (rows_by_out) {
    wcn_rows_layout(const_cast<void*>(rows_by_out), num_out, num_offsets, num_pairs, &vo);
    out_ptr = vo.row_ptr;
  }
  const bool vec = rows_are_vectors(grad_out, channels, dtype) && rows_are_vectors(grad_in, channels, dtype);
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case WCN_DTYPE_F32:
      launch_pool_bwd<float>(grad_out, num_out, channels, v, num_in, mode, vec, out_ptr, argmax_or_null,
                             grad_in, s);
      break;
    case WCN_DTYPE_F16:
      launch_pool_bwd<_Float16>(grad_out, num_out, channels, v, num_in, mode, vec, out_ptr,
                                argmax_or_null, grad_in, s);
      break;
    default:
      launch_pool_bwd<__bf16>(grad_out, num_out, channels, v, num_in, mode, vec, out_ptr, argmax_or_null,
                              grad_in, s);
      break;
  }
  WCN_LAUNCH_CHECK();
  return WCN_OK;
}

int wcn_segment_reduce(const void* features, int64_t num_in, int32_t channels, int32_t dtype,
                       const int64_t* segment_offsets, const int64_t* indices_or_null,
                       int64_t num_entries, int64_t num_segments, int32_t mode, void* out,
                       int64_t* argmax_or_null, void* stream) {
  if (dtype < 0 || dtype > 2 || mode < POOL_SUM || mode > POOL_MIN || channels < 1 || num_in < 0 ||
      num_segments < 0 || channels > (1 << 20) || num_entries < 0)
    return WCN_ERR_INVALID_ARGUMENT;
  if (num_segments == 0) return WCN_OK;
  if (!out || !segment_offsets || (num_in > 0 && !features)) return WCN_ERR_INVALID_ARGUMENT;
  const bool vec = rows_are_vectors(features, channels, dtype) && rows_are_vectors(out, channels, dtype);
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case WCN_DTYPE_F32:
      launch_segment_reduce<float>(features, num_in, channels, segment_offsets, indices_or_null,
                                   num_entries, num_segments, mode, vec, out, argmax_or_null, s);
      break;
    case WCN_DTYPE_F16:
      launch_segment_reduce<_Float16>(features, num_in, channels, segment_offsets, indices_or_null,
                                      num_entries, num_segments, mode, vec, out, argmax_or_null, s);
      break;
    default:
      launch_segment_reduce<__bf16>(features, num_in, channels, segment_offsets, indices_or_null,
                                    num_entries, num_segments, mode, vec, out, argmax_or_null, s);
      break;
  }
  WCN_LAUNCH_CHECK();
  return WCN_OK;
}

int wcn_segment_reduce_bwd(const void* grad_out, int64_t num_segments, int32_t channels, int32_t dtype,
                           const int64_t* segment_offsets, const int64_t* segment_of_row, int64_t num_in,
                           int32_t mode, const int64_t* argmax_or_null, void* grad_in, void* stream) {
  if (dtype < 0 || dtype > 2 || mode < POOL_SUM || mode > POOL_MIN || channels < 1 || num_in < 0 ||
      num_segments < 0 || channels > (1 << 20))
    return WCN_ERR_INVALID_ARGUMENT;
  if (mode >= POOL_MAX && !argmax_or_null) return WCN_ERR_INVALID_ARGUMENT;
  if (num_in == 0) return WCN_OK;
  if (!grad_in || !segment_of_row || !segment_offsets || (num_segments > 0 && !grad_out))
    return WCN_ERR_INVALID_ARGUMENT;
  const bool vec = rows_are_vectors(grad_out, channels, dtype) && rows_are_vectors(grad_in, channels, dtype);
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case WCN_DTYPE_F32:
      launch_segment_reduce_bwd<float>(grad_out, num_segments, channels, segment_offsets, segment_of_row,
                                       num_in, mode, vec, argmax_or_null, grad_in, s);
      break;
    case WCN_DTYPE_F16:
      launch_segment_reduce_bwd<_Float16>(grad_out, num_segments, channels, segment_offsets,
                                          segment_of_row, num_in, mode, vec, argmax_or_null, grad_in, s);
      break;
    default:
      launch_segment_reduce_bwd<__bf16>(grad_out, num_segments, channels, segment_offsets, segment_of_row,
                                        num_in, mode, vec, argmax_or_null, grad_in, s);
      break;
  }
  WCN_LAUNCH_CHECK();
  return WCN_OK;
}

/* Depthwise convolution and its input gradient (the same call over the exchanged rows form with
 * grad_out as features). */
int wcn_sparse_depthwise_fwd(const void* features, int64_t num_in, int32_t channels, int32_t dtype,
                             const void* weight, int32_t weight_dtype, const void* rows_by_out,
                             int64_t num_out, int32_t num_offsets, int64_t num_pairs,
                             int32_t identity_offset, void* out, void* stream) {
  if (dtype < 0 || dtype > 2 || (weight_dtype != dtype && weight_dtype != WCN_DTYPE_F32) ||
      channels < 1 || num_in < 0 || num_out < 0 || num_pairs < 0 || !rows_by_out || !weight ||
      num_offsets < 1 || num_offsets > WCN_MAX_OFFSETS || identity_offset >= num_offsets)
    return WCN_ERR_INVALID_ARGUMENT;
  if (num_out == 0) return WCN_OK;
  if (!out || (num_in > 0 && !features)) return WCN_ERR_INVALID_ARGUMENT;
  WcnRowsView v;
  wcn_rows_layout(const_cast<void*>(rows_by_out), num_out, num_offsets, num_pairs, &v);
  const bool vec = rows_are_vectors(features, channels, dtype) && rows_are_vectors(out, channels, dtype);
  hipStream_t s = (hipStream_t)stream;
  const int per = dtype == WCN_DTYPE_F32 ? 4 : 8;
  const int64_t items = num_out * ((channels + per - 1) / per);
  const dim3 grid((unsigned)((items + 255) / 256)), block(256);
#define WCN_DW_LAUNCH(T, WT)                                                                        \
  hipLaunchKernelGGL((depthwise_fwd<T, WT>), grid, block, 0, s, (const T*)features, num_in, channels, \
                     (const WT*)weight, num_offsets, identity_offset, (const uint32_t*)v.row_mask,  \
                     v.words, (const int32_t*)v.row_ptr, (const int32_t*)v.row_in, num_out, vec, (T*)out)
  if (dtype == WCN_DTYPE_F32) {
    WCN_DW_LAUNCH(float, float);
  } else if (dtype == WCN_DTYPE_F16) {
    if (weight_dtype == WCN_DTYPE_F32) WCN_DW_LAUNCH(_Float16, float); else WCN_DW_LAUNCH(_Float16, _Float16);
  } else {
    if (weight_dtype == WCN_DTYPE_F32) WCN_DW_LAUNCH(__bf16, float); else WCN_DW_LAUNCH(__bf16, __bf16);
  }
#undef WCN_DW_LAUNCH
  WCN_LAUNCH_CHECK();
  return WCN_OK;
}

size_t wcn_depthwise_wgrad_workspace_bytes(int32_t num_offsets, int32_t channels, int64_t num_pairs,
                                           int64_t identity_rows) {
  if (num_offsets < 1 || num_offsets > WCN_MAX_OFFSETS || channels < 1 || num_pairs < 0 ||
      identity_rows < 0)
    return 0;
  const size_t chunks = (size_t)((num_pairs + identity_rows) / DW_CHUNK + num_offsets);
  return wcn_align256(sizeof(int64_t) * (size_t)(num_offsets + 1)) +
         wcn_align256(sizeof(int32_t) * (size_t)(num_offsets + 1)) +
         wcn_align256(sizeof(float) * chunks * (size_t)channels);
}

int wcn_sparse_depthwise_wgrad(const void* features, int64_t num_in, const void* grad_out,
                               int64_t num_out, int32_t channels, int32_t dtype,
                               const int32_t* in_maps, const int32_t* out_maps,
                               const int64_t* host_offsets, int32_t num_offsets,
                               int32_t identity_offset, void* grad_weight, int32_t weight_dtype,
                               void* workspace, size_t workspace_bytes, void* stream) {
  int64_t pairs = 0;
  if (dtype < 0 || dtype > 2 || (weight_dtype != dtype && weight_dtype != WCN_DTYPE_F32) ||
      channels < 1 || num_in < 0 || num_out < 0 || !grad_weight || !workspace ||
      !map_args_ok(host_offsets, num_offsets, in_maps, out_maps, &pairs) ||
      identity_offset >= num_offsets)
    return WCN_ERR_INVALID_ARGUMENT;
  if ((num_in > 0 && !features) || (num_out > 0 && !grad_out)) return WCN_ERR_INVALID_ARGUMENT;
  const int64_t identity_rows = identity_offset >= 0 ? std::min(num_in, num_out) : 0;
  if (workspace_bytes < wcn_depthwise_wgrad_workspace_bytes(num_offsets, channels, pairs, identity_rows))
    return WCN_ERR_WORKSPACE;
  char* p = (char*)workspace;
  int64_t* offsets = (int64_t*)p;
  p += wcn_align256(sizeof(int64_t) * (size_t)(num_offsets + 1));
  int32_t* chunk_first = (int32_t*)p;
  p += wcn_align256(sizeof(int32_t) * (size_t)(num_offsets + 1));
  float* partial = (float*)p;
  hipStream_t s = (hipStream_t)stream;
  if (hipMemcpyAsync(offsets, host_offsets, sizeof(int64_t) * (size_t)(num_offsets + 1),
                     hipMemcpyHostToDevice, s) != hipSuccess)
    return WCN_ERR_LAUNCH;
  int64_t chunks = 0;
  for (int k = 0; k < num_offsets; ++k) {
    const int64_t n = k == identity_offset ? identity_rows : host_offsets[k + 1] - host_offsets[k];
    chunks += (n + DW_CHUNK - 1) / DW_CHUNK;
  }
  hipLaunchKernelGGL(depthwise_plan, dim3(1), dim3(64), 0, s, (const int64_t*)offsets, num_offsets,
                     identity_offset, identity_rows, chunk_first);
  const bool vec = rows_are_vectors(features, channels, dtype) && rows_are_vectors(grad_out, channels, dtype);
  if (chunks > 0) {
    const dim3 grid((unsigned)chunks), block(256);
#define WCN_DWG_LAUNCH(T)                                                                          \
  hipLaunchKernelGGL(depthwise_wgrad<T>, grid, block, 0, s, (const T*)features, num_in, (const T*)grad_out, \
                     num_out, channels, in_maps, out_maps, (const int64_t*)offsets,                 \
                     (const int32_t*)chunk_first, num_offsets, identity_offset, identity_rows, vec, partial)
    if (dtype == WCN_DTYPE_F32) WCN_DWG_LAUNCH(float);
    else if (dtype == WCN_DTYPE_F16) WCN_DWG_LAUNCH(_Float16);
    else WCN_DWG_LAUNCH(__bf16);
#undef WCN_DWG_LAUNCH
  }
  const int64_t total = (int64_t)num_offsets * channels;
  const dim3 rgrid((unsigned)((total + 255) / 256)), rblock(256);
  if (weight_dtype == WCN_DTYPE_F32)
    hipLaunchKernelGGL(depthwise_wgrad_reduce<float>, rgrid, rblock, 0, s, (const float*)partial,
                       (const int32_t*)chunk_first, num_offsets, channels, (float*)grad_weight);
  else if (dtype == WCN_DTYPE_F16)
    hipLaunchKernelGGL(depthwise_wgrad_reduce<_Float16>, rgrid, rblock, 0, s, (const float*)partial,
                       (const int32_t*)chunk_first, num_offsets, channels, (_Float16*)grad_weight);
  else
    hipLaunchKernelGGL(depthwise_wgrad_reduce<__bf16>, rgrid, rblock, 0, s, (const float*)partial,
                       (const int32_t*)chunk_first, num_offsets, channels, (__bf16*)grad_weight);
  WCN_LAUNCH_CHECK();
  return WCN_OK;
}

}  // extern "C"
