// Feature contraction of the sparse convolution forward (gfx950, MFMA).
//
//   out[m, :] = bias + sum_k sum_{p in offset k, out_maps[p] == m} X[in_maps[p], :] @ W[k]
//
// Output-stationary and atomic-free: a workgroup owns TM consecutive output rows and TN output
// channels and keeps their fp32 accumulators in LDS for the whole kernel.  Because the pairs of
// every offset ascend in output index, the pairs that touch the workgroup's rows are one
// contiguous run per offset, located with the group_start table (number of pairs of offset k
// below output row 64*g).  For each offset the run is processed in chunks of RB pairs: the RB
// input rows are gathered into LDS, multiplied with W[k] (kept transposed so that both MFMA
// operands are 16-byte LDS reads) by v_mfma_f32_16x16x32_{f16,bf16} / v_mfma_f32_16x16x4_f32,
// and the fp32 products are added to the accumulator rows the pairs name.  Rows are rounded to
// the feature dtype once, when the tile is written.
//
// Compulsory HBM bytes: every input row once per offset that uses it (L * C_in * s, served by the
// L2 / Infinity Cache when rows are revisited), the maps once (8 L), the output once
// (M * C_out * s); the weights (K * C_in * C_out * s) stay cache resident.
#include <algorithm>

#include "wcn_common.h"

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int TM = 128;  // output rows per workgroup (two 64-row groups of the kernel map)
constexpr int TN = 64;   // output channels per workgroup
constexpr int RB = 64;   // pairs per chunk (4 waves x 16 MFMA rows)
constexpr int ACC_LD = TN + 4;

template <typename T>
struct Cfg;
template <>
struct Cfg<_Float16> {
  static constexpr int CK = 64;     // input channels staged per chunk
  static constexpr int LD = CK + 8; // LDS row pitch in elements (144 B: spreads rows over banks)
};
template <>
struct Cfg<__bf16> {
  static constexpr int CK = 64;
  static constexpr int LD = CK + 8;
};
template <>
struct Cfg<float> {
  static constexpr int CK = 32;
  static constexpr int LD = CK + 4;
};

__device__ __forceinline__ float to_float(_Float16 v) { return (float)v; }
__device__ __forceinline__ float to_float(__bf16 v) { return (float)v; }
__device__ __forceinline__ float to_float(float v) { return v; }
template <typename T>
__device__ __forceinline__ T from_float(float v) {
  return (T)v;
}

// One 16x16 output block: acc += A(16 x CK, rows of As) * B(CK x 16, rows of Bs are columns).
// Operand layout of the 16x16x32 MFMAs: lane l holds row (l & 15), k = 8 * (l >> 4) .. +7 of A
// and column (l & 15), same k of B; the result holds column (l & 15), rows 4 * (l >> 4) .. +3.
__device__ __forceinline__ f32x4 mma_block(const _Float16* a_row, const _Float16* b_row, int lane,
                                           f32x4 acc) {
#pragma unroll
  for (int ks = 0; ks < Cfg<_Float16>::CK / 32; ++ks) {
    const f16x8 a = *reinterpret_cast<const f16x8*>(a_row + ks * 32 + (lane >> 4) * 8);
    const f16x8 b = *reinterpret_cast<const f16x8*>(b_row + ks * 32 + (lane >> 4) * 8);
    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc, 0, 0, 0);
  }
  return acc;
}
__device__ __forceinline__ f32x4 mma_block(const __bf16* a_row, const __bf16* b_row, int lane,
                                           f32x4 acc) {
#pragma unroll
  for (int ks = 0; ks < Cfg<__bf16>::CK / 32; ++ks) {
    const bf16x8 a = *reinterpret_cast<const bf16x8*>(a_row + ks * 32 + (lane >> 4) * 8);
    const bf16x8 b = *reinterpret_cast<const bf16x8*>(b_row + ks * 32 + (lane >> 4) * 8);
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
  }
  return acc;
}
// fp32: v_mfma_f32_16x16x4_f32, lane l holds A[row l & 15][k = l >> 4] and B[k = l >> 4][col l & 15].
__device__ __forceinline__ f32x4 mma_block(const float* a_row, const float* b_row, int lane,
                                           f32x4 acc) {
#pragma unroll
  for (int ks = 0; ks < Cfg<float>::CK / 4; ++ks) {
    const float a = a_row[ks * 4 + (lane >> 4)];
    const float b = b_row[ks * 4 + (lane >> 4)];
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc, 0, 0, 0);
  }
  return acc;
}

// Wt[k][n][c] = W[k][c][n] converted to T, zero padded to (c_out_pad, c_in_pad).
template <typename T, typename WT>
__global__ void __launch_bounds__(256) conv_prep_weight(const WT* __restrict__ W, int K, int c_in,
                                                        int c_out, int c_in_pad, int c_out_pad,
                                                        T* __restrict__ Wt) {
  const int64_t total = (int64_t)K * c_out_pad * c_in_pad;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int c = (int)(i % c_in_pad);
    const int n = (int)((i / c_in_pad) % c_out_pad);
    const int k = (int)(i / ((int64_t)c_in_pad * c_out_pad));
    float v = 0.f;
    if (c < c_in && n < c_out) v = to_float(W[((int64_t)k * c_in + c) * c_out + n]);
    Wt[i] = from_float<T>(v);
  }
}

// group_start[k][g] = number of pairs of offset k with out_maps < 64 * g (binary search).
__global__ void __launch_bounds__(256) conv_group_start(const int32_t* __restrict__ out_maps,
                                                        const int64_t* __restrict__ offsets, int K,
                                                        int64_t G, int32_t* __restrict__ gs) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)K * (G + 1)) return;
  const int k = (int)(i / (G + 1));
  const int64_t g = i % (G + 1);
  const int64_t lo0 = offsets[k], hi0 = offsets[k + 1];
  int64_t lo = lo0, hi = hi0;
  const int64_t target = g * 64;
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if ((int64_t)out_maps[mid] < target) lo = mid + 1; else hi = mid;
  }
  gs[i] = (int32_t)(lo - lo0);
}

struct ConvArgs {
  const void* X;
  const void* Wt;
  const void* bias;         // same dtype as X, or null
  const int32_t* in_maps;
  const int32_t* out_maps;
  const int64_t* offsets;   // device copy, K+1
  const int32_t* group_start;  // (K, G+1)
  void* out;
  int64_t num_in, num_out, G;
  int32_t K, c_in, c_out, c_in_pad, c_out_pad, identity;
  int32_t vec_rows;  // feature rows are 16-byte aligned and a whole number of 16-byte vectors
};

__device__ __forceinline__ int64_t imin(int64_t x, int64_t y) { return x < y ? x : y; }
__device__ __forceinline__ int64_t imax(int64_t x, int64_t y) { return x > y ? x : y; }

template <typename T>
__global__ void __launch_bounds__(256) conv_fwd(ConvArgs a) {
  constexpr int CK = Cfg<T>::CK;
  constexpr int LD = Cfg<T>::LD;
  constexpr int VEC = 16 / sizeof(T);  // elements per 16-byte vector
  __shared__ float accs[TM * ACC_LD];
  __shared__ __attribute__((aligned(16))) T As[RB * LD];
  __shared__ __attribute__((aligned(16))) T Bs[TN * LD];
  __shared__ int32_t s_in[RB];
  __shared__ int32_t s_out[RB];

  const T* __restrict__ X = (const T*)a.X;
  const T* __restrict__ Wt = (const T*)a.Wt;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t m0 = (int64_t)blockIdx.x * TM;
  const int n0 = blockIdx.y * TN;
  const int tile_rows = (int)imin(TM, a.num_out - m0);
  const int64_t g0 = m0 >> 6;
  const int64_t g1 = imin(g0 + TM / 64, a.G);
  const bool vec_rows = a.vec_rows != 0;
  const int64_t num_pairs = a.offsets[a.K];

  for (int i = tid; i < TM * ACC_LD; i += 256) accs[i] = 0.f;
  __syncthreads();

  for (int k = 0; k < a.K; ++k) {
    int64_t p0, cnt;
    const bool iden = (k == a.identity);
    if (iden) {
      p0 = 0;
      cnt = imax(0, imin(tile_rows, a.num_in - m0));
    } else {
      const int32_t* gs = a.group_start + (int64_t)k * (a.G + 1);
      p0 = a.offsets[k] + gs[g0];
      cnt = imin(gs[g1] - gs[g0], num_pairs - p0);  // never read past the maps
    }
    for (int64_t r0 = 0; r0 < cnt; r0 += RB) {
      const int rows = (int)imin(RB, cnt - r0);
      __syncthreads();  // previous chunk's readers of s_in / s_out are done
      if (tid < RB) {
        int32_t ii = 0, oo = 0;
        if (tid < rows) {
          if (iden) {
            ii = (int32_t)(m0 + r0 + tid);
            oo = (int32_t)(r0 + tid);
          } else {
            ii = a.in_maps[p0 + r0 + tid];
            oo = (int32_t)(a.out_maps[p0 + r0 + tid] - m0);
          }
          // a malformed map must not turn into a wild access: such a pair contributes nothing
          if ((uint32_t)ii >= (uint64_t)a.num_in || (uint32_t)oo >= (uint32_t)tile_rows) {
            ii = -1;
            oo = -1;
          }
        }
        s_in[tid] = ii;
        s_out[tid] = oo;
      }
      f32x4 acc[TN / 16];
#pragma unroll
      for (int nb = 0; nb < TN / 16; ++nb) acc[nb] = (f32x4){0.f, 0.f, 0.f, 0.f};

      for (int c0 = 0; c0 < a.c_in_pad; c0 += CK) {
        __syncthreads();  // s_in visible; previous channel chunk's MFMA reads are done
        // stage the gathered input rows: RB rows x CK channels
        if (vec_rows) {
          for (int v = tid; v < RB * (CK / VEC); v += 256) {
            const int r = v / (CK / VEC), cv = (v % (CK / VEC)) * VEC;
            uint4 val = make_uint4(0u, 0u, 0u, 0u);
            if (r < rows && c0 + cv < a.c_in && s_in[r] >= 0)
              val = *reinterpret_cast<const uint4*>(X + (int64_t)s_in[r] * a.c_in + c0 + cv);
            *reinterpret_cast<uint4*>(&As[r * LD + cv]) = val;
          }
        } else {
          for (int e = tid; e < RB * CK; e += 256) {
            const int r = e / CK, c = e % CK;
            T val = from_float<T>(0.f);
            if (r < rows && c0 + c < a.c_in && s_in[r] >= 0)
              val = X[(int64_t)s_in[r] * a.c_in + c0 + c];
            As[r * LD + c] = val;
          }
        }
        // stage W[k]^T: TN output channels x CK input channels (already padded, always aligned)
        for (int v = tid; v < TN * (CK / VEC); v += 256) {
          const int n = v / (CK / VEC), cv = (v % (CK / VEC)) * VEC;
          const uint4 val = *reinterpret_cast<const uint4*>(
              Wt + ((int64_t)k * a.c_out_pad + n0 + n) * a.c_in_pad + c0 + cv);
          *reinterpret_cast<uint4*>(&Bs[n * LD + cv]) = val;
        }
        __syncthreads();
        if (wave * 16 < rows) {
          const T* a_row = &As[(wave * 16 + (lane & 15)) * LD];
#pragma unroll
          for (int nb = 0; nb < TN / 16; ++nb)
            acc[nb] = mma_block(a_row, &Bs[(nb * 16 + (lane & 15)) * LD], lane, acc[nb]);
        }
      }
      // add the chunk's products to the accumulator rows its pairs name (rows of one offset
      // are distinct, so plain read-modify-write is race free)
      if (wave * 16 < rows) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int row = wave * 16 + (lane >> 4) * 4 + r;
          if (row < rows && s_out[row] >= 0) {
            float* dst = &accs[s_out[row] * ACC_LD + (lane & 15)];
#pragma unroll
            for (int nb = 0; nb < TN / 16; ++nb) dst[nb * 16] += acc[nb][r];
          }
        }
      }
    }
  }
  __syncthreads();

  // write the tile: bias add, one rounding to T
  T* __restrict__ out = (T*)a.out;
  const T* __restrict__ bias = (const T*)a.bias;
  for (int e = tid; e < TM * TN; e += 256) {
    const int r = e / TN, c = e % TN;
    if (r < tile_rows && n0 + c < a.c_out) {
      float v = accs[r * ACC_LD + c];
      if (bias) v += to_float(bias[n0 + c]);
      out[(m0 + r) * a.c_out + n0 + c] = from_float<T>(v);
    }
  }
}

inline int round_up(int x, int m) { return (x + m - 1) / m * m; }

struct ConvWorkspace {
  int64_t* offsets;      // K+1
  int32_t* group_start;  // (K, G+1)
  void* Wt;              // K * c_out_pad * c_in_pad elements
  int64_t G;
  int c_in_pad, c_out_pad;
};

inline size_t elem_size(int dtype) { return dtype == WCN_DTYPE_F32 ? 4 : 2; }

inline int ck_of(int dtype) { return dtype == WCN_DTYPE_F32 ? Cfg<float>::CK : Cfg<_Float16>::CK; }

inline size_t conv_layout(void* base, int64_t num_out, int K, int c_in, int c_out, int dtype,
                          ConvWorkspace* w) {
  char* p = (char*)base;
  size_t off = 0;
  const int64_t G = (num_out + 63) / 64;
  const int cip = round_up(c_in, ck_of(dtype)), cop = round_up(c_out, TN);
  if (w) w->offsets = (int64_t*)(p + off);
  off += wcn_align256(sizeof(int64_t) * (size_t)(K + 1));
  if (w) w->group_start = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * (size_t)K * (size_t)(G + 1));
  if (w) w->Wt = (void*)(p + off);
  off += wcn_align256(elem_size(dtype) * (size_t)K * cop * cip);
  if (w) {
    w->G = G;
    w->c_in_pad = cip;
    w->c_out_pad = cop;
  }
  return off;
}

// Optional timing hook: events armed by wcn_conv_set_timing_events bracket the next conv_fwd
// launch of this thread (and only that kernel), then disarm.
thread_local hipEvent_t g_time_start = nullptr;
thread_local hipEvent_t g_time_stop = nullptr;

template <typename T>
int launch_conv(const ConvArgs& a, const void* weight, int weight_dtype, int dtype,
                hipStream_t s) {
  const int64_t total = (int64_t)a.K * a.c_out_pad * a.c_in_pad;
  const int pgrid = (int)std::min<int64_t>(4096, (total + 255) / 256);
  if (weight_dtype == dtype) {
    hipLaunchKernelGGL((conv_prep_weight<T, T>), dim3(pgrid), dim3(256), 0, s, (const T*)weight,
                       a.K, a.c_in, a.c_out, a.c_in_pad, a.c_out_pad, (T*)a.Wt);
  } else {
    hipLaunchKernelGGL((conv_prep_weight<T, float>), dim3(pgrid), dim3(256), 0, s,
                       (const float*)weight, a.K, a.c_in, a.c_out, a.c_in_pad, a.c_out_pad,
                       (T*)a.Wt);
  }
  const dim3 grid((unsigned)((a.num_out + TM - 1) / TM), (unsigned)(a.c_out_pad / TN));
  if (g_time_start) (void)hipEventRecord(g_time_start, s);
  hipLaunchKernelGGL(conv_fwd<T>, grid, dim3(256), 0, s, a);
  if (g_time_stop) (void)hipEventRecord(g_time_stop, s);
  g_time_start = g_time_stop = nullptr;
  WCN_LAUNCH_CHECK();
  return WCN_OK;
}

}  // namespace

extern "C" {

int wcn_conv_set_timing_events(void* start_event, void* stop_event) {
  g_time_start = (hipEvent_t)start_event;
  g_time_stop = (hipEvent_t)stop_event;
  return WCN_OK;
}

size_t wcn_conv_workspace_bytes(int64_t num_out, int32_t num_offsets, int32_t c_in, int32_t c_out,
                                int32_t dtype) {
  if (num_out < 0 || num_offsets < 1 || c_in < 1 || c_out < 1 || dtype < 0 || dtype > 2) return 0;
  return conv_layout(nullptr, num_out, num_offsets, c_in, c_out, dtype, nullptr);
}

int wcn_sparse_conv_fwd(const void* features, int64_t num_in, int32_t c_in, int32_t dtype,
                        const void* weight, int32_t weight_dtype, int32_t num_offsets,
                        int32_t c_out, const void* bias_or_null, const int32_t* in_maps,
                        const int32_t* out_maps, const int64_t* host_offsets,
                        int32_t identity_offset, const int32_t* group_start_or_null, void* out,
                        int64_t num_out, void* workspace, size_t workspace_bytes, void* stream) {
  if (dtype < 0 || dtype > 2 || (weight_dtype != dtype && weight_dtype != WCN_DTYPE_F32))
    return WCN_ERR_INVALID_ARGUMENT;
  if (num_in < 0 || num_out < 0 || num_offsets < 1 || c_in < 1 || c_out < 1 || !weight ||
      !host_offsets || !workspace)
    return WCN_ERR_INVALID_ARGUMENT;
  if (num_in >= (1ll << 31) || num_out >= (1ll << 31)) return WCN_ERR_INVALID_ARGUMENT;
  if (identity_offset >= num_offsets) return WCN_ERR_INVALID_ARGUMENT;
  if (num_out == 0) return WCN_OK;
  if (!out || (num_in > 0 && !features)) return WCN_ERR_INVALID_ARGUMENT;
  const int64_t L = host_offsets[num_offsets];
  if (host_offsets[0] != 0 || L < 0) return WCN_ERR_INVALID_ARGUMENT;
  for (int k = 0; k < num_offsets; ++k)
    if (host_offsets[k + 1] < host_offsets[k]) return WCN_ERR_INVALID_ARGUMENT;
  if (L > 0 && (!in_maps || !out_maps)) return WCN_ERR_INVALID_ARGUMENT;
  if (workspace_bytes < wcn_conv_workspace_bytes(num_out, num_offsets, c_in, c_out, dtype))
    return WCN_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  ConvWorkspace w;
  conv_layout(workspace, num_out, num_offsets, c_in, c_out, dtype, &w);
  if (hipMemcpyAsync(w.offsets, host_offsets, sizeof(int64_t) * (size_t)(num_offsets + 1),
                     hipMemcpyHostToDevice, s) != hipSuccess)
    return WCN_ERR_LAUNCH;
  const int32_t* gs = group_start_or_null;
  if (!gs) {
    const int64_t items = (int64_t)num_offsets * (w.G + 1);
    hipLaunchKernelGGL(conv_group_start, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, s,
                       out_maps, (const int64_t*)w.offsets, num_offsets, w.G, w.group_start);
    gs = w.group_start;
  }
  ConvArgs a;
  a.X = features;
  a.Wt = w.Wt;
  a.bias = bias_or_null;
  a.in_maps = in_maps;
  a.out_maps = out_maps;
  a.offsets = w.offsets;
  a.group_start = gs;
  a.out = out;
  a.num_in = num_in;
  a.num_out = num_out;
  a.G = w.G;
  a.K = num_offsets;
  a.c_in = c_in;
  a.c_out = c_out;
  a.c_in_pad = w.c_in_pad;
  a.c_out_pad = w.c_out_pad;
  a.identity = identity_offset;
  a.vec_rows = (((size_t)c_in * elem_size(dtype)) % 16 == 0 && ((uintptr_t)features % 16) == 0) ? 1 : 0;
  switch (dtype) {
    case WCN_DTYPE_F32: return launch_conv<float>(a, weight, weight_dtype, dtype, s);
    case WCN_DTYPE_F16: return launch_conv<_Float16>(a, weight, weight_dtype, dtype, s);
    default: return launch_conv<__bf16>(a, weight, weight_dtype, dtype, s);
  }
}

}  // extern "C"
