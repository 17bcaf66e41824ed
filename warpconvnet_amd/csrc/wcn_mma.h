// MFMA operand traits and the LDS row format shared by the contraction kernels (gfx950).
#ifndef WCN_MMA_H_
#define WCN_MMA_H_
#include "wcn_common.h"

namespace wcn_mma {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));  // one 16-byte piece

__device__ __forceinline__ float to_float(_Float16 v) { return (float)v; }
__device__ __forceinline__ float to_float(__bf16 v) { return (float)v; }
__device__ __forceinline__ float to_float(float v) { return v; }
template <typename T>
__device__ __forceinline__ T from_float(float v) {
  return (T)v;
}
// N consecutive entries of a residual row as floats (N * sizeof(T) = 8 or 16 bytes: one load).
template <typename T, int N>
__device__ __forceinline__ void load_floats(const T* p, float (&v)[N]) {
  static_assert(N * sizeof(T) == 8 || N * sizeof(T) == 16, "one 8- or 16-byte load");
  T t[N];
  if (N * sizeof(T) == 16)
    *reinterpret_cast<u32x4*>(t) = *reinterpret_cast<const u32x4*>(p);
  else
    *reinterpret_cast<uint2*>(t) = *reinterpret_cast<const uint2*>(p);
#pragma unroll
  for (int e = 0; e < N; ++e) v[e] = to_float(t[e]);
}
// The fused part of a contraction's epilogue, on the fp32 sum (bias already added) of output row
// `row`, channel `col`: plus the residual's entry, then clamped at zero (a NaN stays a NaN).
template <typename T>
__device__ __forceinline__ float finish_sum(float v, const void* residual, int relu, int64_t row, int c_out, int col) {
  if (residual) v += to_float(static_cast<const T*>(residual)[row * c_out + col]);
  if (relu) v = v < 0.f ? 0.f : v;
  return v;
}

// MFMA operand handling per element type.  16x16x32 (f16/bf16): lane l holds row (l & 15),
// k = 8 * (l >> 4) .. +7 of A and column (l & 15), same k of B; 16x16x4 (f32): lane l holds
// A[row l & 15][k = l >> 4], B[k = l >> 4][col l & 15].  The result holds column (l & 15), rows
// 4 * (l >> 4) .. +3.  Both operands are read from rows of CK contiguous k values.
template <typename T>
struct Mma;
template <>
struct Mma<_Float16> {
  typedef f16x8 V;
  static constexpr int CK = 64, KS = 2;
  // 8 consecutive k of row `r`: logical part ks * 4 + kgrp, stored at its swizzled position
  static __device__ __forceinline__ V load(const _Float16* row, int r, int ks, int kgrp) {
    return *reinterpret_cast<const V*>(row + ((ks * 4 + kgrp) ^ ((r >> 1) & 7)) * 8);
  }
  static __device__ __forceinline__ V zero() { return (V){0, 0, 0, 0, 0, 0, 0, 0}; }
  static __device__ __forceinline__ f32x4 mma(V a, V b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};
template <>
struct Mma<__bf16> {
  typedef bf16x8 V;
  static constexpr int CK = 64, KS = 2;
  static __device__ __forceinline__ V load(const __bf16* row, int r, int ks, int kgrp) {
    return *reinterpret_cast<const V*>(row + ((ks * 4 + kgrp) ^ ((r >> 1) & 7)) * 8);
  }
  static __device__ __forceinline__ V zero() { return (V){0, 0, 0, 0, 0, 0, 0, 0}; }
  static __device__ __forceinline__ f32x4 mma(V a, V b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct Mma<float> {
  typedef float V;
  static constexpr int CK = 32, KS = 8;
  // element ks * 4 + kgrp of row `r`: part ks (four floats), swizzled, then the float inside it
  static __device__ __forceinline__ V load(const float* row, int r, int ks, int kgrp) {
    return row[(ks ^ ((r >> 1) & 7)) * 4 + kgrp];
  }
  static __device__ __forceinline__ V zero() { return 0.f; }
  static __device__ __forceinline__ f32x4 mma(V a, V b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
  }
};

// LDS rows are 128 bytes (eight 16-byte parts) with no padding; part p of row r is stored at
// part p ^ ((r >> 1) & 7), which makes the 16-byte operand reads of 16 consecutive rows (and of
// most scattered row sets) hit distinct banks.
__device__ __forceinline__ int lds_part(int row, int part) { return part ^ ((row >> 1) & 7); }

}  // namespace wcn_mma
#endif  // WCN_MMA_H_
