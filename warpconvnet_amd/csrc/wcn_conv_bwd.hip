// Weight gradient of the sparse convolution (gfx950, MFMA).
//
//   dW[k][ci][co] = sum over the pairs p of offset k of  X[in_maps[p]][ci] * dY[out_maps[p]][co]
//
// (reference: warpconvnet/nn/functional/sparse_conv.py:314-355, the per-offset
// `curr_in_feats.T @ curr_grad_output`; its native forms are _C.gemm.cutlass_gemm_trAB_gather and
// _C.gemm.split_k_implicit_gemm).  The identity offset of a same-size map is the dense product
// X[m]^T dY[m] over all rows, as in the reference.
//
// The reduction runs over pairs, so the pairs of every offset are cut into chunks; a workgroup
// owns one chunk and one 64 x 64 tile of (ci, co), keeps the fp32 sum in MFMA accumulators and
// writes it once to a partial buffer; a second kernel adds the chunks of every offset in a fixed
// order (no atomics: the result is bitwise reproducible) and rounds once to the weight dtype.
//
// The MFMA operands want, per lane, consecutive *pairs* of one channel, while a gathered feature
// row holds consecutive channels of one pair.  The transposition happens on the way into LDS: a
// lane fetches 16 bytes of a gathered row and writes its elements to the LDS rows of their
// channels, at the pair's position.  Four adjacent lanes fetch 64 contiguous bytes of one row (one
// request to the vector cache instead of four), sixteen rows per load instruction; a transposing
// write of the wave then covers 32 contiguous bytes in each of four LDS rows.
#include <algorithm>

#include "wcn_common.h"
#include "wcn_mma.h"

namespace {

using namespace wcn_mma;

constexpr int WG_THREADS = 256;
constexpr int TILE = 64;  // channels of X and of dY per workgroup
#ifndef WCN_WGRAD_LPR
#define WCN_WGRAD_LPR 4
#endif

struct WgradArgs {
  const void* X;
  const void* dY;
  const int32_t* in_maps;
  const int32_t* out_maps;
  const int64_t* offsets;      // (K + 1), device
  const int32_t* chunk_first;  // (K + 1), device: first chunk of every offset
  float* partial;              // (chunks, c_in_pad, c_out_pad)
  int64_t num_in, num_out, identity_rows;
  int32_t K, c_in, c_out, c_in_pad, c_out_pad, identity, pairs_per_chunk;
  int32_t vec_in, vec_out;  // rows of X / dY are 16-byte aligned whole vectors
};

// chunk_first[k] = number of chunks of the offsets before k (one workgroup of K + 1 <= 1025 threads
// rounded up to waves; a serial scan by thread 0 over at most 1024 entries).
__global__ void __launch_bounds__(64) wgrad_plan(const int64_t* __restrict__ offsets, int K,
                                                 int identity, int64_t identity_rows,
                                                 int pairs_per_chunk, int32_t* __restrict__ chunk_first) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  int32_t run = 0;
  for (int k = 0; k < K; ++k) {
    chunk_first[k] = run;
    const int64_t n = k == identity ? identity_rows : offsets[k + 1] - offsets[k];
    run += (int32_t)((n + pairs_per_chunk - 1) / pairs_per_chunk);
  }
  chunk_first[K] = run;
}

// 16 bytes (VEC elements) of row `row` starting at channel ch0, zeros where there is nothing.
// With VECIO (rows are whole 16-byte vectors) every call is exactly one load, so the number of
// loads in flight is known when the code is compiled and a wait for the oldest ones does not
// wait for the newest; pieces that do not exist read the first bytes of the matrix instead and
// are replaced by zeros afterwards.
template <typename T, bool VECIO>
__device__ __forceinline__ u32x4 load_piece(const T* __restrict__ base, int64_t row, int64_t num_rows,
                                            int channels, int ch0) {
  constexpr int VEC = 16 / sizeof(T);
  const u32x4 zero = (u32x4){0u, 0u, 0u, 0u};
  const bool valid = row >= 0 && row < num_rows && ch0 < channels;
  if (VECIO) {
    const T* src = base + (valid ? row * channels + ch0 : 0);
    const u32x4 got = *reinterpret_cast<const u32x4*>(src);
    return valid ? got : zero;
  }
  if (!valid) return zero;
  const T* src = base + row * channels + ch0;
  T tmp[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) tmp[j] = ch0 + j < channels ? src[j] : from_float<T>(0.f);
  return *reinterpret_cast<const u32x4*>(tmp);
}

// IDENT: the workgroups of this launch are the chunks of the identity offset (pair p is row p of
// both matrices, no map is read); otherwise the launch covers every chunk and the workgroups of
// the identity offset leave at once.  Two instances keep the hot loop free of branches.
template <typename T, bool VECIO, bool IDENT>
__global__ void __launch_bounds__(WG_THREADS) conv_wgrad(WgradArgs a) {
  typedef Mma<T> M;
  typedef typename M::V V;
  constexpr int CK = M::CK, KS = M::KS;      // pairs per step (one LDS row), MFMA k-steps per step
  constexpr int VEC = 16 / sizeof(T);
  constexpr int PARTS = TILE / VEC;           // 16-byte pieces of a 64-channel row
  constexpr int NPI = CK * PARTS / 128;       // pieces per thread and step (two waves per operand)
  constexpr int LPR = WCN_WGRAD_LPR;          // adjacent lanes on one gathered row
  constexpr int RPI = 64 / LPR;               // rows per load instruction
  constexpr int GROUPS = PARTS / LPR;         // groups of LPR pieces in a 64-channel row
  static_assert(CK * sizeof(T) == 128 && NPI * RPI * 2 * LPR == CK * PARTS, "a step fills 128-byte LDS rows");
  // [buffer][operand][channel][pair]
  __shared__ __attribute__((aligned(16))) T tiles[2][2][TILE * CK];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kgrp = lane >> 4;
  const int chunk = IDENT ? a.chunk_first[a.identity] + (int)blockIdx.x : (int)blockIdx.x;
  const int ci0 = blockIdx.y * TILE, co0 = blockIdx.z * TILE;

  // which offset this chunk belongs to: the last k with chunk_first[k] <= chunk
  int lo = 0, hi = a.K;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (a.chunk_first[mid] <= chunk) lo = mid; else hi = mid;
  }
  const int k = lo;
  if ((k == a.identity) != IDENT) return;  // the same for the whole workgroup
  const int64_t n_k = IDENT ? a.identity_rows : a.offsets[k + 1] - a.offsets[k];
  const int64_t first = (int64_t)(chunk - a.chunk_first[k]) * a.pairs_per_chunk;  // inside the offset
  const int64_t left = n_k - first;
  const int count = (int)(left < a.pairs_per_chunk ? left : a.pairs_per_chunk);
  const int64_t pbase = a.offsets[k] + first;
  const int steps = (count + CK - 1) / CK;

  // this thread's share of a step: operand (wave & 1); piece i is 16 bytes of the row of pair
  // pair_of(i), channels part_of(i) * VEC .. of the tile.  The wave pair (wave >> 1 = 0, 1) covers
  // the step's CK pairs x PARTS pieces as 2 * NPI instructions of RPI rows x LPR pieces.
  const int operand = wave & 1;
  auto pair_of = [&](int i) { return (((wave >> 1) * NPI + i) / GROUPS) * RPI + lane / LPR; };
  auto part_of = [&](int i) { return (((wave >> 1) * NPI + i) % GROUPS) * LPR + lane % LPR; };
  constexpr int NROW = (NPI + GROUPS - 1) / GROUPS;  // distinct pairs among a thread's pieces
  const T* const src = (const T*)(operand ? a.dY : a.X);
  const int32_t* const map = operand ? a.out_maps : a.in_maps;
  const int64_t src_rows = operand ? a.num_out : a.num_in;
  const int src_ch = operand ? a.c_out : a.c_in;
  const int ch_base = operand ? co0 : ci0;

  // The map entry of piece i's pair in step s: always exactly one load, and the value is not
  // touched until the rows are requested DEPTH steps later (a use right here would make the wave
  // wait for the load at once).  Pairs past the chunk's end read its last entry; row_from sorts
  // that out at the time of use.
  auto raw_of = [&](int s, int i) -> int32_t {
    if (IDENT) return 0;
    const int p = s * CK + pair_of(i);
    return map[pbase + (p < count ? p : count - 1)];  // count >= 1 in every launched chunk
  };
  auto row_from = [&](int32_t raw, int s, int i) -> int64_t {  // source row, or -1
    const int p = s * CK + pair_of(i);
    const int64_t row = IDENT ? first + p : (int64_t)raw;
    return p < count ? row : -1;
  };
  // the rows of DEPTH steps are in flight at any time (a step multiplies for a few hundred
  // cycles, a gathered row takes a few thousand to arrive)
  constexpr int DEPTH = 3;
  u32x4 piece[DEPTH][NPI];
  int32_t row_ahead[DEPTH][NROW];  // pieces i with the same i / GROUPS share a pair
  auto rows_of = [&](int s, int32_t* raw) {
#pragma unroll
    for (int g = 0; g < NROW; ++g) raw[g] = raw_of(s, g * GROUPS);
  };
  auto fetch = [&](const int32_t* raw, int s, u32x4* dst) {
#pragma unroll
    for (int i = 0; i < NPI; ++i)
      dst[i] = load_piece<T, VECIO>(src, row_from(raw[i / GROUPS], s, i), src_rows, src_ch,
                                    ch_base + part_of(i) * VEC);
  };

  // the wave's quadrant of the tile: 32 channels of X by 32 channels of dY
  const int qi = (wave & 1) * 32, qo = (wave >> 1) * 32;
  f32x4 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};

#pragma unroll
  for (int u = 0; u < DEPTH; ++u) rows_of(u, row_ahead[u]);
#pragma unroll
  for (int u = 0; u < DEPTH; ++u) {
    fetch(row_ahead[u], u, piece[u]);
    rows_of(DEPTH + u, row_ahead[u]);
  }
  // the step count is rounded up to a multiple of DEPTH (the extra steps multiply zeros), which
  // keeps the loop free of exits in the middle
  for (int s0 = 0; s0 < steps; s0 += DEPTH) {
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) {
      const int s = s0 + u;
      // transpose into LDS: element j of piece i goes to row (channel) part * VEC + j, position pr
      T* const dst = tiles[s & 1][operand];
#pragma unroll
      for (int i = 0; i < NPI; ++i) {
        const int part = part_of(i), pr = pair_of(i);
        const T* v = reinterpret_cast<const T*>(&piece[u][i]);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const int ch = part * VEC + j;
          dst[ch * CK + lds_part(ch, pr / VEC) * VEC + pr % VEC] = v[j];
        }
      }
      // step s is in LDS; everyone is done reading the other buffer.  (Written out because
      // __syncthreads would also wait for the global loads in flight.)
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      fetch(row_ahead[u], s + DEPTH, piece[u]);  // rows of step s + DEPTH
      rows_of(s + 2 * DEPTH, row_ahead[u]);
      const T* const xt = tiles[s & 1][0];
      const T* const yt = tiles[s & 1][1];
      V xf[2][KS], yf[2][KS];
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const int rx = qi + b * 16 + (lane & 15), ry = qo + b * 16 + (lane & 15);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          xf[b][ks] = M::load(xt + rx * CK, rx, ks, kgrp);
          yf[b][ks] = M::load(yt + ry * CK, ry, ks, kgrp);
        }
      }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j) acc[i][j] = M::mma(xf[i][ks], yf[j][ks], acc[i][j]);
    }
  }

  // a lane holds column (lane & 15) = channel of dY, rows 4 * kgrp .. + 3 = channels of X
  float* const part_tile = a.partial + (int64_t)chunk * a.c_in_pad * a.c_out_pad;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int ci = ci0 + qi + i * 16 + kgrp * 4 + r;
        const int co = co0 + qo + j * 16 + (lane & 15);
        part_tile[(int64_t)ci * a.c_out_pad + co] = acc[i][j][r];
      }
}

// dW[k][ci][co] = sum of the offset's chunks, rounded once.  A workgroup owns 256 consecutive
// elements of one offset's padded (ci, co) plane; thread (j, e) adds the chunks c = j, j + 4, ...
// of four adjacent elements, and the four partial sums are combined as (0 + 1) + (2 + 3): the
// order of the additions is fixed, so the result is bitwise reproducible.
template <typename WT>
__global__ void __launch_bounds__(256) wgrad_reduce(const float* __restrict__ partial,
                                                    const int32_t* __restrict__ chunk_first, int K,
                                                    int c_in, int c_out, int c_in_pad, int c_out_pad,
                                                    WT* __restrict__ dW) {
  __shared__ f32x4 part[4][64];
  const int plane = c_in_pad * c_out_pad;
  const int slices = plane / 256;
  const int k = blockIdx.x / slices, slice = blockIdx.x % slices;
  const int j = threadIdx.x >> 6, e = threadIdx.x & 63;
  const int elem = slice * 256 + e * 4;  // first of this thread's four elements in the plane
  const int c0 = chunk_first[k], c1 = chunk_first[k + 1];
  f32x4 sum = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
  for (int c = c0 + j; c < c1; c += 4)
    sum += *reinterpret_cast<const f32x4*>(partial + (int64_t)c * plane + elem);
  part[j][e] = sum;
  __syncthreads();
  if (j == 0) {
    const f32x4 total = (part[0][e] + part[1][e]) + (part[2][e] + part[3][e]);
    const int ci = elem / c_out_pad, co = elem % c_out_pad;
    if (ci < c_in) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (co + r < c_out) dW[((int64_t)k * c_in + ci) * c_out + co + r] = from_float<WT>(total[r]);
    }
  }
}

inline int pad_to_tile(int c) { return (c + TILE - 1) / TILE * TILE; }

// Pairs per chunk: about 2048 workgroups in all (8 per CU), never fewer than 256 pairs.
inline int64_t plan_pairs_per_chunk(int64_t pairs, int c_in, int c_out) {
  const int64_t tiles = (int64_t)(pad_to_tile(c_in) / TILE) * (pad_to_tile(c_out) / TILE);
  const int64_t want = std::max<int64_t>(64, 2048 / tiles);
  int64_t p = std::max<int64_t>(256, (pairs + want - 1) / want);
  p = (p + 63) / 64 * 64;
  return std::min<int64_t>(p, 1 << 30);
}
inline int64_t plan_max_chunks(int64_t pairs, int K, int c_in, int c_out) {
  return pairs / plan_pairs_per_chunk(pairs, c_in, c_out) + K;
}

struct WgradWorkspace {
  int64_t* offsets;
  int32_t* chunk_first;
  float* partial;
};
inline size_t wgrad_layout(void* base, int K, int c_in, int c_out, int64_t pairs, WgradWorkspace* w) {
  char* p = (char*)base;
  size_t off = 0;
  if (w) w->offsets = (int64_t*)(p + off);
  off += wcn_align256(sizeof(int64_t) * (size_t)(K + 1));
  if (w) w->chunk_first = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * (size_t)(K + 1));
  if (w) w->partial = (float*)(p + off);
  off += wcn_align256(sizeof(float) * (size_t)plan_max_chunks(pairs, K, c_in, c_out) *
                      pad_to_tile(c_in) * pad_to_tile(c_out));
  return off;
}

template <typename T, bool VECIO>
void launch_wgrad_io(const WgradArgs& a, int chunks, int identity_chunks, bool have_pairs, hipStream_t s) {
  const dim3 grid((unsigned)chunks, (unsigned)(a.c_in_pad / TILE), (unsigned)(a.c_out_pad / TILE));
  if (have_pairs) hipLaunchKernelGGL((conv_wgrad<T, VECIO, false>), grid, dim3(WG_THREADS), 0, s, a);
  if (identity_chunks > 0) {
    const dim3 igrid((unsigned)identity_chunks, grid.y, grid.z);
    hipLaunchKernelGGL((conv_wgrad<T, VECIO, true>), igrid, dim3(WG_THREADS), 0, s, a);
  }
}
template <typename T>
void launch_wgrad(const WgradArgs& a, int chunks, int identity_chunks, bool have_pairs, hipStream_t s) {
  if (a.vec_in && a.vec_out)
    launch_wgrad_io<T, true>(a, chunks, identity_chunks, have_pairs, s);
  else
    launch_wgrad_io<T, false>(a, chunks, identity_chunks, have_pairs, s);
}

}  // namespace

extern "C" {

size_t wcn_conv_wgrad_workspace_bytes(int32_t num_offsets, int32_t c_in, int32_t c_out,
                                      int64_t num_pairs, int64_t identity_rows) {
  if (num_offsets < 1 || num_offsets > WCN_MAX_OFFSETS || c_in < 1 || c_out < 1 || num_pairs < 0 ||
      identity_rows < 0)
    return 0;
  return wgrad_layout(nullptr, num_offsets, c_in, c_out, num_pairs + identity_rows, nullptr);
}

int wcn_sparse_conv_wgrad(const void* features, int64_t num_in, int32_t c_in, const void* grad_out,
                          int64_t num_out, int32_t c_out, int32_t dtype, const int32_t* in_maps,
                          const int32_t* out_maps, const int64_t* host_offsets,
                          int32_t num_offsets, int32_t identity_offset, void* grad_weight,
                          int32_t weight_dtype, void* workspace, size_t workspace_bytes,
                          void* stream) {
  if (dtype < 0 || dtype > 2 || (weight_dtype != dtype && weight_dtype != WCN_DTYPE_F32))
    return WCN_ERR_INVALID_ARGUMENT;
  if (num_in < 0 || num_out < 0 || num_offsets < 1 || num_offsets > WCN_MAX_OFFSETS || c_in < 1 ||
      c_out < 1 || !grad_weight || !workspace || !host_offsets || identity_offset >= num_offsets)
    return WCN_ERR_INVALID_ARGUMENT;
  if (num_in >= (1ll << 31) || num_out >= (1ll << 31)) return WCN_ERR_INVALID_ARGUMENT;
  const int64_t L = host_offsets[num_offsets];
  if (host_offsets[0] != 0 || L < 0 || L > INT32_MAX) return WCN_ERR_INVALID_ARGUMENT;
  for (int k = 0; k < num_offsets; ++k)
    if (host_offsets[k + 1] < host_offsets[k]) return WCN_ERR_INVALID_ARGUMENT;
  if (L > 0 && (!in_maps || !out_maps)) return WCN_ERR_INVALID_ARGUMENT;
  if ((num_in > 0 && !features) || (num_out > 0 && !grad_out)) return WCN_ERR_INVALID_ARGUMENT;
  const int64_t identity_rows = identity_offset >= 0 ? std::min(num_in, num_out) : 0;
  if (workspace_bytes < wcn_conv_wgrad_workspace_bytes(num_offsets, c_in, c_out, L, identity_rows))
    return WCN_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  WgradWorkspace w;
  wgrad_layout(workspace, num_offsets, c_in, c_out, L + identity_rows, &w);
  if (hipMemcpyAsync(w.offsets, host_offsets, sizeof(int64_t) * (size_t)(num_offsets + 1),
                     hipMemcpyHostToDevice, s) != hipSuccess)
    return WCN_ERR_LAUNCH;
  const int ppc = (int)plan_pairs_per_chunk(L + identity_rows, c_in, c_out);
  int64_t chunks = 0;  // the device computes the same numbers from the same inputs
  for (int k = 0; k < num_offsets; ++k) {
    const int64_t n = k == identity_offset ? identity_rows : host_offsets[k + 1] - host_offsets[k];
    chunks += (n + ppc - 1) / ppc;
  }
  if (chunks > plan_max_chunks(L + identity_rows, num_offsets, c_in, c_out)) return WCN_ERR_WORKSPACE;
  hipLaunchKernelGGL(wgrad_plan, dim3(1), dim3(64), 0, s, (const int64_t*)w.offsets, num_offsets,
                     identity_offset, identity_rows, ppc, w.chunk_first);

  WgradArgs a;
  a.X = features;
  a.dY = grad_out;
  a.in_maps = in_maps;
  a.out_maps = out_maps;
  a.offsets = w.offsets;
  a.chunk_first = w.chunk_first;
  a.partial = w.partial;
  a.num_in = num_in;
  a.num_out = num_out;
  a.identity_rows = identity_rows;
  a.K = num_offsets;
  a.c_in = c_in;
  a.c_out = c_out;
  a.c_in_pad = pad_to_tile(c_in);
  a.c_out_pad = pad_to_tile(c_out);
  a.identity = identity_offset;
  a.pairs_per_chunk = ppc;
  const size_t es = dtype == WCN_DTYPE_F32 ? 4 : 2;
  a.vec_in = (((size_t)c_in * es) % 16 == 0 && ((uintptr_t)features % 16) == 0) ? 1 : 0;
  a.vec_out = (((size_t)c_out * es) % 16 == 0 && ((uintptr_t)grad_out % 16) == 0) ? 1 : 0;
  if (chunks > 0) {
    const int ichunks = (int)((identity_rows + ppc - 1) / ppc);
    const bool have_pairs = chunks > ichunks && L > 0;  // the map is only read if it is not empty
    switch (dtype) {
      case WCN_DTYPE_F32: launch_wgrad<float>(a, (int)chunks, ichunks, have_pairs, s); break;
      case WCN_DTYPE_F16: launch_wgrad<_Float16>(a, (int)chunks, ichunks, have_pairs, s); break;
      default: launch_wgrad<__bf16>(a, (int)chunks, ichunks, have_pairs, s); break;
    }
  }
  const unsigned rgrid = (unsigned)((int64_t)num_offsets * (a.c_in_pad * a.c_out_pad / 256));
  if (weight_dtype == WCN_DTYPE_F32) {
    hipLaunchKernelGGL(wgrad_reduce<float>, dim3(rgrid), dim3(256), 0, s, (const float*)w.partial,
                       (const int32_t*)w.chunk_first, num_offsets, c_in, c_out, a.c_in_pad,
                       a.c_out_pad, (float*)grad_weight);
  } else if (dtype == WCN_DTYPE_F16) {
    hipLaunchKernelGGL(wgrad_reduce<_Float16>, dim3(rgrid), dim3(256), 0, s, (const float*)w.partial,
                       (const int32_t*)w.chunk_first, num_offsets, c_in, c_out, a.c_in_pad,
                       a.c_out_pad, (_Float16*)grad_weight);
  } else {
    hipLaunchKernelGGL(wgrad_reduce<__bf16>, dim3(rgrid), dim3(256), 0, s, (const float*)w.partial,
                       (const int32_t*)w.chunk_first, num_offsets, c_in, c_out, a.c_in_pad,
                       a.c_out_pad, (__bf16*)grad_weight);
  }
  WCN_LAUNCH_CHECK();
  return WCN_OK;
}

}  // extern "C"
