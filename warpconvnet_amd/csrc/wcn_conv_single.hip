// Feature contraction for maps in which every output row has exactly one pair (gfx950, MFMA): the
// transposed convolution that undoes a strided one whose kernel is as large as its stride (the
// decoder's up-sampling of a U-Net: every fine voxel has one parent and lies at one offset from it).
//
//   out[out_k[p], :] = act(bias + X[in_k[p], :] @ W[k] + residual[out_k[p], :])     for every pair p
//
// Nothing is accumulated across pairs, so there are no sums to keep anywhere, no phases and no order
// the pairs of an offset have to be in: the lists are taken as they are (a forward map with its
// lists exchanged is not re-ordered first), cut into tiles of 256 pairs of one offset.  A workgroup
// of four waves walks a contiguous stretch of tiles with W[k]^T of the current offset in LDS (loaded
// again when the offset changes); a wave takes 64 pairs as four blocks of 16.  The product is
// transposed: W[k]^T is the A operand (rows = output channels, read from LDS), the gathered rows
// are the B operand and go from memory straight into registers in operand layout (lane = pair,
// 8 channels), so a lane ends up with 4 consecutive output channels of one pair and stores them
// with one 8-byte store.  Output channels are walked 64 at a time with the gathered rows kept.
// Replaces the same reference path as the other kernels (sparse_conv.py:495-544 + the native GEMMs
// it calls) for this kind of map.
#include <algorithm>
#include <mutex>

#include "wcn_common.h"
#include "wcn_conv_args.h"
#include "wcn_mma.h"

namespace {

using namespace wcn_mma;

constexpr int SINGLE_WAVES = 4, SINGLE_BPW = 4;               // waves per workgroup, 16-pair blocks per wave
constexpr int SINGLE_TILE = SINGLE_WAVES * SINGLE_BPW * 16;   // pairs per tile

// KS: 32-channel steps of the gathered rows (c_in = 32 KS)
template <typename T, int KS>
__global__ void __launch_bounds__(SINGLE_WAVES * 64) conv_fwd_single(ConvArgs a, WcnSingleTiles tt) {
  typedef typename Mma<T>::V V;
  extern __shared__ __attribute__((aligned(16))) unsigned char single_smem[];
  constexpr int ROW_BYTES = KS * 64 + 16;  // a row of W[k]^T (c_in values) plus 16 bytes: the operand reads of
                                           // 16 consecutive rows then fall into distinct banks
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int p = lane & 15, kg = lane >> 4;
  const int ncb = (a.c_out + 15) / 16;     // 16-channel blocks of output channels
  const int wrows = ncb * 16;              // rows of W[k]^T that are used (the tiles are zero padded beyond c_out)
  const T* __restrict__ X = (const T*)a.X;
  const T* __restrict__ Wt = (const T*)a.Wt;
  T* __restrict__ out = (T*)a.out;
  const int per_wg = (tt.total + (int)gridDim.x - 1) / (int)gridDim.x;
  const int t_begin = (int)blockIdx.x * per_wg;
  const int t_end = t_begin + per_wg < tt.total ? t_begin + per_wg : tt.total;
  int k = 0, loaded = -1;
  for (int tile = t_begin; tile < t_end; ++tile) {
    while (k + 1 < a.K && tile >= tt.first_tile[k + 1]) ++k;  // tiles ascend in offset
    if (k != loaded) {
      __syncthreads();  // everybody has finished with the previous offset's tile
      const u32x4* src = reinterpret_cast<const u32x4*>(Wt + (int64_t)k * a.c_out_pad * a.c_in_pad);
      const int pieces = wrows * KS * 4;  // 16-byte pieces: KS * 4 per row
      for (int i = tid; i < pieces; i += SINGLE_WAVES * 64) {
        const int row = i / (KS * 4), part = i % (KS * 4);
        *reinterpret_cast<u32x4*>(single_smem + row * ROW_BYTES + part * 16) =
            src[(int64_t)row * (a.c_in_pad / 8) + part];
      }
      __syncthreads();
      loaded = k;
    }
    const int run_end = tt.first_pair[k + 1];
    const int p0 = tt.first_pair[k] + (tile - tt.first_tile[k]) * SINGLE_TILE + wave * (SINGLE_BPW * 16);
    if (p0 >= run_end) continue;  // wave-uniform: this wave's share of the offset's last tile is empty
    // the wave's pairs and their rows, in MFMA operand layout
    int32_t orow[SINGLE_BPW];
    V B[SINGLE_BPW][KS];
#pragma unroll
    for (int b = 0; b < SINGLE_BPW; ++b) {
      const int pi = p0 + b * 16 + p;
      const bool live = pi < run_end;
      const int32_t irow = live ? a.in_maps[pi] : -1;
      orow[b] = live ? a.out_maps[pi] : -1;
      const bool ok = live && (uint32_t)irow < (uint64_t)a.num_in && (uint32_t)orow[b] < (uint64_t)a.num_out;
      if (!ok) orow[b] = -1;
      const T* row = X + (int64_t)(ok ? irow : 0) * a.c_in + kg * 8;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        B[b][ks] = ok ? *reinterpret_cast<const V*>(row + ks * 32) : Mma<T>::zero();
    }
    // 64 output channels at a time
    for (int cg = 0; cg * 4 < ncb; ++cg) {
      f32x4 acc[SINGLE_BPW][4];
#pragma unroll
      for (int b = 0; b < SINGLE_BPW; ++b)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[b][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int cb = cg * 4 + j;
          if (cb < ncb) {  // uniform
            const V A = *reinterpret_cast<const V*>(single_smem + (cb * 16 + p) * ROW_BYTES + (ks * 32 + kg * 8) * 2);
#pragma unroll
            for (int b = 0; b < SINGLE_BPW; ++b) acc[b][j] = Mma<T>::mma(A, B[b][ks], acc[b][j]);
          }
        }
      }
      // lane (p, kg) holds channels cb * 16 + 4 kg .. + 3 of pair p of every block
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int col = (cg * 4 + j) * 16 + 4 * kg;
        if (col < a.c_out) {  // c_out is a multiple of 8: all four or none
          float bias[4] = {0.f, 0.f, 0.f, 0.f};
          if (a.bias) load_floats<T, 4>((const T*)a.bias + col, bias);
#pragma unroll
          for (int b = 0; b < SINGLE_BPW; ++b) {
            if (orow[b] >= 0) {
              float r[4] = {0.f, 0.f, 0.f, 0.f};
              if (a.residual) load_floats<T, 4>((const T*)a.residual + (int64_t)orow[b] * a.c_out + col, r);
              T t[4];
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                float f = acc[b][j][e] + bias[e] + r[e];
                if (a.relu) f = f < 0.f ? 0.f : f;
                t[e] = from_float<T>(f);
              }
              *reinterpret_cast<uint2*>(out + (int64_t)orow[b] * a.c_out + col) = *reinterpret_cast<const uint2*>(t);
            }
          }
        }
      }
    }
  }
}

inline int single_cus() {
  static std::mutex mu;
  static int cus[64] = {};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 256;
  std::lock_guard<std::mutex> hold(mu);
  if (cus[device] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || n < 1) n = 256;
    cus[device] = n;
  }
  return cus[device];
}

template <typename T, int KS>
int launch_single(const ConvArgs& a, const WcnSingleTiles& tt, hipStream_t s) {
  const int ncb = (a.c_out + 15) / 16;
  const int lds = ncb * 16 * (KS * 64 + 16);
  if (lds > 160 * 1024) return WCN_ERR_INVALID_ARGUMENT;
  const void* fn = (const void*)conv_fwd_single<T, KS>;
  // more than 64 KiB of dynamic LDS has to be allowed once per device and kernel (the largest is asked for)
  static std::mutex mu;
  static bool allowed[64] = {};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return WCN_ERR_LAUNCH;
  {
    std::lock_guard<std::mutex> hold(mu);
    if (!allowed[device]) {
      if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess)
        return WCN_ERR_LAUNCH;
      allowed[device] = true;
    }
  }
  // workgroups per CU: what the registers admit (130 to 166 a lane for rows of up to 96 channels: three
  // waves per SIMD; 180 for 128 channels: two; 214 and 244 beyond: one) and LDS holds
  const int per_cu = std::max(1, std::min(KS <= 3 ? 3 : (KS <= 4 ? 2 : 1), (160 * 1024) / lds));
  const unsigned grid = (unsigned)std::min<int64_t>(tt.total, (int64_t)single_cus() * per_cu);
  hipLaunchKernelGGL((conv_fwd_single<T, KS>), dim3(grid), dim3(SINGLE_WAVES * 64), lds, s, a, tt);
  wcn_conv_note_kernel("conv_fwd_single<%s, %d>", wcn_type_text<T>(), KS);
  return hipGetLastError() == hipSuccess ? WCN_OK : WCN_ERR_LAUNCH;
}

template <typename T>
int launch_single_typed(const ConvArgs& a, const WcnSingleTiles& tt, hipStream_t s) {
  switch (a.c_in / 32) {
    case 1: return launch_single<T, 1>(a, tt, s);
    case 2: return launch_single<T, 2>(a, tt, s);
    case 3: return launch_single<T, 3>(a, tt, s);
    case 4: return launch_single<T, 4>(a, tt, s);
    case 6: return launch_single<T, 6>(a, tt, s);
    case 8: return launch_single<T, 8>(a, tt, s);
    default: return WCN_ERR_INVALID_ARGUMENT;
  }
}

}  // namespace

// 16-bit rows of 32, 64, 96, 128, 192 or 256 input channels that are whole 16-byte vectors on both
// sides, at most 64 offsets, at most 256 output channels.
bool wcn_conv_single_takes(int dtype, int c_in, int c_out, int num_offsets) {
  if (dtype != WCN_DTYPE_F16 && dtype != WCN_DTYPE_BF16) return false;
  if (c_in % 32 != 0 || c_out % 8 != 0 || c_out < 8 || c_out > 256 || num_offsets < 1 || num_offsets > WCN_SINGLE_MAX_OFFSETS)
    return false;
  const int ks = c_in / 32;
  return ks == 1 || ks == 2 || ks == 3 || ks == 4 || ks == 6 || ks == 8;
}

int wcn_conv_single_launch(const ConvArgs& a, int dtype, const int64_t* host_offsets, hipStream_t s) {
  WcnSingleTiles tt;
  int64_t tiles = 0;
  for (int k = 0; k < a.K; ++k) {
    tt.first_tile[k] = (int32_t)tiles;
    tt.first_pair[k] = (int32_t)host_offsets[k];
    tiles += (host_offsets[k + 1] - host_offsets[k] + SINGLE_TILE - 1) / SINGLE_TILE;
  }
  if (tiles > INT32_MAX || host_offsets[a.K] > INT32_MAX) return WCN_ERR_INVALID_ARGUMENT;
  for (int k = a.K; k <= WCN_SINGLE_MAX_OFFSETS; ++k) {
    tt.first_tile[k] = (int32_t)tiles;
    tt.first_pair[k] = (int32_t)host_offsets[a.K];
  }
  tt.total = (int32_t)tiles;
  if (tiles == 0) return WCN_OK;
  return dtype == WCN_DTYPE_F16 ? launch_single_typed<_Float16>(a, tt, s) : launch_single_typed<__bf16>(a, tt, s);
}
