// Feature contraction of the sparse convolution (gfx950, MFMA): forward product and, through the
// same kernels, the input gradient.
//
//   out[m, :] = bias + sum_k sum_{p in offset k, out_maps[p] == m} X[in_maps[p], :] @ W[k]
//
// Output-stationary, atomic-free, fp32 accumulators in registers in MFMA result layout for the
// whole kernel, one rounding at the end: the result is bitwise reproducible.
//
// The map is consumed as the reference's pair lists, which ascend in output row inside every
// offset: the pairs of one offset that touch a tile's rows are one contiguous run, found with the
// group_start table (pairs of offset k below output row 64 * g).  Lists that do not ascend (the
// exchanged lists of a transposed convolution or of an input gradient) are first re-ordered
// inside the workspace (rows_* kernels below).
//
// Two kernels:
//   conv_fwd_ring  feature rows that are whole 16-byte vectors (every case the Python entry points
//                  produce): rows, weight tiles and pairs go from memory straight into LDS rings,
//                  eight waves in two roles; described where it is defined.
//   conv_fwd       any channel count: a workgroup of four waves owns 256 output rows x 64 output
//                  channels; the offsets are cut into batches (up to 4 offsets, up to 128 pairs)
//                  that run as a software pipeline through registers: while batch b is multiplied,
//                  the gathered rows and W[k]^T tiles of batch b + 1 are in flight and the pairs
//                  of batch b + 2 are being read.
// In both, lane l of a 16-row block reads the gathered row of output row (l & 15) through a slot
// table, or a row of zeros if that output row has no pair for the offset, so the product lands in
// the accumulator rows directly (v_mfma_f32_16x16x32_{f16,bf16}, v_mfma_f32_16x16x4_f32); 16-row
// blocks without any pair skip their MFMAs.
//
// Compulsory HBM bytes: every gathered input row once (L * C_in * s; revisits are served by the
// L2 / Infinity Cache when the voxel order has locality), the map once (8 L), the output once
// (M * C_out * s); the weights (K * C_in * C_out * s) stay cache resident.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <type_traits>

#include <stdarg.h>
#include <stdio.h>

#include "wcn_common.h"
#include "wcn_conv_args.h"
#include "wcn_mma.h"

void wcn_scan_rows_launch(int32_t* groups, int64_t G, int rows, int64_t* row_total, hipStream_t s);

namespace {

using namespace wcn_mma;

constexpr int ROWS = 256;    // output rows per workgroup
constexpr int TN = 64;       // output channels per workgroup
constexpr int THREADS = 256; // wave w owns rows 64 * (w & 3) .. +63 and channel blocks of column group (w >> 2)
constexpr int NBW = TN / 16 / (THREADS / 256);  // 16-channel blocks per wave
constexpr int A_ROWS = 128;  // gathered input rows resident in LDS (pairs per batch)
constexpr int BATCH = 4;     // offsets per batch, at most

// Up to 128 offsets of a kernel map (K + 1 <= 128) travel as a kernel argument.
constexpr int OFFSETS_BY_VALUE = 128;
struct OffsetsByValue {
  int64_t v[OFFSETS_BY_VALUE];
};

// The kernels multiply by tiles Wt[k][n][c] (n: channel of the result, c: channel of the gathered
// rows), converted to T and zero padded to (c_out_pad, c_in_pad).
//   forward        Wt[k][n][c] = W[k][c][n]            (W is (K, c_in, c_out))
//   input gradient Wt[k][n][c] = W[k'][n][c], k' = k or K - 1 - k   (W is (K, c_out, c_in) in the
//                  kernel's terms: the product is dY @ W[k']^T)
template <typename T, typename WT>
__global__ void __launch_bounds__(256) conv_prep_weight(const WT* __restrict__ W, int K, int c_in,
                                                        int c_out, int c_in_pad, int c_out_pad,
                                                        int as_stored, int flip_k,
                                                        T* __restrict__ Wt, uint32_t* __restrict__ zeros,
                                                        int64_t* __restrict__ offsets_dst,
                                                        int n_offsets, OffsetsByValue ov) {
  if (blockIdx.x == 0 && zeros) {
    zeros[threadIdx.x] = 0u;  // 256 threads x 4 bytes
    // the map's offsets, handed over in the kernel arguments (saves a copy command per call)
    if ((int)threadIdx.x < n_offsets) offsets_dst[threadIdx.x] = ov.v[threadIdx.x];
  }
  const int64_t total = (int64_t)K * c_out_pad * c_in_pad;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int c = (int)(i % c_in_pad);
    const int n = (int)((i / c_in_pad) % c_out_pad);
    const int k = (int)(i / ((int64_t)c_in_pad * c_out_pad));
    const int ks = flip_k ? K - 1 - k : k;
    float v = 0.f;
    if (c < c_in && n < c_out)
      v = to_float(as_stored ? W[((int64_t)ks * c_out + n) * c_in + c] : W[((int64_t)ks * c_in + c) * c_out + n]);
    Wt[i] = from_float<T>(v);
  }
}

// One batch = up to BATCH offsets and A_ROWS pairs; the pairs of one offset may be split over
// consecutive batches.  Packed descriptor of one (batch, offset) entry.
__device__ __forceinline__ uint32_t pack_run(int k, int first, int num) {
  return (uint32_t)k | ((uint32_t)first << 8) | ((uint32_t)num << 20);  // k < 32, first <= 256, num <= 128
}
__device__ __forceinline__ int run_k(uint32_t r) { return (int)(r & 0xFFu); }
__device__ __forceinline__ int run_first(uint32_t r) { return (int)((r >> 8) & 0xFFFu); }
__device__ __forceinline__ int run_num(uint32_t r) { return (int)(r >> 20); }

template <typename T>
__global__ void __launch_bounds__(THREADS, 2) conv_fwd(ConvArgs a) {
  typedef Mma<T> M;
  typedef typename M::V V;
  constexpr int CK = M::CK, KS = M::KS;
  constexpr int VEC = 16 / sizeof(T);  // elements per 16-byte part; a row is CK = 8 * VEC elements
  static_assert(CK == 8 * VEC, "a staged row is eight 16-byte parts");
  constexpr int A_PIECES = A_ROWS * 8 / THREADS;      // 16-byte parts of gathered rows per thread
  constexpr int B_PIECES = BATCH * TN * 8 / THREADS;  // 16-byte parts of the batch's weight tiles
  constexpr int MAX_BATCHES = 32 * ROWS / A_ROWS + 32 / BATCH + 2;  // per chunk of 32 offsets
  static_assert(A_ROWS <= 128 && A_ROWS <= THREADS, "slot ids take 7 bits; one pair per thread");
  __shared__ __attribute__((aligned(16))) T As[(A_ROWS + 1) * CK];  // last row: zeros
  __shared__ __attribute__((aligned(16))) T Bs[BATCH][TN * CK];
  // gathered row of (batch offset, output row), tagged with the batch it was written for:
  // entry = (batch & 255) << 8 | row; an entry of another batch means "no pair"
  __shared__ __attribute__((aligned(8))) uint16_t s_slot[2][ROWS][BATCH];
  __shared__ int32_t s_gidx[2][A_ROWS];
  __shared__ __attribute__((aligned(16))) uint32_t s_run[MAX_BATCHES + 2][BATCH];  // two empty batches after the last
  __shared__ int32_t s_cnt[32];
  __shared__ int32_t s_start[32];
  __shared__ int32_t s_num_batches;

  const T* __restrict__ X = (const T*)a.X;
  const T* __restrict__ Wt = (const T*)a.Wt;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wrow = (wave & 3) * 64, wcol = (wave >> 2) * (NBW * 16);
  const int64_t m0 = (int64_t)blockIdx.x * ROWS;
  const int n0 = blockIdx.y * TN;
  const int tile_rows = (int)(a.num_out - m0 < ROWS ? a.num_out - m0 : ROWS);
  const int64_t g0 = m0 >> 6;
  const int64_t g1 = g0 + ROWS / 64 < a.G ? g0 + ROWS / 64 : a.G;

  f32x4 acc[4][NBW];
#pragma unroll
  for (int rb = 0; rb < 4; ++rb)
#pragma unroll
    for (int nb = 0; nb < NBW; ++nb) acc[rb][nb] = (f32x4){0.f, 0.f, 0.f, 0.f};
  if (tid < 8) *reinterpret_cast<u32x4*>(&As[A_ROWS * CK + tid * VEC]) = (u32x4){0u, 0u, 0u, 0u};

  // MFMA operand addressing: lane l reads row (l & 15) of a 16-row block, k-group (l >> 4)
  const int kgrp = lane >> 4;

  const size_t w_tile_stride = (size_t)a.c_out_pad * a.c_in_pad;
  const uint32_t w_step = (uint32_t)(THREADS / 8) * (uint32_t)a.c_in_pad;  // weight rows one piece apart
  for (int c0 = 0; c0 < a.c_in_pad; c0 += CK) {
    const uint32_t w_lane_off = (uint32_t)(n0 + (tid >> 3)) * (uint32_t)a.c_in_pad + c0 + (tid & 7) * VEC;
    const uint32_t x_lane_off = (uint32_t)(c0 + (tid & 7) * VEC);
    const bool x_part_ok = (int)x_lane_off < a.c_in;
    for (int kbase = 0; kbase < a.K; kbase += 32) {
      const int nk = a.K - kbase < 32 ? a.K - kbase : 32;
      __syncthreads();  // the previous chunk is completely done with the shared tables
      if (tid < 32) {
        int cnt = 0;
        int32_t start = 0;
        const int k = kbase + tid;
        if (tid < nk) {
          if (k == a.identity) {  // every row reads its own input row; the map's pairs are ignored
            const int64_t left = a.num_in - m0;
            cnt = (int)(left < 0 ? 0 : (left < tile_rows ? left : tile_rows));
          } else {
            const int32_t* gs = a.group_start + (int64_t)k * (a.G + 1);
            start = (int32_t)(a.offsets[k] + gs[g0]);
            cnt = gs[g1] - gs[g0];
            if (cnt < 0 || cnt > ROWS) cnt = 0;  // inconsistent table: contribute nothing
          }
        }
        s_cnt[tid] = cnt;
        s_start[tid] = start;
      }
      for (int i = tid; i < 2 * BATCH * ROWS; i += THREADS) (&s_slot[0][0][0])[i] = 0xFFFFu;
      __syncthreads();
      if (tid == 0) {  // cut the chunk into batches (a few dozen steps at most)
        int nb = 0, k = 0, done = 0;
        while (k < nk && s_cnt[k] == 0) ++k;
        while (k < nk && nb < MAX_BATCHES) {
          int total = 0;
          for (int j = 0; j < BATCH; ++j) {
            uint32_t run = pack_run(0, 0, 0);
            if (k < nk && total < A_ROWS) {
              const int left = s_cnt[k] - done;
              const int take = left < A_ROWS - total ? left : A_ROWS - total;
              run = pack_run(k, done, take);
              total += take;
              done += take;
              if (done == s_cnt[k]) {
                done = 0;
                ++k;
                while (k < nk && s_cnt[k] == 0) ++k;
              }
            }
            s_run[nb][j] = run;
          }
          ++nb;
        }
        for (int j = 0; j < BATCH; ++j) s_run[nb][j] = s_run[nb + 1][j] = pack_run(0, 0, 0);
        s_num_batches = nb;
      }
      __syncthreads();
      const int num_batches = s_num_batches;

      // ---- software pipeline over the batches ------------------------------------------------
      // While batch b is multiplied, the input rows and weight tiles of batch b + 1 are in flight
      // (held in registers until the multiply is over) and so are the pairs of batch b + 2.
      int pr_j = -1, pr_in = -1, pr_out = -1;  // this thread's pair of the batch after the next store
      auto load_pair = [&](int b) {
        pr_j = -1;
        if (b < num_batches && tid < A_ROWS) {
          int before = 0;
#pragma unroll
          for (int j = 0; j < BATCH; ++j) {
            const uint32_t run = s_run[b][j];
            const int num = run_num(run);
            if (pr_j < 0 && tid >= before && tid < before + num) {
              pr_j = j;
              const int k = run_k(run), i = run_first(run) + tid - before;
              if (kbase + k == a.identity) {
                pr_in = (int)(m0 + i);
                pr_out = i;
              } else {
                const int64_t p = (int64_t)s_start[k] + i;
                pr_in = a.in_maps[p];
                pr_out = (int)(a.out_maps[p] - m0);
              }
            }
            before += num;
          }
        }
      };
      auto publish_pair = [&](int b) {  // slot table and row list of batch b
        if (b < num_batches && tid < A_ROWS) {
          int32_t g = -1;
          if (pr_j >= 0) {
            g = pr_in;
            if ((uint32_t)g >= (uint64_t)a.num_in) g = -1;  // malformed map: zeros
            if ((uint32_t)pr_out < (uint32_t)tile_rows)
              s_slot[b & 1][pr_out][pr_j] = (uint16_t)(((b & 255) << 8) | tid);
          }
          s_gidx[b & 1][tid] = g;
        }
      };
      u32x4 piece[A_PIECES], wpiece[B_PIECES];
      // runs of a batch as wave-uniform scalars (one 16-byte LDS read)
      auto read_runs = [&](int b, uint32_t (&run)[BATCH]) {
        static_assert(BATCH == 4, "one 16-byte read");
        const u32x4 r = *reinterpret_cast<const u32x4*>(&s_run[b][0]);
#pragma unroll
        for (int j = 0; j < BATCH; ++j) run[j] = __builtin_amdgcn_readfirstlane(r[j]);
      };
      auto fetch_rows = [&](int b, const uint32_t (&run)[BATCH]) {  // rows and weight tiles of batch b -> registers
        if (b >= num_batches) return;
        int32_t g[A_PIECES];
#pragma unroll
        for (int i = 0; i < A_PIECES; ++i) g[i] = s_gidx[b & 1][(tid >> 3) + i * (THREADS / 8)];
#pragma unroll
        for (int i = 0; i < B_PIECES; ++i) {
          constexpr int PER = TN * 8 / THREADS;  // pieces of one weight tile per thread
          const int j = i / PER;
          wpiece[i] = (u32x4){0u, 0u, 0u, 0u};
          if (run_num(run[j]) > 0) {  // uniform
            const T* wk = Wt + (size_t)(kbase + run_k(run[j])) * w_tile_stride;
            wpiece[i] = *reinterpret_cast<const u32x4*>(wk + w_lane_off + (uint32_t)(i % PER) * w_step);
          }
        }
        if (a.vec_in) {
#pragma unroll
          for (int i = 0; i < A_PIECES; ++i) {
            piece[i] = (u32x4){0u, 0u, 0u, 0u};
            if (g[i] >= 0 && x_part_ok)
              piece[i] = *reinterpret_cast<const u32x4*>(X + ((uint64_t)(uint32_t)g[i] * (uint32_t)a.c_in + x_lane_off));
          }
        } else {  // rows that are not whole 16-byte vectors: element by element
#pragma unroll
          for (int i = 0; i < A_PIECES; ++i) {
            piece[i] = (u32x4){0u, 0u, 0u, 0u};
            if (g[i] >= 0 && x_part_ok) {
              T tmp[VEC];
#pragma unroll
              for (int e = 0; e < VEC; ++e) {
                const int c = (int)x_lane_off + e;
                tmp[e] = c < a.c_in ? X[(uint64_t)(uint32_t)g[i] * (uint32_t)a.c_in + c] : from_float<T>(0.f);
              }
              piece[i] = *reinterpret_cast<const u32x4*>(tmp);
            }
          }
        }
      };

      uint32_t run_cur[BATCH], run_next[BATCH];
      if (num_batches > 0) {
        load_pair(0);
        publish_pair(0);
        load_pair(1);
        __syncthreads();
        read_runs(0, run_next);
        fetch_rows(0, run_next);
      }
      for (int b = 0; b < num_batches; ++b) {
#pragma unroll
        for (int j = 0; j < BATCH; ++j) run_cur[j] = run_next[j];
        // registers -> LDS for batch b (this is where the loads issued one batch ago are awaited)
#pragma unroll
        for (int i = 0; i < A_PIECES; ++i) {
          const int seg = tid + i * THREADS, sl = seg >> 3, part = seg & 7;
          *reinterpret_cast<u32x4*>(&As[sl * CK + lds_part(sl, part) * VEC]) = piece[i];
        }
#pragma unroll
        for (int i = 0; i < B_PIECES; ++i) {
          const int v = tid + i * THREADS, j = v / (TN * 8), n = (v >> 3) % TN, part = v & 7;
          *reinterpret_cast<u32x4*>(&Bs[j][n * CK + lds_part(n, part) * VEC]) = wpiece[i];
        }
        publish_pair(b + 1);
        load_pair(b + 2);
        __syncthreads();
        // slot entries of this lane's four row blocks, all offsets of the batch (8 bytes each)
        uint32_t se[4][2];
#pragma unroll
        for (int rb = 0; rb < 4; ++rb) {
          const uint2 t = *reinterpret_cast<const uint2*>(&s_slot[b & 1][wrow + rb * 16 + (lane & 15)][0]);
          se[rb][0] = t.x;
          se[rb][1] = t.y;
        }
        read_runs(b + 1, run_next);
        fetch_rows(b + 1, run_next);

        // multiply batch b: no barrier between its offsets, the waves run freely
        const uint16_t tag = (uint16_t)(b & 255);
#pragma unroll
        for (int j = 0; j < BATCH; ++j) {
          if (run_num(run_cur[j]) == 0) continue;  // uniform
          int sl[4];
#pragma unroll
          for (int rb = 0; rb < 4; ++rb) {
            const uint32_t e = (se[rb][j >> 1] >> (16 * (j & 1))) & 0xFFFFu;
            sl[rb] = (e >> 8) == tag ? (int)(e & 0xFFu) : A_ROWS;  // no pair: the row of zeros
          }
          V bfr[NBW][KS];
#pragma unroll
          for (int nb = 0; nb < NBW; ++nb) {
            const int n = wcol + nb * 16 + (lane & 15);
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) bfr[nb][ks] = M::load(&Bs[j][n * CK], n, ks, kgrp);
          }
          V av[4][KS];
#pragma unroll
          for (int rb = 0; rb < 4; ++rb)
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) av[rb][ks] = M::load(&As[sl[rb] * CK], sl[rb], ks, kgrp);
#pragma unroll
          for (int rb = 0; rb < 4; ++rb) {
            if (__ballot(sl[rb] < A_ROWS) == 0ull) continue;  // no pair in these 16 rows
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
#pragma unroll
              for (int nb = 0; nb < NBW; ++nb) acc[rb][nb] = M::mma(av[rb][ks], bfr[nb][ks], acc[rb][nb]);
          }
        }
        __syncthreads();  // every wave is done with the gathered rows and weight tiles of batch b
      }
    }
  }
  // epilogue: bias add, one rounding to T
  T* __restrict__ out = (T*)a.out;
  const T* __restrict__ bias = (const T*)a.bias;
  float bias_v[NBW];  // this lane's bias values, fetched together
#pragma unroll
  for (int nb = 0; nb < NBW; ++nb) {
    const int col = n0 + wcol + nb * 16 + (lane & 15);
    bias_v[nb] = (bias && col < a.c_out) ? to_float(bias[col]) : 0.f;
  }
  if (sizeof(T) == 2 && a.vec_out) {
    // stage the tile in LDS (the weight buffers are free: the last batch ended with a barrier) for
    // 16-byte stores
    static_assert(BATCH * TN >= ROWS, "the weight buffers hold one output tile");
    T* stage = &Bs[0][0];
    __syncthreads();
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
      for (int nb = 0; nb < NBW; ++nb) {
        const int col = wcol + nb * 16 + (lane & 15);
        const float bv = bias_v[nb];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int lr = wrow + rb * 16 + kgrp * 4 + r;
          float v = acc[rb][nb][r] + bv;
          if ((a.residual || a.relu) && m0 + lr < a.num_out && n0 + col < a.c_out)
            v = finish_sum<T>(v, a.residual, a.relu, m0 + lr, a.c_out, n0 + col);
          stage[lr * CK + lds_part(lr, col / VEC) * VEC + col % VEC] = from_float<T>(v);
        }
      }
    __syncthreads();
    for (int v = tid; v < ROWS * 8; v += THREADS) {
      const int r = v >> 3, part = v & 7;
      if (m0 + r < a.num_out && n0 + part * VEC < a.c_out)
        *reinterpret_cast<u32x4*>(out + (m0 + r) * a.c_out + n0 + part * VEC) =
            *reinterpret_cast<const u32x4*>(&stage[r * CK + lds_part(r, part) * VEC]);
    }
  } else {
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
      for (int nb = 0; nb < NBW; ++nb) {
        const int col = n0 + wcol + nb * 16 + (lane & 15);
        if (col >= a.c_out) continue;
        const float bv = bias_v[nb];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int64_t orow = m0 + wrow + rb * 16 + kgrp * 4 + r;
          if (orow < a.num_out)
            out[orow * a.c_out + col] = from_float<T>(finish_sum<T>(acc[rb][nb][r] + bv, a.residual, a.relu, orow, a.c_out, col));
        }
      }
  }
}

// ---- ring kernel: input rows, weight tiles and pairs go from memory straight into LDS ------------
//
// Used when feature rows are whole 16-byte vectors.  The offsets of a tile are cut into steps of
// at most 64 pairs of one offset.  A workgroup has eight waves in two roles; NC of them multiply,
// 8 - NC request (NC = 6 by default: tiles of 384 rows; NC = 4 gives 256-row tiles):
//   multiplying waves  each owns four 16-row blocks of the tile (dealt in turn) and their
//                      accumulators; per step it reads its operands from LDS and issues the
//                      MFMAs, nothing else
//   requesting waves   each an equal share of W[k]^T of step r + DW (weight ring, 4 tiles) and of
//                      the input rows of step r + DG (row ring, 5 x 64 rows); the first two also
//                      the in_maps / out_maps entries of step r + DP (pair ring); the last but
//                      one writes the slot table of step r + DG, the last clears the next one
// The requests are global_load_lds: the data goes from memory into LDS without passing through
// registers.  A wave issues at most one instruction every four cycles, so the bookkeeping of the
// requests would otherwise sit between the MFMAs of every wave; here it runs beside them.
// (Workgroups of more than four waves are co-resident on a CU only if every SIMD has room for
// two waves of each, hence the budget of 128 vector registers.)
// A requesting wave issues the same loads in every iteration, in the order weights, rows, pairs
// (lanes without work read a block of zeros), so "what step r needs has landed" is one fixed
// s_waitcnt vmcnt(n): the counter retires in order, and with DG = DW + 1 and DP = 2 DG the rows of
// step r, the pairs of step r + DG and the weights of step r are the oldest loads still wanted.
// One barrier per step publishes what has landed and hands the slots read in the previous step
// back to the requesting waves.  A slot table per step (one byte per output row: the row's
// position in the step's slot, or none) is written when the rows are requested and read when
// the step is multiplied.
#ifndef WCN_RING_NC
#define WCN_RING_NC 6
#endif
constexpr int RING_THREADS = 512;
constexpr int STEP_ROWS = 64;
constexpr int A_SLOTS = 5, W_SLOTS = 4;
constexpr int DG = A_SLOTS - 1, DW = W_SLOTS - 1, DP = 2 * DG;
constexpr int SLOT_BYTES = STEP_ROWS * 128;   // a row of the rings is 128 bytes for every dtype
static_assert(TN * 128 == SLOT_BYTES, "weight tile and row slot have the same size");
static_assert(DG == DW + 1, "rows and weights share the requesting waves");

// Layout for NC multiplying waves (tile of 64 NC rows) and 8 - NC requesting waves.
template <int NC>
struct RingCfg {
  static constexpr int RROWS = 64 * NC;
  static constexpr int NP = 8 - NC;
  static constexpr int PER = 8 / NP;                 // row loads and weight loads per requesting wave and step
  static constexpr int P_SLOTS = NC == 4 ? 8 : 6;    // pair ring
  static constexpr int T_SLOTS = NC == 4 ? 8 : 6;    // slot tables
  static constexpr int MAX_STEPS = 32 * NC;
  static constexpr int RING_OFF = 0;
  static constexpr int WRING_OFF = RING_OFF + A_SLOTS * SLOT_BYTES;
  static constexpr int PIN_OFF = WRING_OFF + W_SLOTS * SLOT_BYTES;
  static constexpr int POUT_OFF = PIN_OFF + P_SLOTS * STEP_ROWS * 4;
  static constexpr int TAB_OFF = POUT_OFF + P_SLOTS * STEP_ROWS * 4;
  static constexpr int ZERO_OFF = TAB_OFF + T_SLOTS * RROWS;
  static constexpr int STEP_OFF = ZERO_OFF + 128;  // after the row of zeros
  static constexpr int MISC_OFF = STEP_OFF + (MAX_STEPS + 2 * DP) * 8;  // DP empty steps before and after the plan
  static constexpr int LDS_BYTES = (MISC_OFF + 16 + 511) / 512 * 512;
  static_assert(NP == 4 || NP == 2, "8 loads per step split evenly");
  static_assert(DP < P_SLOTS + DG && T_SLOTS > DG + 1, "ring reuse distances");
  static_assert(DG * (2 * PER + 1) < 64, "outstanding loads per wave fit the 6-bit vmcnt");
  static_assert(2 * LDS_BYTES <= 160 * 1024, "two workgroups per CU");
  static_assert(A_SLOTS * SLOT_BYTES + W_SLOTS * SLOT_BYTES >= RROWS * 128, "the rings hold a staged output tile");
  // position in a ring of P_SLOTS / T_SLOTS entries (x >= -48)
  static __device__ __forceinline__ int pslot(int x) { return (int)((uint32_t)(x + 48) % (uint32_t)P_SLOTS); }
  static __device__ __forceinline__ int tslot(int x) { return (int)((uint32_t)(x + 48) % (uint32_t)T_SLOTS); }
  // The 16-row blocks of a tile are dealt to the multiplying waves in turn (block b belongs to
  // wave b % NC as its block b / NC), so that the pairs of a step, which cover a contiguous range
  // of output rows, spread over all of them.  Byte of tile row t in a slot table: the four blocks
  // of a wave's row (t & 15) are adjacent.
  static __device__ __forceinline__ int tab_index(int t) {
    const uint32_t b = (uint32_t)t >> 4, rb = b / (uint32_t)NC, w = b - rb * (uint32_t)NC;
    return (int)(w * 64u + ((uint32_t)t & 15u) * 4u + rb);
  }
};

// global_load_lds_*: lane l of the wave copies 16 (4) bytes from its own global address to LDS
// byte offset `lds_off` + 16 (4) * l; the data never passes through registers and the load is
// counted by vmcnt.  Written as inline assembly so that the placement of the s_waitcnt for these
// loads stays with this file (the compiler would wait for all of them before every LDS read).
__device__ __forceinline__ uint32_t lds_offset(const void* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}
__device__ __forceinline__ void load_to_lds_16(const void* g, uint32_t lds_off) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(lds_off)
               : "memory", "m0");
}
// the same with a wave-uniform base address and a 32-bit unsigned byte offset per lane
__device__ __forceinline__ void load_to_lds_16(const void* base, uint32_t lane_off, uint32_t lds_off) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(base),
               "s"(lds_off)
               : "memory", "m0");
}
__device__ __forceinline__ void load_to_lds_4(const void* base, uint32_t lane_off, uint32_t lds_off) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" ::"v"(lane_off), "s"(base),
               "s"(lds_off)
               : "memory", "m0");
}
__device__ __forceinline__ void load_to_lds_4(const void* g, uint32_t lds_off) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(g), "s"(lds_off)
               : "memory", "m0");
}

// Step descriptor: w0 = k (in chunk) | num << 8 | first << 16 | identity << 31, w1 = first pair.
__device__ __forceinline__ int step_k(uint32_t w0) { return (int)(w0 & 0xFFu); }
__device__ __forceinline__ int step_num(uint32_t w0) { return (int)((w0 >> 8) & 0xFFu); }
__device__ __forceinline__ int step_first(uint32_t w0) { return (int)((w0 >> 16) & 0x1FFu); }
__device__ __forceinline__ bool step_identity(uint32_t w0) { return (w0 >> 31) != 0u; }

// NARROW: bit 0 = at most TN / 2 output channels, bit 1 = at most CK / 2 input channels.  The
// multiplying waves then leave out the half of the channel blocks / k-steps that is padding (the
// requests and the LDS layout stay as they are).
template <typename T, int NC, bool SPLIT, int NARROW>
__global__ void __launch_bounds__(RING_THREADS, 4) conv_fwd_ring(ConvArgs a) {
  typedef Mma<T> M;
  typedef typename M::V V;
  typedef RingCfg<NC> C;
  constexpr int CK = M::CK, KS = (NARROW & 2) ? M::KS / 2 : M::KS;
  constexpr int VEC = 16 / sizeof(T);
  constexpr int NB = (NARROW & 1) ? TN / 32 : TN / 16;
  constexpr int RROWS = C::RROWS, NP = C::NP, PER = C::PER;
  static_assert(CK * sizeof(T) == 128, "ring rows are 128 bytes");
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint8_t* const ring = smem + C::RING_OFF;
  uint8_t* const wring = smem + C::WRING_OFF;
  int32_t* const s_pin = (int32_t*)(smem + C::PIN_OFF);
  int32_t* const s_pout = (int32_t*)(smem + C::POUT_OFF);
  uint8_t* const s_tab = smem + C::TAB_OFF;
  const T* const s_zero = (const T*)(smem + C::ZERO_OFF);
  uint2* const s_step = (uint2*)(smem + C::STEP_OFF);
  int32_t* const s_nsteps = (int32_t*)(smem + C::MISC_OFF);

  const T* __restrict__ X = (const T*)a.X;
  const T* __restrict__ Wt = (const T*)a.Wt;
  const uint8_t* const zsrc = (const uint8_t*)a.zeros;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wrow = (wave < NC ? wave : 0) * 64;  // multiplying waves: first byte of the wave's entries in a slot table
  const int64_t m0 = (int64_t)blockIdx.x * RROWS;
  const int n0 = blockIdx.y * TN;
  const int tile_rows = (int)(a.num_out - m0 < RROWS ? a.num_out - m0 : RROWS);
  const int64_t g0 = m0 >> 6;
  const int64_t g1 = g0 + RROWS / 64 < a.G ? g0 + RROWS / 64 : a.G;
  const int kgrp = lane >> 4;
  const int sub = lane >> 3, lpart = lane & 7;  // row inside an 8-row load, 16-byte part in LDS

  if (tid < 32) ((uint32_t*)(smem + C::ZERO_OFF))[tid] = 0u;
  T* __restrict__ out = (T*)a.out;
  T* const stage = (T*)ring;  // output tile staged for 16-byte stores: RROWS x 128 bytes (the rings are contiguous)
  const bool staged = sizeof(T) == 2 && a.vec_out && !SPLIT;
  const int c0_begin = SPLIT ? (int)blockIdx.z * CK : 0;       // this workgroup's input-channel slices
  const int c0_end = SPLIT ? c0_begin + CK : a.c_in_pad;

  // Start of a chunk (up to 32 offsets of one slice of input channels): the step plan and clean
  // slot tables.  Every wave runs it; returns the number of steps.
  auto begin_chunk = [&](int kbase) -> int {
    const int nk = a.K - kbase < 32 ? a.K - kbase : 32;
    // the previous chunk is completely done: every load_to_lds has landed, every wave is past
    // its last multiply
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (wave == 0) {  // cut the chunk into steps
      int cnt = 0;
      int32_t start = 0;
      bool ident = false;
      if (lane < nk) {
        const int k = kbase + lane;
        if (k == a.identity) {  // every row reads its own input row; the map's pairs are ignored
          const int64_t left = a.num_in - m0;
          cnt = (int)(left < 0 ? 0 : (left < tile_rows ? left : tile_rows));
          ident = true;
        } else {
          const int32_t* gs = a.group_start + (int64_t)k * (a.G + 1);
          start = (int32_t)(a.offsets[k] + gs[g0]);
          cnt = gs[g1] - gs[g0];
          if (cnt < 0 || cnt > RROWS) cnt = 0;  // inconsistent table: contribute nothing
        }
      }
      const int ns = (cnt + STEP_ROWS - 1) / STEP_ROWS;
      const int incl = wcn_wave_inclusive_sum(ns);
      for (int j = 0; j < ns; ++j) {
        const int num = cnt - j * STEP_ROWS < STEP_ROWS ? cnt - j * STEP_ROWS : STEP_ROWS;
        s_step[DP + incl - ns + j] =
            make_uint2((uint32_t)lane | ((uint32_t)num << 8) | ((uint32_t)(j * STEP_ROWS) << 16) |
                           (ident ? 0x80000000u : 0u),
                       (uint32_t)(start + j * STEP_ROWS));
      }
      const int total = __builtin_amdgcn_readlane(incl, 63);
      if (lane < DP) s_step[lane] = s_step[DP + total + lane] = make_uint2(0u, 0u);
      if (lane == 63) *s_nsteps = total;
    }
    for (int i = tid; i < C::T_SLOTS * RROWS / 4; i += RING_THREADS) ((uint32_t*)s_tab)[i] = 0xFFFFFFFFu;
    __syncthreads();
    return *s_nsteps;
  };
  // descriptors are fetched one iteration ahead (raw, made wave-uniform when used)
  auto step_raw = [&](int s, int S) -> uint2 {  // -DP <= s; steps past the plan's padding read as its last entry
    const int idx = s + DP < S + 2 * DP - 1 ? s + DP : S + 2 * DP - 1;
    return s_step[idx];
  };
  auto uniform = [&](uint2 d) -> uint2 {
    d.x = __builtin_amdgcn_readfirstlane(d.x);
    d.y = __builtin_amdgcn_readfirstlane(d.y);
    return d;
  };

  // The two kinds of waves run separate code from here on (the accumulators exist only in the
  // multiplying waves); both pass the same sequence of barriers.
  if (wave < NC) {
    f32x4 acc[4][NB];
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) acc[rb][nb] = (f32x4){0.f, 0.f, 0.f, 0.f};
    for (int c0 = c0_begin; c0 < c0_end; c0 += CK) {
      for (int kbase = 0; kbase < a.K; kbase += 32) {
        const int S = begin_chunk(kbase);
        if (S == 0) continue;
        // ================= multiplying waves =================
        uint2 rR = step_raw(-DP, S);
        uint32_t sw = 0xFFFFFFFFu;  // slot entries of this lane's four row blocks for step r
        int im = (A_SLOTS - DP % A_SLOTS) % A_SLOTS;   // r mod A_SLOTS, kept incrementally
        int imw = (W_SLOTS - DP % W_SLOTS) % W_SLOTS;  // r mod W_SLOTS
#pragma nounroll
        for (int r = -DP; r < S; ++r) {
          const uint2 dR = uniform(rR);
          asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
          rR = step_raw(r + 1, S);
          const uint32_t sw_cur = sw;
          sw = *(const uint32_t*)(s_tab + C::tslot(r + 1) * RROWS + wrow + (lane & 15) * 4);
          if (r >= 0 && step_num(dR.x) > 0) {
            const T* const abase = (const T*)(ring + im * SLOT_BYTES);
            const T* const bbase = (const T*)(wring + imw * SLOT_BYTES);
            V bfr[NB][KS], av[2][KS];  // the A operands of a row block are read while the one before multiplies
            bool any[4];
            const T* arow[4];
            int aswz[4];
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
              const int n = nb * 16 + (lane & 15);
#pragma unroll
              for (int ks = 0; ks < KS; ++ks) bfr[nb][ks] = M::load(bbase + n * CK, n, ks, kgrp);
            }
#pragma unroll
            for (int rb = 0; rb < 4; ++rb) {
              const int e = (int)((sw_cur >> (8 * rb)) & 0xFFu);
              const bool has = e != 0xFF;
              any[rb] = __ballot(has) != 0ull;  // no pair in these 16 rows: skipped
              arow[rb] = has ? abase + e * CK : s_zero;
              aswz[rb] = has ? e : 0;
            }
            if (any[0]) {
#pragma unroll
              for (int ks = 0; ks < KS; ++ks) av[0][ks] = M::load(arow[0], aswz[0], ks, kgrp);
            }
#pragma unroll
            for (int rb = 0; rb < 4; ++rb) {
              if (rb + 1 < 4 && any[rb + 1]) {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
                  av[(rb + 1) & 1][ks] = M::load(arow[rb + 1], aswz[rb + 1], ks, kgrp);
              }
              if (!any[rb]) continue;
#pragma unroll
              for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
                  acc[rb][nb] = M::mma(bfr[nb][ks], av[rb & 1][ks], acc[rb][nb]);  // (W^T X^T): channels x rows
            }
          }
          im = im + 1 == A_SLOTS ? 0 : im + 1;
          imw = imw + 1 == W_SLOTS ? 0 : imw + 1;
        }
      }
    }
    // epilogue: bias add, one rounding to T.  The products were taken transposed, so a lane holds
    // four consecutive output channels (4 * kgrp ..) of output row (lane & 15) of every 16 x 16
    // block.  16-bit outputs are staged in LDS (8 bytes per lane and block) for whole-row stores.
    const T* __restrict__ bias = (const T*)a.bias;
    float bias_v[NB][4];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int col = n0 + nb * 16 + kgrp * 4 + r;
        bias_v[nb][r] = (bias && !SPLIT && col < a.c_out) ? to_float(bias[col]) : 0.f;
      }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();  // every wave is done with the rings, every load has landed
    if (SPLIT) {  // fp32 sums of this slice, 16 bytes per lane and block; bias and rounding come later
      float* const slice = a.partial + (int64_t)blockIdx.z * a.num_out * a.c_out_pad;
#pragma unroll
      for (int rb = 0; rb < 4; ++rb) {
        const int lr = (rb * NC + wave) * 16 + (lane & 15);
        if (m0 + lr < a.num_out) {
#pragma unroll
          for (int nb = 0; nb < NB; ++nb)
            *reinterpret_cast<f32x4*>(slice + (m0 + lr) * a.c_out_pad + n0 + nb * 16 + kgrp * 4) = acc[rb][nb];
        }
      }
      return;
    }
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) {
      const int lr = (rb * NC + wave) * 16 + (lane & 15);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        const int col = nb * 16 + kgrp * 4;
        T v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float f = acc[rb][nb][r] + bias_v[nb][r];
          if ((a.residual || a.relu) && m0 + lr < a.num_out && n0 + col + r < a.c_out)
            f = finish_sum<T>(f, a.residual, a.relu, m0 + lr, a.c_out, n0 + col + r);
          v[r] = from_float<T>(f);
        }
        if (staged) {
          *reinterpret_cast<uint2*>(&stage[lr * CK + lds_part(lr, col / VEC) * VEC + col % VEC]) =
              *reinterpret_cast<const uint2*>(v);
        } else if (m0 + lr < a.num_out) {
          T* dst = out + (m0 + lr) * a.c_out + n0 + col;
          if (sizeof(T) == 4 && a.vec_out && n0 + col + 3 < a.c_out) {
            *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(v);
          } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (n0 + col + r < a.c_out) dst[r] = v[r];
          }
        }
      }
    }
  } else {
    for (int c0 = c0_begin; c0 < c0_end; c0 += CK) {
      for (int kbase = 0; kbase < a.K; kbase += 32) {
        const int S = begin_chunk(kbase);
        if (S == 0) continue;
        // ================= requesting waves =================
        const int q = wave - NC;  // which share of the weight tile and of the step's rows
        const size_t w_tile_bytes = (size_t)a.c_out_pad * a.c_in_pad * sizeof(T);
        const uint8_t* const wbase0 = (const uint8_t*)(Wt + (size_t)n0 * a.c_in_pad + c0);
        const uint8_t* const xbase0 = a.num_in > 0 ? (const uint8_t*)(X + c0) : zsrc;
        const uint32_t row_bytes = (uint32_t)a.c_in * (uint32_t)sizeof(T);
        uint32_t w_lane_off[PER], x_lane_off[PER];
#pragma unroll
        for (int j = 0; j < PER; ++j) {
          const int n = (q * PER + j) * 8 + sub;  // also the row inside the step's slot
          const uint32_t part_off = (uint32_t)(lpart ^ ((n >> 1) & 7)) * 16u;  // source part kept at this LDS position
          w_lane_off[j] = (uint32_t)n * (uint32_t)a.c_in_pad * (uint32_t)sizeof(T) + part_off;
          x_lane_off[j] = part_off;
        }
        uint2 rW = step_raw(-DP + DW, S), rG = step_raw(-DP + DG, S), rP = step_raw(0, S);
        int iw = (W_SLOTS - (DP - DW) % W_SLOTS) % W_SLOTS;  // (r + DW) mod W_SLOTS
        int ia = (A_SLOTS - (DP - DG) % A_SLOTS) % A_SLOTS;  // (r + DG) mod A_SLOTS
#pragma nounroll
        for (int r = -DP; r < S; ++r) {
          const uint2 dW = uniform(rW), dG = uniform(rG), dP = uniform(rP);
          // this wave's share of what step r needs, and of the pairs of step r + DG, has landed:
          // everything but the rows and pairs requested DW iterations ago and all that came later
          if (q < 2) {
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"((PER + 1) + (2 * PER + 1) * (DW - 1)) : "memory");
          } else {
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(PER + 2 * PER * (DW - 1)) : "memory");
          }
          asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
          const int gi = r + DG;
          const int32_t* pin = s_pin + C::pslot(gi) * STEP_ROWS;
          const int32_t* pout = s_pout + C::pslot(gi) * STEP_ROWS;
          // all LDS reads first and unconditionally (slots past the step's pairs hold stale
          // values that are not used)
          int32_t pv[PER];
#pragma unroll
          for (int j = 0; j < PER; ++j) pv[j] = pin[(q * PER + j) * 8 + sub];
          const int32_t pin_l = pin[lane], pout_l = pout[lane];
          rW = step_raw(r + 1 + DW, S);
          rG = step_raw(r + 1 + DG, S);
          rP = step_raw(r + 1 + DP, S);
          const int numG = step_num(dG.x);
          const bool identG = step_identity(dG.x);
          const int firstG = step_first(dG.x);
          const int kW = kbase + step_k(dW.x);
          const uint32_t wdst = lds_offset(wring + iw * SLOT_BYTES + q * PER * 1024);
          const uint32_t xdst = lds_offset(ring + ia * SLOT_BYTES + q * PER * 1024);
          // weights: uniform base of the tile, this lane's fixed offset inside it
          const uint8_t* const wk = wbase0 + (size_t)kW * w_tile_bytes;
#pragma unroll
          for (int j = 0; j < PER; ++j) load_to_lds_16(wk, w_lane_off[j], __builtin_amdgcn_readfirstlane(wdst + j * 1024));
          if (a.flat_in) {
            // rows: uniform base, row index times row size plus this lane's part (rows past the
            // step's pairs and malformed indices fetch row 0; no slot entry ever points at them)
            uint32_t xoff[PER];
#pragma unroll
            for (int j = 0; j < PER; ++j) {
              const int row = (q * PER + j) * 8 + sub;
              uint32_t in = identG ? (uint32_t)(m0 + firstG + row) : (uint32_t)pv[j];
              if (row >= numG || in >= (uint32_t)a.num_in) in = 0u;
              xoff[j] = in * row_bytes + x_lane_off[j];
            }
#pragma unroll
            for (int j = 0; j < PER; ++j) load_to_lds_16(xbase0, xoff[j], __builtin_amdgcn_readfirstlane(xdst + j * 1024));
          } else {
            const uint8_t* xsrc[PER];
#pragma unroll
            for (int j = 0; j < PER; ++j) {
              const int row = (q * PER + j) * 8 + sub;
              int32_t in = identG ? (int32_t)(m0 + firstG + row) : pv[j];
              if (row >= numG) in = -1;
              const int ps = lpart ^ ((row >> 1) & 7);  // source part kept at this LDS position
              const bool ok = (uint32_t)in < (uint64_t)a.num_in && c0 + ps * VEC < a.c_in;
              const uint8_t* real =
                  (const uint8_t*)(X + ((uint64_t)(uint32_t)in * (uint32_t)a.c_in + (uint32_t)(c0 + ps * VEC)));
              xsrc[j] = ok ? real : zsrc + lane * 16;
            }
#pragma unroll
            for (int j = 0; j < PER; ++j) load_to_lds_16(xsrc[j], __builtin_amdgcn_readfirstlane(xdst + j * 1024));
          }
          if (q < 2) {  // pairs of step r + DP: wave 4 the input rows, wave 5 the output rows
            const int numP = step_identity(dP.x) ? 0 : step_num(dP.x);
            const int32_t* list = q == 0 ? a.in_maps : a.out_maps;
            // lanes past the step's pairs repeat its last pair (never used); empty steps read zeros
            const uint8_t* pbase = numP > 0 ? (const uint8_t*)(list + (int64_t)dP.y) : zsrc;
            const uint32_t poff = (uint32_t)(numP > 0 ? (lane < numP ? lane : numP - 1) : lane) * 4u;
            const uint32_t pdst = lds_offset(q == 0 ? s_pin : s_pout) +
                                  (uint32_t)(C::pslot(r + DP) * STEP_ROWS * 4);
            load_to_lds_4(pbase, poff, __builtin_amdgcn_readfirstlane(pdst));
          }
          if (q == NP - 2) {  // slot table of step r + DG
            int32_t pub_in = identG ? (int32_t)(m0 + firstG + lane) : pin_l;
            const int pub_out = identG ? firstG + lane : (int)(pout_l - m0);
            if (lane >= numG) pub_in = -1;
            if ((uint32_t)pub_in < (uint64_t)a.num_in && (uint32_t)pub_out < (uint32_t)tile_rows)
              s_tab[C::tslot(gi) * RROWS + C::tab_index(pub_out)] = (uint8_t)lane;
          } else if (q == NP - 1) {  // the slot table after it starts empty
            for (int i = lane; i < RROWS / 4; i += 64)
              ((uint32_t*)(s_tab + C::tslot(gi + 1) * RROWS))[i] = 0xFFFFFFFFu;
          }
          iw = iw + 1 == W_SLOTS ? 0 : iw + 1;
          ia = ia + 1 == A_SLOTS ? 0 : ia + 1;
        }
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the loads of the empty steps after the last one
    __syncthreads();  // every wave is done with the rings, every load has landed
  }
  if (staged) {
    __syncthreads();
    for (int v = tid; v < RROWS * 8; v += RING_THREADS) {
      const int r = v >> 3, part = v & 7;
      if (m0 + r < a.num_out && n0 + part * VEC < a.c_out)
        *reinterpret_cast<u32x4*>(out + (m0 + r) * a.c_out + n0 + part * VEC) =
            *reinterpret_cast<const u32x4*>(&stage[r * CK + lds_part(r, part) * VEC]);
    }
  }
}

// out[m][c] = bias[c] + the slices' partial sums added in slice order, rounded once (one thread per
// four channels).
template <typename T>
__global__ void __launch_bounds__(256) conv_split_reduce(const float* __restrict__ partial, int slices,
                                                         int64_t num_out, int c_out, int c_out_pad,
                                                         const T* __restrict__ bias, T* __restrict__ out,
                                                         const void* residual, int relu) {
  const int quads = c_out_pad / 4;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= num_out * quads) return;
  const int64_t m = i / quads;
  const int col = (int)(i % quads) * 4;
  if (col >= c_out) return;
  f32x4 sum = (f32x4){0.f, 0.f, 0.f, 0.f};
  for (int z = 0; z < slices; ++z)
    sum += *reinterpret_cast<const f32x4*>(partial + ((int64_t)z * num_out + m) * c_out_pad + col);
#pragma unroll
  for (int r = 0; r < 4; ++r)
    if (col + r < c_out)
      out[m * c_out + col + r] = from_float<T>(finish_sum<T>(sum[r] + (bias ? to_float(bias[col + r]) : 0.f),
                                                             residual, relu, m, c_out, col + r));
}

// group_start[k][g] = number of pairs of offset k with out_maps < 64 * g (binary search; needs
// out_maps ascending inside every offset).
__global__ void __launch_bounds__(256) conv_group_start(const int32_t* __restrict__ out_maps,
                                                        const int64_t* __restrict__ offsets, int K,
                                                        int64_t G, int32_t* __restrict__ gs) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)K * (G + 1)) return;
  const int k = (int)(i / (G + 1));
  const int64_t g = i % (G + 1);
  const int64_t lo0 = offsets[k];
  int64_t lo = lo0, hi = offsets[k + 1];
  const int64_t target = g * 64;
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if ((int64_t)out_maps[mid] < target) lo = mid + 1; else hi = mid;
  }
  gs[i] = (int32_t)(lo - lo0);
}

// ---- pair lists -> output-row form (for maps that were not built by wcn_kmap_fill) ---------------

__device__ __forceinline__ int offset_of_pair(const int64_t* __restrict__ offsets, int K, int64_t p) {
  int lo = 0, hi = K;  // largest k with offsets[k] <= p
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (offsets[mid] <= p) lo = mid; else hi = mid;
  }
  return lo;
}

__global__ void __launch_bounds__(256) rows_clear(uint32_t* __restrict__ words, int64_t n, uint32_t value) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x)
    words[i] = value;
}

__global__ void __launch_bounds__(256) rows_mark(const int32_t* __restrict__ out_maps,
                                                 const int64_t* __restrict__ offsets, int K,
                                                 int words, int64_t num_out,
                                                 uint32_t* __restrict__ row_mask) {
  const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= offsets[K]) return;
  const int k = offset_of_pair(offsets, K, p);
  const int32_t o = out_maps[p];
  if ((uint32_t)o < (uint64_t)num_out) atomicOr(&row_mask[(int64_t)o * words + (k >> 5)], 1u << (k & 31));
}

template <bool WRITE_PTR>
__global__ void __launch_bounds__(256) rows_count(const uint32_t* __restrict__ row_mask, int words,
                                                  int64_t num_out, int32_t* __restrict__ groups,
                                                  int32_t* __restrict__ row_ptr) {
  const int64_t m = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t group = m >> 6;
  if (group >= (num_out + 63) / 64) return;
  int cnt = 0;
  if (m < num_out)
    for (int w = 0; w < words; ++w) cnt += __popc(row_mask[m * words + w]);
  const int incl = wcn_wave_inclusive_sum(cnt);
  if (!WRITE_PTR) {
    if (wcn_lane() == 63) groups[group] = incl;
  } else if (m < num_out) {
    row_ptr[m] = groups[group] + incl - cnt;
    if (m == num_out - 1) row_ptr[num_out] = groups[group] + incl;
  }
}

__global__ void __launch_bounds__(256) rows_fill(const int32_t* __restrict__ in_maps,
                                                 const int32_t* __restrict__ out_maps,
                                                 const int64_t* __restrict__ offsets, int K,
                                                 int words, int64_t num_out,
                                                 const uint32_t* __restrict__ row_mask,
                                                 const int32_t* __restrict__ row_ptr,
                                                 int32_t* __restrict__ row_in) {
  // row_in starts at INT32_MAX everywhere: of several pairs with the same (offset, output row),
  // which a kernel map never holds but a caller's lists may, the lowest input row survives,
  // whatever order the threads run in.
  const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= offsets[K]) return;
  const int k = offset_of_pair(offsets, K, p);
  const int32_t o = out_maps[p];
  if ((uint32_t)o >= (uint64_t)num_out) return;
  const uint32_t* mw = row_mask + (int64_t)o * words;
  int rank = 0;
  for (int w = 0; w < (k >> 5); ++w) rank += __popc(mw[w]);
  rank += __popc(mw[k >> 5] & ((1u << (k & 31)) - 1u));
  atomicMin(&row_in[row_ptr[o] + rank], in_maps[p]);
}

// The re-ordering of pair lists (pairs_sort_by_out) needs no row form in between.  First the rows of
// every 64-row group that carry offset k, as a count (scanned afterwards into group_start) and as a
// 64-bit mask ...
__global__ void __launch_bounds__(256) pairs_group_hits(const uint32_t* __restrict__ row_mask, int K,
                                                        int words, int64_t num_out,
                                                        int32_t* __restrict__ gs, int64_t G,
                                                        unsigned long long* __restrict__ hits) {
  const int64_t m = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t group = m >> 6;
  if (group >= G) return;
  const int lane = wcn_lane();
  const bool live = m < num_out;
  for (int w = 0; w < words; ++w) {
    const uint32_t word = live ? row_mask[m * words + w] : 0u;
    const int nbits = K - w * 32 < 32 ? K - w * 32 : 32;
    for (int b = 0; b < nbits; ++b) {
      const int k = w * 32 + b;
      const unsigned long long h = __ballot((word >> b) & 1u);
      if (lane == 0) {
        gs[(int64_t)k * (G + 1) + group] = __popcll(h);
        hits[group * K + k] = h;
      }
    }
  }
}

// ... from which every pair finds its place by itself: behind the pairs of its offset whose output
// row is lower.  in_sorted starts at INT32_MAX everywhere: of several pairs with the same (offset,
// output row), which a kernel map never holds but a caller's lists may, the lowest input row
// survives, whatever order the threads run in.
__global__ void __launch_bounds__(256) pairs_place(const int32_t* __restrict__ in_maps,
                                                   const int32_t* __restrict__ out_maps,
                                                   const int64_t* __restrict__ offsets, int K,
                                                   int64_t num_out, const int32_t* __restrict__ gs,
                                                   int64_t G, const unsigned long long* __restrict__ hits,
                                                   int32_t* __restrict__ in_sorted,
                                                   int32_t* __restrict__ out_sorted) {
  const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= offsets[K]) return;
  const int k = offset_of_pair(offsets, K, p);
  const int32_t o = out_maps[p];
  if ((uint32_t)o >= (uint64_t)num_out) return;
  const int64_t group = o >> 6;
  const unsigned long long h = hits[group * K + k];
  const int64_t dest = offsets[k] + gs[(int64_t)k * (G + 1) + group] + __popcll(h & ((1ull << (o & 63)) - 1ull));
  atomicMin(&in_sorted[dest], in_maps[p]);
  out_sorted[dest] = o;
}

// Two ranges of words set to two values in one launch.
__global__ void __launch_bounds__(256) rows_clear_two(uint32_t* __restrict__ a, int64_t n_a, uint32_t value_a,
                                                      uint32_t* __restrict__ b, int64_t n_b, uint32_t value_b) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_a + n_b;
       i += (int64_t)gridDim.x * blockDim.x) {
    if (i < n_a) a[i] = value_a; else b[i - n_a] = value_b;
  }
}

inline int round_up(int x, int m) { return (x + m - 1) / m * m; }
inline size_t elem_size(int dtype) { return dtype == WCN_DTYPE_F32 ? 4 : 2; }
inline int ck_of(int dtype) { return dtype == WCN_DTYPE_F32 ? Mma<float>::CK : Mma<_Float16>::CK; }

// Slices of input channels go to separate workgroups when the output tiles alone would leave most
// of the 256 CUs (two workgroups each) idle.
inline bool conv_wants_split(int64_t num_out, int c_in_pad, int c_out_pad, int ck) {
  const int64_t tiles = (num_out + 64 * WCN_RING_NC - 1) / (64 * WCN_RING_NC) * (c_out_pad / TN);
  return c_in_pad / ck > 1 && tiles <= 256;
}

struct ConvWorkspace {
  int64_t* offsets;      // K+1 (device copy of the host offsets)
  void* Wt;              // K * c_out_pad * c_in_pad elements
  void* zeros;           // 1 KiB
  int32_t* group_start;  // (K, G+1), when not supplied by the caller
  int64_t* row_total;    // K+1 scratch of the scans
  uint32_t* row_mask;    // the rest only when the pair lists have to be re-ordered here
  unsigned long long* hits;
  int32_t* in_sorted;
  int32_t* out_sorted;
  float* partial;        // (slices, num_out, c_out_pad) when the input-channel slices are split
  int c_in_pad, c_out_pad, words;
  int64_t G;
};

inline size_t conv_layout(void* base, int64_t num_out, int K, int c_in, int c_out, int dtype,
                          int64_t resort_pairs, ConvWorkspace* w) {
  char* p = (char*)base;
  size_t off = 0;
  const int64_t G = (num_out + 63) / 64;
  const int words = (K + 31) / 32;
  const int cip = round_up(c_in, ck_of(dtype)), cop = round_up(c_out, TN);
  if (w) w->offsets = (int64_t*)(p + off);
  off += wcn_align256(sizeof(int64_t) * (size_t)(K + 1));
  if (w) w->Wt = (void*)(p + off);
  off += wcn_align256(elem_size(dtype) * (size_t)K * cop * cip);
  if (w) w->zeros = (void*)(p + off);
  off += 1024;
  if (w) w->group_start = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * (size_t)K * (size_t)(G + 1));
  if (w) w->row_total = (int64_t*)(p + off);
  off += wcn_align256(sizeof(int64_t) * (size_t)(K + 1));
  if (w) w->partial = nullptr;
  if (conv_wants_split(num_out, cip, cop, ck_of(dtype))) {
    if (w) w->partial = (float*)(p + off);
    off += wcn_align256(sizeof(float) * (size_t)(cip / ck_of(dtype)) * (size_t)num_out * cop);
  }
  if (resort_pairs >= 0) {
    if (w) w->row_mask = (uint32_t*)(p + off);
    off += wcn_align256(sizeof(uint32_t) * (size_t)num_out * words);
    if (w) w->hits = (unsigned long long*)(p + off);
    off += wcn_align256(sizeof(unsigned long long) * (size_t)K * (size_t)G);
    if (w) w->in_sorted = (int32_t*)(p + off);
    off += wcn_align256(sizeof(int32_t) * (size_t)resort_pairs);
    if (w) w->out_sorted = (int32_t*)(p + off);
    off += wcn_align256(sizeof(int32_t) * (size_t)resort_pairs);
  }
  if (w) {
    w->G = G;
    w->c_in_pad = cip;
    w->c_out_pad = cop;
    w->words = words;
  }
  return off;
}

// Optional timing hook: events armed by wcn_conv_set_timing_events bracket the next conv_fwd
// launch of this thread (and only that kernel), then disarm.
thread_local hipEvent_t g_time_start = nullptr;
thread_local hipEvent_t g_time_stop = nullptr;

// Weight tiles, the block of zeros and (when given) the map's offsets: first launch of every call.
template <typename T>
void launch_prep(const ConvArgs& a, const void* weight, int weight_dtype, int dtype, int as_stored,
                 int flip_k, const int64_t* host_offsets_or_null, hipStream_t s) {
  OffsetsByValue ov;
  const int n_ov = host_offsets_or_null ? a.K + 1 : 0;
  for (int i = 0; i < OFFSETS_BY_VALUE; ++i) ov.v[i] = i < n_ov ? host_offsets_or_null[i] : 0;
  const int64_t total = (int64_t)a.K * a.c_out_pad * a.c_in_pad;
  const int pgrid = (int)std::min<int64_t>(4096, (total + 255) / 256);
  if (weight_dtype == dtype) {
    hipLaunchKernelGGL((conv_prep_weight<T, T>), dim3(pgrid), dim3(256), 0, s, (const T*)weight,
                       a.K, a.c_in, a.c_out, a.c_in_pad, a.c_out_pad, as_stored, flip_k, (T*)a.Wt,
                       (uint32_t*)a.zeros, const_cast<int64_t*>(a.offsets), n_ov, ov);
  } else {
    hipLaunchKernelGGL((conv_prep_weight<T, float>), dim3(pgrid), dim3(256), 0, s,
                       (const float*)weight, a.K, a.c_in, a.c_out, a.c_in_pad, a.c_out_pad,
                       as_stored, flip_k, (T*)a.Wt, (uint32_t*)a.zeros, const_cast<int64_t*>(a.offsets),
                       n_ov, ov);
  }
}

template <typename T>
int launch_conv(const ConvArgs& a, hipStream_t s) {
  constexpr int dtype = std::is_same<T, float>::value ? WCN_DTYPE_F32
                        : std::is_same<T, _Float16>::value ? WCN_DTYPE_F16 : WCN_DTYPE_BF16;
  // Wide rows on both sides go to the output-stationary kernel of wcn_conv_dense.hip, 16-bit rows of
  // at most 32 channels on both sides to the kernel of wcn_conv_group.hip, rows of up to four
  // k-slices to the pair-packed kernel.  WCN_CONV_KERNEL=ring in the environment keeps everything on
  // the kernels below, WCN_CONV_KERNEL=pack skips the first two of the three (for comparisons).
  // (read at every call, a fraction of a microsecond, so that one process can compare them)
  const char* const choice = getenv("WCN_CONV_KERNEL");
  const int only = !choice ? 0 : strcmp(choice, "ring") == 0 ? 1 : strcmp(choice, "pack") == 0 ? 2 : 0;
  const bool ring_only = only == 1;
  if (only == 0 && wcn_conv_dense_takes(a, dtype)) {
    if (g_time_start) (void)hipEventRecord(g_time_start, s);
    const int st = wcn_conv_dense_launch(a, dtype, s);
    if (g_time_stop) (void)hipEventRecord(g_time_stop, s);
    g_time_start = g_time_stop = nullptr;
    return st;
  }
  if (only == 0 && wcn_conv_group_takes(a, dtype)) {
    if (g_time_start) (void)hipEventRecord(g_time_start, s);
    const int st = wcn_conv_group_launch(a, dtype, s);
    if (g_time_stop) (void)hipEventRecord(g_time_stop, s);
    g_time_start = g_time_stop = nullptr;
    return st;
  }
  if (!ring_only && wcn_conv_pack_takes(a, dtype)) {
    if (g_time_start) (void)hipEventRecord(g_time_start, s);
    const int st = wcn_conv_pack_launch(a, dtype, s);
    if (g_time_stop) (void)hipEventRecord(g_time_stop, s);
    g_time_start = g_time_stop = nullptr;
    return st;
  }
  const dim3 grid((unsigned)((a.num_out + ROWS - 1) / ROWS), (unsigned)(a.c_out_pad / TN));
  constexpr int NC = WCN_RING_NC;  // multiplying waves per workgroup of the ring kernel
  if (a.vec_in) {
    // more than 64 KiB of dynamic LDS has to be allowed once per device
    static thread_local int allowed_device = -1;
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) return WCN_ERR_LAUNCH;
    if (allowed_device != device) {
      const void* instances[5] = {(const void*)conv_fwd_ring<T, NC, false, 0>, (const void*)conv_fwd_ring<T, NC, false, 1>,
                                  (const void*)conv_fwd_ring<T, NC, false, 2>, (const void*)conv_fwd_ring<T, NC, false, 3>,
                                  (const void*)conv_fwd_ring<T, NC, true, 0>};
      for (const void* f : instances)
        if (hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, RingCfg<NC>::LDS_BYTES) != hipSuccess)
          return WCN_ERR_LAUNCH;
      allowed_device = device;
    }
  }
  if (g_time_start) (void)hipEventRecord(g_time_start, s);
  if (a.vec_in) {
    const unsigned slices = a.split ? (unsigned)(a.c_in_pad / Mma<T>::CK) : 1u;
    const dim3 rgrid((unsigned)((a.num_out + RingCfg<NC>::RROWS - 1) / RingCfg<NC>::RROWS), grid.y, slices);
    // channel counts of at most half a tile leave out the padding half of the multiplications
    const int narrow = (a.c_out <= TN / 2 ? 1 : 0) | (a.c_in <= Mma<T>::CK / 2 ? 2 : 0);
    if (a.split)
      hipLaunchKernelGGL((conv_fwd_ring<T, NC, true, 0>), rgrid, dim3(RING_THREADS), RingCfg<NC>::LDS_BYTES, s, a);
    else if (narrow == 0)
      hipLaunchKernelGGL((conv_fwd_ring<T, NC, false, 0>), rgrid, dim3(RING_THREADS), RingCfg<NC>::LDS_BYTES, s, a);
    else if (narrow == 1)
      hipLaunchKernelGGL((conv_fwd_ring<T, NC, false, 1>), rgrid, dim3(RING_THREADS), RingCfg<NC>::LDS_BYTES, s, a);
    else if (narrow == 2)
      hipLaunchKernelGGL((conv_fwd_ring<T, NC, false, 2>), rgrid, dim3(RING_THREADS), RingCfg<NC>::LDS_BYTES, s, a);
    else
      hipLaunchKernelGGL((conv_fwd_ring<T, NC, false, 3>), rgrid, dim3(RING_THREADS), RingCfg<NC>::LDS_BYTES, s, a);
    wcn_conv_note_kernel("conv_fwd_ring<%s, %d, %s, %d>", wcn_type_text<T>(), NC, a.split ? "true" : "false",
                         a.split ? 0 : narrow);
    if (a.split) {
      const int64_t items = a.num_out * (a.c_out_pad / 4);
      hipLaunchKernelGGL(conv_split_reduce<T>, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, s,
                         (const float*)a.partial, (int)slices, a.num_out, a.c_out, a.c_out_pad,
                         (const T*)a.bias, (T*)a.out, a.residual, a.relu);
    }
  } else {
    hipLaunchKernelGGL(conv_fwd<T>, grid, dim3(THREADS), 0, s, a);
    wcn_conv_note_kernel("conv_fwd<%s>", wcn_type_text<T>());
  }
  if (g_time_stop) (void)hipEventRecord(g_time_stop, s);
  g_time_start = g_time_stop = nullptr;
  WCN_LAUNCH_CHECK();
  return WCN_OK;
}

}  // namespace

size_t wcn_rows_layout(void* base, int64_t num_out, int num_offsets, int64_t pairs, WcnRowsView* v) {
  char* p = (char*)base;
  size_t off = 0;
  const int64_t G = (num_out + 63) / 64;
  const int words = (num_offsets + 31) / 32;
  if (v) v->offsets = (int64_t*)(p + off);
  off += wcn_align256(sizeof(int64_t) * (size_t)(num_offsets + 1));
  if (v) v->row_mask = (uint32_t*)(p + off);
  off += wcn_align256(sizeof(uint32_t) * (size_t)num_out * words);
  if (v) v->row_ptr = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * (size_t)(num_out + 1));
  if (v) v->row_in = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * (size_t)pairs);
  if (v) v->groups = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * (size_t)(G + 1));
  if (v) v->row_total = (int64_t*)(p + off);
  off += 256;
  if (v) {
    v->words = words;
    v->G = G;
  }
  return off;
}

int wcn_rows_build(const int32_t* in_maps, const int32_t* out_maps, int num_offsets, int64_t num_out,
                   int64_t pairs, const WcnRowsView& v, hipStream_t s) {
  const unsigned rows_grid = (unsigned)((num_out + 255) / 256);
  const int64_t mask_words = num_out * v.words;
  hipLaunchKernelGGL(rows_clear, dim3((unsigned)std::min<int64_t>(4096, (mask_words + 255) / 256)),
                     dim3(256), 0, s, v.row_mask, mask_words, 0u);
  if (pairs > 0)
    hipLaunchKernelGGL(rows_clear, dim3((unsigned)std::min<int64_t>(4096, (pairs + 255) / 256)),
                       dim3(256), 0, s, (uint32_t*)v.row_in, pairs, 0x7fffffffu);
  if (pairs > 0)
    hipLaunchKernelGGL(rows_mark, dim3((unsigned)((pairs + 255) / 256)), dim3(256), 0, s, out_maps,
                       (const int64_t*)v.offsets, num_offsets, v.words, num_out, v.row_mask);
  hipLaunchKernelGGL(rows_count<false>, dim3(rows_grid), dim3(256), 0, s,
                     (const uint32_t*)v.row_mask, v.words, num_out, v.groups, v.row_ptr);
  wcn_scan_rows_launch(v.groups, v.G, 1, v.row_total, s);
  hipLaunchKernelGGL(rows_count<true>, dim3(rows_grid), dim3(256), 0, s,
                     (const uint32_t*)v.row_mask, v.words, num_out, v.groups, v.row_ptr);
  if (pairs > 0)
    hipLaunchKernelGGL(rows_fill, dim3((unsigned)((pairs + 255) / 256)), dim3(256), 0, s, in_maps,
                       out_maps, (const int64_t*)v.offsets, num_offsets, v.words, num_out,
                       (const uint32_t*)v.row_mask, (const int32_t*)v.row_ptr, v.row_in);
  WCN_LAUNCH_CHECK();
  return WCN_OK;
}

namespace {
thread_local char g_last_kernel[160] = "";
}
void wcn_conv_note_kernel(const char* format, ...) {
  va_list ap;
  va_start(ap, format);
  vsnprintf(g_last_kernel, sizeof(g_last_kernel), format, ap);
  va_end(ap);
}

extern "C" {

const char* wcn_conv_last_kernel(void) { return g_last_kernel; }

int wcn_conv_set_timing_events(void* start_event, void* stop_event) {
  g_time_start = (hipEvent_t)start_event;
  g_time_stop = (hipEvent_t)stop_event;
  return WCN_OK;
}

// pair lists -> pair lists ascending in output row inside every offset, with their group_start
// table.  Of several pairs with the same (offset, output row) one is kept.  Five launches: clear,
// mark the (row, offset) bits, per-group counts and masks, scan, place.
static void pairs_sort_by_out(const int32_t* in_maps, const int32_t* out_maps, const int64_t* offsets_dev,
                              int K, int64_t num_out, int64_t L, uint32_t* row_mask,
                              unsigned long long* hits, int64_t* row_total, int32_t* in_sorted,
                              int32_t* out_sorted, int32_t* group_start, hipStream_t s) {
  const int words = (K + 31) / 32;
  const int64_t G = (num_out + 63) / 64;
  const unsigned rows_grid = (unsigned)((num_out + 255) / 256);
  const int64_t mask_words = num_out * words;
  hipLaunchKernelGGL(rows_clear_two, dim3((unsigned)std::min<int64_t>(4096, (mask_words + L + 255) / 256)),
                     dim3(256), 0, s, row_mask, mask_words, 0u, (uint32_t*)in_sorted, L, 0x7fffffffu);
  if (L > 0)
    hipLaunchKernelGGL(rows_mark, dim3((unsigned)((L + 255) / 256)), dim3(256), 0, s, out_maps,
                       offsets_dev, K, words, num_out, row_mask);
  hipLaunchKernelGGL(pairs_group_hits, dim3(rows_grid), dim3(256), 0, s, (const uint32_t*)row_mask, K,
                     words, num_out, group_start, G, hits);
  wcn_scan_rows_launch(group_start, G, K, row_total, s);
  if (L > 0)
    hipLaunchKernelGGL(pairs_place, dim3((unsigned)((L + 255) / 256)), dim3(256), 0, s, in_maps, out_maps,
                       offsets_dev, K, num_out, (const int32_t*)group_start, G,
                       (const unsigned long long*)hits, in_sorted, out_sorted);
}

struct SortWorkspace {
  int64_t* offsets;
  int64_t* row_total;
  uint32_t* row_mask;
  unsigned long long* hits;
};

inline size_t sort_layout(void* base, int64_t num_out, int K, int64_t L, SortWorkspace* w) {
  char* p = (char*)base;
  size_t off = 0;
  const int64_t G = (num_out + 63) / 64;
  const int words = (K + 31) / 32;
  if (w) w->offsets = (int64_t*)(p + off);
  off += wcn_align256(sizeof(int64_t) * (size_t)(K + 1));
  if (w) w->row_total = (int64_t*)(p + off);
  off += wcn_align256(sizeof(int64_t) * (size_t)(K + 1));
  if (w) w->row_mask = (uint32_t*)(p + off);
  off += wcn_align256(sizeof(uint32_t) * (size_t)num_out * words);
  if (w) w->hits = (unsigned long long*)(p + off);
  off += wcn_align256(sizeof(unsigned long long) * (size_t)K * (size_t)G);
  return off;
}

__global__ void offsets_store(OffsetsByValue ov, int n, int64_t* __restrict__ dst) {
  if ((int)threadIdx.x < n) dst[threadIdx.x] = ov.v[threadIdx.x];
}

size_t wcn_conv_workspace_bytes(int64_t num_out, int32_t num_offsets, int32_t c_in, int32_t c_out,
                                int32_t dtype, int64_t num_pairs, int32_t out_maps_ascend) {
  if (num_out < 0 || num_offsets < 1 || num_offsets > WCN_MAX_OFFSETS || c_in < 1 || c_out < 1 ||
      dtype < 0 || dtype > 2 || num_pairs < 0)
    return 0;
  return conv_layout(nullptr, num_out, num_offsets, c_in, c_out, dtype,
                     out_maps_ascend ? -1 : num_pairs, nullptr);
}

// 1 KiB of zeros that no kernel writes (the source of loads that have nothing to fetch), for calls
// that bring prepared weight tiles and so run no preparation kernel that could write such a block
// into the workspace.  Host code uses the address hipGetSymbolAddress reports for the current
// device, never the array's name.
static __device__ __align__(256) uint32_t zero_page[256];

namespace {
std::mutex g_zero_page_mutex;
void* g_zero_page_ptr[64] = {};

int static_zero_page(void** ptr) {
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return WCN_ERR_LAUNCH;
  std::lock_guard<std::mutex> hold(g_zero_page_mutex);
  if (!g_zero_page_ptr[device]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(zero_page)) != hipSuccess || !p) return WCN_ERR_LAUNCH;
    g_zero_page_ptr[device] = p;
  }
  *ptr = g_zero_page_ptr[device];
  return WCN_OK;
}
}  // namespace

size_t wcn_conv_prepared_workspace_bytes(int64_t num_out, int32_t num_offsets, int32_t c_in, int32_t c_out,
                                         int32_t dtype) {
  if (num_out < 0 || num_offsets < 1 || num_offsets > WCN_MAX_OFFSETS || c_in < 1 || c_out < 1 ||
      dtype < 0 || dtype > 2)
    return 0;
  const int cip = round_up(c_in, ck_of(dtype)), cop = round_up(c_out, TN);
  if (!conv_wants_split(num_out, cip, cop, ck_of(dtype))) return 0;
  return wcn_align256(sizeof(float) * (size_t)(cip / ck_of(dtype)) * (size_t)num_out * cop);
}

// Shared body of the forward product and the input gradient.  weight_as_stored / flip_offsets
// choose how the caller's weight becomes the kernels' tiles (see conv_prep_weight).  With
// `no_copy_commands` the call enqueues kernels only (the offsets must then fit the kernel
// arguments of the weight preparation).
static int conv_run(const void* features, int64_t num_in, int32_t c_in, int32_t dtype,
                    const void* weight, int32_t weight_dtype, int32_t num_offsets, int32_t c_out,
                    const void* bias_or_null, const int32_t* in_maps, const int32_t* out_maps,
                    const int64_t* host_offsets, int32_t identity_offset, int32_t out_maps_ascend,
                    const int32_t* group_start_or_null, void* out, int64_t num_out,
                    void* workspace, size_t workspace_bytes, int weight_as_stored,
                    int flip_offsets, bool no_copy_commands, void* stream,
                    const void* residual_or_null = nullptr, int relu = 0,
                    const int64_t* device_offsets_of_prepared = nullptr) {
  // With device_offsets_of_prepared, `weight` is the tiles wcn_conv_prepare_weight made and the
  // call enqueues nothing but the contraction.
  const bool prepared = device_offsets_of_prepared != nullptr;
  if (dtype < 0 || dtype > 2 || (!prepared && weight_dtype != dtype && weight_dtype != WCN_DTYPE_F32))
    return WCN_ERR_INVALID_ARGUMENT;
  if (prepared && (!out_maps_ascend || !group_start_or_null)) return WCN_ERR_INVALID_ARGUMENT;
  if (num_in < 0 || num_out < 0 || num_offsets < 1 || num_offsets > WCN_MAX_OFFSETS || c_in < 1 ||
      c_out < 1 || !weight || (!workspace && !prepared) || !host_offsets)
    return WCN_ERR_INVALID_ARGUMENT;
  if (num_in >= (1ll << 31) || num_out >= (1ll << 31)) return WCN_ERR_INVALID_ARGUMENT;
  if (identity_offset >= num_offsets) return WCN_ERR_INVALID_ARGUMENT;
  if (group_start_or_null && !out_maps_ascend) return WCN_ERR_INVALID_ARGUMENT;
  const int64_t L = host_offsets[num_offsets];
  if (host_offsets[0] != 0 || L < 0 || L > INT32_MAX) return WCN_ERR_INVALID_ARGUMENT;
  for (int k = 0; k < num_offsets; ++k)
    if (host_offsets[k + 1] < host_offsets[k]) return WCN_ERR_INVALID_ARGUMENT;
  if (L > 0 && (!in_maps || !out_maps)) return WCN_ERR_INVALID_ARGUMENT;
  if (num_out == 0) return WCN_OK;
  if (!out || (num_in > 0 && !features)) return WCN_ERR_INVALID_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  ConvWorkspace w;
  if (prepared) {
    // tiles, zeros, offsets and group starts all come from elsewhere: the workspace is the partial
    // sums of split input-channel slices, where the problem's shape asks for them, and nothing else
    const size_t need = wcn_conv_prepared_workspace_bytes(num_out, num_offsets, c_in, c_out, dtype);
    if (need > 0 && (!workspace || workspace_bytes < need)) return WCN_ERR_WORKSPACE;
    conv_layout(nullptr, num_out, num_offsets, c_in, c_out, dtype, -1, &w);
    w.partial = need > 0 ? (float*)workspace : nullptr;
  } else {
    if (workspace_bytes <
        wcn_conv_workspace_bytes(num_out, num_offsets, c_in, c_out, dtype, L, out_maps_ascend))
      return WCN_ERR_WORKSPACE;
    conv_layout(workspace, num_out, num_offsets, c_in, c_out, dtype, out_maps_ascend ? -1 : L, &w);
  }
  // Up to 127 offsets reach the device in the arguments of the weight preparation, which is the
  // first launch of the call: no copy command.
  const bool offsets_by_value = num_offsets + 1 <= OFFSETS_BY_VALUE;
  if (!offsets_by_value && !prepared) {
    if (no_copy_commands) return WCN_ERR_INVALID_ARGUMENT;
    if (hipMemcpyAsync(w.offsets, host_offsets, sizeof(int64_t) * (size_t)(num_offsets + 1),
                       hipMemcpyHostToDevice, s) != hipSuccess)
      return WCN_ERR_LAUNCH;
  }

  ConvArgs a;
  a.offsets = w.offsets;
  a.X = features;
  a.Wt = w.Wt;
  a.zeros = w.zeros;
  a.bias = bias_or_null;
  a.residual = residual_or_null;
  a.relu = relu ? 1 : 0;
  a.out = out;
  a.num_in = num_in;
  a.num_out = num_out;
  a.num_pairs = L;
  a.G = w.G;
  a.K = num_offsets;
  a.c_in = c_in;
  a.c_out = c_out;
  a.c_in_pad = w.c_in_pad;
  a.c_out_pad = w.c_out_pad;
  a.identity = identity_offset;
  const int64_t* by_value = offsets_by_value ? host_offsets : nullptr;
  if (prepared) {
    void* zero_page_address = nullptr;
    if (const int st = static_zero_page(&zero_page_address)) return st;
    a.Wt = weight;
    a.zeros = zero_page_address;
    a.offsets = device_offsets_of_prepared;
  } else {
    switch (dtype) {
      case WCN_DTYPE_F32:
        launch_prep<float>(a, weight, weight_dtype, dtype, weight_as_stored, flip_offsets, by_value, s);
        break;
      case WCN_DTYPE_F16:
        launch_prep<_Float16>(a, weight, weight_dtype, dtype, weight_as_stored, flip_offsets, by_value, s);
        break;
      default:
        launch_prep<__bf16>(a, weight, weight_dtype, dtype, weight_as_stored, flip_offsets, by_value, s);
        break;
    }
  }

  a.in_maps = in_maps;
  a.out_maps = out_maps;
  a.group_start = group_start_or_null;
  if (!out_maps_ascend) {
    pairs_sort_by_out(in_maps, out_maps, (const int64_t*)w.offsets, num_offsets, num_out, L, w.row_mask,
                      w.hits, w.row_total, w.in_sorted, w.out_sorted, w.group_start, s);
    a.in_maps = w.in_sorted;
    a.out_maps = w.out_sorted;
    a.group_start = w.group_start;
  } else if (!a.group_start) {
    const int64_t items = (int64_t)num_offsets * (w.G + 1);
    hipLaunchKernelGGL(conv_group_start, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, s,
                       out_maps, (const int64_t*)w.offsets, num_offsets, w.G, w.group_start);
    a.group_start = w.group_start;
  }
  const size_t es = elem_size(dtype);
  a.vec_in = (((size_t)c_in * es) % 16 == 0 && ((uintptr_t)features % 16) == 0) ? 1 : 0;
  a.vec_out = (((size_t)c_out * es) % 16 == 0 && ((uintptr_t)out % 16) == 0) ? 1 : 0;
  a.vec_res = (a.residual && ((size_t)c_out * es) % 16 == 0 && ((uintptr_t)a.residual % 16) == 0) ? 1 : 0;
  a.flat_in = (c_in % ck_of(dtype) == 0 && (uint64_t)num_in * c_in * es < (1ull << 32)) ? 1 : 0;
  a.partial = w.partial;
  a.split = (a.vec_in && w.partial != nullptr) ? 1 : 0;
  switch (dtype) {
    case WCN_DTYPE_F32:
      return launch_conv<float>(a, s);
    case WCN_DTYPE_F16:
      return launch_conv<_Float16>(a, s);
    default:
      return launch_conv<__bf16>(a, s);
  }
}

// ---- the contraction for callers that cannot allocate ------------------------------------------
// One device-resident scratch array per GPU serves as the workspace of wcn_sparse_conv_fwd_static.
// Host code never uses the array's name as an address: the per-device address comes from
// hipGetSymbolAddress, once per device, and is what the kernels receive.
static __device__ __align__(256) unsigned char scratch[WCN_CONV_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// Address of `scratch` on the current device (looked up on the first call on that device).
int static_scratch(void** ptr) {
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return WCN_ERR_LAUNCH;
  std::lock_guard<std::mutex> hold(g_scratch_mutex);
  if (!g_scratch_ptr[device]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return WCN_ERR_LAUNCH;
    g_scratch_ptr[device] = p;
  }
  *ptr = g_scratch_ptr[device];
  return WCN_OK;
}
}  // namespace

int wcn_sparse_conv_fwd_static(const void* features, int64_t num_in, int32_t c_in, int32_t dtype,
                               const void* weight, int32_t weight_dtype, int32_t num_offsets,
                               int32_t c_out, const void* bias_or_null, const int32_t* in_maps,
                               const int32_t* out_maps, const int64_t* host_offsets,
                               int32_t identity_offset, int32_t out_maps_ascend,
                               const int32_t* group_start_or_null, void* out, int64_t num_out,
                               void* stream) {
  if (!host_offsets || num_offsets < 1 || num_offsets + 1 > OFFSETS_BY_VALUE)
    return WCN_ERR_INVALID_ARGUMENT;
  const size_t need = wcn_conv_workspace_bytes(num_out, num_offsets, c_in, c_out, dtype,
                                               host_offsets[num_offsets], out_maps_ascend);
  if (need == 0) return WCN_ERR_INVALID_ARGUMENT;
  if (need > (size_t)WCN_CONV_STATIC_SCRATCH_BYTES) return WCN_ERR_WORKSPACE;
  void* ws = nullptr;
  const int st = static_scratch(&ws);
  if (st != WCN_OK) return st;
  return conv_run(features, num_in, c_in, dtype, weight, weight_dtype, num_offsets, c_out,
                  bias_or_null, in_maps, out_maps, host_offsets, identity_offset, out_maps_ascend,
                  group_start_or_null, out, num_out, ws, WCN_CONV_STATIC_SCRATCH_BYTES, 0, 0, true,
                  stream);
}

size_t wcn_pairs_sort_workspace_bytes(int64_t num_out, int32_t num_offsets, int64_t num_pairs) {
  if (num_out < 0 || num_offsets < 1 || num_offsets > WCN_MAX_OFFSETS || num_pairs < 0) return 0;
  return sort_layout(nullptr, num_out, num_offsets, num_pairs, nullptr);
}

int wcn_pairs_sort_by_out(const int32_t* in_maps, const int32_t* out_maps, const int64_t* host_offsets,
                          int32_t num_offsets, int64_t num_out, int32_t* in_sorted,
                          int32_t* out_sorted, int32_t* group_start, void* workspace,
                          size_t workspace_bytes, void* stream) {
  if (!host_offsets || num_offsets < 1 || num_offsets > WCN_MAX_OFFSETS || num_out < 0 ||
      num_out >= (1ll << 31) || !group_start || !workspace)
    return WCN_ERR_INVALID_ARGUMENT;
  const int64_t L = host_offsets[num_offsets];
  if (host_offsets[0] != 0 || L < 0 || L > INT32_MAX) return WCN_ERR_INVALID_ARGUMENT;
  for (int k = 0; k < num_offsets; ++k)
    if (host_offsets[k + 1] < host_offsets[k]) return WCN_ERR_INVALID_ARGUMENT;
  if (L > 0 && (!in_maps || !out_maps || !in_sorted || !out_sorted)) return WCN_ERR_INVALID_ARGUMENT;
  if (workspace_bytes < sort_layout(nullptr, num_out, num_offsets, L, nullptr)) return WCN_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  SortWorkspace w;
  sort_layout(workspace, num_out, num_offsets, L, &w);
  if (num_offsets + 1 <= OFFSETS_BY_VALUE) {
    OffsetsByValue ov;
    for (int i = 0; i < OFFSETS_BY_VALUE; ++i) ov.v[i] = i <= num_offsets ? host_offsets[i] : 0;
    hipLaunchKernelGGL(offsets_store, dim3(1), dim3(OFFSETS_BY_VALUE), 0, s, ov, num_offsets + 1, w.offsets);
  } else if (hipMemcpyAsync(w.offsets, host_offsets, sizeof(int64_t) * (size_t)(num_offsets + 1),
                            hipMemcpyHostToDevice, s) != hipSuccess) {
    return WCN_ERR_LAUNCH;
  }
  pairs_sort_by_out(in_maps, out_maps, w.offsets, num_offsets, num_out, L, w.row_mask, w.hits,
                    w.row_total, in_sorted, out_sorted, group_start, s);
  return hipGetLastError() == hipSuccess ? WCN_OK : WCN_ERR_LAUNCH;
}

int wcn_sparse_conv_fwd(const void* features, int64_t num_in, int32_t c_in, int32_t dtype,
                        const void* weight, int32_t weight_dtype, int32_t num_offsets,
                        int32_t c_out, const void* bias_or_null, const int32_t* in_maps,
                        const int32_t* out_maps, const int64_t* host_offsets,
                        int32_t identity_offset, int32_t out_maps_ascend,
                        const int32_t* group_start_or_null, void* out, int64_t num_out,
                        void* workspace, size_t workspace_bytes, void* stream) {
  return conv_run(features, num_in, c_in, dtype, weight, weight_dtype, num_offsets, c_out,
                  bias_or_null, in_maps, out_maps, host_offsets, identity_offset, out_maps_ascend,
                  group_start_or_null, out, num_out, workspace, workspace_bytes, 0, 0, false, stream);
}

int wcn_sparse_conv_fwd_fused(const void* features, int64_t num_in, int32_t c_in, int32_t dtype,
                              const void* weight, int32_t weight_dtype, int32_t num_offsets,
                              int32_t c_out, const void* bias_or_null, const int32_t* in_maps,
                              const int32_t* out_maps, const int64_t* host_offsets,
                              int32_t identity_offset, int32_t out_maps_ascend,
                              const int32_t* group_start_or_null, const void* residual_or_null,
                              int32_t relu, void* out, int64_t num_out, void* workspace,
                              size_t workspace_bytes, void* stream) {
  if (residual_or_null && residual_or_null == out) return WCN_ERR_INVALID_ARGUMENT;  // rows are read and written by different threads
  return conv_run(features, num_in, c_in, dtype, weight, weight_dtype, num_offsets, c_out,
                  bias_or_null, in_maps, out_maps, host_offsets, identity_offset, out_maps_ascend,
                  group_start_or_null, out, num_out, workspace, workspace_bytes, 0, 0, false, stream,
                  residual_or_null, relu);
}

size_t wcn_conv_prepared_weight_bytes(int32_t num_offsets, int32_t c_in, int32_t c_out, int32_t dtype) {
  if (num_offsets < 1 || num_offsets > WCN_MAX_OFFSETS || c_in < 1 || c_out < 1 || dtype < 0 || dtype > 2)
    return 0;
  return wcn_align256(elem_size(dtype) * (size_t)num_offsets * round_up(c_out, TN) *
                      round_up(c_in, ck_of(dtype)));
}

int wcn_conv_prepare_weight(const void* weight, int32_t weight_dtype, int32_t num_offsets, int32_t c_in,
                            int32_t c_out, int32_t dtype, void* prepared, size_t prepared_bytes,
                            void* stream) {
  const size_t need = wcn_conv_prepared_weight_bytes(num_offsets, c_in, c_out, dtype);
  if (need == 0 || !weight || !prepared || (weight_dtype != dtype && weight_dtype != WCN_DTYPE_F32))
    return WCN_ERR_INVALID_ARGUMENT;
  if (prepared_bytes < need) return WCN_ERR_WORKSPACE;
  ConvArgs a = {};
  a.K = num_offsets;
  a.c_in = c_in;
  a.c_out = c_out;
  a.c_in_pad = round_up(c_in, ck_of(dtype));
  a.c_out_pad = round_up(c_out, TN);
  a.Wt = prepared;  // zeros and offsets stay null: the kernel then writes the tiles only
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case WCN_DTYPE_F32: launch_prep<float>(a, weight, weight_dtype, dtype, 0, 0, nullptr, s); break;
    case WCN_DTYPE_F16: launch_prep<_Float16>(a, weight, weight_dtype, dtype, 0, 0, nullptr, s); break;
    default: launch_prep<__bf16>(a, weight, weight_dtype, dtype, 0, 0, nullptr, s); break;
  }
  return hipGetLastError() == hipSuccess ? WCN_OK : WCN_ERR_LAUNCH;
}

int wcn_sparse_conv_fwd_prepared(const void* features, int64_t num_in, int32_t c_in, int32_t dtype,
                                 const void* prepared_weight, size_t prepared_bytes,
                                 int32_t num_offsets, int32_t c_out, const void* bias_or_null,
                                 const int32_t* in_maps, const int32_t* out_maps,
                                 const int64_t* host_offsets, const int64_t* device_offsets,
                                 int32_t identity_offset, const int32_t* group_start,
                                 const void* residual_or_null, int32_t relu, void* out,
                                 int64_t num_out, void* workspace, size_t workspace_bytes,
                                 void* stream) {
  if (residual_or_null && residual_or_null == out) return WCN_ERR_INVALID_ARGUMENT;
  if (!device_offsets || !group_start) return WCN_ERR_INVALID_ARGUMENT;
  const size_t need = wcn_conv_prepared_weight_bytes(num_offsets, c_in, c_out, dtype);
  if (need == 0) return WCN_ERR_INVALID_ARGUMENT;
  if (prepared_bytes < need) return WCN_ERR_WORKSPACE;
  return conv_run(features, num_in, c_in, dtype, prepared_weight, dtype, num_offsets, c_out,
                  bias_or_null, in_maps, out_maps, host_offsets, identity_offset, 1, group_start, out,
                  num_out, workspace, workspace_bytes, 0, 0, true, stream, residual_or_null, relu,
                  device_offsets);
}

int wcn_conv_single_supported(int32_t dtype, int32_t c_in, int32_t c_out, int32_t num_offsets) {
  return wcn_conv_single_takes(dtype, c_in, c_out, num_offsets) ? 1 : 0;
}

int wcn_sparse_conv_fwd_single(const void* features, int64_t num_in, int32_t c_in, int32_t dtype,
                               const void* weight, int32_t weight_dtype, int32_t weight_is_prepared,
                               int32_t num_offsets, int32_t c_out, const void* bias_or_null,
                               const int32_t* in_maps, const int32_t* out_maps,
                               const int64_t* host_offsets, const void* residual_or_null, int32_t relu,
                               void* out, int64_t num_out, void* workspace, size_t workspace_bytes,
                               void* stream) {
  if (!wcn_conv_single_takes(dtype, c_in, c_out, num_offsets) || !features || !weight || !host_offsets || !out ||
      num_in <= 0 || num_out <= 0 || num_in >= (1ll << 31) || num_out >= (1ll << 31))
    return WCN_ERR_INVALID_ARGUMENT;
  if (residual_or_null && residual_or_null == out) return WCN_ERR_INVALID_ARGUMENT;
  if (weight_is_prepared < 0 || weight_is_prepared > 2) return WCN_ERR_INVALID_ARGUMENT;
  if (weight_is_prepared != 1 && weight_dtype != dtype && weight_dtype != WCN_DTYPE_F32) return WCN_ERR_INVALID_ARGUMENT;
  const int64_t L = host_offsets[num_offsets];
  if (host_offsets[0] != 0 || L != num_out || !in_maps || !out_maps) return WCN_ERR_INVALID_ARGUMENT;  // one pair per output row
  for (int k = 0; k < num_offsets; ++k)
    if (host_offsets[k + 1] < host_offsets[k]) return WCN_ERR_INVALID_ARGUMENT;
  const size_t es = elem_size(dtype);
  if ((uintptr_t)features % 16 != 0 || (uintptr_t)out % 16 != 0 || ((size_t)c_out * es) % 16 != 0 ||
      (bias_or_null && (uintptr_t)bias_or_null % 8 != 0) || (residual_or_null && (uintptr_t)residual_or_null % 16 != 0))
    return WCN_ERR_INVALID_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  ConvArgs a = {};
  a.X = features;
  a.bias = bias_or_null;
  a.residual = residual_or_null;
  a.relu = relu ? 1 : 0;
  a.in_maps = in_maps;
  a.out_maps = out_maps;
  a.out = out;
  a.num_in = num_in;
  a.num_out = num_out;
  a.num_pairs = L;
  a.K = num_offsets;
  a.c_in = c_in;
  a.c_out = c_out;
  a.c_in_pad = round_up(c_in, ck_of(dtype));
  a.c_out_pad = round_up(c_out, TN);
  a.identity = -1;
  if (weight_is_prepared == 1) {
    a.Wt = weight;
  } else {
    const size_t need = wcn_conv_prepared_weight_bytes(num_offsets, c_in, c_out, dtype);
    if (!workspace || workspace_bytes < need) return WCN_ERR_WORKSPACE;
    a.Wt = workspace;
    const int as_stored = weight_is_prepared == 2 ? 1 : 0;  // 2: W is (K, c_out, c_in): rows of the tiles already
    if (dtype == WCN_DTYPE_F16) launch_prep<_Float16>(a, weight, weight_dtype, dtype, as_stored, 0, nullptr, s);
    else launch_prep<__bf16>(a, weight, weight_dtype, dtype, as_stored, 0, nullptr, s);
  }
  if (g_time_start) (void)hipEventRecord(g_time_start, s);
  const int rc = wcn_conv_single_launch(a, dtype, host_offsets, s);
  if (g_time_stop) (void)hipEventRecord(g_time_stop, s);
  g_time_start = g_time_stop = nullptr;
  return rc;
}

int wcn_sparse_conv_dgrad(const void* grad_out, int64_t num_out, int32_t c_out, int32_t dtype,
                          const void* weight, int32_t weight_dtype, int32_t num_offsets,
                          int32_t c_in, const int32_t* in_maps, const int32_t* out_maps,
                          const int64_t* host_offsets, int32_t identity_offset,
                          int32_t map_is_symmetric, int32_t in_maps_ascend,
                          const int32_t* group_start_or_null, void* grad_in, int64_t num_in,
                          void* workspace, size_t workspace_bytes, void* stream) {
  if (map_is_symmetric) {
    // the pairs of offset k with in and out exchanged are the pairs of offset K - 1 - k: the map
    // is used as it stands (with its group starts) and the weight tiles are taken in reverse
    if (num_in != num_out) return WCN_ERR_INVALID_ARGUMENT;
    return conv_run(grad_out, num_out, c_out, dtype, weight, weight_dtype, num_offsets, c_in,
                    nullptr, in_maps, out_maps, host_offsets,
                    identity_offset < 0 ? -1 : num_offsets - 1 - identity_offset, 1,
                    group_start_or_null, grad_in, num_in, workspace, workspace_bytes, 1, 1, false,
                    stream);
  }
  // in general: the same contraction over the map with in and out exchanged
  return conv_run(grad_out, num_out, c_out, dtype, weight, weight_dtype, num_offsets, c_in, nullptr,
                  out_maps, in_maps, host_offsets, identity_offset, in_maps_ascend,
                  in_maps_ascend ? group_start_or_null : nullptr, grad_in, num_in, workspace,
                  workspace_bytes, 1, 0, false, stream);
}

}  // extern "C"



