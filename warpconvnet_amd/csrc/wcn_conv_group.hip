// Feature contraction for narrow layers (at most 32 channels in and out, 16-bit features): a wave
// owns a group of 64 output rows from the first kernel offset to the last.
//
//   out[m, :] = bias + sum_k X[in_k(m), :] @ W[k]
//
// The pair-packed kernel (wcn_conv_pack_impl.h) walks a tile of output rows offset by offset with a
// workgroup barrier between offsets, because its waves add into each other's rows and share one
// weight tile at a time.  With narrow rows neither is needed: the fp32 sums of 64 rows x 32 channels
// are 8 KB, so every wave keeps the sums of its own group in LDS and no other wave touches them, and
// all K weight tiles W[k]^T fit LDS together (27 x 2 KB, or 125 x 512 B for 16 channels), loaded
// once per workgroup.  After that load there is no barrier and no atomic in the kernel:
//
//   * the pairs of offset k whose output row lies in the group are one run of the pair lists
//     (bounds from group_start); a run is cut into blocks of 16 pairs, and the blocks of all offsets
//     of a group form one list that the wave walks from end to end;
//   * a block is multiplied transposed: the gathered rows are the B operand (lane = (pair, 8 or 4
//     channels)), W[k]^T the A operand, so that a lane ends up with 4 consecutive output channels of
//     one pair and hands that pair's row of sums to the MFMA as its C operand: one 16-byte LDS read
//     and write per 16 channels.  Pairs that do not exist read row 0 and add into a spare row;
//   * requests run a fixed distance ahead of the multiplications (the rows 8 blocks, the pair-list
//     entries 16), in a ring whose 16 steps are written out: plain loads, and the compiler's own
//     waits for them come out exact because the start-up issues its requests in the loop's order;
//   * the additions of a row happen in a fixed order: results are bitwise reproducible.
#include <algorithm>
#include <mutex>

#include "wcn_common.h"
#include "wcn_conv_args.h"
#include "wcn_mma.h"

using namespace wcn_mma;

namespace {

constexpr int GROUP_AHEAD = 8;     // blocks of 16 pairs whose gathered rows are on their way
constexpr int GROUP_ENTRIES = 16;  // blocks whose pair-list entries are on their way or held

typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

// MFMA operands of a block of 16 pairs: 8 channels per lane (16x16x32) or, for rows of at most 16
// channels, 4 (16x16x16).
template <typename T, bool HALF_K>
struct GroupOp;
template <typename T>
struct GroupOp<T, false> {
  typedef typename Mma<T>::V V;
  static constexpr int PER_LANE = 8;
  static __device__ __forceinline__ V zero() { return Mma<T>::zero(); }
  static __device__ __forceinline__ f32x4 mma(V a, V b, f32x4 c) { return Mma<T>::mma(a, b, c); }
};
template <>
struct GroupOp<_Float16, true> {
  typedef f16x4 V;
  static constexpr int PER_LANE = 4;
  static __device__ __forceinline__ V zero() { return (V){0, 0, 0, 0}; }
  static __device__ __forceinline__ f32x4 mma(V a, V b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(a, b, c, 0, 0, 0);
  }
};
template <>
struct GroupOp<__bf16, true> {
  typedef s16x4 V;
  static constexpr int PER_LANE = 4;
  static __device__ __forceinline__ V zero() { return (V){0, 0, 0, 0}; }
  static __device__ __forceinline__ f32x4 mma(V a, V b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, c, 0, 0, 0);
  }
};

// NCB: 16-channel blocks of output; NCH: 64s of kernel offsets; WAVES: groups in work per workgroup
template <typename T, int NCB, bool HALF_K, int NCH, int WAVES>
__global__ void __launch_bounds__(WAVES * 64) conv_fwd_group(ConvArgs a) {
  typedef GroupOp<T, HALF_K> Op;
  typedef typename Op::V V;
  constexpr int PER = Op::PER_LANE;
  constexpr int ROWF = NCB * 16;  // floats per row of sums
  constexpr int ACC_FLOATS = 65 * ROWF;  // row 64: sums of pairs that do not exist
  extern __shared__ __attribute__((aligned(16))) unsigned char group_smem[];
  // LDS: the weight operands of all offsets, [k][cb][lane], then the sums of every wave
  V* __restrict__ s_w = reinterpret_cast<V*>(group_smem);
  const int K = a.K;
  float* __restrict__ acc = reinterpret_cast<float*>(group_smem + (size_t)K * NCB * 64 * sizeof(V)) +
                            (threadIdx.x >> 6) * ACC_FLOATS;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int pr = lane & 15, kg = lane >> 4;
  const T* __restrict__ X = (const T*)a.X;
  const int c_in = a.c_in;
  const bool has_c = kg * PER < c_in;  // this lane's input channels exist
  const uint32_t row_bytes = (uint32_t)c_in * sizeof(T);
  const uint32_t lane_bytes = has_c ? (uint32_t)(kg * PER * sizeof(T)) : 0u;

  // weight operands: lane (pr, kg) of block cb holds W[k]^T[cb * 16 + pr][kg * PER ..]
  {
    const T* __restrict__ Wt = (const T*)a.Wt;
    for (int i = threadIdx.x; i < K * NCB * 64; i += WAVES * 64) {
      const int l = i & 63, cb = (i >> 6) % NCB, k = (i >> 6) / NCB;
      s_w[i] = *reinterpret_cast<const V*>(Wt + ((int64_t)(k * a.c_out_pad + cb * 16 + (l & 15)) * a.c_in_pad + (l >> 4) * PER));
    }
  }
  __syncthreads();  // the only barrier: from here on a wave works alone

  // granule gi (4 channels) of row r of the sums: the sums are kept granule by granule, 65 rows of
  // 16 bytes each, so that the 16 rows one instruction touches spread over the banks and an
  // address is one shift-and-add away from the row number
  auto granule = [&](int r, int gi) -> f32x4* { return reinterpret_cast<f32x4*>(acc) + gi * 65 + r; };
  // 8 (4) channels of input row idx.  No lane is switched off and nothing is replaced by zeros
  // afterwards (a select fed by a load is turned into a branch around the load, and the straight
  // line is gone): a pair that does not exist reads row 0 and adds its product to the spare row of
  // sums, and a lane whose channels lie beyond c_in reads the row's first channels, which meet the
  // zero padding of the weight operand.
  auto x_operand = [&](int32_t idx) -> V {
    const uint32_t at = __umul24((uint32_t)idx, row_bytes) + lane_bytes;  // rows number below 2^24
    return *reinterpret_cast<const V*>(reinterpret_cast<const unsigned char*>(X) + at);
  };
  auto add_block = [&](int k, V xv, int r) {  // r: the pair's row in the group, 64 if it does not exist
    f32x4* at[NCB];
    f32x4 sum[NCB];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
      at[cb] = granule(r, cb * 4 + kg);
      sum[cb] = *at[cb];
    }
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) sum[cb] = Op::mma(s_w[(k * NCB + cb) * 64 + lane], xv, sum[cb]);
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) *at[cb] = sum[cb];
  };
  // the bias of the 8 channels this lane writes out
  const int cpart = lane & 3;
  float bias_v[8];
#pragma unroll
  for (int e = 0; e < 8; ++e)
    bias_v[e] = (a.bias && cpart * 8 + e < a.c_out) ? to_float(((const T*)a.bias)[cpart * 8 + e]) : 0.f;
  const bool with_identity = a.identity >= 0 && a.identity < K;
  const int64_t total_waves = (int64_t)gridDim.x * WAVES;
  const int32_t* __restrict__ in_maps = a.in_maps;
  const int32_t* __restrict__ out_maps = a.out_maps;

  // lane j looks after the kernel offsets j, 64 + j, ..: where their pair lists start, and where
  // their group bounds are
  int list_at[NCH], bounds_at[NCH];
  bool mine[NCH];
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int k = c * 64 + lane;
    mine[c] = k < K && k != a.identity;
    list_at[c] = mine[c] ? (int)a.offsets[k] : 0;
    bounds_at[c] = mine[c] ? k * (int)(a.G + 1) : 0;
  }
  const int64_t g_first = (int64_t)blockIdx.x * WAVES + wave;
  int next_lo[NCH], next_hi[NCH];  // the bounds of the group after this one, requested a group ahead
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int64_t gg = g_first < a.G ? g_first : 0;
    next_lo[c] = a.group_start[bounds_at[c] + gg];
    next_hi[c] = a.group_start[bounds_at[c] + gg + 1];
  }

  for (int64_t g = g_first; g < a.G; g += total_waves) {
    const int64_t m0 = g * 64;
    // every offset's run of pairs in this group, cut into blocks of 16: the blocks of all offsets
    // form one list, walked from end to end with requests a fixed number of blocks ahead
    int run_lo[NCH], run_cnt[NCH], ends[NCH];  // ends: blocks up to and including this lane's offset
    int blocks = 0;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      int cnt = next_hi[c] - next_lo[c];
      if (!mine[c] || cnt < 0 || cnt > 64) cnt = 0;  // inconsistent table: contribute nothing
      run_lo[c] = list_at[c] + next_lo[c];
      run_cnt[c] = cnt;
      ends[c] = blocks + wcn_wave_inclusive_sum((cnt + 15) >> 4);
      blocks = __builtin_amdgcn_readlane(ends[c], 63);
      const int64_t gn = g + total_waves < a.G ? g + total_waves : g;
      next_lo[c] = a.group_start[bounds_at[c] + gn];
      next_hi[c] = a.group_start[bounds_at[c] + gn + 1];
    }
    // What block t of the list is: its offset, the first of its pairs in the lists, and how many
    // pairs of its run it and the blocks after it hold.  Worked out for 64 blocks at a time, a lane
    // per block (a search of the running block counts), and read from that lane when the block's
    // entries are requested; past the end of the list: offset 0, no pairs.
    int page_k = 0, page_first = 0, page_left = 0;
    auto turn_page = [&](int page) {
      const int t = page * 64 + lane;
      int c = 0, at = 0;  // the first offset whose count of blocks exceeds t
      if (NCH == 2) c = __builtin_amdgcn_readlane(ends[0], 63) <= t ? 1 : 0;
#pragma unroll
      for (int step = 32; step >= 1; step >>= 1) {
        int e = __shfl(ends[0], at + step - 1, 64);
        if (NCH == 2) {
          const int e1 = __shfl(ends[NCH - 1], at + step - 1, 64);
          e = c ? e1 : e;
        }
        if (e <= t) at += step;
      }
      int e = __shfl(ends[0], at, 64), lo = __shfl(run_lo[0], at, 64), cnt = __shfl(run_cnt[0], at, 64);
      if (NCH == 2) {
        const int e1 = __shfl(ends[NCH - 1], at, 64), lo1 = __shfl(run_lo[NCH - 1], at, 64),
                  cnt1 = __shfl(run_cnt[NCH - 1], at, 64);
        e = c ? e1 : e;
        lo = c ? lo1 : lo;
        cnt = c ? cnt1 : cnt;
      }
      const int b = t - (e - ((cnt + 15) >> 4));  // which block of its run
      const bool live = t < blocks;
      page_k = live ? c * 64 + at : 0;
      page_first = live ? lo + b * 16 : 0;
      page_left = live ? cnt - b * 16 : 0;
    };

    // the sums start as the identity offset's product (every row reads its own input row; the
    // map's pairs of that offset are ignored), or as zeros, plus the row of the residual if one
    // is given (requested here, where the group's first requests are on their way anyway, and not
    // in the epilogue, where the wave would wait for it with nothing else to do)
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) {
      const int64_t m = m0 + rb * 16 + pr;
      const bool here = with_identity && m < a.num_out && m < a.num_in;
      V xv = Op::zero();
      if (with_identity) xv = x_operand(here ? (int32_t)m : 0);
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) {
        float start[4] = {0.f, 0.f, 0.f, 0.f};
        const int col = cb * 16 + kg * 4;
        if (a.residual && m < a.num_out && col < a.c_out) {
          const T* rs = static_cast<const T*>(a.residual) + m * a.c_out + col;
          if (a.vec_res) {  // whole 16-byte vectors per row: c_out is a multiple of 8
            load_floats<T, 4>(rs, start);
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (col + e < a.c_out) start[e] = to_float(rs[e]);
          }
        }
        f32x4 d = (f32x4){0.f, 0.f, 0.f, 0.f};
        if (with_identity) d = Op::mma(s_w[(a.identity * NCB + cb) * 64 + lane], xv, d);
        if (!here) d = (f32x4){0.f, 0.f, 0.f, 0.f};
        *granule(rb * 16 + pr, cb * 4 + kg) = d + (f32x4){start[0], start[1], start[2], start[3]};
      }
    }

    // A ring of GROUP_ENTRIES blocks whose pair-list entries are on their way or here, of which the
    // oldest GROUP_AHEAD also have their gathered rows requested.  The scheduling barriers keep
    // the requests where they are written (left to itself the scheduler sinks them until three
    // are in flight, a few hundred cycles ahead of their use).
    int32_t e_in[GROUP_ENTRIES], e_row[GROUP_ENTRIES];
    int b_k[GROUP_ENTRIES], b_left[GROUP_ENTRIES];
    V xv[GROUP_AHEAD];
    auto request_entries = [&](int slot, int on_page) {
      b_k[slot] = __builtin_amdgcn_readlane(page_k, on_page);
      b_left[slot] = __builtin_amdgcn_readlane(page_left, on_page);
      const int first = __builtin_amdgcn_readlane(page_first, on_page);
      const int last = b_left[slot] > 0 ? b_left[slot] - 1 : 0;
      const uint32_t at = (uint32_t)(first + (pr < last ? pr : last)) * 4u;  // fewer than 2^30 pairs
      e_in[slot] = *reinterpret_cast<const int32_t*>(reinterpret_cast<const unsigned char*>(in_maps) + at);
      e_row[slot] = *reinterpret_cast<const int32_t*>(reinterpret_cast<const unsigned char*>(out_maps) + at);
    };
    auto request_rows = [&](int slot, int xslot) {
      const uint32_t row = (uint32_t)(e_row[slot] - (int32_t)m0);
      const bool ok = pr < b_left[slot] && (uint32_t)e_in[slot] < (uint32_t)a.num_in && row < 64u;
      xv[xslot] = x_operand(ok ? e_in[slot] : 0);
      e_row[slot] = ok ? (int)row : 64;
    };
    // (the requests of the first blocks come in the order the loop issues them, so that one count
    // of requests issued since holds for a wait on either way into the loop)
    turn_page(0);
#pragma unroll
    for (int u = 0; u < GROUP_ENTRIES; ++u) {
      if (u >= GROUP_AHEAD) request_rows(u - GROUP_AHEAD, u - GROUP_AHEAD);
      request_entries(u, u);
      __builtin_amdgcn_sched_barrier(0);
    }
    static_assert(GROUP_ENTRIES == 16 && GROUP_AHEAD == 8, "the turn below is written out for a ring of 16 and 8");
    for (int t0 = 0; t0 < blocks; t0 += GROUP_ENTRIES) {
      const int ask = t0 + GROUP_ENTRIES;  // the first block whose entries this turn requests
      if ((ask & 63) == 0) turn_page(ask >> 6);
      const int todo = blocks - t0, on_page = ask & 63;
      // one block: multiply it, request the rows of the block 8 further on (whose entries have
      // arrived) and the entries of the block 16 further on (into the slot just multiplied).
      // Written out rather than left to the unroller: the turn ends at the list's last block from
      // any of its 16 places, and the register of every slot has to be fixed at compile time.
#define WCN_GROUP_STEP(u)                                                      \
  if ((u) >= todo) goto turn_done;                                             \
  add_block(b_k[(u)], xv[(u) % GROUP_AHEAD], e_row[(u)]);                      \
  request_rows(((u) + GROUP_AHEAD) % GROUP_ENTRIES, (u) % GROUP_AHEAD);        \
  request_entries((u), on_page + (u));                                         \
  __builtin_amdgcn_sched_barrier(0);
      WCN_GROUP_STEP(0) WCN_GROUP_STEP(1) WCN_GROUP_STEP(2) WCN_GROUP_STEP(3)
      WCN_GROUP_STEP(4) WCN_GROUP_STEP(5) WCN_GROUP_STEP(6) WCN_GROUP_STEP(7)
      WCN_GROUP_STEP(8) WCN_GROUP_STEP(9) WCN_GROUP_STEP(10) WCN_GROUP_STEP(11)
      WCN_GROUP_STEP(12) WCN_GROUP_STEP(13) WCN_GROUP_STEP(14) WCN_GROUP_STEP(15)
#undef WCN_GROUP_STEP
    turn_done:;
    }

    // bias, one rounding, 16-byte stores: lane (row = lane >> 2 (+16 per turn), 8 channels = lane & 3)
    T* __restrict__ out = (T*)a.out;
#pragma unroll
    for (int turn = 0; turn < 4; ++turn) {
      const int r = turn * 16 + (lane >> 2);
      const int64_t m = m0 + r;
      if (cpart * 8 < NCB * 16 && m < a.num_out) {
        const f32x4 lo4 = *granule(r, cpart * 2);
        const f32x4 hi4 = *granule(r, cpart * 2 + 1);
        float v[8] = {lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
        const int col = cpart * 8;
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += bias_v[e];
        if (a.relu) {  // (the residual went into the sums at the group's start)
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] = v[e] < 0.f ? 0.f : v[e];
        }
        T* dst = out + m * a.c_out + col;
        if (a.vec_out && col + 8 <= a.c_out) {
          T t[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) t[e] = from_float<T>(v[e]);
          *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(t);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (col + e < a.c_out) dst[e] = from_float<T>(v[e]);
        }
      }
    }
  }
}

inline int group_cus() {
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

template <typename T, int NCB, bool HALF_K>
size_t group_lds(int K, int waves) {
  typedef typename GroupOp<T, HALF_K>::V V;
  return (size_t)K * NCB * 64 * sizeof(V) + (size_t)waves * 65 * NCB * 16 * sizeof(float);
}

constexpr size_t GROUP_LDS_MAX = 160 * 1024;

template <typename T, int NCB, bool HALF_K, int NCH, int WAVES>
int launch_group_waves(const ConvArgs& a, hipStream_t s) {
  const size_t lds = group_lds<T, NCB, HALF_K>(a.K, WAVES);
  const void* fn = (const void*)conv_fwd_group<T, NCB, HALF_K, NCH, WAVES>;
  {  // more than 64 KiB of dynamic LDS has to be allowed per device and kernel
    static std::mutex mu;
    static size_t allowed[64] = {};
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return WCN_ERR_LAUNCH;
    std::lock_guard<std::mutex> hold(mu);
    if (allowed[device] < lds) {
      if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)GROUP_LDS_MAX) != hipSuccess)
        return WCN_ERR_LAUNCH;
      allowed[device] = GROUP_LDS_MAX;
    }
  }
  const int64_t wgs = (a.G + WAVES - 1) / WAVES;
  const unsigned grid = (unsigned)std::min<int64_t>(wgs, group_cus());
  hipLaunchKernelGGL((conv_fwd_group<T, NCB, HALF_K, NCH, WAVES>), dim3(grid), dim3(WAVES * 64), lds, s, a);
  wcn_conv_note_kernel("conv_fwd_group<%s, %d, %s, %d, %d>", wcn_type_text<T>(), NCB, HALF_K ? "true" : "false", NCH, WAVES);
  return hipGetLastError() == hipSuccess ? WCN_OK : WCN_ERR_LAUNCH;
}

// Sixteen waves per workgroup (four per SIMD) where the sums of sixteen groups fit LDS beside the
// weights, twelve otherwise (3x3x3 with 32 channels on both sides: 54 KB of weights and 8 KB of
// sums per wave).  The instances for 32 input channels under more than 64 offsets do not stay
// within the 128 registers of sixteen waves (one has weights that fit LDS for no such kernel anyway,
// the other would spill a few registers): they are built for twelve waves only.
template <typename T, int NCB, bool HALF_K, int NCH>
int launch_group_chunks(const ConvArgs& a, hipStream_t s) {
  if constexpr (!(!HALF_K && NCH == 2)) {
    if (group_lds<T, NCB, HALF_K>(a.K, 16) <= GROUP_LDS_MAX) return launch_group_waves<T, NCB, HALF_K, NCH, 16>(a, s);
  }
  return launch_group_waves<T, NCB, HALF_K, NCH, 12>(a, s);
}

template <typename T, int NCB, bool HALF_K>
int launch_group_instance(const ConvArgs& a, hipStream_t s) {
  return a.K <= 64 ? launch_group_chunks<T, NCB, HALF_K, 1>(a, s) : launch_group_chunks<T, NCB, HALF_K, 2>(a, s);
}

template <typename T>
int launch_group(const ConvArgs& a, hipStream_t s) {
  if (a.c_in <= 16) {
    return a.c_out <= 16 ? launch_group_instance<T, 1, true>(a, s) : launch_group_instance<T, 2, true>(a, s);
  }
  return a.c_out <= 16 ? launch_group_instance<T, 1, false>(a, s) : launch_group_instance<T, 2, false>(a, s);
}

template <typename T>
bool group_fits(const ConvArgs& a) {
  const bool half_k = a.c_in <= 16;
  const size_t lds = a.c_out <= 16 ? (half_k ? group_lds<T, 1, true>(a.K, 12) : group_lds<T, 1, false>(a.K, 12))
                                   : (half_k ? group_lds<T, 2, true>(a.K, 12) : group_lds<T, 2, false>(a.K, 12));
  return lds <= GROUP_LDS_MAX;
}

}  // namespace

// 16-bit rows of whole 16-byte pieces (8-byte pieces for rows of at most 16 channels), at most 32
// channels on either side, all weight tiles and the waves' sums within LDS, a feature matrix that
// 32-bit byte offsets reach, a map that comes with its group starts (pairs ascending in output row
// inside every offset).
bool wcn_conv_group_takes(const ConvArgs& a, int dtype) {
  if (dtype != WCN_DTYPE_F16 && dtype != WCN_DTYPE_BF16) return false;
  if (!a.vec_in || a.split || !a.group_start || a.G <= 0 || a.num_pairs <= 0) return false;
  if (a.c_in > 32 || a.c_out > 32 || (a.c_in <= 16 && a.c_in % 4 != 0)) return false;
  if ((uint64_t)a.num_in * (uint64_t)a.c_in * 2u >= (1ull << 32)) return false;
  if (a.K > 128 || (int64_t)a.K * (a.G + 1) >= (1ll << 31) || a.num_pairs >= (1ll << 30) ||
      a.num_in > (1ll << 24))
    return false;
  return dtype == WCN_DTYPE_F16 ? group_fits<_Float16>(a) : group_fits<__bf16>(a);
}

int wcn_conv_group_launch(const ConvArgs& a, int dtype, hipStream_t s) {
  return dtype == WCN_DTYPE_F16 ? launch_group<_Float16>(a, s) : launch_group<__bf16>(a, s);
}
