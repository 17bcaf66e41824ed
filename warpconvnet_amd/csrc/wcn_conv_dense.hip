// Output-stationary feature contraction for wide rows (gfx950, MFMA): the kernel behind
// wcn_sparse_conv_fwd / _dgrad when both channel counts are wide (C_in a multiple of 64 and at least
// 128, C_out 128 or 256, 16-bit features).
//
//   out[m, :] = bias + sum_k X[in_k(m), :] @ W[k]        (in_k(m): the input row paired with output
//                                                          row m in offset k, if there is one)
//
// With rows this wide the multiplications dominate, and what has to be kept small is the traffic
// that feeds them.  A workgroup of four waves (one per SIMD, so that a wave may use all 512
// registers) owns a tile of 256 output rows, wave w rows 64 w .. 64 w + 63 as four 16-row MFMA
// blocks, and keeps their fp32 sums in REGISTERS from the first offset to the last
// (4 x C_out / 16 accumulators of four floats per lane): nothing is
// added in LDS and nothing is written before the tile is complete.  The work is walked offset by
// offset and, inside an offset, in chunks of 64 input channels:
//
//   * W[k]^T of a chunk (C_out rows of 128 bytes) travels memory -> registers -> LDS, two buffers,
//     one workgroup barrier per chunk; every wave reads each 16-row block of it once and uses it
//     for all four of its row blocks (eight MFMAs per two 16-byte LDS reads per lane);
//   * the gathered rows of the next chunk travel memory -> registers (MFMA operand layout: lane =
//     output row, 16 bytes of the chunk) while the current chunk is multiplied; an output row
//     without a pair in the offset multiplies zeros (read from a small buffer of zeros);
//   * which input row belongs to which of a wave's 64 output rows in offset k ("dense index") comes
//     from the pair lists: the pairs of the wave's 64-row group in offset k are one run of at most 64
//     entries (out_maps ascends inside an offset; the run's bounds are in the group_start table),
//     the lanes fetch them one offset ahead and scatter the input rows into 64 words of LDS.
//
// The additions into a sum happen in a fixed order (k ascending, channels ascending), so results
// are bitwise reproducible.  Against the pair-packed kernel (wcn_conv_pack_impl.h) this one
// multiplies zeros where an output row has no pair, but pays one barrier per 64 x C_out x 256
// multiply-adds instead of one per 16-pair block and offset, and gathers every row once instead of
// once per 64 output channels.
#include <algorithm>
#include <mutex>

#include "wcn_common.h"
#include "wcn_conv_args.h"
#include "wcn_mma.h"

namespace {

using namespace wcn_mma;

// NCB: 16-channel blocks of output channels (C_out / 16); DENSE_WAVES waves with DENSE_RB 16-row
// blocks of output rows each: a tile is DENSE_WAVES * DENSE_RB * 16 output rows
// RES: the instance that reads a residual in its epilogue (those loads keep more registers alive
// beside the sums, so calls without a residual get an instance without them)
template <typename T, int NCB, int DENSE_WAVES, int DENSE_RB, bool RES>
__global__ void __launch_bounds__(DENSE_WAVES * 64) conv_fwd_dense(ConvArgs a, int num_tiles) {
  constexpr int DENSE_THREADS = DENSE_WAVES * 64, DENSE_ROWS = DENSE_WAVES * DENSE_RB * 16;
  typedef typename Mma<T>::V V;
  extern __shared__ __attribute__((aligned(16))) uint32_t dense_smem[];
  constexpr int WROWS = NCB * 16;              // rows of a weight chunk (output channels)
  constexpr int WGRAN = WROWS * 8;             // its 16-byte granules (64 input channels per row)
  constexpr int WPT = WGRAN / DENSE_THREADS;   // granules per thread
  static_assert(WGRAN % DENSE_THREADS == 0, "the threads share a weight chunk evenly");
  u32x4* const wbuf = (u32x4*)dense_smem;                              // two chunks
  constexpr int RB = DENSE_RB, WROWS_OUT = RB * 16;  // output rows of a wave
  constexpr int NE = 64 % WROWS_OUT == 0 ? 1 : 2;    // 64-row groups its rows can lie in
  static_assert(WROWS_OUT <= 64, "a wave's dense index is one word per lane");
  volatile int32_t* const tab = (volatile int32_t*)(wbuf + 2 * WGRAN);  // DENSE_WAVES x WROWS_OUT words
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 15, g = lane >> 4;
  const int K = a.K;
  const int NC = a.c_in_pad / 64;  // chunks of input channels
  const size_t row_bytes = (size_t)a.c_in * sizeof(T);
  const size_t w_row_bytes = (size_t)a.c_in_pad * sizeof(T);
  const size_t w_tile_bytes = (size_t)a.c_out_pad * w_row_bytes;
  const char* const zsrc = (const char*)a.zeros;
  volatile int32_t* const mytab = tab + wave * WROWS_OUT;

  // this thread's granules of a weight chunk: granule tid % 8 of rows tid / 8, tid / 8 + 64, ...; in
  // an LDS buffer granule j of row r sits at j ^ (r % 8)
  const uint32_t w_src0 = (uint32_t)(tid >> 3) * (uint32_t)w_row_bytes + (uint32_t)(tid & 7) * 16u;
  const uint32_t w_src_step = (uint32_t)(DENSE_THREADS / 8) * (uint32_t)w_row_bytes;
  const int w_dst0 = (tid >> 3) * 8 + ((tid & 7) ^ ((tid >> 3) & 7));
  // this lane's operand granules in a 16-row block of the chunk: row c, granules g and 4 + g
  int w_op[2];
#pragma unroll
  for (int l = 0; l < 2; ++l) w_op[l] = c * 8 + ((l * 4 + g) ^ (c & 7));

  auto load_w = [&](int k, int chunk, u32x4 (&regs)[WPT]) {
    const char* p = (const char*)a.Wt + (size_t)k * w_tile_bytes + (size_t)chunk * 128;
#pragma unroll
    for (int j = 0; j < WPT; ++j) regs[j] = *reinterpret_cast<const u32x4*>(p + (w_src0 + (uint32_t)j * w_src_step));
  };
  auto store_w = [&](int buf, const u32x4 (&regs)[WPT]) {
#pragma unroll
    for (int j = 0; j < WPT; ++j) wbuf[buf * WGRAN + w_dst0 + j * DENSE_THREADS] = regs[j];
  };
  auto load_rows = [&](const int32_t (&in)[RB], int chunk, V (&A)[RB][2]) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const char* p = in[rb] >= 0 ? (const char*)a.X + (size_t)in[rb] * row_bytes + (size_t)chunk * 128 + g * 16
                                  : zsrc + g * 16;
      A[rb][0] = *reinterpret_cast<const V*>(p);
      A[rb][1] = *reinterpret_cast<const V*>(p + 64);
    }
  };

  for (int tile = (int)blockIdx.x; tile < num_tiles; tile += (int)gridDim.x) {
    const int64_t m0 = (int64_t)tile * DENSE_ROWS;
    const int tile_rows = (int)(a.num_out - m0 < DENSE_ROWS ? a.num_out - m0 : DENSE_ROWS);
    const int32_t base = (int32_t)(m0 + wave * WROWS_OUT);  // first output row of this wave
    // its rows lie in one 64-row group or two (48-row waves): the groups' pairs in an offset are one
    // run of at most NE * 64 entries
    const int64_t grp = (int64_t)base >> 6, grp_end = (((int64_t)base + WROWS_OUT - 1) >> 6) + 1;
    // the run in every offset: lane k looks after offset k
    int run_lo = 0, run_cnt = 0;
    if (lane < K && lane != a.identity && grp < a.G) {
      const int32_t* gs = a.group_start + (int64_t)lane * (a.G + 1);
      const int lo = gs[grp], hi = gs[grp_end < a.G ? grp_end : a.G];
      run_lo = (int)a.offsets[lane] + lo;
      run_cnt = hi - lo;
      if (run_cnt < 0 || run_cnt > NE * 64) run_cnt = 0;  // inconsistent table: contribute nothing
    }
    // the entries of offset k's run, NE per lane (requested an offset ahead)
    auto request = [&](int k, int32_t (&e_in)[NE], int32_t (&e_out)[NE]) {
      const int lo = __builtin_amdgcn_readlane(run_lo, k), cnt = __builtin_amdgcn_readlane(run_cnt, k);
      // no branches (the loads sit between the MFMAs of a chunk): lanes past the run read its last
      // entry, an empty run reads zeros; settle() looks at the count again
      const int32_t* pin = cnt > 0 ? a.in_maps + lo : (const int32_t*)a.zeros;
      const int32_t* pout = cnt > 0 ? a.out_maps + lo : (const int32_t*)a.zeros;
      const int last = cnt > 0 ? cnt - 1 : 0;
#pragma unroll
      for (int h = 0; h < NE; ++h) {
        const int i = lane + 64 * h < last ? lane + 64 * h : last;
        e_in[h] = pin[i];
        e_out[h] = pout[i];
      }
    };
    // ... turned into the input row of each of the wave's output rows (lane (c, *): rows c, 16 + c, 32 + c, 48 + c)
    auto settle = [&](int k, const int32_t (&e_in)[NE], const int32_t (&e_out)[NE], int32_t (&in)[RB]) {
      if (k == a.identity) {  // every row reads its own input row; the map's pairs are ignored
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          const int64_t r = (int64_t)base + rb * 16 + c;
          in[rb] = (r < a.num_out && r < a.num_in) ? (int32_t)r : -1;
        }
        return;
      }
      if (lane < WROWS_OUT) mytab[lane] = -1;
      const int cnt = __builtin_amdgcn_readlane(run_cnt, k);
#pragma unroll
      for (int h = 0; h < NE; ++h) {
        const uint32_t slot = (uint32_t)(e_out[h] - base);
        if (lane + 64 * h < cnt && e_in[h] >= 0 && slot < (uint32_t)WROWS_OUT && (uint32_t)e_in[h] < (uint32_t)a.num_in &&
            (int64_t)e_out[h] < a.num_out)
          mytab[slot] = e_in[h];
      }
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) in[rb] = mytab[rb * 16 + c];
    };

    f32x4 acc[RB][NCB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) acc[rb][cb] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // ---- the tile's first chunk ----
    int32_t e_in[NE], e_out[NE], in_cur[RB], in_next[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) in_next[rb] = -1;
    V a_cur[RB][2], a_next[RB][2];
    u32x4 wr[WPT];
    request(0, e_in, e_out);
    load_w(0, 0, wr);
    settle(0, e_in, e_out, in_cur);
    load_rows(in_cur, 0, a_cur);
    __syncthreads();  // the workgroup is done with the buffers of the tile before
    store_w(0, wr);
    __syncthreads();

    const int steps = K * NC;
    int k = 0, chunk = 0, buf = 0;
    for (int s = 0; s < steps; ++s) {
      const bool more = s + 1 < steps;
      const int nchunk = chunk + 1 < NC ? chunk + 1 : 0;
      const int nk = (nchunk == 0 && k + 1 < K) ? k + 1 : k;
      // Every step issues the same loads in the same order, needed or not (the last step of a tile
      // fetches its own chunk again, every step of an offset fetches the next offset's entries),
      // and nothing loaded in a step is used in it: the waits for loaded data are then the same
      // counts on every path.  The loads are issued between the first MFMAs of the chunk, whose
      // operands are at hand, so that their address arithmetic runs beside the multiplications.
      if (nchunk == 0 && more) settle(nk, e_in, e_out, in_next);  // entries requested a step ago
      int32_t in_sel[RB];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) in_sel[rb] = nchunk == 0 ? in_next[rb] : in_cur[rb];
      // ---- multiply the current chunk: the operands of the 16-channel blocks to come are read
      //      AHEAD blocks before they are multiplied ----
      constexpr int AHEAD = 3;
      u32x4 wq[AHEAD + 1][2];
#pragma unroll
      for (int cb = 0; cb < AHEAD && cb < NCB; ++cb) {
        wq[cb][0] = wbuf[buf * WGRAN + cb * 128 + w_op[0]];
        wq[cb][1] = wbuf[buf * WGRAN + cb * 128 + w_op[1]];
      }
      __builtin_amdgcn_sched_group_barrier(0x100, 2 * AHEAD, 0);  // LDS reads: the first operands
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) {
        if (cb + AHEAD < NCB) {
          wq[(cb + AHEAD) % (AHEAD + 1)][0] = wbuf[buf * WGRAN + (cb + AHEAD) * 128 + w_op[0]];
          wq[(cb + AHEAD) % (AHEAD + 1)][1] = wbuf[buf * WGRAN + (cb + AHEAD) * 128 + w_op[1]];
        }
#pragma unroll
        for (int l = 0; l < 2; ++l)
#pragma unroll
          for (int rb = 0; rb < RB; ++rb)
            acc[rb][cb] = Mma<T>::mma(__builtin_bit_cast(V, wq[cb % (AHEAD + 1)][l]), a_cur[rb][l], acc[rb][cb]);
        if (cb == 0) load_w(nk, nchunk, wr);
        if (cb == 1) request(k + 1 < K ? k + 1 : k, e_in, e_out);
        if (cb == 2) load_rows(in_sel, nchunk, a_next);
        __builtin_amdgcn_sched_group_barrier(0x008, 2 * RB, 0);  // this block's MFMAs
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);       // the operands AHEAD blocks on
        if (cb == 0) __builtin_amdgcn_sched_group_barrier(0x020, WPT, 0);     // the next chunk's weights
        if (cb == 1) __builtin_amdgcn_sched_group_barrier(0x020, 2 * NE, 0);  // the next offset's entries
        if (cb == 2) __builtin_amdgcn_sched_group_barrier(0x020, 2 * RB, 0);  // the next chunk's rows
      }
      if (more) store_w(buf ^ 1, wr);
      __syncthreads();  // everybody has read this chunk's buffer and written the next one's
      buf ^= 1;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        a_cur[rb][0] = a_next[rb][0];
        a_cur[rb][1] = a_next[rb][1];
        if (nchunk == 0 && more) in_cur[rb] = in_next[rb];
      }
      k = nk;
      chunk = nchunk;
    }

    // ---- the tile is complete: bias, one rounding, 8-byte stores (lane (c, g): channels
    //      cb * 16 + 4 g .. + 3 of rows c, 16 + c, 32 + c, 48 + c of the wave) ----
    T* __restrict__ out = (T*)a.out;
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
      const int col = cb * 16 + 4 * g;
      float b[4] = {0.f, 0.f, 0.f, 0.f};
      if (a.bias) {
#pragma unroll
        for (int e = 0; e < 4; ++e) b[e] = to_float(((const T*)a.bias)[col + e]);
      }
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const int row = wave * WROWS_OUT + rb * 16 + c;
        if (row < tile_rows) {
          T t[4];
          float r[4] = {0.f, 0.f, 0.f, 0.f};  // rows are whole 16-byte vectors here: 128 or 256 channels
          if (RES) load_floats<T, 4>(static_cast<const T*>(a.residual) + (m0 + row) * a.c_out + col, r);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float f = acc[rb][cb][e] + b[e] + r[e];
            if (a.relu) f = f < 0.f ? 0.f : f;
            t[e] = from_float<T>(f);
          }
          *reinterpret_cast<uint2*>(out + (m0 + row) * a.c_out + col) = *reinterpret_cast<const uint2*>(t);
        }
      }
    }
  }
}

inline int dense_cus() {
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

template <typename T, int NCB, int WAVES, int RB, bool RES>
int launch_dense_instance(const ConvArgs& a, hipStream_t s) {
  constexpr int ROWS = WAVES * RB * 16;
  constexpr int lds = 2 * NCB * 16 * 8 * 16 + WAVES * RB * 16 * 4;
  static_assert(lds <= 160 * 1024, "LDS of one workgroup");
  const void* fn = (const void*)conv_fwd_dense<T, NCB, WAVES, RB, RES>;
  // more than 64 KiB of dynamic LDS has to be allowed once per device and kernel
  static std::mutex mu;
  static bool allowed[64] = {};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return WCN_ERR_LAUNCH;
  {
    std::lock_guard<std::mutex> hold(mu);
    if (!allowed[device]) {
      if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
        return WCN_ERR_LAUNCH;
      allowed[device] = true;
    }
  }
  const int64_t tiles = (a.num_out + ROWS - 1) / ROWS;
  if (tiles <= 0 || tiles > INT32_MAX) return WCN_ERR_INVALID_ARGUMENT;
  const unsigned grid = (unsigned)std::min<int64_t>(tiles, dense_cus());
  hipLaunchKernelGGL((conv_fwd_dense<T, NCB, WAVES, RB, RES>), dim3(grid), dim3(WAVES * 64), lds, s, a, (int)tiles);
  wcn_conv_note_kernel("conv_fwd_dense<%s, %d, %d, %d, %s>", wcn_type_text<T>(), NCB, WAVES, RB, RES ? "true" : "false");
  return hipGetLastError() == hipSuccess ? WCN_OK : WCN_ERR_LAUNCH;
}

template <typename T, int NCB, int WAVES, int RB>
int launch_dense(const ConvArgs& a, hipStream_t s) {
  return a.residual ? launch_dense_instance<T, NCB, WAVES, RB, true>(a, s)
                    : launch_dense_instance<T, NCB, WAVES, RB, false>(a, s);
}

// Two tile shapes: 256 rows (eight waves of 32 rows, two per SIMD) and 192 rows (four waves of 48
// rows, one per SIMD).  The multiplications of a tile take a SIMD 4 and 3 units of time per chunk
// (waves per SIMD times row blocks per wave) and they are what the kernel waits for, so the shape is
// chosen by rounds of the grid times that: the shorter tile wins where it saves a round or, on a
// small map, where the taller one would not use more CUs anyway.
template <typename T, int NCB>
int launch_dense_shaped(const ConvArgs& a, hipStream_t s) {
  const int64_t cus = dense_cus();
  const int64_t rounds_256 = ((a.num_out + 255) / 256 + cus - 1) / cus;
  const int64_t rounds_192 = ((a.num_out + 191) / 192 + cus - 1) / cus;
  if (rounds_192 * 3 < rounds_256 * 4) return launch_dense<T, NCB, 4, 3>(a, s);
  return launch_dense<T, NCB, 8, 2>(a, s);
}

template <typename T>
int launch_dense_typed(const ConvArgs& a, hipStream_t s) {
  return a.c_out_pad == 256 ? launch_dense_shaped<T, 16>(a, s) : launch_dense_shaped<T, 8>(a, s);
}

}  // namespace

// Wide 16-bit rows on both sides, whole 64-channel chunks, a map of at most 64 offsets with its
// group starts, and enough tiles to occupy a good part of the chip (a tile is 192 or 256 output rows
// and runs on one CU from the first offset to the last).
bool wcn_conv_dense_takes(const ConvArgs& a, int dtype) {
  if (dtype == WCN_DTYPE_F32 || !a.vec_in || !a.vec_out || !a.group_start) return false;
  if (a.residual && !a.vec_res) return false;  // the epilogue reads the residual in 8-byte pieces
  if (a.c_in != a.c_in_pad || a.c_in % 64 != 0 || a.c_in < 128) return false;
  if (a.c_out != a.c_out_pad || (a.c_out != 128 && a.c_out != 256)) return false;
  if (a.K < 1 || a.K > 64 || a.num_in >= (1ll << 31) || a.num_out >= (1ll << 31)) return false;
  return (a.num_out + 255) / 256 >= 96;
}

int wcn_conv_dense_launch(const ConvArgs& a, int dtype, hipStream_t s) {
  return dtype == WCN_DTYPE_F16 ? launch_dense_typed<_Float16>(a, s) : launch_dense_typed<__bf16>(a, s);
}
