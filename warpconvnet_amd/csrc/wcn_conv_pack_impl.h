// Pair-packed feature contraction (gfx950, MFMA): the kernel behind wcn_sparse_conv_fwd / _dgrad
// for feature rows of one to four 128-byte slices (64 channels of 16-bit data, 32 of fp32, per
// slice) and maps of at most 128 offsets (64 when a row has several slices).
//
//   out[m, :] = bias + sum_k sum_{p in offset k, out_maps[p] == m} X[in_maps[p], :] @ W[k]
//
// On surface-like data an output row has a pair for only a few of the K offsets (4 of 27 on the
// benchmark scenes), so a product laid out by output rows multiplies mostly zeros.  Here the
// multiplications are laid out by PAIRS:
//
//   * a workgroup owns a tile of R output rows at a time and keeps their fp32 sums in LDS; it is
//     persistent and walks tiles blockIdx.x, blockIdx.x + gridDim.x, ...;
//   * the pairs of one offset that land in a tile are one contiguous run of the pair lists
//     (out_maps ascends inside an offset; the run's bounds come from the group_start table); a run
//     is cut into blocks of 16 pairs, block j goes to wave j % NW: every MFMA multiplies 16 real
//     gathered rows (but for the last block of a run);
//   * the tile is worked through one offset after the other (a "phase" per offset -- per offset and
//     slice for rows of several slices -- one barrier between phases).  Inside a phase every output
//     row occurs at most once, so the waves add their 16 x C_out products into the sums with plain
//     LDS reads and writes: no atomics, and the order of the additions is fixed (k ascending), so
//     results are bitwise reproducible;
//   * W[k]^T of the next phases travels memory -> registers -> LDS (two buffers) while the
//     current phase runs; a wave reads the tile into registers once per phase;
//   * a wave fetches the 16 gathered rows of a block straight from memory into registers in MFMA
//     operand layout (lane = pair, 16 bytes of the row).  Memory latency is covered inside the
//     wave by a ring of U steps: while step s is multiplied, the rows of steps s+1 .. s+DG and
//     the pair-list entries of steps up to s+U are in flight, across phase and tile boundaries.
//
// A wave's steps are the blocks it has, plus one step (empty if need be) in a tile's last phase;
// a step says how many phase barriers the wave passes before it, so every wave passes every barrier
// and the phases line up although the waves walk different sequences of steps.
#ifndef WCN_CONV_PACK_IMPL_H_
#define WCN_CONV_PACK_IMPL_H_
#include <algorithm>
#include <cmath>
#include <mutex>

#include "wcn_common.h"
#include "wcn_conv_args.h"
#include "wcn_mma.h"

namespace {

using namespace wcn_mma;

constexpr int PB = 16;  // pairs per block (rows of one MFMA)
constexpr int U = 4;    // steps in the ring (unroll factor of the step loop)
constexpr int DG = 2;   // gathered rows are requested DG steps before they are multiplied

// Step descriptor (wave-uniform).
constexpr uint32_t F_NEW_TILE = 1u << 16;  // this wave's first step of a tile
constexpr uint32_t F_TILE_END = 2u << 16;  // last step of a tile
constexpr uint32_t F_END = 4u << 16;       // no work left: leave the loop
constexpr uint32_t F_IDENT = 8u << 16;     // identity offset: pair i of the block is (m0 + p0 + i, p0 + i)
struct Step {
  uint32_t w0;  // pairs of this wave's block (0..16) | k << 8 | flags | slice << 20 | phase barriers to pass before the step << 24
  int32_t p0;   // first pair of the block (index into the pair lists; tile row for F_IDENT)
  int32_t m0;   // first output row of the step's tile
};

template <typename T>
struct PackMma;
template <>
struct PackMma<_Float16> {
  template <int NL>
  static __device__ __forceinline__ f32x4 run(const u32x4 (&W)[NL], const u32x4 (&A)[NL], f32x4 c) {
#pragma unroll
    for (int l = 0; l < NL; ++l)
      c = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, W[l]),
                                                 __builtin_bit_cast(f16x8, A[l]), c, 0, 0, 0);
    return c;
  }
};
template <>
struct PackMma<__bf16> {
  template <int NL>
  static __device__ __forceinline__ f32x4 run(const u32x4 (&W)[NL], const u32x4 (&A)[NL], f32x4 c) {
#pragma unroll
    for (int l = 0; l < NL; ++l)
      c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, W[l]),
                                                  __builtin_bit_cast(bf16x8, A[l]), c, 0, 0, 0);
    return c;
  }
};
// fp32: a lane's 16 bytes are four channels, one per 16x16x4 step (the steps may sum the channels in
// any order as long as both operands agree: step (l, e) covers channels 16 l + 4 (lane >> 4) + e)
template <>
struct PackMma<float> {
  template <int NL>
  static __device__ __forceinline__ f32x4 run(const u32x4 (&W)[NL], const u32x4 (&A)[NL], f32x4 c) {
#pragma unroll
    for (int l = 0; l < NL; ++l) {
      const f32x4 wv = __builtin_bit_cast(f32x4, W[l]), av = __builtin_bit_cast(f32x4, A[l]);
#pragma unroll
      for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_16x16x4f32(wv[e], av[e], c, 0, 0, 0);
    }
    return c;
  }
};

// The ring's loads and the waits for them are written out: every step of a multiplying wave issues
// exactly NL row loads and two pair-list loads, always, in that order, so "the loads of d steps ago
// have landed" is a fixed count for s_waitcnt vmcnt (loads retire in order).  The compiler's own
// bookkeeping merges the loop's many paths and ends up waiting for nearly everything in every step.
// The waits name the registers they vouch for, so that no use can move ahead of them.
template <int NL>
__device__ __forceinline__ void load_row(u32x4 (&dst)[NL], const char* p0, const char* p1) {
  asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(dst[0]) : "v"(p0));
  if (NL == 2) asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(dst[NL - 1]) : "v"(p1));
}
// The same loads with the address as a uniform base (a scalar register pair) plus an unsigned
// 32-bit byte offset per lane: one vector instruction makes the offset, against three or four for
// a 64-bit address per lane.
__device__ __forceinline__ void load_dword_at(int32_t& dst, const int32_t* base, uint32_t off) {
  asm volatile("global_load_dword %0, %1, %2" : "=&v"(dst) : "v"(off), "s"(base));
}
template <int NL>
__device__ __forceinline__ void load_row_at(u32x4 (&dst)[NL], const char* base, uint32_t off) {
  asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(dst[0]) : "v"(off), "s"(base));
  if (NL == 2) asm volatile("global_load_dwordx4 %0, %1, %2 offset:64" : "=&v"(dst[NL - 1]) : "v"(off), "s"(base));
}
template <int N>
__device__ __forceinline__ void wait_loads(int32_t& a, int32_t& b) {
  asm volatile("s_waitcnt vmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N));
}
template <int N, int NL>
__device__ __forceinline__ void wait_rows(u32x4 (&r)[NL]) {
  if (NL == 2)
    asm volatile("s_waitcnt vmcnt(%2)" : "+v"(r[0]), "+v"(r[NL - 1]) : "n"(N));
  else
    asm volatile("s_waitcnt vmcnt(%1)" : "+v"(r[0]) : "n"(N));
}

// LDS traffic is ordered by lgkmcnt alone; a plain s_barrier (no wait for the loads in flight).
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

constexpr int PLAN_AHEAD = 10;              // the supplier publishes a tile's runs this many tiles early
constexpr int PLAN_SLOTS = PLAN_AHEAD + 2;  // ring of published plans
constexpr int LW = 3;                       // weight tiles the supplier holds in registers
constexpr int MAX_BIAS = WCN_PACK_MAX_BIAS;  // output channels (padded) whose bias fits the LDS copy

// The runs of a tile's offsets, in two halves so that the loads can be in flight for a while:
// lane k < K requests its offset's entries of the group_start table, later turns them into the
// pair count and the first pair of the offset's run in the tile.
struct RunsRaw {
  int32_t lo, hi, off;
};
struct Runs2 {  // a lane looks after two offsets: lane and lane + 64
  RunsRaw half[2];
};
template <int R>
__device__ __forceinline__ RunsRaw runs_request(const ConvArgs& a, int vt, int num_vtiles, int ny, int k) {
  RunsRaw r = {0, 0, 0};
  const int lane = k;  // the offset this lane looks after in this call
  if (vt < num_vtiles && lane < a.K && lane != a.identity) {
    const int64_t m0 = (int64_t)(vt / ny) * R;
    const int64_t g0 = m0 >> 6;
    const int64_t g1 = g0 + R / 64 < a.G ? g0 + R / 64 : a.G;
    const int32_t* gs = a.group_start + (int64_t)lane * (a.G + 1);
    r.lo = gs[g0];
    r.hi = gs[g1];
    r.off = (int32_t)a.offsets[lane];
  }
  return r;
}
template <int R>
__device__ __forceinline__ void runs_finish(const ConvArgs& a, int vt, int num_vtiles, int ny, int k,
                                            const RunsRaw& r, int& cnt, int& start) {
  const int lane = k;  // the offset this lane looks after in this call
  cnt = 0;
  start = 0;
  if (vt < num_vtiles && lane < a.K) {
    const int64_t m0 = (int64_t)(vt / ny) * R;
    const int tile_rows = (int)(a.num_out - m0 < R ? a.num_out - m0 : R);
    if (lane == a.identity) {  // every row reads its own input row; the map's pairs are ignored
      const int64_t left = a.num_in - m0;
      cnt = (int)(left < 0 ? 0 : (left < tile_rows ? left : tile_rows));
    } else {
      cnt = r.hi - r.lo;
      start = r.off + r.lo;
      if (cnt < 0 || cnt > R) cnt = 0;  // inconsistent table: contribute nothing
    }
  }
}

// R output rows per tile, NW multiplying waves (+ 1 supplier wave), NB 16-channel blocks of output
// channels per tile column, NL 16-byte loads per gathered row and lane (a row is at most NL * 64
// bytes); FULL = exactly that long.
//
// The supplier wave keeps everything that is not a gathered row or a pair-list entry out of the
// multiplying waves' load stream (whose waits are counts of loads still in flight, and loads retire
// in order: one slow or oddly timed load in that stream stalls the ring): it brings W[k]^T of the
// coming phases into LDS and publishes the runs of the coming tiles there.
//
// WIDE: feature rows of several 128-byte slices (up to four).  A phase is then one slice of one
// offset -- K * NS phases per tile, the weight tile of a phase is the slice's 64 x 64 part of W[k]^T,
// the gathered rows are the slice's 128 bytes -- and everything else stays as it is: the sums stay
// in LDS across the slices.
template <typename T, int R, int NW, int NB, int NL, bool FULL, bool K2, bool WIDE>
__global__ void __launch_bounds__((NW + 1) * 64) conv_fwd_pack(ConvArgs a, int num_vtiles, int ny) {
  static_assert(!WIDE || (NL == 2 && !K2), "slices are 128 bytes; the barrier count of a step has 8 bits");
  constexpr int KH = K2 ? 2 : 1;  // offsets a lane looks after: lane (and lane + 64 for maps of more than 64 offsets)
  extern __shared__ __attribute__((aligned(16))) float smem[];
  constexpr int THREADS = NW * 64;           // multiplying threads
  constexpr int RS = NB * 16;                // floats per row of sums
  constexpr int WPARTS = NL * 4;             // 16-byte parts of a row of W[k]^T
  constexpr int WTILE = NB * 16 * WPARTS;    // 16-byte parts of a weight tile (one column group)
  constexpr int WPL = WTILE / 64;            // parts per supplier lane
  static_assert(R % 64 == 0 && (NB == 4 || NB == 2) && (NL == 1 || NL == 2), "tile shape");
  static_assert(WTILE % 64 == 0, "the supplier's lanes share a weight tile evenly");
  float* const acc = smem;                                   // R x RS sums
  u32x4* const wbuf = (u32x4*)(smem + R * RS);               // 2 weight tiles
  int32_t* const s_plan = (int32_t*)(wbuf + 2 * WTILE);      // PLAN_SLOTS x {cnt[128], start[128]}
  float* const s_bias = (float*)(s_plan + PLAN_SLOTS * 256); // MAX_BIAS
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int K = a.K;
  const int NS = WIDE ? (int)((size_t)a.c_in_pad * sizeof(T) / (NL * 64)) : 1;  // slices of a row
  const int KP = K * NS;                                                       // phases of a tile
  // Tiles of a workgroup: tile0, tile0 + gridDim.x, ...  With several column groups (ny > 1) the
  // tiles of one row tile gather the same rows, so they should meet in one L2: workgroups go to the
  // eight XCDs in turn (blockIdx.x % 8), and the ny workgroups that are neighbours on an XCD
  // (blockIdx.x / 8 = ny * set + column group) take the column groups of row tile 8 * set + XCD.
  // A permutation of [0, gridDim.x) when the grid divides that way; blockIdx.x itself otherwise.
  int tile0 = (int)blockIdx.x;
  {
    const int grid = (int)gridDim.x, per_xcd = grid / 8;
    if (ny > 1 && grid % 8 == 0 && per_xcd % ny == 0) {
      const int xcd = (int)blockIdx.x % 8, q = (int)blockIdx.x / 8;
      tile0 = ((q / ny) * 8 + xcd) * ny + q % ny;
    }
  }
  tile0 = __builtin_amdgcn_readfirstlane(tile0);
  const int tile_step = __builtin_amdgcn_readfirstlane((int)gridDim.x);
  auto tile_of = [&](int iter) -> int { return tile0 + iter * tile_step; };

  if (wave == NW) {
    // ================= supplier wave =================
    const size_t w_tile_bytes = (size_t)a.c_out_pad * a.c_in_pad * sizeof(T);
    const uint32_t w_row_bytes = (uint32_t)a.c_in_pad * (uint32_t)sizeof(T);
    uint32_t w_src[WPL];  // byte offset of this lane's parts inside a tile (column group 0)
    int w_dst[WPL];       // their places in an LDS buffer
#pragma unroll
    for (int j = 0; j < WPL; ++j) {
      const int q = j * 64 + lane, row = q / WPARTS, part = q % WPARTS;
      w_src[j] = (uint32_t)row * w_row_bytes + (uint32_t)part * 16u;
      w_dst[j] = row * WPARTS + (part ^ ((row >> 1) & (WPARTS - 1)));
    }
    auto w_load = [&](int i, u32x4 (&regs)[WPL]) {  // the tile of phase i (counted over all tiles)
      const int it = i / KP, q = i - it * KP, k = WIDE ? q / NS : q, sl = WIDE ? q - k * NS : 0;
      const int vt = tile_of(it);
      const int n0 = vt < num_vtiles ? (vt % ny) * RS : 0;
      const char* p = (const char*)a.Wt + (size_t)k * w_tile_bytes + (size_t)n0 * w_row_bytes + (size_t)sl * (NL * 64);
#pragma unroll
      for (int j = 0; j < WPL; ++j) regs[j] = *reinterpret_cast<const u32x4*>(p + w_src[j]);
    };
    auto w_store = [&](int buf, const u32x4 (&regs)[WPL]) {
#pragma unroll
      for (int j = 0; j < WPL; ++j) wbuf[buf * WTILE + w_dst[j]] = regs[j];
    };
    auto plan_store = [&](int iter, const Runs2& r) {  // offsets lane and lane + 64
      int32_t* slot = s_plan + (iter % PLAN_SLOTS) * 256;
#pragma unroll
      for (int h = 0; h < KH; ++h) {
        int cnt, start;
        runs_finish<R>(a, tile_of(iter), num_vtiles, ny, lane + 64 * h, r.half[h], cnt, start);
        slot[64 * h + lane] = cnt;
        slot[128 + 64 * h + lane] = start;
      }
    };
    auto plan_request = [&](int iter) -> Runs2 {
      Runs2 r = {{{0, 0, 0}, {0, 0, 0}}};
#pragma unroll
      for (int h = 0; h < KH; ++h) r.half[h] = runs_request<R>(a, tile_of(iter), num_vtiles, ny, lane + 64 * h);
      return r;
    };
    for (int i = lane; i < MAX_BIAS; i += 64)
      s_bias[i] = (a.bias && i < a.c_out) ? to_float(((const T*)a.bias)[i]) : 0.f;
    {
      Runs2 first[PLAN_AHEAD];
#pragma unroll
      for (int it = 0; it < PLAN_AHEAD; ++it) first[it] = plan_request(it);
#pragma unroll
      for (int it = 0; it < PLAN_AHEAD; ++it) plan_store(it, first[it]);
    }
    Runs2 pending = {{{0, 0, 0}, {0, 0, 0}}};  // requested at a tile's first phase, published at its last
    u32x4 wr[LW][WPL];
    w_load(0, wr[0]);
    w_store(0, wr[0]);  // phase 0's tile
#pragma unroll
    for (int j = 1; j <= LW; ++j) w_load(j, wr[j % LW]);  // phases 1 .. LW are on their way
    lds_barrier();  // start: plans, bias and the first weight tile are published
    int num_iters = 0;
    while (tile_of(num_iters) < num_vtiles) ++num_iters;
    const int num_phases = num_iters * KP;
    int k = 0, iter = 0;  // k: the phase inside the tile
    for (int i0 = 0; i0 < num_phases; i0 += LW) {
#pragma unroll
      for (int j = 0; j < LW; ++j) {
        const int i = i0 + j;
        if (i >= num_phases) break;
        lds_barrier();  // phase i begins: the buffer of phase i - 1 is free
        // the tile of phase i + 1 (requested LW phases ago) goes to LDS, its registers take phase i + 1 + LW
        if (k == KP - 1 && KP > 1) plan_store(iter + PLAN_AHEAD, pending);
        w_store((i + 1) & 1, wr[(j + 1) % LW]);
        w_load(i + 1 + LW, wr[(j + 1) % LW]);
        if (k == 0) {
          pending = plan_request(iter + PLAN_AHEAD);
          if (KP == 1) plan_store(iter + PLAN_AHEAD, pending);
        }
        if (++k == KP) {
          k = 0;
          ++iter;
          lds_barrier();  // the tile's sums are complete (the multiplying waves write them out)
        }
      }
    }
    return;
  }

  // ================= multiplying waves =================
  const int c = lane & 15, g = lane >> 4;
  const uint32_t row_bytes = (uint32_t)a.c_in * (uint32_t)sizeof(T);
  const char* const zsrc = (const char*)a.zeros;
  const char* const xbase = a.num_in > 0 ? (const char*)a.X : zsrc;
  const int32_t* const zidx = (const int32_t*)a.zeros;

  // sums start at zero (every tile's epilogue leaves them zero again)
  for (int i = tid; i < R * RS / 4; i += THREADS) ((f32x4*)acc)[i] = (f32x4){0.f, 0.f, 0.f, 0.f};

  // this lane's operand parts of a weight tile in LDS: rows cb * 16 + c, parts l * 4 + g
  int w_opnd[NB][NL];
#pragma unroll
  for (int cb = 0; cb < NB; ++cb)
#pragma unroll
    for (int l = 0; l < NL; ++l) {
      const int row = cb * 16 + c;
      w_opnd[cb][l] = row * WPARTS + ((l * 4 + g) ^ ((row >> 1) & (WPARTS - 1)));
    }
  const uint32_t c4 = (uint32_t)c * 4u;
  uint32_t col_off[NL];
  bool col_ok[NL];
#pragma unroll
  for (int l = 0; l < NL; ++l) {
    col_off[l] = (uint32_t)(l * 4 + g) * 16u;
    col_ok[l] = FULL || col_off[l] < row_bytes;
  }

  // ---- the step generator (runs U steps ahead of the multiplications) -----------------------------
  // A wave's steps are the blocks it has to multiply, plus one step (empty if need be) in a tile's
  // last phase, where the tile is written out by all waves together.  Phases in which the wave has
  // no block cost it a barrier each and nothing else: the step that follows says how many.
  // Per tile, lane k % 64 prepares what the wave's steps in offset k need (offsets below 64 in [0],
  // the others in [1]): the descriptor word and the first pair of its first block there, the number
  // of its blocks, the run's pairs; a step then takes its descriptor out of these registers.
  uint32_t plan_w0[2] = {0u, 0u};
  int plan_p0[2] = {0, 0}, plan_mine[2] = {0, 0}, plan_cnt[2] = {0, 0};
  unsigned long long plan_work[2] = {0ull, 0ull};  // the offsets in which this wave has a step
  int gen_iter = -1;                 // tiles this generator has entered, minus one
  int gen_k = K - 1, gen_sl = NS - 1, gen_sip = 0, gen_mine = 0;  // "past the last step of a tile": the first advance enters tile 0
  uint32_t gen_w0 = 0u;              // the first block of the wave in offset gen_k: descriptor word,
  int gen_p0 = 0;                    //   first pair
  int64_t gen_m0 = 0;
  bool gen_live = true;              // false once the tiles are used up
  auto next_step = [&]() -> Step {
    Step d = {F_END, 0, 0};
    if (!gen_live) return d;
    uint32_t extra = 0, bars = 0;
    if (gen_sip >= gen_mine && WIDE && gen_sl + 1 < NS) {  // the same blocks, next slice
      gen_sip = 0;
      ++gen_sl;
      bars = 1;
    } else if (gen_sip >= gen_mine) {  // this wave's steps of the offset are used up
      gen_sip = 0;
      gen_sl = 0;
      if (gen_k == K - 1) {        // next tile
        gen_k = -1;
        ++gen_iter;
        if (tile_of(gen_iter) >= num_vtiles) {
          gen_live = false;
          return d;
        }
        extra |= F_NEW_TILE;
        gen_m0 = (int64_t)(tile_of(gen_iter) / ny) * R;
        const int32_t* slot = s_plan + (gen_iter % PLAN_SLOTS) * 256;
#pragma unroll
        for (int h = 0; h < KH; ++h) {
          const int off = 64 * h + lane;
          const int cnt = slot[off], start = slot[128 + off];
          const int nb = (cnt + PB - 1) / PB;
          int mine = nb > wave ? (nb - wave + NW - 1) / NW : 0;
          if (off == K - 1 && mine == 0) mine = 1;  // the step that ends the tile
          int n1 = cnt - wave * PB;                 // pairs of the wave's first block
          n1 = n1 < 0 ? 0 : (n1 > PB ? PB : n1);
          uint32_t w0 = (uint32_t)n1 | ((uint32_t)off << 8);
          if (off == a.identity) w0 |= F_IDENT;
          if (off == K - 1 && mine == 1) w0 |= F_TILE_END;
          plan_w0[h] = w0;
          plan_p0[h] = start + wave * PB;
          plan_mine[h] = mine;
          plan_cnt[h] = cnt;
          plan_work[h] = __ballot(mine > 0);
        }
      }
      // the next offset with a step of this wave (the last offset always has one)
      const int from = gen_k + 1;
      int nk;
      const unsigned long long w0m = from < 64 ? plan_work[0] & (~0ull << from) : 0ull;
      if (!K2 || w0m != 0ull) {
        nk = (int)__builtin_ctzll(w0m);
      } else {
        const int f1 = from > 64 ? from - 64 : 0;
        nk = 64 + (int)__builtin_ctzll(plan_work[1] & (~0ull << f1));
      }
      bars = (uint32_t)((nk - gen_k - 1) * NS + 1);  // from the last slice of gen_k to the first of nk
      gen_k = nk;
      if (!K2 || gen_k < 64) {
        gen_w0 = __builtin_amdgcn_readlane(plan_w0[0], gen_k);
        gen_p0 = __builtin_amdgcn_readlane(plan_p0[0], gen_k);
        gen_mine = __builtin_amdgcn_readlane(plan_mine[0], gen_k);
      } else {
        gen_w0 = __builtin_amdgcn_readlane(plan_w0[1], gen_k - 64);
        gen_p0 = __builtin_amdgcn_readlane(plan_p0[1], gen_k - 64);
        gen_mine = __builtin_amdgcn_readlane(plan_mine[1], gen_k - 64);
      }
    }
    uint32_t w0 = gen_w0;
    int p0 = gen_p0;
    if (gen_sip > 0) {  // a run of more than NW blocks: the wave's further blocks in the offset
      const int cnt = (!K2 || gen_k < 64) ? __builtin_amdgcn_readlane(plan_cnt[0], gen_k)
                                          : __builtin_amdgcn_readlane(plan_cnt[1], gen_k - 64);
      int n = cnt - (gen_sip * NW + wave) * PB;
      n = n < 0 ? 0 : (n > PB ? PB : n);
      w0 = (uint32_t)n | (gen_w0 & (0xFF00u | F_IDENT));
      p0 = gen_p0 + gen_sip * NW * PB;
      if (gen_k == K - 1 && gen_sip == gen_mine - 1) w0 |= F_TILE_END;
    }
    if (WIDE && gen_sl != NS - 1) w0 &= ~F_TILE_END;  // the tile ends with the last slice
    ++gen_sip;
    d.w0 = w0 | extra | ((uint32_t)gen_sl << 20) | (bars << 24);
    d.p0 = p0;
    d.m0 = (int32_t)gen_m0;
    return d;
  };

  // ---- ring state ---------------------------------------------------------------------------------
  Step ring[U];
  int32_t in_raw[U], out_raw[U];
  u32x4 A[U][NL];
  auto issue_idx = [&](int u) {  // the block's pair-list entries: lane (c, *) reads pair c
    const Step d = next_step();
    ring[u] = d;
    const int n = (int)(d.w0 & 0xFFu);
    const bool use = n > 0 && !(d.w0 & F_IDENT);
    const int32_t* pin = use ? a.in_maps + d.p0 : zidx;
    const int32_t* pout = use ? a.out_maps + d.p0 : zidx;
    const uint32_t last4 = use ? (uint32_t)(n - 1) * 4u : 0u;  // slots past the block's pairs repeat its last pair
    const uint32_t slot4 = c4 < last4 ? c4 : last4;
    load_dword_at(in_raw[u], pin, slot4);
    load_dword_at(out_raw[u], pout, slot4);
  };
  auto issue_gather = [&](int u) {
    const Step d = ring[u];
    const int n = (int)(d.w0 & 0xFFu);
    const int last = n > 0 ? n - 1 : 0;
    // the entries were requested U - DG steps ago: (U - DG - 1) whole steps of loads came after them
    wait_loads<(U - DG - 1) * (NL + 2)>(in_raw[u], out_raw[u]);
    int in = (d.w0 & F_IDENT) ? d.m0 + d.p0 + (c < last ? c : last) : in_raw[u];
    if ((uint32_t)in >= (uint32_t)a.num_in) {  // malformed map: the pair contributes nothing
      in = 0;
      out_raw[u] = -1;
    }
    const uint32_t sl_off = WIDE ? ((d.w0 >> 20) & 3u) * (uint32_t)(NL * 64) : 0u;  // the step's slice of the row
    if (FULL) {  // whole slices; all of X within 4 GiB of its start, fewer than 2^24 rows (the launch checks)
      if (WIDE)
        load_row_at<NL>(A[u], xbase, __umul24((uint32_t)in, row_bytes) + (sl_off + col_off[0]));
      else
        load_row_at<NL>(A[u], xbase, ((uint32_t)in << (NL == 2 ? 7 : 6)) + col_off[0]);
      return;
    }
    const char* p = xbase + (uint64_t)(uint32_t)in * row_bytes + sl_off;
    const char* q[2];
#pragma unroll
    for (int l = 0; l < NL; ++l) {
      q[l] = p + col_off[l];
      const bool ok = WIDE ? sl_off + col_off[l] < row_bytes : col_ok[l];
      if (!FULL) q[l] = ok ? q[l] : zsrc + lane * 16;
    }
    load_row<NL>(A[u], q[0], q[NL - 1]);
  };

  // The ring starts with U empty steps and fills itself through the loop's own code: a separate
  // fill sequence would issue its loads in another order, and the waits inside the loop (counts of
  // loads that may still be in flight) have to hold for every way into it.
#pragma unroll
  for (int u = 0; u < U; ++u) {
    ring[u] = Step{0u, 0, 0};
    in_raw[u] = 0;
    out_raw[u] = 0;
#pragma unroll
    for (int l = 0; l < NL; ++l) A[u][l] = (u32x4){0u, 0u, 0u, 0u};
  }
  lds_barrier();  // start: plans, bias and the first weight tile are published, the sums are zero

  int cmp_iter = -1;    // tile the multiplications are in
  int phase = -1;       // phases passed by the multiplications (over all tiles)
  int64_t m0 = 0;
  int n0 = 0, tile_rows = 0;
  u32x4 Wop[NB][NL];
  bool running = true;
#pragma nounroll
  while (running) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const Step d = ring[u];
      if (d.w0 & F_END) {
        running = false;
        break;
      }
      const int n = (int)(d.w0 & 0xFFu);
      const int bars = (int)(d.w0 >> 24);
      if (bars > 0) {
        // a barrier per phase: everybody is done with the phase before, its additions and its reads
        // of the weight tile
        for (int i = 0; i < bars; ++i) lds_barrier();
        phase += bars;
        if (d.w0 & F_NEW_TILE) {
          ++cmp_iter;
          const int vt = tile_of(cmp_iter);
          m0 = (int64_t)(vt / ny) * R;
          n0 = (vt % ny) * RS;
          tile_rows = (int)(a.num_out - m0 < R ? a.num_out - m0 : R);
        }
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): nothing pending after the barrier (said so that the compiler knows)
        // this phase's tile -> operand registers (only if this wave has a block in the phase)
        if (n > 0) {
#pragma unroll
          for (int cb = 0; cb < NB; ++cb)
#pragma unroll
            for (int l = 0; l < NL; ++l) Wop[cb][l] = wbuf[(phase & 1) * WTILE + w_opnd[cb][l]];
        }
      }
      // The sums this block adds to (the pair-list entries landed DG steps ago, when the rows were
      // requested): read now and handed to the MFMAs as their starting value, so that the read's
      // latency and that of the weight operands pass while the next steps are prepared below.
      const int orow = (d.w0 & F_IDENT) ? d.p0 + c : out_raw[u] - d.m0;
      const bool mine = c < n && (uint32_t)orow < (uint32_t)tile_rows;
      f32x4* sums[NB];
      f32x4 P[NB];
      {
        const int row = mine ? orow : 0;  // lanes without a pair read along (and write nothing)
        float* const rowp = acc + row * RS;
        const int sw = row & 7;  // 16-byte granule cb * 4 + g of the row is stored at granule ^ (row % 8)
#pragma unroll
        for (int cb = 0; cb < NB; ++cb) sums[cb] = reinterpret_cast<f32x4*>(rowp + (((cb * 4 + g) ^ sw) << 2));
      }
      if (n > 0) {
#pragma unroll
        for (int cb = 0; cb < NB; ++cb) P[cb] = *sums[cb];
      }
      const bool tile_end = (d.w0 & F_TILE_END) != 0;
      issue_gather((u + DG) % U);
      issue_idx(u);  // from here on ring[u], in_raw[u] and out_raw[u] belong to a later step
      // The step's rows were requested DG steps ago: that step's two pair-list loads, DG - 1 whole
      // steps of loads and this step's own came after them.  Waited for in every step, also the
      // empty ones: a register is free for other values only once the load into it has landed.
      wait_rows<2 + DG * (NL + 2), NL>(A[u]);
      if (n > 0) {
        // products: lane (c, g) gets channels cb * 16 + 4 g .. + 3 of pair c
#pragma unroll
        for (int cb = 0; cb < NB; ++cb) P[cb] = PackMma<T>::template run<NL>(Wop[cb], A[u], P[cb]);
        if (mine) {
#pragma unroll
          for (int cb = 0; cb < NB; ++cb) *sums[cb] = P[cb];
        }
      }
      if (tile_end) {
        // ---- the tile is complete: bias, one rounding, whole 16-byte stores; sums back to zero ----
        lds_barrier();
        T* __restrict__ out = (T*)a.out;
        constexpr int PARTS = NB * 2;  // 8-channel parts of a row
        static_assert(THREADS % PARTS == 0, "a thread keeps its part");
        const int part = tid % PARTS;
        const int col = n0 + part * 8;
        float bias_v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) bias_v[e] = s_bias[(col + e) & (MAX_BIAS - 1)];
        if (col < a.c_out) {
          for (int i = tid; i < R * PARTS; i += THREADS) {
            const int row = i / PARTS;
            if (row >= tile_rows) break;
            const int sw = row & 7;
            f32x4* const s0 = reinterpret_cast<f32x4*>(acc + row * RS + (((2 * part) ^ sw) << 2));
            f32x4* const s1 = reinterpret_cast<f32x4*>(acc + row * RS + (((2 * part + 1) ^ sw) << 2));
            const f32x4 v0 = *s0, v1 = *s1;
            *s0 = (f32x4){0.f, 0.f, 0.f, 0.f};
            *s1 = (f32x4){0.f, 0.f, 0.f, 0.f};
            float v[8] = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] += bias_v[e];
            if (a.residual) {
              const T* rs = static_cast<const T*>(a.residual) + (m0 + row) * a.c_out + col;
              if (a.vec_res && col + 8 <= a.c_out) {
                constexpr int PER = 16 / sizeof(T);  // entries per 16-byte load
                float r[8];
#pragma unroll
                for (int h = 0; h < 8 / PER; ++h) load_floats<T, PER>(rs + h * PER, *reinterpret_cast<float (*)[PER]>(r + h * PER));
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] += r[e];
              } else {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                  if (col + e < a.c_out) v[e] += to_float(rs[e]);
              }
            }
            if (a.relu) {
#pragma unroll
              for (int e = 0; e < 8; ++e) v[e] = v[e] < 0.f ? 0.f : v[e];
            }
            T* dst = out + (m0 + row) * a.c_out + col;
            if (a.vec_out && col + 8 <= a.c_out) {
              T t[8];
#pragma unroll
              for (int e = 0; e < 8; ++e) t[e] = from_float<T>(v[e]);
              *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(t);
              if (sizeof(T) == 4) *reinterpret_cast<u32x4*>(dst + 4) = *reinterpret_cast<const u32x4*>(t + 4);
            } else {
#pragma unroll
              for (int e = 0; e < 8; ++e)
                if (col + e < a.c_out) dst[e] = from_float<T>(v[e]);
            }
          }
        } else {  // a column part beyond the last channel: only the sums go back to zero
          for (int i = tid; i < R * PARTS; i += THREADS) {
            const int row = i / PARTS, sw = row & 7;
            *reinterpret_cast<f32x4*>(acc + row * RS + (((2 * part) ^ sw) << 2)) = (f32x4){0.f, 0.f, 0.f, 0.f};
            *reinterpret_cast<f32x4*>(acc + row * RS + (((2 * part + 1) ^ sw) << 2)) = (f32x4){0.f, 0.f, 0.f, 0.f};
          }
        }
        // Stores and loads complete in no fixed order relative to each other, so while stores are
        // pending no partial wait can vouch for a load: let them finish here, once per tile,
        // instead of turning every later wait of the ring into a full one.
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
      }
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the ring's last loads land before the registers are given up
}

template <typename T, int R, int NW, int NB, int NL, bool FULL, bool K2, bool WIDE>
int launch_instance(const ConvArgs& a, hipStream_t s) {
  constexpr int lds = R * NB * 16 * 4 + 2 * NB * 16 * NL * 64 + PLAN_SLOTS * 1024 + MAX_BIAS * 4;
  static_assert(lds <= 160 * 1024, "LDS of one workgroup");
  const void* fn = (const void*)conv_fwd_pack<T, R, NW, NB, NL, FULL, K2, WIDE>;
  // more than 64 KiB of dynamic LDS has to be allowed once per device and kernel
  static std::mutex mu;
  static bool allowed[64] = {};
  static int cus[64] = {};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return WCN_ERR_LAUNCH;
  {
    std::lock_guard<std::mutex> hold(mu);
    if (!allowed[device]) {
      if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
        return WCN_ERR_LAUNCH;
      int n = 0;
      if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || n < 1)
        return WCN_ERR_LAUNCH;
      cus[device] = n;
      allowed[device] = true;
    }
  }
  const int ny = (a.c_out + NB * 16 - 1) / (NB * 16);
  const int64_t vtiles = ((a.num_out + R - 1) / R) * ny;
  if (vtiles <= 0 || vtiles > INT32_MAX) return WCN_ERR_INVALID_ARGUMENT;
  const int per_cu = lds * 2 <= 160 * 1024 ? 2 : 1;  // workgroups resident per CU
  const unsigned grid = (unsigned)std::min<int64_t>(vtiles, (int64_t)cus[device] * per_cu);
  hipLaunchKernelGGL((conv_fwd_pack<T, R, NW, NB, NL, FULL, K2, WIDE>), dim3(grid), dim3((NW + 1) * 64), lds, s, a,
                     (int)vtiles, ny);
  wcn_conv_note_kernel("conv_fwd_pack<%s, %d, %d, %d, %d, %s, %s, %s>", wcn_type_text<T>(), R, NW, NB, NL,
                       FULL ? "true" : "false", K2 ? "true" : "false", WIDE ? "true" : "false");
  return hipGetLastError() == hipSuccess ? WCN_OK : WCN_ERR_LAUNCH;
}

#ifndef WCN_PACK_R
#define WCN_PACK_R 512
#endif
#ifndef WCN_PACK_NW
#define WCN_PACK_NW 11  // 12 waves: three per SIMD, 168 registers each; a 512-row tile's run of ~160 pairs is one step
#endif

// CUs of the current device (asked once per device).
inline int device_cus() {
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

// Tile height: R, 3/4 R or 1/2 R rows for column groups of 64 channels, twice that for 32 (same
// LDS), whichever an estimate of the run time likes best: rounds of the persistent grid times the
// phases of a tile, a phase costing its barrier, weight tile and set-up (about one step's worth)
// plus its steps.  Small tiles put more CUs to work on small maps; tall ones need fewer phases.
template <typename T, int NL, bool FULL, bool K2, bool WIDE>
int launch_shaped(const ConvArgs& a, hipStream_t s) {
  // fp32 rows that are not whole 128-byte slices under more than 64 offsets need a few registers
  // more than twelve waves leave a lane (the kernel's waits are counted by hand: nothing may spill);
  // that instance runs with eight waves
  constexpr int R = WCN_PACK_R, NW = (sizeof(T) == 4 && !FULL && K2) ? 7 : WCN_PACK_NW;
  const bool wide_out = a.c_out > 32;
  const int64_t ny = wide_out ? (a.c_out + 63) / 64 : 1;
  const int cus = device_cus();
  const double rows = (double)std::max<int64_t>(a.num_out, 1);
  const bool has_identity = a.identity >= 0 && a.identity < a.K;
  const double others = std::max(1, a.K - (has_identity ? 1 : 0));
  const double per_row = std::max(0.0, (double)a.num_pairs - (has_identity ? rows : 0.0)) / (others * rows);
  auto cost = [&](int r) {
    const int64_t tiles = (a.num_out + r - 1) / r * ny;
    const double rounds = (double)((tiles + cus - 1) / cus);
    const double steps = std::max(1.0, std::ceil(r * per_row / PB / NW));
    const double centre = has_identity ? 1.0 + std::ceil((double)r / PB / NW) : 0.0;
    return rounds * (others * (1.0 + steps) + centre);
  };
  const int unit = wide_out ? R / 4 : R / 2;  // candidates: 2, 3, 4 units
  int best = 4;
  for (int q = 3; q >= 2; --q)
    if (cost(q * unit) < cost(best * unit)) best = q;
  if (wide_out) {
    if (best == 2) return launch_instance<T, R / 2, NW, 4, NL, FULL, K2, WIDE>(a, s);
    if (best == 3) return launch_instance<T, R / 4 * 3, NW, 4, NL, FULL, K2, WIDE>(a, s);
    return launch_instance<T, R, NW, 4, NL, FULL, K2, WIDE>(a, s);
  }
  if (best == 2) return launch_instance<T, R, NW, 2, NL, FULL, K2, WIDE>(a, s);
  if (best == 3) return launch_instance<T, R / 2 * 3, NW, 2, NL, FULL, K2, WIDE>(a, s);
  return launch_instance<T, 2 * R, NW, 2, NL, FULL, K2, WIDE>(a, s);
}

template <typename T, int NL, bool FULL>
int launch_sized(const ConvArgs& a, hipStream_t s) {
  return a.K > 64 ? launch_shaped<T, NL, FULL, true, false>(a, s) : launch_shaped<T, NL, FULL, false, false>(a, s);
}

template <typename T>
int launch_typed(const ConvArgs& a, hipStream_t s) {
  const uint32_t row_bytes = (uint32_t)a.c_in * (uint32_t)sizeof(T);
  // the instances for whole rows address X with 32-bit byte offsets
  const bool near = (uint64_t)a.num_in * row_bytes < (1ull << 32);
  if (row_bytes > 128) {  // several slices (wcn_conv_pack_takes has checked the limits)
    const bool whole = row_bytes % 128 == 0 && near && a.num_in < (1 << 24);
    return whole ? launch_shaped<T, 2, true, false, true>(a, s) : launch_shaped<T, 2, false, false, true>(a, s);
  }
  if (row_bytes == 128 && near) return launch_sized<T, 2, true>(a, s);
  if (row_bytes == 64 && near) return launch_sized<T, 1, true>(a, s);
  if (row_bytes > 64) return launch_sized<T, 2, false>(a, s);
  return launch_sized<T, 1, false>(a, s);
}

}  // namespace

#endif  // WCN_CONV_PACK_IMPL_H_
