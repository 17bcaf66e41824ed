// Coordinate table of 4x4x4-voxel blocks: build and point queries (gfx950).
//
// Build pipeline (all on the caller's stream, no host round trip).  The keys are first grouped into
// bins of one to two thousand (a bin is a hash of the key's 16x16x16-voxel cell, so every 4x4x4
// block lies in exactly one bin); one workgroup per bin then sees all voxels of its blocks and
// builds their masks with LDS atomics:
//   table_hist     per part of the keys (a workgroup): keys per bin (LDS counters) and the part's
//                  bounding box
//   table_colscan  per bin (a wave): prefix sums over the parts; the last workgroup to finish turns
//                  the bin totals into bin starts, merges the boxes and initialises the header
//   table_scatter  per part: every key and its row to its place in its bin; clears the slots
//   table_bins     per bin: block masks and entry counts in an LDS table, their prefix sums, one
//                  64-bit CAS per BLOCK to claim a slot of the table in memory (mask and base are
//                  plain stores), then per key: its place in block order and perm[base + rank] = row
//
// HBM traffic per key: 16 B read twice (histogram, scatter), 20 B written and read (binned entry),
// 20 B written (entry in block order) + 4 B (perm), plus 32 B per table slot to clear.
#include <stdlib.h>
#include <string.h>

#include <chrono>
#include <mutex>
#include <thread>

#include "wcn_common.h"

namespace {

// Bin of a key: a hash of (batch, x >> 4, y >> 4, z >> 4).  Block boundaries are multiples of four
// in absolute coordinates (the table's origin is rounded down to one), so a block never straddles
// two cells.
__device__ __forceinline__ uint32_t bin_of(const int4 c, uint32_t bin_mask) {
  const unsigned long long a = ((unsigned long long)(uint32_t)c.x << 32) | (uint32_t)(c.y >> 4);
  const unsigned long long b = ((unsigned long long)(uint32_t)(c.z >> 4) << 32) | (uint32_t)(c.w >> 4);
  return wcn_mix(a * 0x9E3779B97F4A7C15ull + b, bin_mask);
}

struct PartRange {
  int64_t lo, hi;
};
__device__ __forceinline__ PartRange part_range(int64_t n_keys) {
  const int64_t chunk = (n_keys + gridDim.x - 1) / gridDim.x;
  PartRange r;
  r.lo = (int64_t)blockIdx.x * chunk;
  r.hi = r.lo + chunk < n_keys ? r.lo + chunk : n_keys;
  return r;
}

// Bins: capacity / 2048, at most WCN_MAX_BINS.  The histogram and scatter passes keep one counter
// per bin in LDS (dynamic: 4 bytes per bin, 128 KB at the most), and a thread of the scatter pass
// scans BINS_PER_THREAD bin totals: 4 up to 4096 bins, 32 beyond.
constexpr int SMALL_BINS = 4096;

// Keys per bin of one part of the keys, the part's bounding box; the part's share of the slots is
// set to empty on the way (each slot is two 16-byte stores, {EMPTY, 0} and {0, 0, 0, 0}).
__global__ void __launch_bounds__(1024) table_hist(const int4* __restrict__ keys, int64_t n_keys,
                                                   int32_t bins, int32_t* __restrict__ hist,
                                                   int32_t* __restrict__ part_box,
                                                   WcnSlot* __restrict__ slots, int64_t capacity) {
  extern __shared__ int s_cnt[];  // [bins]
  __shared__ int s_mn[16][4];
  __shared__ int s_mx[16][4];
  const int tid = threadIdx.x, parts = gridDim.x, part = blockIdx.x;
  for (int b = tid; b < bins; b += 1024) s_cnt[b] = 0;
  __syncthreads();
  int mn[4] = {INT32_MAX, INT32_MAX, INT32_MAX, INT32_MAX};
  int mx[4] = {INT32_MIN, INT32_MIN, INT32_MIN, INT32_MIN};
  const PartRange r = part_range(n_keys);
  const uint32_t bin_mask = (uint32_t)bins - 1u;
  constexpr int PER = 4;  // keys a thread has in flight together
  for (int64_t i0 = r.lo + tid; i0 < r.hi; i0 += 1024 * PER) {
    int4 c[PER];
#pragma unroll
    for (int t = 0; t < PER; ++t) {
      const int64_t i = i0 + t * 1024;
      c[t] = keys[i < r.hi ? i : i0];
    }
#pragma unroll
    for (int t = 0; t < PER; ++t) {
      if (i0 + t * 1024 < r.hi) atomicAdd(&s_cnt[bin_of(c[t], bin_mask)], 1);
      mn[0] = min(mn[0], c[t].x); mx[0] = max(mx[0], c[t].x);
      mn[1] = min(mn[1], c[t].y); mx[1] = max(mx[1], c[t].y);
      mn[2] = min(mn[2], c[t].z); mx[2] = max(mx[2], c[t].z);
      mn[3] = min(mn[3], c[t].w); mx[3] = max(mx[3], c[t].w);
    }
  }
  {
    uint4* raw = reinterpret_cast<uint4*>(slots);
    const int64_t items = 2 * capacity, chunk = (items + parts - 1) / parts;
    const int64_t lo = (int64_t)part * chunk, hi = lo + chunk < items ? lo + chunk : items;
    for (int64_t i = lo + tid; i < hi; i += 1024)
      raw[i] = (i & 1) ? make_uint4(0u, 0u, 0u, 0u) : make_uint4(0xFFFFFFFFu, 0xFFFFFFFFu, 0u, 0u);
  }
#pragma unroll
  for (int d = 0; d < 4; ++d) {
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) {
      mn[d] = min(mn[d], __shfl_xor(mn[d], s, 64));
      mx[d] = max(mx[d], __shfl_xor(mx[d], s, 64));
    }
  }
  const int wave = tid >> 6;
  if (wcn_lane() == 0) {
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      s_mn[wave][d] = mn[d];
      s_mx[wave][d] = mx[d];
    }
  }
  __syncthreads();
  for (int b = tid; b < bins; b += 1024) hist[(int64_t)b * parts + part] = s_cnt[b];
  if (tid < 4) {
    int a = s_mn[0][tid], b = s_mx[0][tid];
    for (int w = 1; w < 16; ++w) {
      a = min(a, s_mn[w][tid]);
      b = max(b, s_mx[w][tid]);
    }
    part_box[part * 8 + tid] = a;
    part_box[part * 8 + 4 + tid] = b;
  }
}

// One wave per bin: hist[bin][0..parts) becomes its exclusive prefix sum, bin_total[bin] its sum.
// All loads of a column are issued before the first is used (parts <= 256: four per lane).
__global__ void __launch_bounds__(256) table_colscan(int32_t* __restrict__ hist, int32_t bins,
                                                     int32_t parts, int32_t* __restrict__ bin_total) {
  const int lane = wcn_lane(), wave = threadIdx.x >> 6;
  const int bin = blockIdx.x * 4 + wave;
  if (bin >= bins) return;
  int32_t* col = hist + (int64_t)bin * parts;
  int v[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) v[t] = t * 64 + lane < parts ? col[t * 64 + lane] : 0;
  int carry = 0;
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int incl = wcn_wave_inclusive_sum(v[t]);
    if (t * 64 + lane < parts) col[t * 64 + lane] = carry + incl - v[t];
    carry += __shfl(incl, 63, 64);
  }
  if (lane == 0) bin_total[bin] = carry;
}

// Every key and its row to its place in its bin.  Each workgroup scans the bin totals into bin
// starts for itself (1024 x BPT numbers); workgroup 0 also stores them for the next pass,
// merges the parts' bounding boxes and writes the header.
template <int BPT>
__global__ void __launch_bounds__(1024) table_scatter(const int4* __restrict__ keys, int64_t n_keys,
                                                      int32_t bins, const int32_t* __restrict__ hist,
                                                      const int32_t* __restrict__ bin_total,
                                                      int32_t* __restrict__ bin_start,
                                                      const int32_t* __restrict__ part_box,
                                                      WcnTableHeader* __restrict__ hdr,
                                                      int64_t stats_offset,
                                                      int4* __restrict__ bin_coords,
                                                      int32_t* __restrict__ bin_row) {
  extern __shared__ int s_cur[];  // [bins]
  __shared__ int s_wave[16];
  const int tid = threadIdx.x, lane = wcn_lane(), wave = tid >> 6;
  const int parts = gridDim.x, part = blockIdx.x;
  const PartRange r = part_range(n_keys);
  constexpr int PER = 4;
  int4 c[PER];  // the first keys are requested before anything else
#pragma unroll
  for (int t = 0; t < PER; ++t) {
    const int64_t i = r.lo + tid + t * 1024;
    c[t] = i < r.hi ? keys[i] : make_int4(0, 0, 0, 0);
  }
  int v[BPT], mine[BPT], sum = 0;
#pragma unroll
  for (int t = 0; t < BPT; ++t) {
    const int b = tid * BPT + t;
    v[t] = b < bins ? bin_total[b] : 0;
    mine[t] = b < bins ? hist[(int64_t)b * parts + part] : 0;
    sum += v[t];
  }
  const int incl = wcn_wave_inclusive_sum(sum);
  if (lane == 63) s_wave[wave] = incl;
  __syncthreads();
  int run = incl - sum;
  for (int w = 0; w < wave; ++w) run += s_wave[w];
#pragma unroll
  for (int t = 0; t < BPT; ++t) {
    const int b = tid * BPT + t;
    if (b < bins) {
      s_cur[b] = run + mine[t];
      if (part == 0) bin_start[b] = run;
    }
    run += v[t];
  }
  if (part == 0) {
    if (tid == 0) bin_start[bins] = (int32_t)n_keys;
    if (wave == 1) {  // the boxes: lane d + 8 j merges column d of parts j, j + 8, ...
      const int d = lane & 7;
      int acc = d < 4 ? INT32_MAX : INT32_MIN;
      for (int p = lane >> 3; p < parts; p += 8) {
        const int x = part_box[p * 8 + d];
        acc = d < 4 ? min(acc, x) : max(acc, x);
      }
#pragma unroll
      for (int s = 8; s < 64; s <<= 1) {
        const int o = __shfl_xor(acc, s, 64);
        acc = d < 4 ? min(acc, o) : max(acc, o);
      }
      if (lane < 4) hdr->mn[lane] = acc;
      else if (lane < 8) hdr->mx[lane - 4] = acc;
      if (lane == 8) {
        hdr->num_blocks = 0;
        hdr->status = 0;
        hdr->total = 0;
        hdr->num_keys = (int32_t)n_keys;
        hdr->bins = bins;
        hdr->stats_offset = stats_offset;
      }
    }
  }
  __syncthreads();
  const uint32_t bin_mask = (uint32_t)bins - 1u;
  for (int64_t i0 = r.lo + tid; i0 < r.hi; i0 += 1024 * PER) {
    if (i0 != r.lo + tid) {
#pragma unroll
      for (int t = 0; t < PER; ++t) {
        const int64_t i = i0 + t * 1024;
        c[t] = keys[i < r.hi ? i : i0];
      }
    }
#pragma unroll
    for (int t = 0; t < PER; ++t) {
      const int64_t i = i0 + t * 1024;
      if (i < r.hi) {
        const int pos = atomicAdd(&s_cur[bin_of(c[t], bin_mask)], 1);
        bin_coords[pos] = c[t];
        bin_row[pos] = (int32_t)i;
      }
    }
  }
}

// One workgroup per bin.  LDS holds an open-addressing table of the bin's blocks: key, occupancy
// mask, number of entries (keys, duplicates included), later their prefix sums.
struct BinLds {
  unsigned long long key[WCN_BIN_SLOTS];
  unsigned long long mask[WCN_BIN_SLOTS];
  uint32_t cursor[WCN_BIN_SLOTS];   // entries of the block, then the next free place among them
  uint32_t base[WCN_BIN_SLOTS];     // voxels of the blocks before this one
  int32_t where[WCN_BIN_SLOTS];     // the block's slot in the table in memory
  int32_t low[WCN_BIN_SLOTS];       // lowest row per voxel when keys repeat
  int32_t index[WCN_BIN_SLOTS];     // the block's number in the bin's block list
  int32_t part[3][16];
};

// Entry e of the bin: claims / finds its block in the LDS table, sets its bit, counts itself.
// Returns the block's place in the LDS table, or -1 if the table is full.
__device__ __forceinline__ int bin_insert(BinLds* s, unsigned long long key, uint32_t bit) {
  uint32_t h = wcn_mix(key, WCN_BIN_SLOTS - 1);
  for (int p = 0; p < WCN_BIN_SLOTS; ++p) {
    unsigned long long seen = s->key[h];
    if (seen == WCN_EMPTY_KEY) {
      seen = atomicCAS(&s->key[h], WCN_EMPTY_KEY, key);
      if (seen == WCN_EMPTY_KEY) seen = key;
    }
    if (seen == key) {
      atomicOr(&s->mask[h], 1ull << bit);
      atomicAdd(&s->cursor[h], 1u);
      return (int)h;
    }
    h = (h + 1) & (WCN_BIN_SLOTS - 1);
  }
  return -1;
}

template <bool WANT_SLOT_OF>
__global__ void __launch_bounds__(1024) table_bins(WcnTableHeader* __restrict__ hdr,
                                                   WcnSlot* __restrict__ slots, uint32_t cap_mask,
                                                   const int32_t* __restrict__ bin_start,
                                                   const int4* __restrict__ bin_coords,
                                                   const int32_t* __restrict__ bin_row,
                                                   int32_t* __restrict__ order_tag,
                                                   int32_t* __restrict__ order_row,
                                                   WcnSlot* __restrict__ block_list,
                                                   int32_t* __restrict__ perm,
                                                   int32_t* __restrict__ slot_of,
                                                   int32_t* __restrict__ bin_stats) {
  extern __shared__ __attribute__((aligned(16))) unsigned char bin_smem[];
  BinLds* s = reinterpret_cast<BinLds*>(bin_smem);
  const int tid = threadIdx.x, lane = wcn_lane(), wave = tid >> 6;
  const int lo = bin_start[blockIdx.x], hi = bin_start[blockIdx.x + 1];
  if (tid == 0) {
    bin_stats[2 * blockIdx.x] = 0;
    bin_stats[2 * blockIdx.x + 1] = 0;
  }
  if (lo >= hi) return;
  // A thread keeps its first E entries in registers from the first pass to the last (bins hold
  // one to two thousand keys: one or two entries per thread); entries beyond that are read again.
  constexpr int E = 4;
  int4 c[E];
  int32_t row[E];
  int where[E];
#pragma unroll
  for (int t = 0; t < E; ++t) {
    const int e = lo + tid + t * 1024;
    c[t] = bin_coords[e < hi ? e : lo];
    row[t] = bin_row[e < hi ? e : lo];
  }
  const WcnLayout L = wcn_make_layout(hdr);
  if (!L.ok) {
    if (tid == 0) atomicOr(&hdr->status, WCN_DEV_RANGE);
    for (int e = lo + tid; e < hi; e += 1024) {
      if (WANT_SLOT_OF) slot_of[bin_row[e]] = -1;
      order_row[e] = bin_row[e];
      order_tag[e] = 0;
    }
    return;
  }
  for (int h = tid; h < WCN_BIN_SLOTS; h += 1024) {
    s->key[h] = WCN_EMPTY_KEY;
    s->mask[h] = 0ull;
    s->cursor[h] = 0u;
    s->where[h] = -1;
  }
  __syncthreads();
  // masks and entry counts
  bool lost = false;
#pragma unroll
  for (int t = 0; t < E; ++t) {
    where[t] = -1;
    if (lo + tid + t * 1024 < hi) {
      uint32_t r[4];
      wcn_relative(L, c[t].x, c[t].y, c[t].z, c[t].w, r);  // always inside: the box was built from these keys
      where[t] = bin_insert(s, wcn_block_key(L, r), wcn_block_bit(r));
      lost |= where[t] < 0;
    }
  }
  for (int e = lo + tid + E * 1024; e < hi; e += 1024) {
    const int4 ce = bin_coords[e];
    uint32_t r[4];
    wcn_relative(L, ce.x, ce.y, ce.z, ce.w, r);
    lost |= bin_insert(s, wcn_block_key(L, r), wcn_block_bit(r)) < 0;
  }
  if (lost) atomicOr(&hdr->status, WCN_DEV_OVERFLOW);  // more distinct blocks in this bin than its table holds
  __syncthreads();
  // Prefix sums over the table's slots, entries and voxels.  Thread t owns slots t, t + 1024, ...
  // and counts them as neighbours in the order of the sums (any fixed order will do, and this one
  // reads LDS without bank conflicts and spreads the occupied slots over the threads).
  constexpr int PER = WCN_BIN_SLOTS / 1024;
  uint32_t ne[PER], nv[PER], se = 0, sv = 0, sb = 0;
  unsigned long long bkey[PER], bmask[PER];
#pragma unroll
  for (int t = 0; t < PER; ++t) {
    const int h = tid + t * 1024;
    bkey[t] = s->key[h];
    bmask[t] = s->mask[h];
    ne[t] = s->cursor[h];
    nv[t] = (uint32_t)__popcll(bmask[t]);
    se += ne[t];
    sv += nv[t];
    sb += bkey[t] != WCN_EMPTY_KEY ? 1u : 0u;
  }
  const int ie = wcn_wave_inclusive_sum((int)se), iv = wcn_wave_inclusive_sum((int)sv);
  const int ib = wcn_wave_inclusive_sum((int)sb);
  if (lane == 63) {
    s->part[0][wave] = ie;
    s->part[1][wave] = iv;
    s->part[2][wave] = ib;
  }
  __syncthreads();
  int be = 0, bv = 0, bb = 0, total_v = 0, total_b = 0;
  for (int w = 0; w < 16; ++w) {
    if (w < wave) {
      be += s->part[0][w];
      bv += s->part[1][w];
      bb += s->part[2][w];
    }
    total_v += s->part[1][w];
    total_b += s->part[2][w];
  }
  const bool repeats = total_v != hi - lo;          // some key of this bin came more than once
  const bool low_in_lds = total_v <= WCN_BIN_SLOTS;  // room for one word per voxel
  uint32_t re = (uint32_t)(be + ie) - se, rv = (uint32_t)(bv + iv) - sv;
  int rb = bb + ib - (int)sb;
  // Every block claims a slot of the table in memory: one claimant per block in the whole grid,
  // so the compare-and-swap only ever meets other blocks' keys.
  int claimed = 0;
#pragma unroll
  for (int t = 0; t < PER; ++t) {
    const int h = tid + t * 1024;
    s->cursor[h] = re;
    s->base[h] = rv;
    if (bkey[t] != WCN_EMPTY_KEY) {
      uint32_t g = wcn_mix(bkey[t], cap_mask);
      int p = 0;
      for (; p < WCN_MAX_PROBE; ++p) {
        if (atomicCAS(&slots[g].key, WCN_EMPTY_KEY, bkey[t]) == WCN_EMPTY_KEY) break;
        g = (g + 1) & cap_mask;
      }
      if (p < WCN_MAX_PROBE) {
        slots[g].mask = bmask[t];
        slots[g].base = lo + (int32_t)rv;
        if (WANT_SLOT_OF) s->where[h] = (int32_t)g;
        ++claimed;
      } else {
        atomicOr(&hdr->status, WCN_DEV_OVERFLOW);
      }
      // the block's line of the bin's block list (two 16-byte stores)
      uint4* line = reinterpret_cast<uint4*>(&block_list[lo + rb]);
      line[0] = make_uint4((uint32_t)bkey[t], (uint32_t)(bkey[t] >> 32), (uint32_t)bmask[t], (uint32_t)(bmask[t] >> 32));
      line[1] = make_uint4((uint32_t)(lo + (int32_t)rv), re, 0u, 0u);
      s->index[h] = rb;
      ++rb;
    }
    re += ne[t];
    rv += nv[t];
  }
  (void)claimed;
  if (repeats) {
    if (low_in_lds) {
      for (int j = tid; j < total_v; j += 1024) s->low[j] = INT32_MAX;
    } else {
      for (int j = lo + tid; j < lo + total_v; j += 1024) perm[j] = INT32_MAX;
      __threadfence();
    }
  }
  __syncthreads();
  // every key to its place in block order; the row of every voxel into perm
  auto place = [&](const int4 ce, int32_t rw, int h, int e) {
    if (h < 0) {  // its block did not fit (overflow is flagged): the entry stays where it is
      order_tag[e] = 0;
      order_row[e] = rw;
      if (WANT_SLOT_OF) slot_of[rw] = -1;
      return;
    }
    uint32_t r[4];
    wcn_relative(L, ce.x, ce.y, ce.z, ce.w, r);
    const int v = (int)s->base[h] + wcn_rank_below(s->mask[h], wcn_block_bit(r));
    // without repeated keys the entries of a block are its voxels: block order is perm's order
    const int q = lo + (repeats ? (int)atomicAdd(&s->cursor[h], 1u) : v);
    order_tag[q] = (s->index[h] << 6) | (int32_t)wcn_block_bit(r);
    order_row[q] = rw;
    if (!repeats) perm[lo + v] = rw;
    else if (low_in_lds) atomicMin(&s->low[v], rw);
    else atomicMin(&perm[lo + v], rw);
  };
#pragma unroll
  for (int t = 0; t < E; ++t) {
    const int e = lo + tid + t * 1024;
    if (e < hi) place(c[t], row[t], where[t], e);
  }
  for (int e = lo + tid + E * 1024; e < hi; e += 1024) {
    const int4 ce = bin_coords[e];
    uint32_t r[4];
    wcn_relative(L, ce.x, ce.y, ce.z, ce.w, r);
    const unsigned long long key = wcn_block_key(L, r);
    uint32_t h = wcn_mix(key, WCN_BIN_SLOTS - 1);
    int found = -1;
    for (int p = 0; p < WCN_BIN_SLOTS && found < 0; ++p) {
      if (s->key[h] == key) found = (int)h;
      h = (h + 1) & (WCN_BIN_SLOTS - 1);
    }
    place(ce, bin_row[e], found, e);
  }
  __syncthreads();
  if (WANT_SLOT_OF) {  // the claims have landed: the slot of every key
#pragma unroll
    for (int t = 0; t < E; ++t) {
      const int e = lo + tid + t * 1024;
      if (e < hi && where[t] >= 0) slot_of[row[t]] = s->where[where[t]];
    }
    for (int e = lo + tid + E * 1024; e < hi; e += 1024) {
      const int4 ce = bin_coords[e];
      uint32_t r[4];
      wcn_relative(L, ce.x, ce.y, ce.z, ce.w, r);
      const unsigned long long key = wcn_block_key(L, r);
      uint32_t h = wcn_mix(key, WCN_BIN_SLOTS - 1);
      for (int p = 0; p < WCN_BIN_SLOTS; ++p) {
        if (s->key[h] == key) {
          slot_of[bin_row[e]] = s->where[h];
          break;
        }
        h = (h + 1) & (WCN_BIN_SLOTS - 1);
      }
    }
  }
  if (repeats && low_in_lds)
    for (int j = tid; j < total_v; j += 1024) perm[lo + j] = s->low[j];
  if (tid == 0) {
    bin_stats[2 * blockIdx.x] = total_v;
    bin_stats[2 * blockIdx.x + 1] = total_b;
  }
}

// Sums the bins' voxel and block counts into the header (for the host's status read; the
// kernel-map builder adds them up itself).
__global__ void __launch_bounds__(1024) table_sum_stats(WcnTableHeader* __restrict__ hdr) {
  __shared__ int s_v[16], s_b[16];
  const int32_t bins = hdr->bins;
  const int32_t* bin_stats = reinterpret_cast<const int32_t*>(reinterpret_cast<const char*>(hdr) + hdr->stats_offset);
  int v = 0, b = 0;
  for (int i = threadIdx.x; i < bins; i += 1024) {
    v += bin_stats[2 * i];
    b += bin_stats[2 * i + 1];
  }
#pragma unroll
  for (int s = 32; s > 0; s >>= 1) {
    v += __shfl_xor(v, s, 64);
    b += __shfl_xor(b, s, 64);
  }
  if (wcn_lane() == 0) {
    s_v[threadIdx.x >> 6] = v;
    s_b[threadIdx.x >> 6] = b;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    v = b = 0;
    for (int w = 0; w < 16; ++w) {
      v += s_v[w];
      b += s_b[w];
    }
    hdr->total = v;
    hdr->num_blocks = b;
  }
}

__global__ void __launch_bounds__(256) table_query(const WcnTableHeader* __restrict__ hdr,
                                                   const WcnSlot* __restrict__ slots,
                                                   uint32_t cap_mask,
                                                   const int32_t* __restrict__ perm,
                                                   const int4* __restrict__ queries,
                                                   int64_t num_queries,
                                                   int32_t* __restrict__ results) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= num_queries) return;
  const WcnLayout L = wcn_make_layout(hdr);
  const int4 c = queries[i];
  uint32_t r[4];
  int32_t res = -1;
  if (L.ok && wcn_relative(L, c.x, c.y, c.z, c.w, r)) {
    int32_t base;
    const unsigned long long mask = wcn_lookup_block(slots, cap_mask, wcn_block_key(L, r), &base);
    const uint32_t bit = wcn_block_bit(r);
    if ((mask >> bit) & 1ull) res = perm[base + wcn_rank_below(mask, bit)];
  }
  results[i] = res;
}

inline bool is_pow2(int64_t x) { return x > 0 && (x & (x - 1)) == 0; }

// One-item-per-thread kernels take the uncapped grid (a grid's x extent reaches 2^31 - 1 blocks, and
// item counts here stay below 2^31); a cap is for kernels that loop with a grid stride.
inline int grid_for(int64_t n, int block, int cap = 0x7fffffff) {
  int64_t g = (n + block - 1) / block;
  if (g < 1) g = 1;
  if (g > cap) g = cap;
  return (int)g;
}

}  // namespace

// Enqueue the build kernels.  Shared with the strided-coordinate path, which also wants the slot of
// every key (`want_slot_of`).
int wcn_table_build_impl(const int32_t* keys, int64_t n_keys, const WcnTableView& v,
                         bool want_slot_of, hipStream_t s) {
  const uint32_t cap_mask = (uint32_t)(v.capacity - 1);
  const int4* k4 = (const int4*)keys;
  if (v.bins < 1 || v.bins > WCN_MAX_BINS || (v.bins & (v.bins - 1))) return WCN_ERR_INVALID_ARGUMENT;
  const bool many_bins = v.bins > SMALL_BINS;
  const size_t counters = sizeof(int) * (size_t)v.bins;
  auto scatter = many_bins ? table_scatter<WCN_MAX_BINS / 1024> : table_scatter<SMALL_BINS / 1024>;
  auto fn = want_slot_of ? table_bins<true> : table_bins<false>;
  {  // LDS beyond the default limit: lifted once per device and kernel
    static std::mutex mu;
    static bool allowed[4][64] = {};
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return WCN_ERR_LAUNCH;
    std::lock_guard<std::mutex> hold(mu);
    if (!allowed[want_slot_of][device]) {
      if (hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)sizeof(BinLds)) != hipSuccess)
        return WCN_ERR_LAUNCH;
      allowed[want_slot_of][device] = true;
    }
    if (many_bins && !allowed[2][device]) {
      const int most = (int)(sizeof(int) * WCN_MAX_BINS);
      if (hipFuncSetAttribute((const void*)table_hist, hipFuncAttributeMaxDynamicSharedMemorySize,
                              most) != hipSuccess ||
          hipFuncSetAttribute((const void*)scatter, hipFuncAttributeMaxDynamicSharedMemorySize,
                              most) != hipSuccess)
        return WCN_ERR_LAUNCH;
      allowed[2][device] = true;
    }
  }
  hipLaunchKernelGGL(table_hist, dim3(v.parts), dim3(1024), counters, s, k4, n_keys, v.bins, v.hist,
                     v.part_box, v.slots, v.capacity);
  hipLaunchKernelGGL(table_colscan, dim3((v.bins + 3) / 4), dim3(256), 0, s, v.hist, v.bins,
                     v.parts, v.bin_total);
  hipLaunchKernelGGL(scatter, dim3(v.parts), dim3(1024), counters, s, k4, n_keys, v.bins, v.hist,
                     v.bin_total, v.bin_start, v.part_box, v.hdr,
                     (int64_t)((const char*)v.bin_stats - (const char*)v.hdr), (int4*)v.bin_coords,
                     v.bin_row);
  hipLaunchKernelGGL(fn, dim3(v.bins), dim3(1024), sizeof(BinLds), s, v.hdr, v.slots, cap_mask,
                     v.bin_start, (const int4*)v.bin_coords, v.bin_row, v.order_tag, v.order_row,
                     v.block_list, v.perm, v.slot_of, v.bin_stats);
  WCN_LAUNCH_CHECK();
  return WCN_OK;
}


// Host waits are polls (a blocking stream synchronisation wakes the host tens of microseconds
// late) with an upper bound: WCN_WAIT_LIMIT_MS milliseconds (environment, default 60000), after
// which the call gives up with WCN_ERR_LAUNCH instead of spinning for ever on a stream that is
// stuck.  After a short spin the poll yields the core between looks.
namespace {
int64_t wait_limit_ns() {
  static const int64_t limit = [] {
    const char* e = getenv("WCN_WAIT_LIMIT_MS");
    const long long ms = e ? atoll(e) : 0;
    return (int64_t)(ms > 0 ? ms : 60000) * 1000000;
  }();
  return limit;
}
struct BoundedPoll {
  std::chrono::steady_clock::time_point start = std::chrono::steady_clock::now();
  unsigned looks = 0;
  // false once the time limit has passed
  bool again() {
    if ((++looks & 0xFFu) != 0) return true;
    const int64_t ns = std::chrono::duration_cast<std::chrono::nanoseconds>(
                           std::chrono::steady_clock::now() - start).count();
    if (ns > wait_limit_ns()) return false;
    if (ns > 200000) std::this_thread::yield();
    return true;
  }
};
int wait_for_event(hipEvent_t ev) {
  BoundedPoll poll;
  for (;;) {
    const hipError_t e = hipEventQuery(ev);
    if (e == hipSuccess) return WCN_OK;
    if (e != hipErrorNotReady || !poll.again()) return WCN_ERR_LAUNCH;
  }
}
// per-thread pinned staging of wcn_read_small (released by wcn_thread_release)
thread_local void* g_small_staging = nullptr;
thread_local hipEvent_t g_small_done = nullptr;
thread_local int g_small_device = -1;
}  // namespace

int wcn_read_small(void* host_dst, const void* device_src, size_t bytes, hipStream_t stream) {
  constexpr size_t kStaging = 16384;
  void*& staging = g_small_staging;
  hipEvent_t& done = g_small_done;
  int& staging_device = g_small_device;
  if (bytes > kStaging) return WCN_ERR_INVALID_ARGUMENT;
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return WCN_ERR_LAUNCH;
  if (!staging) {
    if (hipHostMalloc(&staging, kStaging, hipHostMallocDefault) != hipSuccess) {
      staging = nullptr;
      return WCN_ERR_LAUNCH;
    }
  }
  if (!done || staging_device != device) {  // events belong to the device they were created on
    if (done) (void)hipEventDestroy(done);
    if (hipEventCreateWithFlags(&done, hipEventDisableTiming) != hipSuccess) {
      done = nullptr;
      return WCN_ERR_LAUNCH;
    }
    staging_device = device;
  }
  if (hipMemcpyAsync(staging, device_src, bytes, hipMemcpyDeviceToHost, stream) != hipSuccess)
    return WCN_ERR_LAUNCH;
  if (hipEventRecord(done, stream) != hipSuccess) return WCN_ERR_LAUNCH;
  if (wait_for_event(done) != WCN_OK) return WCN_ERR_LAUNCH;
  memcpy(host_dst, staging, bytes);
  return WCN_OK;
}

// A read that is requested where the data is produced and collected later: the copy into the
// thread's second staging buffer is enqueued at once (so that it runs before whatever the caller
// enqueues next), the wait happens in wcn_read_early_end.  One pending read per host thread; an
// end without a matching begin is a plain wcn_read_small.
namespace {
constexpr size_t kEarlyStaging = 16384;
thread_local void* g_early_staging = nullptr;
thread_local hipEvent_t g_early_done = nullptr;
thread_local int g_early_device = -1;
thread_local const void* g_early_src = nullptr;
thread_local size_t g_early_bytes = 0;
}  // namespace

int wcn_read_early_begin(const void* device_src, size_t bytes, hipStream_t stream) {
  g_early_src = nullptr;
  if (bytes > kEarlyStaging) return WCN_ERR_INVALID_ARGUMENT;
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return WCN_ERR_LAUNCH;
  if (!g_early_staging &&
      hipHostMalloc(&g_early_staging, kEarlyStaging, hipHostMallocDefault) != hipSuccess) {
    g_early_staging = nullptr;
    return WCN_ERR_LAUNCH;
  }
  if (!g_early_done || g_early_device != device) {
    if (g_early_done) (void)hipEventDestroy(g_early_done);
    if (hipEventCreateWithFlags(&g_early_done, hipEventDisableTiming) != hipSuccess) {
      g_early_done = nullptr;
      return WCN_ERR_LAUNCH;
    }
    g_early_device = device;
  }
  if (hipMemcpyAsync(g_early_staging, device_src, bytes, hipMemcpyDeviceToHost, stream) != hipSuccess)
    return WCN_ERR_LAUNCH;
  if (hipEventRecord(g_early_done, stream) != hipSuccess) return WCN_ERR_LAUNCH;
  g_early_src = device_src;
  g_early_bytes = bytes;
  return WCN_OK;
}

int wcn_read_early_end(void* host_dst, const void* device_src, size_t bytes, hipStream_t stream) {
  if (g_early_src != device_src || g_early_bytes != bytes)
    return wcn_read_small(host_dst, device_src, bytes, stream);
  g_early_src = nullptr;
  if (wait_for_event(g_early_done) != WCN_OK) return WCN_ERR_LAUNCH;
  memcpy(host_dst, g_early_staging, bytes);
  return WCN_OK;
}

namespace {
constexpr size_t kMailboxBytes = 16384;
thread_local int64_t* g_box = nullptr;        // pinned, coherent, mapped
thread_local hipEvent_t g_box_done = nullptr;
thread_local int g_box_device = -1;
thread_local int64_t g_box_sequence = 0;
}  // namespace

int wcn_mailbox_begin(int64_t** device_visible_box, int64_t* sequence) {
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return WCN_ERR_LAUNCH;
  if (!g_box) {
    void* p = nullptr;
    if (hipHostMalloc(&p, kMailboxBytes, hipHostMallocCoherent | hipHostMallocMapped) != hipSuccess)
      return WCN_ERR_LAUNCH;
    g_box = (int64_t*)p;
    g_box[0] = 0;
  }
  if (!g_box_done || g_box_device != device) {
    if (g_box_done) (void)hipEventDestroy(g_box_done);
    if (hipEventCreateWithFlags(&g_box_done, hipEventDisableTiming) != hipSuccess) {
      g_box_done = nullptr;
      return WCN_ERR_LAUNCH;
    }
    g_box_device = device;
  }
  void* dev = nullptr;
  if (hipHostGetDevicePointer(&dev, g_box, 0) != hipSuccess) return WCN_ERR_LAUNCH;
  *device_visible_box = (int64_t*)dev;
  *sequence = ++g_box_sequence;
  return WCN_OK;
}

int wcn_mailbox_mark(hipStream_t stream) {
  if (!g_box_done) return WCN_ERR_LAUNCH;
  return hipEventRecord(g_box_done, stream) == hipSuccess ? WCN_OK : WCN_ERR_LAUNCH;
}

int wcn_mailbox_end(void* host_dst, size_t payload_bytes, int64_t sequence) {
  if (!g_box || !g_box_done || payload_bytes + 8 > kMailboxBytes) return WCN_ERR_INVALID_ARGUMENT;
  volatile int64_t* word0 = g_box;
  BoundedPoll poll;
  for (;;) {
    if (*word0 == sequence) break;
    const hipError_t e = hipEventQuery(g_box_done);
    if (e == hipErrorNotReady) {
      if (!poll.again()) return WCN_ERR_LAUNCH;
      continue;
    }
    if (e != hipSuccess) return WCN_ERR_LAUNCH;
    // the kernel is over: its write must be there by now, or it never happened
    if (*word0 == sequence) break;
    return WCN_ERR_LAUNCH;
  }
  __atomic_thread_fence(__ATOMIC_ACQUIRE);
  memcpy(host_dst, (const void*)(g_box + 1), payload_bytes);
  return WCN_OK;
}

int wcn_table_status_from_bits(int32_t bits) {
  if (bits & WCN_DEV_RANGE) return WCN_ERR_COORD_RANGE;
  if (bits & WCN_DEV_OVERFLOW) return WCN_ERR_TABLE_OVERFLOW;
  return WCN_OK;
}

extern "C" {

int wcn_version(void) { return 200; }

int wcn_thread_release(void) {
  int st = WCN_OK;
  if (g_small_done && hipEventDestroy(g_small_done) != hipSuccess) st = WCN_ERR_LAUNCH;
  if (g_early_done && hipEventDestroy(g_early_done) != hipSuccess) st = WCN_ERR_LAUNCH;
  if (g_box_done && hipEventDestroy(g_box_done) != hipSuccess) st = WCN_ERR_LAUNCH;
  if (g_small_staging && hipHostFree(g_small_staging) != hipSuccess) st = WCN_ERR_LAUNCH;
  if (g_early_staging && hipHostFree(g_early_staging) != hipSuccess) st = WCN_ERR_LAUNCH;
  if (g_box && hipHostFree(g_box) != hipSuccess) st = WCN_ERR_LAUNCH;
  g_small_done = g_early_done = g_box_done = nullptr;
  g_small_staging = g_early_staging = nullptr;
  g_box = nullptr;
  g_small_device = g_early_device = g_box_device = -1;
  g_early_src = nullptr;
  return st;
}

const char* wcn_status_string(int status) {
  switch (status) {
    case WCN_OK: return "success";
    case WCN_ERR_INVALID_ARGUMENT: return "invalid argument";
    case WCN_ERR_LAUNCH: return "HIP launch or copy failed";
    case WCN_ERR_TABLE_OVERFLOW: return "coordinate table probe limit exceeded (capacity too small)";
    case WCN_ERR_COORD_RANGE: return "coordinate bounding box does not fit the 63-bit block key";
    case WCN_ERR_TOO_MANY_PAIRS: return "kernel map exceeds 2^31-1 pairs";
    case WCN_ERR_WORKSPACE: return "workspace too small";
    default: return "unknown status";
  }
}

int64_t wcn_table_default_capacity(int64_t n_keys) {
  // Blocks hold up to 64 voxels; surface-like data fills ~10 per block.  One slot per two keys
  // keeps the load factor under 0.5 unless almost every voxel is alone in its block, in which
  // case the build reports WCN_ERR_TABLE_OVERFLOW and the caller retries with 4x the slots.
  int64_t want = n_keys + 1;
  int64_t cap = 1024;
  while (cap < want) cap <<= 1;
  return cap;
}

size_t wcn_table_bytes(int64_t n_keys, int64_t capacity) {
  if (n_keys < 0 || capacity <= 0) return 0;
  return wcn_table_layout(nullptr, n_keys, capacity, nullptr);
}

int wcn_table_build(const int32_t* keys, int64_t n_keys, void* table, int64_t capacity,
                    void* stream) {
  if (!table || n_keys < 0 || (n_keys > 0 && !keys)) return WCN_ERR_INVALID_ARGUMENT;
  if (!is_pow2(capacity) || capacity < 64 || capacity > (1ll << 31)) return WCN_ERR_INVALID_ARGUMENT;
  if (n_keys >= (1ll << 31)) return WCN_ERR_INVALID_ARGUMENT;
  WcnTableView v;
  wcn_table_layout(table, n_keys, capacity, &v);
  return wcn_table_build_impl(keys, n_keys, v, false, (hipStream_t)stream);
}

int wcn_table_query(const void* table, int64_t n_keys, int64_t capacity, const int32_t* queries,
                    int64_t num_queries, int32_t* results, void* stream) {
  if (!table || num_queries < 0 || (num_queries > 0 && (!queries || !results)))
    return WCN_ERR_INVALID_ARGUMENT;
  if (!is_pow2(capacity) || capacity < 64 || n_keys < 0) return WCN_ERR_INVALID_ARGUMENT;
  if (num_queries == 0) return WCN_OK;
  WcnTableView v;
  wcn_table_layout(const_cast<void*>(table), n_keys, capacity, &v);
  hipLaunchKernelGGL(table_query, dim3(grid_for(num_queries, 256)), dim3(256), 0,
                     (hipStream_t)stream, v.hdr, v.slots, (uint32_t)(capacity - 1), v.perm,
                     (const int4*)queries, num_queries, results);
  WCN_LAUNCH_CHECK();
  return WCN_OK;
}

int wcn_table_read_status(const void* table, int32_t* host_num_blocks, void* stream) {
  if (!table) return WCN_ERR_INVALID_ARGUMENT;
  WcnTableHeader h;
  hipLaunchKernelGGL(table_sum_stats, dim3(1), dim3(1024), 0, (hipStream_t)stream,
                     reinterpret_cast<WcnTableHeader*>(const_cast<void*>(table)));
  WCN_LAUNCH_CHECK();
  if (wcn_read_small(&h, table, sizeof(h), (hipStream_t)stream) != WCN_OK) return WCN_ERR_LAUNCH;
  if (host_num_blocks) *host_num_blocks = h.num_blocks;
  return wcn_table_status_from_bits(h.status);
}

}  // extern "C"
