// Kernel-map generation and strided output coordinates on top of the block table (gfx950).
//
// The reference materialises a dense (K, M) table of probe results and compacts it with several
// passes (torch_discrete.py:80-157).  Here one thread owns one output voxel and resolves its K
// offsets in registers; a wave's 64 voxels form a "group".  The probe pass stores, per offset and
// group, the 64-bit mask of lanes that hit and its popcount, and the hit lanes park the input
// rows they found in the group's stretch of a scratch table, packed offset by offset and in lane
// order (one contiguous piece per group, for the emit pass to read back).  A row-wise
// exclusive scan turns the counts into start positions; the emit pass then reads masks, starts
// and parked rows -- no table probes -- and every hit lane writes its pair at start + (number of
// hits in lower lanes).  Because groups are 64 consecutive output rows and lanes ascend within a
// group, pairs come out in ascending output index for each offset, exactly the reference's order
// (discrete_kernels.cu:183-213).
#include "wcn_common.h"

int wcn_table_build_impl(const int32_t* keys, int64_t n_keys, const WcnTableView& v,
                         bool want_slot_of, hipStream_t s);
int wcn_table_status_from_bits(int32_t bits);

namespace {

struct KmapGeom {
  int32_t kx, ky, kz;  // kernel size
  int32_t sx, sy, sz;  // in-to-out stride ratio applied to the output coordinates
  int32_t cx, cy, cz;  // centre: size/2 for odd sizes, 0 for even (discrete_kernels.cu:291-294), or the caller's
  int32_t dx, dy, dz;  // dilation: offset (i, j, kk) is ((i - cx) dx, (j - cy) dy, (kk - cz) dz)
  int32_t K;
};

struct KmapWorkspace {  // host-computed addresses inside a kmap workspace
  int64_t* result;      // [0..K] offsets, [K+1] = table status bits, [K+2] = occupied slots | duplicates << 32
  int64_t* row_total;   // [K+1] totals of the rows of `groups`
  int32_t* ticket;      // arrival counter of the scan's workgroups (zeroed by the probe pass)
  int32_t* groups;      // (K+1, G+1): rows 0..K-1 per-offset hit counts of each 64-row group, row K
                        // all hits of the group; after the scan, exclusive prefix sums
  unsigned long long* hits;  // (G, K): lanes of the group that hit, per offset
  int32_t* found;       // (G, 64 K): input rows found by the hit lanes of a group, packed offset by offset
  int64_t G;            // number of 64-row groups
};

inline size_t kmap_layout(void* base, int64_t num_out, int32_t K, KmapWorkspace* w) {
  char* p = (char*)base;
  size_t off = 0;
  const int64_t G = (num_out + 63) / 64;
  if (w) w->result = (int64_t*)(p + off);
  off += wcn_align256(sizeof(int64_t) * (size_t)(K + 3));
  if (w) w->row_total = (int64_t*)(p + off);
  off += wcn_align256(sizeof(int64_t) * (size_t)(K + 1));
  if (w) w->ticket = (int32_t*)(p + off);
  off += 256;
  if (w) w->groups = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * (size_t)(K + 1) * (size_t)(G + 1));
  if (w) w->hits = (unsigned long long*)(p + off);
  off += wcn_align256(sizeof(unsigned long long) * (size_t)K * (size_t)G);
  if (w) w->found = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * (size_t)K * (size_t)G * 64);
  if (w) w->G = G;
  return off;
}

inline int grid_for(int64_t n, int block) {
  int64_t g = (n + block - 1) / block;
  return (int)(g < 1 ? 1 : g);
}

struct KmapProbe {      // what the probe pass leaves for the scan and the emit pass
  unsigned long long* hits;
  int32_t* found;
  int32_t* ticket;      // set to zero
};

// ---- generic kernel: any kernel size up to WCN_MAX_OFFSETS offsets -----------------------------
// Probe results are produced offset by offset; consecutive offsets differ in z (the fastest
// digit) and mostly fall in the block of the previous probe, whose slot is kept in registers.
__global__ void __launch_bounds__(256) kmap_pass(const WcnTableHeader* __restrict__ hdr,
                                                 const WcnSlot* __restrict__ slots,
                                                 uint32_t cap_mask,
                                                 const int32_t* __restrict__ perm,
                                                 const int4* __restrict__ out_coords,
                                                 int64_t num_out, KmapGeom g,
                                                 int32_t* __restrict__ groups, int64_t G,
                                                 KmapProbe o) {
  const int64_t m = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (m == 0) *o.ticket = 0;
  const int64_t group = m >> 6;  // wave-uniform
  if (group >= G) return;
  const int lane = wcn_lane();
  const bool live = m < num_out;
  const WcnLayout L = wcn_make_layout(hdr);
  int4 c = make_int4(0, 0, 0, 0);
  if (live) c = out_coords[m];
  // query origin relative to the table's box, modulo 2^32 like the reference's int arithmetic
  const uint32_t rb = (uint32_t)c.x - L.amin[0];
  const uint32_t rx0 = (uint32_t)c.y * (uint32_t)g.sx - (uint32_t)(g.cx * g.dx) - L.amin[1];
  const uint32_t ry0 = (uint32_t)c.z * (uint32_t)g.sy - (uint32_t)(g.cy * g.dy) - L.amin[2];
  const uint32_t rz0 = (uint32_t)c.w * (uint32_t)g.sz - (uint32_t)(g.cz * g.dz) - L.amin[3];
  const bool usable = live && L.ok && rb <= L.span[0];

  unsigned long long cached_key = WCN_EMPTY_KEY, cached_mask = 0ull;
  int32_t cached_base = 0;
  int k = 0, group_hits = 0;
  for (int i = 0; i < g.kx; ++i) {
    for (int j = 0; j < g.ky; ++j) {
      for (int kk = 0; kk < g.kz; ++kk, ++k) {
        int32_t found = -1;
        uint32_t r[4] = {rb, rx0 + (uint32_t)(i * g.dx), ry0 + (uint32_t)(j * g.dy), rz0 + (uint32_t)(kk * g.dz)};
        if (usable && r[1] <= L.span[1] && r[2] <= L.span[2] && r[3] <= L.span[3]) {
          const unsigned long long key = wcn_block_key(L, r);
          if (key != cached_key) {
            cached_mask = wcn_lookup_block(slots, cap_mask, key, &cached_base);
            cached_key = key;
          }
          const uint32_t bit = wcn_block_bit(r);
          if ((cached_mask >> bit) & 1ull) found = perm[cached_base + wcn_rank_below(cached_mask, bit)];
        }
        const unsigned long long hits = __ballot(found >= 0);
        const int cnt = __popcll(hits);
        if (lane == 0) {
          groups[(int64_t)k * (G + 1) + group] = cnt;
          o.hits[group * g.K + k] = hits;
        }
        if (found >= 0)  // hits of a group are parked contiguously: offset by offset, in lane order
          o.found[group * (64 * (int64_t)g.K) + group_hits + __popcll(hits & ((1ull << lane) - 1ull))] = found;
        group_hits += cnt;
      }
    }
  }
  if (lane == 0) groups[(int64_t)g.K * (G + 1) + group] = group_hits;
}

// ---- fixed-size kernel: compile-time kernel size, every dimension spans at most 2 blocks -------
// Phase 1 requests the (up to) 8 block slots the neighbourhood can touch, all at once, so their
// memory latencies overlap; phase 2 derives the hit bit of each of the K offsets from the cached
// masks (no memory traffic); phase 3 reads the hit rows from `perm`, again as independent loads,
// and leaves masks, counts and rows for the emit pass.
template <int KX, int KY, int KZ>
__global__ void __launch_bounds__(256) kmap_pass_fixed(const WcnTableHeader* __restrict__ hdr,
                                                       const WcnSlot* __restrict__ slots,
                                                       uint32_t cap_mask,
                                                       const int32_t* __restrict__ perm,
                                                       const int4* __restrict__ out_coords,
                                                       int64_t num_out, KmapGeom g,
                                                       int32_t* __restrict__ groups, int64_t G,
                                                       KmapProbe o) {
  constexpr int K = KX * KY * KZ;
  static_assert(KX <= 5 && KY <= 5 && KZ <= 5, "a kernel of up to five voxels spans at most two blocks per dimension");
  __shared__ unsigned long long s_mask[8][256];
  __shared__ int32_t s_base[8][256];
  const int tid = threadIdx.x;
  const int64_t m = (int64_t)blockIdx.x * blockDim.x + tid;
  if (m == 0) *o.ticket = 0;
  const int64_t group = m >> 6;  // wave-uniform
  if (group >= G) return;
  const int lane = wcn_lane();
  const bool live = m < num_out;
  const WcnLayout L = wcn_make_layout(hdr);
  int4 c = make_int4(0, 0, 0, 0);
  if (live) c = out_coords[m];
  const uint32_t rb = (uint32_t)c.x - L.amin[0];
  const uint32_t r0[3] = {(uint32_t)c.y * (uint32_t)g.sx - (uint32_t)g.cx - L.amin[1],
                          (uint32_t)c.z * (uint32_t)g.sy - (uint32_t)g.cy - L.amin[2],
                          (uint32_t)c.w * (uint32_t)g.sz - (uint32_t)g.cz - L.amin[3]};
  const bool usable = live && L.ok && rb <= L.span[0];
  constexpr int KD[3] = {KX, KY, KZ};

  // candidate block coordinates per dimension: the block of the first neighbour and the next one
  uint32_t cand[3][2];
  bool cok[3][2];
#pragma unroll
  for (int d = 0; d < 3; ++d) {
    const uint32_t lim = L.span[d + 1] >> 2;
    cand[d][0] = r0[d] >> 2;
    cand[d][1] = (r0[d] + 4u) >> 2;
    cok[d][0] = cand[d][0] <= lim;
    cok[d][1] = cand[d][1] <= lim && ((r0[d] & 3u) + (uint32_t)(KD[d] - 1)) >= 4u;
  }
  unsigned long long key[8];
  uint32_t hh[8];
  bool need[8];
  uint4 lo[8];
  int32_t hi[8];  // only the base is needed of a slot's second half: a 4-byte load
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int dx = e >> 2, dy = (e >> 1) & 1, dz = e & 1;
    need[e] = usable && cok[0][dx] && cok[1][dy] && cok[2][dz];
    key[e] = ((unsigned long long)rb << L.shift[0]) |
             ((unsigned long long)cand[0][dx] << L.shift[1]) |
             ((unsigned long long)cand[1][dy] << L.shift[2]) | (unsigned long long)cand[2][dz];
    hh[e] = wcn_mix(key[e], cap_mask);
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    lo[e] = make_uint4(0xFFFFFFFFu, 0xFFFFFFFFu, 0u, 0u);
    hi[e] = 0;
    if (need[e]) {
      const uint4* raw = reinterpret_cast<const uint4*>(&slots[hh[e]]);
      lo[e] = raw[0];
      hi[e] = slots[hh[e]].base;
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    unsigned long long mask = 0ull;
    int32_t base = 0;
    if (need[e]) {
      const unsigned long long k0 = ((unsigned long long)lo[e].y << 32) | lo[e].x;
      if (k0 == key[e]) {
        mask = ((unsigned long long)lo[e].w << 32) | lo[e].z;
        base = hi[e];
      } else if (k0 != WCN_EMPTY_KEY) {  // collision on the first probe: walk on
        mask = wcn_lookup_block_from(slots, cap_mask, key[e], (hh[e] + 1) & cap_mask, 1, &base);
      }
    }
    s_mask[e][tid] = mask;
    s_base[e][tid] = base;
  }
  // no barrier: every thread reads back only its own column

  // Offsets are handled NI planes (values of the slowest kernel index) at a time: all of a small
  // kernel at once, one plane of KY x KZ offsets at a time for 4x4x4 and 5x5x5 (the per-offset
  // positions and rows live in registers).
  constexpr int NI = K <= 32 ? KX : 1, PER = NI * KY * KZ;
  static_assert(PER <= 32, "one plane fits a 32-bit hit mask");
  int group_hits = 0;
#pragma nounroll
  for (int i0 = 0; i0 < KX; i0 += NI) {
    uint32_t hm = 0;
    int32_t pos[PER];
    {
      int q = 0;
#pragma unroll
      for (int di = 0; di < NI; ++di) {
#pragma unroll
        for (int j = 0; j < KY; ++j) {
#pragma unroll
          for (int kk = 0; kk < KZ; ++kk, ++q) {
            const uint32_t ax = (r0[0] & 3u) + (uint32_t)(i0 + di), ay = (r0[1] & 3u) + j, az = (r0[2] & 3u) + kk;
            const int e = (int)(((ax >> 2) << 2) | ((ay >> 2) << 1) | (az >> 2));
            const uint32_t bit = ((ax & 3u) << 4) | ((ay & 3u) << 2) | (az & 3u);
            const unsigned long long mk = s_mask[e][tid];
            const uint32_t hit = (uint32_t)((mk >> bit) & 1ull);
            hm |= hit << q;
            pos[q] = s_base[e][tid] + wcn_rank_below(mk, bit);
          }
        }
      }
    }

    int32_t found[PER];
#pragma unroll
    for (int q = 0; q < PER; ++q) found[q] = ((hm >> q) & 1u) ? perm[pos[q]] : -1;

#pragma unroll
    for (int q = 0; q < PER; ++q) {
      const int k = i0 * KY * KZ + q;
      const bool hit = (hm >> q) & 1u;
      const unsigned long long hits = __ballot(hit);
      const int cnt = __popcll(hits);
      if (lane == 0) {
        groups[(int64_t)k * (G + 1) + group] = cnt;
        o.hits[group * K + k] = hits;
      }
      if (hit)  // hits of a group are parked contiguously: offset by offset, in lane order
        o.found[group * (64 * (int64_t)K) + group_hits + __popcll(hits & ((1ull << lane) - 1ull))] = found[q];
      group_hits += cnt;
    }
  }
  if (lane == 0) groups[(int64_t)K * (G + 1) + group] = group_hits;
}

// Emit pass: pair lists from the masks, scanned counts and parked rows of the probe pass, a lane per
// PAIR.  The parked rows of a group already lie in the order of its pairs (offset by offset, in lane
// order), so for 64 offsets at a time (lane j fetches mask and start of offset k0 + j) lane p of a
// round takes pair p, p + 64, ... of those offsets, finds the offset it belongs to (binary search
// over the running counts the lanes hold), its rank there, and from rank and mask the output row.
// A group's ~270 pairs of a 3x3x3 map cost five rounds of one load and two stores where a walk over
// the offsets costs one load and two stores of a few lanes each per offset (5x5x5: 154 -> 85 us).
__device__ __forceinline__ int kmap_nth_set_bit(unsigned long long mask, int r) {  // position of the r-th set bit (r counts from 0)
  uint32_t w = (uint32_t)mask;
  int pos = 0;
  int c = __popc(w);
  if (r >= c) {
    r -= c;
    w = (uint32_t)(mask >> 32);
    pos = 32;
  }
#pragma unroll
  for (int half = 16; half >= 1; half >>= 1) {
    const uint32_t low = w & ((1u << half) - 1u);
    c = __popc(low);
    if (r >= c) {
      r -= c;
      w >>= half;
      pos += half;
    } else {
      w = low;
    }
  }
  return pos;
}

__global__ void __launch_bounds__(256) kmap_emit_flat(const unsigned long long* __restrict__ hits,
                                                      const int32_t* __restrict__ found,
                                                      const int32_t* __restrict__ groups,
                                                      const int64_t* __restrict__ offsets, int K,
                                                      int64_t G, int64_t pair_capacity,
                                                      int32_t* __restrict__ in_maps,
                                                      int32_t* __restrict__ out_maps) {
  const int64_t m = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t group = m >> 6;  // wave-uniform
  if (group >= G) return;
  // offsets[K] = number of pairs, offsets[K + 1] = table status bits (written by the scan): the
  // pass may have been enqueued before the host has seen either, so it checks them itself
  if (offsets[K] > pair_capacity || offsets[K + 1] != 0) return;
  const int lane = wcn_lane();
  const int32_t* parked = found + group * (64 * (int64_t)K);
  for (int k0 = 0; k0 < K; k0 += 64) {  // 64 offsets at a time, a lane per offset
    unsigned long long h = 0ull;
    long long st = 0;
    if (k0 + lane < K) {
      h = hits[group * K + k0 + lane];
      st = offsets[k0 + lane] + groups[(int64_t)(k0 + lane) * (G + 1) + group];
    }
    const int cnt = __popcll(h);
    const int incl = wcn_wave_inclusive_sum(cnt);  // pairs of these offsets up to and including this lane's
    const int total = __shfl(incl, 63, 64);
    for (int p0 = 0; p0 < total; p0 += 64) {
      const int p = p0 + lane;
      const bool live = p < total;
      // first offset whose running count exceeds p (lanes past the last offset hold the total: never chosen by a live p)
      int lo = 0, hi = 63;
#pragma unroll
      for (int step = 0; step < 6; ++step) {
        const int mid = (lo + hi) >> 1;
        const int v = __shfl(incl, mid, 64);
        if (v <= p) lo = mid + 1; else hi = mid;
      }
      const int k = lo;
      const unsigned long long hk = __shfl(h, k, 64);
      const long long sk = __shfl(st, k, 64);
      const int rank = p - (__shfl(incl, k, 64) - __popcll(hk));
      if (live) {
        const long long dst = sk + rank;
        in_maps[dst] = parked[p];
        out_maps[dst] = (int32_t)(group * 64 + kmap_nth_set_bit(hk, rank));
      }
    }
    parked += total;  // the next 64 offsets' rows follow
  }
}

// In-place exclusive prefix sum of each row of `groups` (one workgroup per row, G+1 entries; the
// last entry receives the row total).
__global__ void kmap_zero_ticket(int32_t* ticket) { *ticket = 0; }

struct KmapFinish {  // null `result`: no finishing step
  int64_t* result;              // [0..K] offsets, [K+1] table status bits, [K+2] occupied slots | duplicates << 32
  int32_t* ticket;              // zero before the launch; left at zero
  const WcnTableHeader* hdr;
  int32_t K;
  int64_t* mailbox;             // pinned host memory (or null): the same K + 3 words behind a sequence word
  int64_t sequence;
};

__global__ void __launch_bounds__(1024) kmap_scan_rows(int32_t* __restrict__ groups, int64_t G,
                                                       int64_t* __restrict__ row_total,
                                                       KmapFinish fin) {
  __shared__ int s_wave[16];
  __shared__ int s_stat[2][16];
  int32_t* row = groups + (int64_t)blockIdx.x * (G + 1);
  const int lane = wcn_lane(), wave = threadIdx.x >> 6;
  if (fin.result && blockIdx.x == 0) {
    // Occupied slots and distinct keys of the table, for the host's one read: the sums of the
    // bins' counts, final since the table was built.  The first workgroup adds them up with all
    // its threads while its row's entries are on their way; whichever workgroup finishes last
    // finds the word in place.
    const int32_t bins = fin.hdr->bins;
    const int32_t* stats = reinterpret_cast<const int32_t*>(reinterpret_cast<const char*>(fin.hdr) + fin.hdr->stats_offset);
    int voxels = 0, occupied = 0;
    for (int i = threadIdx.x; i < bins; i += 1024) {
      voxels += stats[2 * i];
      occupied += stats[2 * i + 1];
    }
#pragma unroll
    for (int sft = 32; sft > 0; sft >>= 1) {
      voxels += __shfl_xor(voxels, sft, 64);
      occupied += __shfl_xor(occupied, sft, 64);
    }
    if (lane == 0) {
      s_stat[0][wave] = voxels;
      s_stat[1][wave] = occupied;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      voxels = occupied = 0;
      for (int w = 0; w < 16; ++w) {
        voxels += s_stat[0][w];
        occupied += s_stat[1][w];
      }
      // written before this thread's ticket (and the fence in front of it) further down
      fin.result[fin.K + 2] = (int64_t)occupied | ((int64_t)(voxels != fin.hdr->num_keys ? 1 : 0) << 32);
    }
  }
  int64_t carry = 0;
  constexpr int PER = 4;  // entries per thread and round (one 16-byte load)
  for (int64_t start = 0; start < G; start += 1024 * PER) {
    const int64_t idx = start + (int64_t)threadIdx.x * PER;
    int v[PER];
    int sum = 0;
#pragma unroll
    for (int t = 0; t < PER; ++t) {
      v[t] = idx + t < G ? row[idx + t] : 0;
      sum += v[t];
    }
    const int incl = wcn_wave_inclusive_sum(sum);
    if (lane == 63) s_wave[wave] = incl;
    __syncthreads();
    int before = 0, all = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      const int t = s_wave[w];
      if (w < wave) before += t;
      all += t;
    }
    int run = (int)carry + before + incl - sum;
#pragma unroll
    for (int t = 0; t < PER; ++t) {
      if (idx + t < G) row[idx + t] = run;
      run += v[t];
    }
    carry += all;
    __syncthreads();
  }
  __shared__ int s_last;
  if (threadIdx.x == 0) {
    // a row of the per-offset counts holds at most M < 2^31 pairs; the row of all hits can
    // exceed int32, which the host turns into WCN_ERR_TOO_MANY_PAIRS
    row[G] = (int32_t)carry;
    row_total[blockIdx.x] = carry;
    s_last = 0;
    if (fin.result) {
      __threadfence();
      s_last = atomicAdd(fin.ticket, 1) == (int32_t)gridDim.x - 1;
    }
  }
  __syncthreads();
  if (!s_last || wave != 0) return;
  // The workgroup that finishes last turns the row totals into offsets[K+1] and copies the
  // table's status next to them, so the host needs one read for everything.  Its first wave
  // fetches 64 totals at a time (independent loads) and scans them.
  __threadfence();
  int64_t run = 0;
  for (int k0 = 0; k0 < fin.K; k0 += 64) {
    const int k = k0 + lane;
    int64_t v = k < fin.K ? __hip_atomic_load(&row_total[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int64_t t = __shfl_up(v, d, 64);
      if (lane >= d) v += t;
    }
    if (k < fin.K) {
      fin.result[k + 1] = run + v;
      if (fin.mailbox) fin.mailbox[1 + k + 1] = run + v;
    }
    run += __shfl(v, 63, 64);
  }
  if (lane == 0) {
    const int64_t status = fin.hdr->status;
    // occupied slots | duplicates << 32: left there by the first workgroup (see the top)
    const int64_t blocks = __hip_atomic_load(&fin.result[fin.K + 2], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    fin.result[0] = 0;
    fin.result[fin.K + 1] = status;
    if (fin.mailbox) {
      fin.mailbox[1] = 0;
      fin.mailbox[1 + fin.K + 1] = status;
      fin.mailbox[1 + fin.K + 2] = blocks;
    }
    *fin.ticket = 0;
  }
  if (fin.mailbox) {
    // the host polls the sequence word: everything this wave wrote into the mailbox is visible to
    // it before the word changes
    __threadfence_system();
    if (lane == 0) __hip_atomic_store(&fin.mailbox[0], fin.sequence, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

// ---- maps of a coordinate set onto itself (stride 1), probed block by block ----------------------
// The table build leaves, per bin, the list of its blocks and its keys in block order.  This probe
// pass walks the blocks: the 64 voxels of a block are tested against a kernel offset with one
// 64-bit AND of occupancy masks, and the neighbours' slots are fetched once per block instead of
// once per voxel.  What it finds goes back to row order through two small per-row records: the
// hit mask of the row (bit k = offset k has a pair) and the place where the found rows are parked.
// The count and emit passes then run in row order, as the reference's pair order demands.
struct SelfWorkspace {
  int64_t* result;      // as KmapWorkspace (same places: the read-result call serves both)
  int64_t* row_total;
  int32_t* ticket;
  int32_t* groups;      // (K+1, G+1): the finished group starts of every offset (written by the emit pass)
  uint32_t* hm;         // (num_out, words) hit masks per row
  int32_t* ptr;         // num_out: index into park of the row's first found row
  int32_t* park;        // (num_out, K) at most: found rows, row by row of a tile, offsets ascending
  int32_t* chunk;       // (K, C + 1): pairs per offset and chunk of SELF_CHUNK rows, then prefix sums
  int64_t G, C;
  int32_t words;
};
constexpr int SELF_CHUNK = 256;  // rows per workgroup of the count and emit passes

inline size_t self_layout(void* base, int64_t num_out, int32_t K, SelfWorkspace* w) {
  char* p = (char*)base;
  size_t off = 0;
  const int64_t G = (num_out + 63) / 64, C = (num_out + SELF_CHUNK - 1) / SELF_CHUNK;
  const int32_t words = (K + 31) / 32;
  if (w) w->result = (int64_t*)(p + off);
  off += wcn_align256(sizeof(int64_t) * (size_t)(K + 3));
  if (w) w->row_total = (int64_t*)(p + off);
  off += wcn_align256(sizeof(int64_t) * (size_t)(K + 1));
  if (w) w->ticket = (int32_t*)(p + off);
  off += 256;
  if (w) w->groups = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * (size_t)(K + 1) * (size_t)(G + 1));
  if (w) w->hm = (uint32_t*)(p + off);
  off += wcn_align256(sizeof(uint32_t) * (size_t)words * (size_t)num_out);
  if (w) w->ptr = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * (size_t)num_out);
  if (w) w->park = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * (size_t)K * (size_t)num_out);
  if (w) w->chunk = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * (size_t)K * (size_t)(C + 1));
  if (w) {
    w->G = G;
    w->C = C;
    w->words = words;
  }
  return off;
}

// Occupancy of a 4x4x4 block (bit x * 16 + y * 4 + z) as seen from d voxels further along one
// axis, |d| <= 2: A is the block itself, B its neighbour block in the direction of d.
__device__ __forceinline__ unsigned long long shift_z(unsigned long long A, unsigned long long B, int d) {
  const int s = d > 0 ? d : -d;
  const bool up = d > 0;
  const uint32_t nib = up ? ((1u << (4 - s)) - 1u) : (0xFu & ~((1u << s) - 1u));  // z the block itself answers
  const uint32_t m32 = 0x11111111u * nib;
  const unsigned long long m = ((unsigned long long)m32 << 32) | m32;
  const unsigned long long a = up ? A >> s : A << s;
  const unsigned long long b = up ? B << (4 - s) : B >> (4 - s);
  return d == 0 ? A : ((a & m) | (b & ~m));
}
template <int D>
__device__ __forceinline__ unsigned long long shift_y(unsigned long long A, unsigned long long B) {
  if (D == 0) return A;
  constexpr int S = D > 0 ? D : -D;
  constexpr unsigned long long M = D > 0 ? 0x0001000100010001ull * ((1u << (16 - 4 * S)) - 1u)
                                         : 0x0001000100010001ull * (0xFFFFu & ~((1u << (4 * S)) - 1u));
  return D > 0 ? (((A >> (4 * S)) & M) | ((B << (16 - 4 * S)) & ~M))
               : (((A << (4 * S)) & M) | ((B >> (16 - 4 * S)) & ~M));
}
template <int D>
__device__ __forceinline__ unsigned long long shift_x(unsigned long long A, unsigned long long B) {
  if (D == 0) return A;
  constexpr int S = D > 0 ? D : -D;
  return D > 0 ? ((A >> (16 * S)) | (B << (64 - 16 * S))) : ((A << (16 * S)) | (B >> (64 - 16 * S)));
}

// One (dy, dx) pair of hit masks of a block for a fixed dz: Z[i][j] is the z-shifted occupancy of
// the block column (bx + i - 1, by + j - 1).
template <int R, int DY, int DX>
__device__ __forceinline__ void self_hits_xy(const unsigned long long (&Z)[3][3], unsigned long long self,
                                             int dzi, unsigned long long* __restrict__ out) {
  constexpr int S = 2 * R + 1;
  constexpr int J = DY > 0 ? 2 : (DY < 0 ? 0 : 1), I = DX > 0 ? 2 : (DX < 0 ? 0 : 1);
  const unsigned long long y_here = shift_y<DY>(Z[1][1], Z[1][J]);
  const unsigned long long y_next = DX == 0 ? 0ull : shift_y<DY>(Z[I][1], Z[I][J]);
  out[((DX + R) * S + (DY + R)) * S + dzi] = self & shift_x<DX>(y_here, y_next);
}
template <int R, int DY>
__device__ __forceinline__ void self_hits_y(const unsigned long long (&Z)[3][3], unsigned long long self,
                                            int dzi, unsigned long long* __restrict__ out) {
  self_hits_xy<R, DY, -1>(Z, self, dzi, out);
  self_hits_xy<R, DY, 0>(Z, self, dzi, out);
  self_hits_xy<R, DY, 1>(Z, self, dzi, out);
  if (R == 2) {
    self_hits_xy<R, DY, -2>(Z, self, dzi, out);
    self_hits_xy<R, DY, 2>(Z, self, dzi, out);
  }
}

// The probe pass, a workgroup per tile of SELF_TILE consecutive blocks of one bin's block list:
//   1a. a lane per block: its line of the block list, and which of its 26 neighbour blocks matter
//       (a neighbour is looked up only if the block has a voxel within R of the face, edge or
//       corner it lies behind: 9 or 10 of 26 for a block of a surface);
//   1b. a lane per lookup: the neighbour's slot from the table (mask and base into LDS);
//   2.  a lane per (block, dz): the hit masks of all (2R+1)^2 offsets with that dz, 64 voxels at
//       a time, from shifts and ANDs of the occupancy masks;
//   3.  a lane per entry (key) of the tile: its bit of every hit mask makes the row's hit mask;
//       the positions of the found rows go into an LDS list, and the rows are fetched from perm
//       and parked behind one another with a lane per found row.
constexpr int SELF_TILE = 32;
constexpr int SELF_LIST = 1024;  // found rows fetched per turn of a workgroup
template <int R>
__global__ void __launch_bounds__(256) self_probe(const WcnTableHeader* __restrict__ hdr,
                                                  const WcnSlot* __restrict__ slots, uint32_t cap_mask,
                                                  const int32_t* __restrict__ perm,
                                                  const int32_t* __restrict__ bin_start,
                                                  const int32_t* __restrict__ bin_stats,
                                                  const WcnSlot* __restrict__ block_list,
                                                  const int32_t* __restrict__ order_tag,
                                                  const int32_t* __restrict__ order_row,
                                                  uint32_t* __restrict__ hm_out,
                                                  int32_t* __restrict__ ptr_out,
                                                  int32_t* __restrict__ park, int32_t* __restrict__ ticket) {
  constexpr int S = 2 * R + 1, K = S * S * S, WORDS = (K + 31) / 32;
  __shared__ unsigned long long s_nmask[SELF_TILE][27];
  __shared__ int32_t s_nbase[SELF_TILE][27];
  __shared__ unsigned long long s_hit[SELF_TILE][K];
  __shared__ uint32_t s_coord[SELF_TILE][4];  // batch and block coordinates of every block of the tile
  __shared__ int32_t s_first[SELF_TILE + 1];  // first entry of every block of the tile, and the end
  __shared__ int32_t s_wave[4];
  __shared__ int32_t s_list[SELF_LIST];
  __shared__ uint16_t s_task[SELF_TILE * 26];  // (block of the tile) << 5 | neighbour: the lookups to make
  __shared__ int32_t s_tasks;
  const int tid = threadIdx.x, lane = wcn_lane(), wave = tid >> 6;
  if (blockIdx.x == 0 && blockIdx.y == 0 && tid == 0) *ticket = 0;
  const int bin = blockIdx.x;
  const int lo = bin_start[bin], entries = bin_start[bin + 1] - lo, blocks = bin_stats[2 * bin + 1];
  const WcnLayout L = wcn_make_layout(hdr);
  if (!L.ok) return;
  const uint32_t lim[3] = {L.span[1] >> 2, L.span[2] >> 2, L.span[3] >> 2};
  for (int j0 = (int)blockIdx.y * SELF_TILE; j0 < blocks; j0 += (int)gridDim.y * SELF_TILE) {
    const int nblk = blocks - j0 < SELF_TILE ? blocks - j0 : SELF_TILE;
    // neighbours that are not looked up count as empty
    for (int idx = tid; idx < SELF_TILE * 27; idx += 256) {
      const int t = idx / 27, n = idx - t * 27;
      if (n != 13) {
        s_nmask[t][n] = 0ull;
        s_nbase[t][n] = 0;
      }
    }
    // 1a
    if (wave == 0) {
      uint32_t wanted = 0;
      if (lane < nblk) {
        const uint4* line = reinterpret_cast<const uint4*>(&block_list[lo + j0 + lane]);
        const uint4 a = line[0], b = line[1];
        const unsigned long long key = ((unsigned long long)a.y << 32) | a.x;
        const unsigned long long self = ((unsigned long long)a.w << 32) | a.z;
        s_nmask[lane][13] = self;
        s_nbase[lane][13] = (int32_t)b.x;
        s_first[lane] = (int32_t)b.y;
        const uint32_t bz = (uint32_t)(key & ((1ull << L.shift[2]) - 1ull));
        const uint32_t by = (uint32_t)((key >> L.shift[2]) & ((1ull << (L.shift[1] - L.shift[2])) - 1ull));
        const uint32_t bx = (uint32_t)((key >> L.shift[1]) & ((1ull << (L.shift[0] - L.shift[1])) - 1ull));
        s_coord[lane][0] = (uint32_t)(key >> L.shift[0]);
        s_coord[lane][1] = bx;
        s_coord[lane][2] = by;
        s_coord[lane][3] = bz;
        // voxels within R of the low / high end of every axis
        constexpr unsigned long long XL = (1ull << (16 * R)) - 1ull, XH = ~0ull << (64 - 16 * R);
        constexpr unsigned long long YL = 0x0001000100010001ull * ((1u << (4 * R)) - 1u);
        constexpr unsigned long long YH = 0x0001000100010001ull * (0xFFFFu & (0xFFFFu << (16 - 4 * R)));
        constexpr unsigned long long ZL = 0x1111111111111111ull * ((1u << R) - 1u);
        constexpr unsigned long long ZH = 0x1111111111111111ull * (0xFu & (0xFu << (4 - R)));
        const unsigned long long mx[3] = {self & XL, self, self & XH};
        const bool inx[3] = {bx >= 1u, true, bx + 1u <= lim[0]};
        const bool iny[3] = {by >= 1u, true, by + 1u <= lim[1]};
        const bool inz[3] = {bz >= 1u, true, bz + 1u <= lim[2]};
#pragma unroll
        for (int i = 0; i < 3; ++i) {
          const unsigned long long my[3] = {mx[i] & YL, mx[i], mx[i] & YH};
#pragma unroll
          for (int j = 0; j < 3; ++j) {
            const unsigned long long mz[3] = {my[j] & ZL, my[j], my[j] & ZH};
#pragma unroll
            for (int k = 0; k < 3; ++k) {
              const int n = i * 9 + j * 3 + k;
              if (n != 13 && mz[k] != 0ull && inx[i] && iny[j] && inz[k]) wanted |= 1u << n;
            }
          }
        }
      }
      const int cnt = __popc(wanted);
      const int incl = wcn_wave_inclusive_sum(cnt);
      int at = incl - cnt;
      while (wanted) {
        const int n = __builtin_ctz(wanted);
        wanted &= wanted - 1u;
        s_task[at++] = (uint16_t)((lane << 5) | n);
      }
      if (lane == 63) s_tasks = incl;
      if (lane == 0) s_first[nblk] = j0 + nblk < blocks ? block_list[lo + j0 + nblk].pad[0] : entries;
    }
    __syncthreads();
    // the tile's first round of entries is requested now and used in step 3
    const int e0 = s_first[0], ne = s_first[nblk] - e0;
    int32_t tag_ahead = 0, row_ahead = -1;
    if (tid < ne) {
      tag_ahead = order_tag[lo + e0 + tid];
      row_ahead = order_row[lo + e0 + tid];
    }
    // 1b
    const int tasks = s_tasks;
    for (int i = tid; i < tasks; i += 256) {
      const int task = s_task[i], t = task >> 5, n = task & 31;
      const int dx = n / 9 - 1, dy = (n / 3) % 3 - 1, dz = n % 3 - 1;
      const unsigned long long nkey = ((unsigned long long)s_coord[t][0] << L.shift[0]) |
                                      ((unsigned long long)(s_coord[t][1] + (uint32_t)dx) << L.shift[1]) |
                                      ((unsigned long long)(s_coord[t][2] + (uint32_t)dy) << L.shift[2]) |
                                      (unsigned long long)(s_coord[t][3] + (uint32_t)dz);
      int32_t base = 0;
      s_nmask[t][n] = wcn_lookup_block(slots, cap_mask, nkey, &base);
      s_nbase[t][n] = base;
    }
    __syncthreads();
    // 2
    for (int idx = tid; idx < nblk * S; idx += 256) {
      const int t = idx / S, dzi = idx - t * S, dz = dzi - R;
      const int nz = dz > 0 ? 2 : (dz < 0 ? 0 : 1);
      unsigned long long Z[3][3];
#pragma unroll
      for (int i = 0; i < 3; ++i)
#pragma unroll
        for (int j = 0; j < 3; ++j)
          Z[i][j] = shift_z(s_nmask[t][i * 9 + j * 3 + 1], s_nmask[t][i * 9 + j * 3 + nz], dz);
      const unsigned long long self = s_nmask[t][13];
      unsigned long long* out = &s_hit[t][0];
      self_hits_y<R, -1>(Z, self, dzi, out);
      self_hits_y<R, 0>(Z, self, dzi, out);
      self_hits_y<R, 1>(Z, self, dzi, out);
      if (R == 2) {
        self_hits_y<R, -2>(Z, self, dzi, out);
        self_hits_y<R, 2>(Z, self, dzi, out);
      }
    }
    __syncthreads();
    // 3
    int run = 0;  // found rows parked so far (the same in every thread)
    for (int i0 = 0; i0 < ne; i0 += 256) {
      const int i = i0 + tid;
      const bool live = i < ne;
      int32_t tag = tag_ahead, m = row_ahead;
      if (live && i0 > 0) {
        tag = order_tag[lo + e0 + i];
        m = order_row[lo + e0 + i];
      }
      const int t = (tag >> 6) - j0;
      const uint32_t bit = (uint32_t)tag & 63u;
      const bool known = live && t >= 0 && t < nblk;  // an entry whose block overflowed the table's build has no tag
      uint32_t hm[WORDS];
#pragma unroll
      for (int w = 0; w < WORDS; ++w) hm[w] = 0;
      if (known) {
        const uint32_t* half = reinterpret_cast<const uint32_t*>(&s_hit[t][0]) + (bit >> 5);
#pragma unroll
        for (int k = 0; k < K; ++k) hm[k >> 5] |= ((half[2 * k] >> (bit & 31u)) & 1u) << (k & 31);
      }
      int cnt = 0;
#pragma unroll
      for (int w = 0; w < WORDS; ++w) cnt += __popc(hm[w]);
      const int incl = wcn_wave_inclusive_sum(cnt);
      if (lane == 63) s_wave[wave] = incl;
      __syncthreads();
      int before = run + incl - cnt, all = 0;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        if (w < wave) before += s_wave[w];
        all += s_wave[w];
      }
      run += all;
      const int64_t mine = (int64_t)(lo + e0) * K + before;  // the row's place in the tile's piece of park
      if (live) {
#pragma unroll
        for (int w = 0; w < WORDS; ++w) hm_out[(int64_t)m * WORDS + w] = hm[w];
        ptr_out[m] = (int32_t)mine;
      }
      // The positions in perm of this round's found rows go into an LDS list, in the order of
      // their places in park; the rows are then fetched and parked with a lane per found row
      // (independent loads, coalesced stores).  The list holds SELF_LIST positions at a time.
      const int x = (int)(bit >> 4), y = (int)((bit >> 2) & 3u), z = (int)(bit & 3u);
      const int64_t round_base = (int64_t)(lo + e0) * K + (run - all);
      const int first = before - (run - all);  // this row's first place in the round's list
      for (int win = 0; win < all; win += SELF_LIST) {
        int done = 0;
#pragma unroll
        for (int w = 0; w < WORDS; ++w) {
          uint32_t rest = hm[w];
          while (rest) {
            const int k = 32 * w + __builtin_ctz(rest);
            rest &= rest - 1u;
            const int at = first + done - win;
            ++done;
            if (at < 0 || at >= SELF_LIST) continue;
            const int ax = x + k / (S * S) - R, ay = y + (k / S) % S - R, az = z + k % S - R;
            const int n = ((ax >> 2) + 1) * 9 + ((ay >> 2) + 1) * 3 + (az >> 2) + 1;
            const uint32_t nbit = (uint32_t)(((ax & 3) << 4) | ((ay & 3) << 2) | (az & 3));
            s_list[at] = s_nbase[t][n] + wcn_rank_below(s_nmask[t][n], nbit);
          }
        }
        __syncthreads();
        const int have = all - win < SELF_LIST ? all - win : SELF_LIST;
        for (int h0 = 0; h0 < have; h0 += 4 * 256) {
          int32_t got[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int h = h0 + u * 256 + tid;
            got[u] = h < have ? perm[s_list[h]] : 0;
          }
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int h = h0 + u * 256 + tid;
            if (h < have) park[round_base + win + h] = got[u];
          }
        }
        __syncthreads();  // the list (and s_wave) are written again
      }
      if (all == 0) __syncthreads();
    }
    __syncthreads();  // the tile's tables are rewritten by the next tile
  }
}

// Row order again: pairs per offset in every chunk of SELF_CHUNK rows.
template <int K>
__global__ void __launch_bounds__(SELF_CHUNK) self_count(const uint32_t* __restrict__ hm, int64_t num_out,
                                                         int32_t* __restrict__ chunk_count, int64_t C) {
  constexpr int WORDS = (K + 31) / 32, WAVES = SELF_CHUNK / 64;
  __shared__ int s_cnt[WAVES][K];
  const int tid = threadIdx.x, lane = wcn_lane(), wave = tid >> 6;
  const int64_t m = (int64_t)blockIdx.x * SELF_CHUNK + tid;
  uint32_t h[WORDS];
#pragma unroll
  for (int w = 0; w < WORDS; ++w) h[w] = m < num_out ? hm[m * WORDS + w] : 0u;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const int n = __popcll(__ballot((h[k >> 5] >> (k & 31)) & 1u));
    if (lane == 0) s_cnt[wave][k] = n;
  }
  __syncthreads();
  for (int k = tid; k < K; k += SELF_CHUNK) {
    int n = 0;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) n += s_cnt[w][k];
    chunk_count[(int64_t)k * (C + 1) + blockIdx.x] = n;
  }
}

// Row order, a lane per PAIR.  A wave's pairs are numbered offset by offset and, inside an offset,
// by lane; pair number q finds its offset by binary search over the running counts, its rank
// there, from rank and the offset's lane mask its row, and from the row's hit mask the place of the
// found row among that row's parked rows.
template <int K>
__global__ void __launch_bounds__(SELF_CHUNK) self_emit(const uint32_t* __restrict__ hm,
                                                        const int32_t* __restrict__ ptr,
                                                        const int32_t* __restrict__ park,
                                                        const int32_t* __restrict__ chunk_start,
                                                        const int64_t* __restrict__ offsets,
                                                        int64_t num_out, int64_t G, int64_t C,
                                                        int64_t pair_capacity,
                                                        int32_t* __restrict__ groups,
                                                        int32_t* __restrict__ in_maps,
                                                        int32_t* __restrict__ out_maps) {
  constexpr int WORDS = (K + 31) / 32, WAVES = SELF_CHUNK / 64;
  __shared__ unsigned long long s_hits[WAVES][K];
  __shared__ int s_incl[WAVES][K];      // pairs of the wave in offsets 0..k
  __shared__ int s_start[WAVES][K];     // pairs of offset k below the wave's first row
  __shared__ uint32_t s_hm[WAVES][64][WORDS];
  __shared__ int32_t s_ptr[WAVES][64];
  // as in kmap_emit_flat; the group starts are written whatever the room for pairs (the caller keeps them)
  if (offsets[K + 1] != 0) return;
  const bool room = offsets[K] <= pair_capacity;
  const int tid = threadIdx.x, lane = wcn_lane(), wave = tid >> 6;
  const int64_t m = (int64_t)blockIdx.x * SELF_CHUNK + tid;
  const int64_t group = m >> 6;
  uint32_t h[WORDS];
#pragma unroll
  for (int w = 0; w < WORDS; ++w) {
    h[w] = m < num_out ? hm[m * WORDS + w] : 0u;
    s_hm[wave][lane][w] = h[w];
  }
  s_ptr[wave][lane] = m < num_out ? ptr[m] : 0;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const unsigned long long b = __ballot((h[k >> 5] >> (k & 31)) & 1u);
    if (lane == 0) s_hits[wave][k] = b;
  }
  __syncthreads();
  // per offset: pairs of the waves before this one (thread k of the workgroup)
  for (int k = tid; k < K; k += SELF_CHUNK) {
    int run = chunk_start[(int64_t)k * (C + 1) + blockIdx.x];
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      s_start[w][k] = run;
      const int64_t g = (int64_t)blockIdx.x * WAVES + w;
      if (g < G) groups[(int64_t)k * (G + 1) + g] = run;
      run += __popcll(s_hits[w][k]);
    }
    if (blockIdx.x == gridDim.x - 1) groups[(int64_t)k * (G + 1) + G] = run;  // the offset's total
  }
  __syncthreads();
  if (group >= G || !room) return;
  // running counts over the offsets of this wave (lane j sums offsets j, j + 64)
  {
    int carry = 0;
#pragma unroll
    for (int k0 = 0; k0 < K; k0 += 64) {
      const int k = k0 + lane;
      const int n = k < K ? __popcll(s_hits[wave][k]) : 0;
      const int incl = wcn_wave_inclusive_sum(n);
      if (k < K) s_incl[wave][k] = carry + incl;
      carry += __shfl(incl, 63, 64);
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  const int total = s_incl[wave][K - 1];
  for (int q0 = 0; q0 < total; q0 += 64) {
    const int q = q0 + lane;
    if (q >= total) continue;
    // first offset whose running count exceeds q
    int lo = 0, hi = K - 1;
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (s_incl[wave][mid] <= q) lo = mid + 1; else hi = mid;
    }
    const int k = lo;
    const unsigned long long hk = s_hits[wave][k];
    const int rank = q - (s_incl[wave][k] - __popcll(hk));
    const int t = kmap_nth_set_bit(hk, rank);  // the lane (row) of this pair
    // the found row is the j-th parked row of row t, j = hits of that row in the offsets below k
    int j = 0;
#pragma unroll
    for (int w = 0; w < WORDS; ++w) {
      const uint32_t word = s_hm[wave][t][w];
      const int kw = k - 32 * w;
      j += kw >= 32 ? __popc(word) : (kw > 0 ? __popc(word & ((1u << kw) - 1u)) : 0);
    }
    const int64_t dst = offsets[k] + s_start[wave][k] + rank;
    in_maps[dst] = park[s_ptr[wave][t] + j];
    out_maps[dst] = (int32_t)(group * 64 + t);
  }
}

bool make_geom(const int32_t ks[3], const int32_t st[3], const int32_t* dil, const int32_t* centre,
               KmapGeom* g) {
  if (!ks || !st) return false;
  for (int d = 0; d < 3; ++d)
    if (ks[d] < 1 || st[d] < 1 || (dil && dil[d] < 1)) return false;
  const int64_t K = (int64_t)ks[0] * ks[1] * ks[2];
  if (K > WCN_MAX_OFFSETS) return false;
  g->kx = ks[0]; g->ky = ks[1]; g->kz = ks[2];
  g->sx = st[0]; g->sy = st[1]; g->sz = st[2];
  g->cx = centre ? centre[0] : ((ks[0] % 2) ? ks[0] / 2 : 0);
  g->cy = centre ? centre[1] : ((ks[1] % 2) ? ks[1] / 2 : 0);
  g->cz = centre ? centre[2] : ((ks[2] % 2) ? ks[2] / 2 : 0);
  g->dx = dil ? dil[0] : 1; g->dy = dil ? dil[1] : 1; g->dz = dil ? dil[2] : 1;
  g->K = (int32_t)K;
  return true;
}

// The compile-time-size probe kernels assume dilation 1 and the default centre.
inline bool plain_geom(const KmapGeom& g) {
  return g.dx == 1 && g.dy == 1 && g.dz == 1 && g.cx == ((g.kx % 2) ? g.kx / 2 : 0) &&
         g.cy == ((g.ky % 2) ? g.ky / 2 : 0) && g.cz == ((g.kz % 2) ? g.kz / 2 : 0);
}

inline bool is_fixed_size(const KmapGeom& g, int x, int y, int z) {
  return plain_geom(g) && g.kx == x && g.ky == y && g.kz == z;
}

inline bool table_args_ok(const void* table, int64_t n_keys, int64_t capacity) {
  return table && n_keys >= 0 && capacity >= 64 && (capacity & (capacity - 1)) == 0;
}

void launch_probe(const WcnTableView& v, const int32_t* out_coords, int64_t num_out,
                  const KmapGeom& g, const KmapWorkspace& w, hipStream_t s) {
  const dim3 grid(grid_for(num_out, 256)), block(256);
  const uint32_t cap_mask = (uint32_t)(v.capacity - 1);
  const KmapProbe o = {w.hits, w.found, w.ticket};
  if (is_fixed_size(g, 3, 3, 3)) {
    hipLaunchKernelGGL((kmap_pass_fixed<3, 3, 3>), grid, block, 0, s, v.hdr, v.slots, cap_mask,
                       v.perm, (const int4*)out_coords, num_out, g, w.groups, w.G, o);
  } else if (is_fixed_size(g, 2, 2, 2)) {
    hipLaunchKernelGGL((kmap_pass_fixed<2, 2, 2>), grid, block, 0, s, v.hdr, v.slots, cap_mask,
                       v.perm, (const int4*)out_coords, num_out, g, w.groups, w.G, o);
  } else if (is_fixed_size(g, 5, 5, 5)) {
    hipLaunchKernelGGL((kmap_pass_fixed<5, 5, 5>), grid, block, 0, s, v.hdr, v.slots, cap_mask,
                       v.perm, (const int4*)out_coords, num_out, g, w.groups, w.G, o);
  } else {
    hipLaunchKernelGGL(kmap_pass, grid, block, 0, s, v.hdr, v.slots, cap_mask, v.perm,
                       (const int4*)out_coords, num_out, g, w.groups, w.G, o);
  }
}

void launch_emit(int64_t num_out, const KmapGeom& g, const KmapWorkspace& w, int64_t pair_capacity,
                 int32_t* in_maps, int32_t* out_maps, hipStream_t s) {
  const dim3 grid(grid_for(num_out, 256)), block(256);
  const int64_t* offsets = (const int64_t*)w.result;
  hipLaunchKernelGGL(kmap_emit_flat, grid, block, 0, s, w.hits, w.found, w.groups, offsets, g.K,
                     w.G, pair_capacity, in_maps, out_maps);
}

// ---- strided output coordinates -----------------------------------------------------------------

constexpr int STRIDE_BATCH_MARKS = 1025;  // batch ids 0 .. 1024 whose first coarse row is looked up

struct StrideWorkspace {
  int64_t* result;   // [0] = M, [1] = table status bits, [4 + b] = first coarse row of batch id >= b
  int32_t* coarse;   // (n, 4) floor-divided coordinates
  int32_t* groups;   // (1, G+1) winners per 64-row group, then prefix sums
  void* table;       // block table over the coarse coordinates
  int64_t G;
};

inline size_t stride_layout(void* base, int64_t n, int64_t capacity, StrideWorkspace* w) {
  char* p = (char*)base;
  size_t off = 0;
  const int64_t G = (n + 63) / 64;
  if (w) w->result = (int64_t*)(p + off);
  off += wcn_align256(sizeof(int64_t) * (size_t)(4 + STRIDE_BATCH_MARKS));
  if (w) w->coarse = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * 4 * (size_t)n);
  if (w) w->groups = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * (size_t)(G + 1));
  if (w) w->table = (void*)(p + off);
  off += wcn_table_layout(nullptr, n, capacity, nullptr);
  if (w) w->G = G;
  return off;
}

__device__ __forceinline__ int32_t floor_div(int32_t a, int32_t b) {  // b > 0
  int32_t q = a / b;
  return (a % b != 0 && a < 0) ? q - 1 : q;
}

__global__ void __launch_bounds__(256) stride_divide(const int4* __restrict__ coords, int64_t n,
                                                     int32_t sx, int32_t sy, int32_t sz,
                                                     int4* __restrict__ coarse) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int4 c = coords[i];
  coarse[i] = make_int4(c.x, floor_div(c.y, sx), floor_div(c.z, sy), floor_div(c.w, sz));
}

// A row is the representative of its coordinate if perm at its rank holds its own index (perm
// keeps the minimum row index per distinct coordinate).
template <bool FILL>
__global__ void __launch_bounds__(256) stride_pick(const int4* __restrict__ coarse, int64_t n,
                                                   const WcnTableHeader* __restrict__ hdr,
                                                   const WcnSlot* __restrict__ slots,
                                                   const int32_t* __restrict__ slot_of,
                                                   const int32_t* __restrict__ perm,
                                                   int32_t* __restrict__ groups, int64_t G,
                                                   int4* __restrict__ out_coords,
                                                   int32_t* __restrict__ first_index) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t group = i >> 6;
  if (group >= G) return;
  const int lane = wcn_lane();
  bool winner = false;
  int4 c = make_int4(0, 0, 0, 0);
  if (i < n) {
    const int32_t h = slot_of[i];
    if (h >= 0) {
      const WcnLayout L = wcn_make_layout(hdr);
      c = coarse[i];
      uint32_t r[4];
      wcn_relative(L, c.x, c.y, c.z, c.w, r);
      const ulonglong2 km = *reinterpret_cast<const ulonglong2*>(&slots[h]);
      const int64_t pos = (int64_t)slots[h].base + wcn_rank_below(km.y, wcn_block_bit(r));
      winner = pos >= 0 && pos < n && perm[pos] == (int32_t)i;
    }
  }
  const unsigned long long wins = __ballot(winner);
  if (!FILL) {
    if (lane == 0) groups[group] = __popcll(wins);
  } else if (winner) {
    const int64_t pos = (int64_t)groups[group] + __popcll(wins & ((1ull << lane) - 1ull));
    out_coords[pos] = c;
    first_index[pos] = (int32_t)i;
  }
}

// The same selection through the table of the FINE coordinates, for strides of 1, 2 or 4 per
// dimension: such a coarse cell is a sub-box of one 4x4x4 block (the blocks' origins are multiples
// of 4), so its voxels are bits of one slot's mask, their rows stand next to each other in perm, and
// the cell's representative is the lowest of them.  No table over the coarse rows is needed: one
// slot look-up and at most sx * sy * sz loads of perm per row.  LOG: log2 of the strides.
template <bool FILL>
__global__ void __launch_bounds__(256) stride_pick_cells(const int4* __restrict__ coords, int64_t n,
                                                         const WcnTableHeader* __restrict__ hdr,
                                                         const WcnSlot* __restrict__ slots,
                                                         uint32_t cap_mask,
                                                         const int32_t* __restrict__ perm,
                                                         int lx, int ly, int lz,
                                                         int32_t* __restrict__ groups, int64_t G,
                                                         unsigned long long* __restrict__ picked,
                                                         int4* __restrict__ out_coords,
                                                         int32_t* __restrict__ first_index) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t group = i >> 6;
  if (group >= G) return;
  const int lane = wcn_lane();
  if (FILL) {
    // the counting pass left the group's representatives as a mask: no second look-up
    const unsigned long long wins = picked[group];
    if ((wins >> lane) & 1ull) {
      const int4 c = coords[i];
      const int64_t pos = (int64_t)groups[group] + __popcll(wins & ((1ull << lane) - 1ull));
      out_coords[pos] = make_int4(c.x, floor_div(c.y, 1 << lx), floor_div(c.z, 1 << ly), floor_div(c.w, 1 << lz));
      first_index[pos] = (int32_t)i;
    }
    return;
  }
  bool winner = false;
  int4 c = make_int4(0, 0, 0, 0);
  if (i < n) {
    const WcnLayout L = wcn_make_layout(hdr);
    c = coords[i];
    uint32_t r[4];
    if (L.ok && wcn_relative(L, c.x, c.y, c.z, c.w, r)) {
      int32_t base = 0;
      const unsigned long long mask = wcn_lookup_block(slots, cap_mask, wcn_block_key(L, r), &base);
      // the bits of the block that lie in this row's coarse cell
      const uint32_t x0 = (r[1] & 3u) >> lx << lx, y0 = (r[2] & 3u) >> ly << ly, z0 = (r[3] & 3u) >> lz << lz;
      const unsigned long long zs = ((1ull << (1 << lz)) - 1ull) << z0;          // within a row of 4 bits
      unsigned long long ys = 0ull, cell = 0ull;
      for (int dy = 0; dy < (1 << ly); ++dy) ys |= zs << ((y0 + dy) * 4);       // within a plane of 16 bits
      for (int dx = 0; dx < (1 << lx); ++dx) cell |= ys << ((x0 + dx) * 16);
      unsigned long long siblings = mask & cell;
      int32_t lowest = INT32_MAX;
      while (siblings) {
        const int b = __builtin_ctzll(siblings);
        siblings &= siblings - 1ull;
        const int64_t pos = (int64_t)base + wcn_rank_below(mask, (uint32_t)b);
        if (pos >= 0 && pos < n) lowest = min(lowest, perm[pos]);
      }
      winner = lowest == (int32_t)i;
    }
  }
  const unsigned long long wins = __ballot(winner);
  if (lane == 0) {
    groups[group] = __popcll(wins);
    picked[group] = wins;
  }
}

__global__ void stride_finish(int64_t* __restrict__ result, const int32_t* __restrict__ groups,
                              int64_t G, const WcnTableHeader* __restrict__ hdr) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  result[0] = groups[G];
  result[1] = hdr->status;
}

// Where the coarse rows of each batch item begin, for rows whose batch column does not descend
// (the rows of a batch-sorted input): thread b finds the first of the M rows whose batch id is at
// least b.  For other inputs the numbers mean nothing and nobody reads them.
__global__ void __launch_bounds__(1024) stride_batch_bounds(const int4* __restrict__ out_coords,
                                                            int64_t* __restrict__ result) {
  const int64_t m = result[0];
  for (int b = threadIdx.x; b < STRIDE_BATCH_MARKS; b += 1024) {
    int64_t lo = 0, hi = m;
    while (lo < hi) {
      const int64_t mid = (lo + hi) >> 1;
      if (out_coords[mid].x < b) lo = mid + 1; else hi = mid;
    }
    result[4 + b] = lo;
  }
}

}  // namespace

// Row-wise exclusive scan, shared with the contraction's map conversion.
void wcn_scan_rows_launch(int32_t* groups, int64_t G, int rows, int64_t* row_total, hipStream_t s) {
  const KmapFinish none = {nullptr, nullptr, nullptr, 0, nullptr, 0};
  hipLaunchKernelGGL(kmap_scan_rows, dim3(rows), dim3(1024), 0, s, groups, G, row_total, none);
}

// what the last wcn_kmap_read_result of this host thread learned about the table (bit 0: some
// key was inserted more than once)
static thread_local int32_t g_last_table_flags = 0;
// the mailbox write the last count call of this thread armed, and the result block it mirrors
static thread_local int64_t g_pending_sequence = 0;
static thread_local const void* g_pending_result = nullptr;

extern "C" {

size_t wcn_kmap_workspace_bytes(int64_t num_out, int32_t num_offsets) {
  if (num_out < 0 || num_offsets < 1 || num_offsets > WCN_MAX_OFFSETS) return 0;
  const size_t a = kmap_layout(nullptr, num_out, num_offsets, nullptr);
  const size_t b = self_layout(nullptr, num_out, num_offsets, nullptr);
  return a > b ? a : b;
}

static int kmap_count_impl(const void* table, int64_t n_keys, int64_t capacity, const int32_t* out_coords,
                           int64_t num_out, const int32_t host_kernel_size[3],
                           const int32_t host_stride[3], const int32_t* host_dilation,
                           const int32_t* host_centre, void* workspace, void* stream) {
  KmapGeom g;
  if (!make_geom(host_kernel_size, host_stride, host_dilation, host_centre, &g)) return WCN_ERR_INVALID_ARGUMENT;
  if (!table_args_ok(table, n_keys, capacity) || !workspace || num_out < 0 ||
      num_out >= (1ll << 31) || (num_out > 0 && !out_coords))
    return WCN_ERR_INVALID_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  WcnTableView v;
  wcn_table_layout(const_cast<void*>(table), n_keys, capacity, &v);
  KmapWorkspace w;
  kmap_layout(workspace, num_out, g.K, &w);
  if (w.G > 0) {
    launch_probe(v, out_coords, num_out, g, w, s);
  } else {
    hipLaunchKernelGGL(kmap_zero_ticket, dim3(1), dim3(1), 0, s, w.ticket);
  }
  // The scan's finishing wave writes the result into device memory (the emit pass reads it there)
  // and into this thread's pinned mailbox, where wcn_kmap_read_result picks it up without a copy
  // command on the stream, ahead of anything the caller enqueues next (an emit pass into buffers of
  // assumed size, say).
  int64_t* box = nullptr;
  int64_t sequence = 0;
  if (wcn_mailbox_begin(&box, &sequence) != WCN_OK) {  // no mailbox: a copy command instead
    box = nullptr;
    sequence = 0;
  }
  g_pending_sequence = sequence;
  g_pending_result = w.result;
  const KmapFinish fin = {w.result, w.ticket, v.hdr, g.K, box, sequence};
  hipLaunchKernelGGL(kmap_scan_rows, dim3(g.K + 1), dim3(1024), 0, s, w.groups, w.G, w.row_total, fin);
  WCN_LAUNCH_CHECK();
  if (box) {
    if (wcn_mailbox_mark(s) != WCN_OK) return WCN_ERR_LAUNCH;
  } else if (wcn_read_early_begin(w.result, sizeof(int64_t) * (size_t)(g.K + 3), s) != WCN_OK) {
    return WCN_ERR_LAUNCH;
  }
  return WCN_OK;
}

int wcn_kmap_count(const void* table, int64_t n_keys, int64_t capacity, const int32_t* out_coords,
                   int64_t num_out, const int32_t host_kernel_size[3],
                   const int32_t host_stride[3], void* workspace, void* stream) {
  return kmap_count_impl(table, n_keys, capacity, out_coords, num_out, host_kernel_size, host_stride,
                         nullptr, nullptr, workspace, stream);
}

int wcn_kmap_count_dilated(const void* table, int64_t n_keys, int64_t capacity, const int32_t* out_coords,
                           int64_t num_out, const int32_t host_kernel_size[3],
                           const int32_t host_stride[3], const int32_t host_dilation[3],
                           const int32_t host_centre[3], void* workspace, void* stream) {
  if (!host_dilation || !host_centre) return WCN_ERR_INVALID_ARGUMENT;
  return kmap_count_impl(table, n_keys, capacity, out_coords, num_out, host_kernel_size, host_stride,
                         host_dilation, host_centre, workspace, stream);
}

static bool self_size(const int32_t ks[3], int32_t* K) {
  if (!ks) return false;
  if (ks[0] == 3 && ks[1] == 3 && ks[2] == 3) { *K = 27; return true; }
  if (ks[0] == 5 && ks[1] == 5 && ks[2] == 5) { *K = 125; return true; }
  return false;
}

int wcn_kmap_self_supported(const int32_t host_kernel_size[3], int64_t n_keys) {
  int32_t K = 0;
  return self_size(host_kernel_size, &K) && n_keys > 0 && n_keys * (int64_t)K < (1ll << 31);
}

int wcn_kmap_count_self(const void* table, int64_t n_keys, int64_t capacity,
                        const int32_t host_kernel_size[3], void* workspace, void* stream) {
  int32_t K = 0;
  if (!self_size(host_kernel_size, &K) || !table_args_ok(table, n_keys, capacity) || !workspace ||
      n_keys <= 0 || n_keys * (int64_t)K >= (1ll << 31))
    return WCN_ERR_INVALID_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  WcnTableView v;
  wcn_table_layout(const_cast<void*>(table), n_keys, capacity, &v);
  SelfWorkspace w;
  self_layout(workspace, n_keys, K, &w);
  const uint32_t cap_mask = (uint32_t)(capacity - 1);
  // a bin of the usual size has about ten tiles; bins with more are walked in turns
  const dim3 pgrid((unsigned)v.bins, 8), cgrid((unsigned)w.C);
  if (K == 27) {
    hipLaunchKernelGGL(self_probe<1>, pgrid, dim3(256), 0, s, v.hdr, v.slots, cap_mask, v.perm, v.bin_start,
                       v.bin_stats, v.block_list, v.order_tag, v.order_row, w.hm, w.ptr, w.park, w.ticket);
    hipLaunchKernelGGL(self_count<27>, cgrid, dim3(SELF_CHUNK), 0, s, w.hm, n_keys, w.chunk, w.C);
  } else {
    hipLaunchKernelGGL(self_probe<2>, pgrid, dim3(256), 0, s, v.hdr, v.slots, cap_mask, v.perm, v.bin_start,
                       v.bin_stats, v.block_list, v.order_tag, v.order_row, w.hm, w.ptr, w.park, w.ticket);
    hipLaunchKernelGGL(self_count<125>, cgrid, dim3(SELF_CHUNK), 0, s, w.hm, n_keys, w.chunk, w.C);
  }
  int64_t* box = nullptr;
  int64_t sequence = 0;
  if (wcn_mailbox_begin(&box, &sequence) != WCN_OK) {  // no mailbox: a copy command instead
    box = nullptr;
    sequence = 0;
  }
  g_pending_sequence = sequence;
  g_pending_result = w.result;
  const KmapFinish fin = {w.result, w.ticket, v.hdr, K, box, sequence};
  hipLaunchKernelGGL(kmap_scan_rows, dim3(K), dim3(1024), 0, s, w.chunk, w.C, w.row_total, fin);
  WCN_LAUNCH_CHECK();
  if (box) {
    if (wcn_mailbox_mark(s) != WCN_OK) return WCN_ERR_LAUNCH;
  } else if (wcn_read_early_begin(w.result, sizeof(int64_t) * (size_t)(K + 3), s) != WCN_OK) {
    return WCN_ERR_LAUNCH;
  }
  return WCN_OK;
}

int wcn_kmap_fill_self(int64_t n_keys, const int32_t host_kernel_size[3], const void* workspace,
                       int64_t pair_capacity, int32_t* in_maps, int32_t* out_maps, void* stream) {
  int32_t K = 0;
  if (!self_size(host_kernel_size, &K) || !workspace || n_keys <= 0 || pair_capacity < 0 ||
      n_keys * (int64_t)K >= (1ll << 31) || !in_maps || !out_maps)
    return WCN_ERR_INVALID_ARGUMENT;
  SelfWorkspace w;
  self_layout(const_cast<void*>(workspace), n_keys, K, &w);
  const int64_t* offsets = (const int64_t*)w.result;
  const dim3 grid((unsigned)w.C), block(SELF_CHUNK);
  if (K == 27) {
    hipLaunchKernelGGL(self_emit<27>, grid, block, 0, (hipStream_t)stream, w.hm, w.ptr, w.park, w.chunk,
                       offsets, n_keys, w.G, w.C, pair_capacity, w.groups, in_maps, out_maps);
  } else {
    hipLaunchKernelGGL(self_emit<125>, grid, block, 0, (hipStream_t)stream, w.hm, w.ptr, w.park, w.chunk,
                       offsets, n_keys, w.G, w.C, pair_capacity, w.groups, in_maps, out_maps);
  }
  WCN_LAUNCH_CHECK();
  return WCN_OK;
}

int32_t wcn_kmap_last_table_flags(void) { return g_last_table_flags; }

int wcn_kmap_read_result(const void* workspace, int64_t num_out, int32_t num_offsets,
                         int64_t* host_offsets, void* stream) {
  if (!workspace || !host_offsets || num_offsets < 1 || num_offsets > WCN_MAX_OFFSETS)
    return WCN_ERR_INVALID_ARGUMENT;
  KmapWorkspace w;
  kmap_layout(const_cast<void*>(workspace), num_out, num_offsets, &w);
  int64_t tmp[WCN_MAX_OFFSETS + 3];
  const size_t bytes = sizeof(int64_t) * (size_t)(num_offsets + 3);
  // from the mailbox the count call armed; otherwise (another thread, a count call that failed
  // half-way) from the device copy
  const int64_t sequence = g_pending_result == (const void*)w.result ? g_pending_sequence : 0;
  if (sequence != 0) g_pending_sequence = 0;
  if (sequence == 0 || wcn_mailbox_end(tmp, bytes, sequence) != WCN_OK) {
    if (wcn_read_early_end(tmp, w.result, bytes, (hipStream_t)stream) != WCN_OK) return WCN_ERR_LAUNCH;
  }
  for (int k = 0; k <= num_offsets; ++k) host_offsets[k] = tmp[k];
  g_last_table_flags = (int32_t)((tmp[num_offsets + 2] >> 32) & 1);
  const int st = wcn_table_status_from_bits((int32_t)tmp[num_offsets + 1]);
  if (st != WCN_OK) return st;
  if (tmp[num_offsets] > INT32_MAX) return WCN_ERR_TOO_MANY_PAIRS;
  return WCN_OK;
}

int wcn_kmap_fill(const void* table, int64_t n_keys, int64_t capacity, const int32_t* out_coords,
                  int64_t num_out, const int32_t host_kernel_size[3], const int32_t host_stride[3],
                  const void* workspace, int64_t pair_capacity, int32_t* in_maps, int32_t* out_maps,
                  void* stream) {
  KmapGeom g;
  if (!make_geom(host_kernel_size, host_stride, nullptr, nullptr, &g)) return WCN_ERR_INVALID_ARGUMENT;
  if (!table_args_ok(table, n_keys, capacity) || !workspace || num_out < 0 ||
      num_out >= (1ll << 31) || (num_out > 0 && !out_coords) || pair_capacity < 0)
    return WCN_ERR_INVALID_ARGUMENT;
  if (num_out == 0 || pair_capacity == 0) return WCN_OK;
  if (!in_maps || !out_maps) return WCN_ERR_INVALID_ARGUMENT;
  WcnTableView v;
  wcn_table_layout(const_cast<void*>(table), n_keys, capacity, &v);
  KmapWorkspace w;
  kmap_layout(const_cast<void*>(workspace), num_out, g.K, &w);
  launch_emit(num_out, g, w, pair_capacity, in_maps, out_maps, (hipStream_t)stream);
  WCN_LAUNCH_CHECK();
  return WCN_OK;
}

const int32_t* wcn_kmap_group_start(const void* workspace, int64_t num_out, int32_t num_offsets) {
  if (!workspace || num_offsets < 1 || num_offsets > WCN_MAX_OFFSETS) return nullptr;
  KmapWorkspace w;
  kmap_layout(const_cast<void*>(workspace), num_out, num_offsets, &w);
  return w.groups;
}

size_t wcn_stride_unique_workspace_bytes(int64_t n, int64_t capacity) {
  if (n < 0 || capacity < 64) return 0;
  return stride_layout(nullptr, n, capacity, nullptr);
}

int wcn_stride_unique(const int32_t* coords, int64_t n, const int32_t host_stride[3],
                      void* workspace, int64_t capacity, int32_t* out_coords,
                      int32_t* first_index, void* stream) {
  if (!workspace || n < 0 || n >= (1ll << 31) || !host_stride) return WCN_ERR_INVALID_ARGUMENT;
  if (capacity < 64 || (capacity & (capacity - 1)) != 0) return WCN_ERR_INVALID_ARGUMENT;
  if (n > 0 && (!coords || !out_coords || !first_index)) return WCN_ERR_INVALID_ARGUMENT;
  for (int d = 0; d < 3; ++d)
    if (host_stride[d] < 1) return WCN_ERR_INVALID_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  StrideWorkspace w;
  stride_layout(workspace, n, capacity, &w);
  WcnTableView v;
  wcn_table_layout(w.table, n, capacity, &v);
  if (n > 0) {
    hipLaunchKernelGGL(stride_divide, dim3(grid_for(n, 256)), dim3(256), 0, s, (const int4*)coords,
                       n, host_stride[0], host_stride[1], host_stride[2], (int4*)w.coarse);
  }
  const int rc = wcn_table_build_impl(w.coarse, n, v, true, s);
  if (rc != WCN_OK) return rc;
  if (n > 0) {
    hipLaunchKernelGGL(stride_pick<false>, dim3(grid_for(n, 256)), dim3(256), 0, s,
                       (const int4*)w.coarse, n, v.hdr, v.slots, v.slot_of, v.perm, w.groups, w.G,
                       (int4*)nullptr, (int32_t*)nullptr);
  }
  {
    const KmapFinish none = {nullptr, nullptr, nullptr, 0, nullptr, 0};
    hipLaunchKernelGGL(kmap_scan_rows, dim3(1), dim3(1024), 0, s, w.groups, w.G, w.result + 2, none);
  }
  hipLaunchKernelGGL(stride_finish, dim3(1), dim3(64), 0, s, w.result, w.groups, w.G, v.hdr);
  if (n > 0) {
    hipLaunchKernelGGL(stride_pick<true>, dim3(grid_for(n, 256)), dim3(256), 0, s,
                       (const int4*)w.coarse, n, v.hdr, v.slots, v.slot_of, v.perm, w.groups, w.G,
                       (int4*)out_coords, first_index);
    hipLaunchKernelGGL(stride_batch_bounds, dim3(1), dim3(1024), 0, s, (const int4*)out_coords, w.result);
  }
  WCN_LAUNCH_CHECK();
  return WCN_OK;
}

size_t wcn_stride_unique_cells_workspace_bytes(int64_t n) {
  if (n < 0) return 0;
  return wcn_align256(sizeof(int64_t) * (size_t)(4 + STRIDE_BATCH_MARKS)) +
         wcn_align256(sizeof(int32_t) * (size_t)((n + 63) / 64 + 1)) +
         wcn_align256(sizeof(unsigned long long) * (size_t)((n + 63) / 64));
}

int wcn_stride_unique_cells(const void* table, int64_t n_keys, int64_t capacity, const int32_t* coords,
                            const int32_t host_stride[3], void* workspace, int32_t* out_coords,
                            int32_t* first_index, void* stream) {
  if (!table_args_ok(table, n_keys, capacity) || !workspace || !host_stride || n_keys >= (1ll << 31))
    return WCN_ERR_INVALID_ARGUMENT;
  if (n_keys > 0 && (!coords || !out_coords || !first_index)) return WCN_ERR_INVALID_ARGUMENT;
  int lg[3];
  for (int d = 0; d < 3; ++d) {
    if (host_stride[d] != 1 && host_stride[d] != 2 && host_stride[d] != 4) return WCN_ERR_INVALID_ARGUMENT;
    lg[d] = host_stride[d] == 1 ? 0 : (host_stride[d] == 2 ? 1 : 2);
  }
  hipStream_t s = (hipStream_t)stream;
  const int64_t n = n_keys;
  WcnTableView v;
  wcn_table_layout(const_cast<void*>(table), n_keys, capacity, &v);
  // the result block first, as in the workspace of wcn_stride_unique (the read calls find it there)
  int64_t* result = (int64_t*)workspace;
  int32_t* groups = (int32_t*)((char*)workspace + wcn_align256(sizeof(int64_t) * (size_t)(4 + STRIDE_BATCH_MARKS)));
  const int64_t G = (n + 63) / 64;
  unsigned long long* picked = (unsigned long long*)((char*)groups + wcn_align256(sizeof(int32_t) * (size_t)(G + 1)));
  const uint32_t cap_mask = (uint32_t)(capacity - 1);
  if (n > 0) {
    hipLaunchKernelGGL(stride_pick_cells<false>, dim3(grid_for(n, 256)), dim3(256), 0, s, (const int4*)coords,
                       n, v.hdr, v.slots, cap_mask, v.perm, lg[0], lg[1], lg[2], groups, G, picked,
                       (int4*)nullptr, (int32_t*)nullptr);
  }
  {
    const KmapFinish none = {nullptr, nullptr, nullptr, 0, nullptr, 0};
    hipLaunchKernelGGL(kmap_scan_rows, dim3(1), dim3(1024), 0, s, groups, G, result + 2, none);
  }
  hipLaunchKernelGGL(stride_finish, dim3(1), dim3(64), 0, s, result, groups, G, v.hdr);
  if (n > 0) {
    hipLaunchKernelGGL(stride_pick_cells<true>, dim3(grid_for(n, 256)), dim3(256), 0, s, (const int4*)coords,
                       n, v.hdr, v.slots, cap_mask, v.perm, lg[0], lg[1], lg[2], groups, G, picked,
                       (int4*)out_coords, first_index);
    hipLaunchKernelGGL(stride_batch_bounds, dim3(1), dim3(1024), 0, s, (const int4*)out_coords, result);
  }
  WCN_LAUNCH_CHECK();
  return WCN_OK;
}

int wcn_stride_unique_read_bounds(const void* workspace, int64_t n, int64_t capacity,
                                  int64_t* host_count, int64_t* host_bounds, void* stream) {
  if (!workspace || !host_count || !host_bounds) return WCN_ERR_INVALID_ARGUMENT;
  StrideWorkspace w;
  stride_layout(const_cast<void*>(workspace), n, capacity, &w);
  int64_t tmp[4 + STRIDE_BATCH_MARKS];
  if (wcn_read_small(tmp, w.result, sizeof(tmp), (hipStream_t)stream) != WCN_OK) return WCN_ERR_LAUNCH;
  *host_count = tmp[0];
  for (int b = 0; b < STRIDE_BATCH_MARKS; ++b) host_bounds[b] = n > 0 ? tmp[4 + b] : 0;
  return wcn_table_status_from_bits((int32_t)tmp[1]);
}

int wcn_stride_unique_read_count(const void* workspace, int64_t n, int64_t capacity,
                                 int64_t* host_count, void* stream) {
  if (!workspace || !host_count) return WCN_ERR_INVALID_ARGUMENT;
  StrideWorkspace w;
  stride_layout(const_cast<void*>(workspace), n, capacity, &w);
  int64_t tmp[2];
  if (wcn_read_small(tmp, w.result, sizeof(tmp), (hipStream_t)stream) != WCN_OK) return WCN_ERR_LAUNCH;
  *host_count = tmp[0];
  return wcn_table_status_from_bits((int32_t)tmp[1]);
}

}  // extern "C"
