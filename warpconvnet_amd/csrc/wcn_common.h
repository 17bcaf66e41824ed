// Shared host/device definitions of libwcn_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/wcn_hip.h"

#define WCN_WAVE 64
#define WCN_MAX_PROBE 128  // linear-probe bound of the block table (insert and lookup)
#define WCN_EMPTY_KEY 0xFFFFFFFFFFFFFFFFull
#define WCN_MAX_OFFSETS 1024  // kernel volume bound of the kernel-map kernels

// Device-recorded conditions (TableHeader::status, a bit set).
#define WCN_DEV_OVERFLOW 1
#define WCN_DEV_RANGE 2

// ---- coordinate table -------------------------------------------------------------------------
// The table does not store one slot per voxel.  Space is cut into 4x4x4-voxel blocks; a slot
// holds the packed block coordinate, a 64-bit occupancy mask of the block and the rank of its
// first voxel in `perm`, the list of input rows grouped by block.  A voxel's row index is
// perm[base + popcount(mask below its bit)].  One 32-byte slot answers up to 64 probes.
struct __attribute__((aligned(32))) WcnSlot {
  unsigned long long key;   // packed (batch, bx, by, bz) relative to the bounding box, or EMPTY
  unsigned long long mask;  // bit (x&3)*16 + (y&3)*4 + (z&3)
  int32_t base;             // first position of the block's voxels in perm
  int32_t pad[3];
};

struct WcnTableHeader {  // first 256 bytes of a table workspace
  int32_t mn[4];         // bounding box of the keys, per column
  int32_t mx[4];
  int32_t num_blocks;    // occupied slots (valid after table_sum_stats)
  int32_t status;        // WCN_DEV_* bits
  int32_t total;         // number of distinct keys (valid after table_sum_stats)
  int32_t num_keys;      // keys inserted; more keys than set bits (`total`) means some key came twice
  int32_t bins;          // bins of the build
  int32_t pad;
  int64_t stats_offset;  // bytes from the header to the bins' (voxels, blocks) counts
  int32_t reserved[48];
};
static_assert(sizeof(WcnTableHeader) == 256, "header is 256 bytes");

// Valid once the bins' counts have been summed into the header: every distinct key set one bit.
#define WCN_HAS_DUPLICATES(hdr) ((hdr)->total != (hdr)->num_keys)

struct WcnTableView {  // host-computed addresses inside a table workspace
  WcnTableHeader* hdr;
  WcnSlot* slots;
  int32_t* perm;        // n_keys
  int32_t* slot_of;     // n_keys (slot of each key; written on request)
  // The keys in block order: every key once, the keys of one block next to each other, the blocks
  // of one bin next to each other (bin b owns entries bin_start[b] .. bin_start[b + 1]).
  int32_t* order_tag;     // n_keys: (index of the entry's block in its bin's block list) << 6 | voxel bit
  int32_t* order_row;     // n_keys: input row of each entry
  // The blocks of bin b, in the order of its entries: block_list[bin_start[b] + j], j < blocks of
  // the bin.  key, mask and base as in the table's slot; pad[0] = first entry of the block,
  // counted from bin_start[b].
  WcnSlot* block_list;    // n_keys places (a bin has at most as many blocks as keys)
  // build scratch
  int32_t* bin_coords;    // (n_keys, 4) keys grouped by bin
  int32_t* bin_row;       // n_keys
  int32_t* hist;          // (bins, parts) keys of part w in bin b, then their exclusive prefix sums
  int32_t* bin_total;     // bins: keys per bin
  int32_t* bin_start;     // bins + 1
  int32_t* bin_stats;     // (bins, 2): distinct keys and blocks of each bin
  int32_t* part_box;      // (parts, 8) bounding box of each part's keys
  int64_t n_keys;
  int64_t capacity;
  int32_t bins;           // power of two
  int32_t parts;          // workgroups of the histogram and scatter passes
};

static inline size_t wcn_align256(size_t x) { return (x + 255) & ~(size_t)255; }

// Keys are first grouped into bins of one to two thousand (a bin is a hash of the key's 16x16x16-voxel
// cell, so the 4x4x4 blocks of a cell stay together); the bin count follows the slot count, so a
// rebuild with more slots also re-deals the bins.
#define WCN_BIN_SLOTS 2048      // distinct blocks a bin can hold (its table in LDS)
#define WCN_PART_KEYS 4096      // keys per workgroup of the histogram and scatter passes
#define WCN_MAX_BINS 32768      // a counter per bin in LDS during the build: 128 KB
static inline int32_t wcn_table_bins(int64_t capacity) {
  int64_t b = capacity / 2048;
  if (b < 16) b = 16;
  if (b > WCN_MAX_BINS) b = WCN_MAX_BINS;
  return (int32_t)b;
}
static inline int32_t wcn_table_parts(int64_t n_keys) {
  int64_t w = (n_keys + WCN_PART_KEYS - 1) / WCN_PART_KEYS;
  if (w < 1) w = 1;
  if (w > 256) w = 256;
  return (int32_t)w;
}

static inline size_t wcn_table_layout(void* base, int64_t n_keys, int64_t capacity,
                                      WcnTableView* v) {
  char* p = (char*)base;
  size_t off = 0;
  const int32_t bins = wcn_table_bins(capacity), parts = wcn_table_parts(n_keys);
  if (v) v->hdr = (WcnTableHeader*)(p + off);
  off += 256;
  if (v) v->slots = (WcnSlot*)(p + off);
  off += wcn_align256(sizeof(WcnSlot) * (size_t)capacity);
  if (v) v->perm = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * (size_t)n_keys);
  if (v) v->slot_of = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * (size_t)n_keys);
  if (v) v->order_tag = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * (size_t)n_keys);
  if (v) v->order_row = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * (size_t)n_keys);
  if (v) v->block_list = (WcnSlot*)(p + off);
  off += wcn_align256(sizeof(WcnSlot) * (size_t)n_keys);
  if (v) v->bin_coords = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * 4 * (size_t)n_keys);
  if (v) v->bin_row = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * (size_t)n_keys);
  if (v) v->hist = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * (size_t)bins * (size_t)parts);
  if (v) v->bin_total = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * (size_t)bins);
  if (v) v->bin_start = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * (size_t)(bins + 1));
  if (v) v->bin_stats = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * 2 * (size_t)bins);
  if (v) v->part_box = (int32_t*)(p + off);
  off += wcn_align256(sizeof(int32_t) * 8 * (size_t)parts);
  if (v) {
    v->n_keys = n_keys;
    v->capacity = capacity;
    v->bins = bins;
    v->parts = parts;
  }
  return off;
}

#ifdef __HIPCC__

// Bit layout of the packed block key, derived from the bounding box in the header.
struct WcnLayout {
  uint32_t amin[4];   // batch minimum; spatial minima rounded down to a multiple of 4
  uint32_t span[4];   // largest valid (coord - amin) per column
  uint32_t shift[4];  // left shift of each field in the key
  bool ok;            // all fields fit in 63 bits
};

__device__ __forceinline__ WcnLayout wcn_make_layout(const WcnTableHeader* __restrict__ h) {
  WcnLayout L;
  uint32_t bits[4];
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    int32_t mn = h->mn[d], mx = h->mx[d];
    uint32_t a = d == 0 ? (uint32_t)mn : ((uint32_t)mn & ~3u);
    L.amin[d] = a;
    L.span[d] = (uint32_t)mx - a;
    uint32_t cells = d == 0 ? L.span[d] : (L.span[d] >> 2);  // largest field value
    bits[d] = cells == 0 ? 0u : 32u - (uint32_t)__builtin_clz(cells);
  }
  L.shift[3] = 0;
  L.shift[2] = bits[3];
  L.shift[1] = bits[3] + bits[2];
  L.shift[0] = bits[3] + bits[2] + bits[1];
  L.ok = (bits[0] + bits[1] + bits[2] + bits[3]) <= 63u;
  return L;
}

// Relative coordinates of (b,x,y,z); false if the point lies outside the bounding box.
__device__ __forceinline__ bool wcn_relative(const WcnLayout& L, int b, int x, int y, int z,
                                             uint32_t r[4]) {
  r[0] = (uint32_t)b - L.amin[0];
  r[1] = (uint32_t)x - L.amin[1];
  r[2] = (uint32_t)y - L.amin[2];
  r[3] = (uint32_t)z - L.amin[3];
  return r[0] <= L.span[0] && r[1] <= L.span[1] && r[2] <= L.span[2] && r[3] <= L.span[3];
}

__device__ __forceinline__ unsigned long long wcn_block_key(const WcnLayout& L,
                                                            const uint32_t r[4]) {
  return ((unsigned long long)r[0] << L.shift[0]) | ((unsigned long long)(r[1] >> 2) << L.shift[1]) |
         ((unsigned long long)(r[2] >> 2) << L.shift[2]) | (unsigned long long)(r[3] >> 2);
}

__device__ __forceinline__ uint32_t wcn_block_bit(const uint32_t r[4]) {
  return ((r[1] & 3u) << 4) | ((r[2] & 3u) << 2) | (r[3] & 3u);
}

// Slot of a block key: the key's two halves folded into one word, then the 32-bit finaliser of
// MurmurHash3 (neighbouring block keys spread over the table; a third of the instructions of a
// 64-bit mix, and every probe of the kernel-map passes pays for it).
__device__ __forceinline__ uint32_t wcn_mix(unsigned long long k, uint32_t cap_mask) {
  uint32_t h = (uint32_t)k ^ ((uint32_t)(k >> 32) * 0x9E3779B1u);
  h ^= h >> 16;
  h *= 0x85ebca6bu;
  h ^= h >> 13;
  h *= 0xc2b2ae35u;
  h ^= h >> 16;
  return h & cap_mask;
}

// Finds the slot of a block key.  Returns its mask (0 if the block is absent) and base.  Both
// 16-byte halves of the 32-byte slot are requested together, so a hit costs one memory round trip.
__device__ __forceinline__ unsigned long long wcn_lookup_block_from(
    const WcnSlot* __restrict__ slots, uint32_t cap_mask, unsigned long long key, uint32_t h,
    int first_probe, int32_t* base) {
  for (int p = first_probe; p < WCN_MAX_PROBE; ++p) {
    const uint4* raw = reinterpret_cast<const uint4*>(&slots[h]);
    const uint4 lo = raw[0];
    const uint4 hi = raw[1];
    const unsigned long long k = ((unsigned long long)lo.y << 32) | lo.x;
    if (k == key) {
      *base = (int32_t)hi.x;
      return ((unsigned long long)lo.w << 32) | lo.z;
    }
    if (k == WCN_EMPTY_KEY) break;
    h = (h + 1) & cap_mask;
  }
  *base = 0;
  return 0ull;
}

__device__ __forceinline__ unsigned long long wcn_lookup_block(const WcnSlot* __restrict__ slots,
                                                               uint32_t cap_mask,
                                                               unsigned long long key,
                                                               int32_t* base) {
  return wcn_lookup_block_from(slots, cap_mask, key, wcn_mix(key, cap_mask), 0, base);
}

__device__ __forceinline__ int wcn_rank_below(unsigned long long mask, uint32_t bit) {
  return __popcll(mask & ((1ull << bit) - 1ull));
}

__device__ __forceinline__ int wcn_lane() { return (int)(threadIdx.x & 63); }

// Inclusive prefix sum over the 64 lanes of a wave.
__device__ __forceinline__ int wcn_wave_inclusive_sum(int v) {
  const int lane = wcn_lane();
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    int t = __shfl_up(v, d, 64);
    if (lane >= d) v += t;
  }
  return v;
}

#endif  // __HIPCC__

// Small device-to-host reads (map offsets, table status, row counts): copied into pinned memory
// and awaited by polling an event, which returns within a few microseconds of the copy's end (a
// blocking stream synchronisation wakes the host tens of microseconds later).  One staging buffer
// and one event per host thread, created on first use and kept until the process ends.
int wcn_read_small(void* host_dst, const void* device_src, size_t bytes, hipStream_t stream);
// The same read split in two: begin enqueues the copy (before whatever is enqueued next), end waits
// for it; an end without a matching begin on this thread does the whole read.
int wcn_read_early_begin(const void* device_src, size_t bytes, hipStream_t stream);
int wcn_read_early_end(void* host_dst, const void* device_src, size_t bytes, hipStream_t stream);

// A result the device writes straight into pinned host memory (no copy command): `begin` hands out
// this thread's mailbox (device-visible address of up to 16 KiB - 8 bytes of payload behind an
// 8-byte sequence word) and a fresh sequence number; the kernel writes the payload, a system-scope
// fence, then the sequence number into word 0.  `end` polls word 0 (and `done`, an event recorded
// after the kernel, so that a kernel that never wrote cannot stall the host: it then returns
// WCN_ERR_LAUNCH and the caller reads the device copy instead) and copies the payload out.
int wcn_mailbox_begin(int64_t** device_visible_box, int64_t* sequence);
int wcn_mailbox_mark(hipStream_t stream);  // records `done` behind the writing kernel
int wcn_mailbox_end(void* host_dst, size_t payload_bytes, int64_t sequence);

// Output-row form of a pair list (rows of the map grouped by output row, inside a row ascending
// in kernel offset): row_mask[m] has bit k set if offset k has a pair for output row m,
// row_in[row_ptr[m] .. row_ptr[m + 1]) are the input rows of those pairs.  Built by
// wcn_rows_build (wcn_conv.hip) inside a caller-provided workspace; used by the contraction to
// re-order lists that do not ascend and by the pooling kernels.
struct WcnRowsView {
  int64_t* offsets;    // K + 1, device copy of the host offsets
  uint32_t* row_mask;  // num_out * words
  int32_t* row_ptr;    // num_out + 1
  int32_t* row_in;     // pairs
  int32_t* groups;     // G + 1 (scan scratch)
  int64_t* row_total;  // 1 (scan scratch)
  int32_t words;       // ceil(K / 32)
  int64_t G;           // ceil(num_out / 64)
};
size_t wcn_rows_layout(void* base, int64_t num_out, int num_offsets, int64_t pairs, WcnRowsView* v);
// `v.offsets` must already hold the offsets; pairs whose output row is out of range are dropped.
int wcn_rows_build(const int32_t* in_maps, const int32_t* out_maps, int num_offsets, int64_t num_out,
                   int64_t pairs, const WcnRowsView& v, hipStream_t stream);

#ifdef __HIPCC__

#define WCN_LAUNCH_CHECK()                      \
  do {                                          \
    if (hipGetLastError() != hipSuccess) return WCN_ERR_LAUNCH; \
  } while (0)

#endif  // __HIPCC__
