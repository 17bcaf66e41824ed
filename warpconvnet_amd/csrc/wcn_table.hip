// Coordinate table of 4x4x4-voxel blocks: build and point queries (gfx950).
//
// Build pipeline (all on the caller's stream, no host round trip):
//   table_clear   header, slots and perm to their empty values
//   table_bbox    bounding box of the keys (LDS reduction, one atomic min/max per workgroup)
//   table_insert  per key: claim / find the block slot with a 64-bit CAS, OR the voxel bit in
//   table_base    per slot: base = running sum of block populations (one atomic per 1024 slots)
//   table_perm    per key: perm[base + rank of its bit] = min(row index)
//
// HBM traffic per key: 16 B read (bbox) + 16 B read (insert) + 4 B slot_of write + 4 B read +
// 4 B perm write, plus 32 B per table slot to clear and one 32 B slot touched per key.
#include <stdlib.h>
#include <string.h>

#include <chrono>
#include <thread>

#include "wcn_common.h"

namespace {

__global__ void __launch_bounds__(256) table_clear(WcnTableHeader* __restrict__ hdr,
                                                   WcnSlot* __restrict__ slots, int64_t capacity,
                                                   int32_t* __restrict__ perm, int64_t n_keys) {
  const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t nthreads = (int64_t)gridDim.x * blockDim.x;
  if (tid == 0) {
    for (int d = 0; d < 4; ++d) {
      hdr->mn[d] = INT32_MAX;
      hdr->mx[d] = INT32_MIN;
    }
    hdr->num_blocks = 0;
    hdr->status = 0;
    hdr->total = 0;
    hdr->num_keys = (int32_t)n_keys;
  }
  // each slot is two 16-byte stores: {EMPTY, 0} and {0, 0, 0, 0}
  uint4* raw = reinterpret_cast<uint4*>(slots);
  for (int64_t i = tid; i < 2 * capacity; i += nthreads) {
    uint4 v = (i & 1) ? make_uint4(0u, 0u, 0u, 0u) : make_uint4(0xFFFFFFFFu, 0xFFFFFFFFu, 0u, 0u);
    raw[i] = v;
  }
  for (int64_t i = tid; i < n_keys; i += nthreads) perm[i] = INT32_MAX;
}

// Bounding box of the keys.  Few, wide workgroups: the eight atomics a workgroup ends with all
// land on the same eight words and serialise, so their number decides the run time.
__global__ void __launch_bounds__(1024) table_bbox(const int4* __restrict__ keys, int64_t n_keys,
                                                   WcnTableHeader* __restrict__ hdr) {
  __shared__ int s_mn[16][4];
  __shared__ int s_mx[16][4];
  int mn[4] = {INT32_MAX, INT32_MAX, INT32_MAX, INT32_MAX};
  int mx[4] = {INT32_MIN, INT32_MIN, INT32_MIN, INT32_MIN};
  const int64_t nthreads = (int64_t)gridDim.x * blockDim.x;
  constexpr int PER = 8;  // keys a thread has in flight together
  for (int64_t i0 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i0 < n_keys; i0 += nthreads * PER) {
    int4 c[PER];
#pragma unroll
    for (int t = 0; t < PER; ++t) {
      const int64_t i = i0 + t * nthreads;
      c[t] = keys[i < n_keys ? i : i0];  // past the end: the thread's first key again
    }
#pragma unroll
    for (int t = 0; t < PER; ++t) {
      mn[0] = min(mn[0], c[t].x); mx[0] = max(mx[0], c[t].x);
      mn[1] = min(mn[1], c[t].y); mx[1] = max(mx[1], c[t].y);
      mn[2] = min(mn[2], c[t].z); mx[2] = max(mx[2], c[t].z);
      mn[3] = min(mn[3], c[t].w); mx[3] = max(mx[3], c[t].w);
    }
  }
#pragma unroll
  for (int d = 0; d < 4; ++d) {
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) {
      mn[d] = min(mn[d], __shfl_xor(mn[d], s, 64));
      mx[d] = max(mx[d], __shfl_xor(mx[d], s, 64));
    }
  }
  const int wave = threadIdx.x >> 6;
  if (wcn_lane() == 0) {
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      s_mn[wave][d] = mn[d];
      s_mx[wave][d] = mx[d];
    }
  }
  __syncthreads();
  if (threadIdx.x < 4) {
    const int d = threadIdx.x;
    int a = s_mn[0][d], b = s_mx[0][d];
    for (int w = 1; w < (int)(blockDim.x >> 6); ++w) {
      a = min(a, s_mn[w][d]);
      b = max(b, s_mx[w][d]);
    }
    atomicMin(&hdr->mn[d], a);
    atomicMax(&hdr->mx[d], b);
  }
}

__global__ void __launch_bounds__(256) table_insert(const int4* __restrict__ keys, int64_t n_keys,
                                                    WcnTableHeader* __restrict__ hdr,
                                                    WcnSlot* __restrict__ slots, uint32_t cap_mask,
                                                    int32_t* __restrict__ slot_of) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_keys) return;
  const WcnLayout L = wcn_make_layout(hdr);
  if (!L.ok) {
    if (i == 0) atomicOr(&hdr->status, WCN_DEV_RANGE);
    slot_of[i] = -1;
    return;
  }
  const int4 c = keys[i];
  uint32_t r[4];
  wcn_relative(L, c.x, c.y, c.z, c.w, r);  // always inside: the box was built from these keys
  const unsigned long long key = wcn_block_key(L, r);
  const uint32_t bit_index = wcn_block_bit(r);
  const uint32_t bit = 1u << (bit_index & 31u);  // within the 32-bit half of the mask that holds it
  uint32_t h = wcn_mix(key, cap_mask);
  int32_t placed = -1;
  for (int p = 0; p < WCN_MAX_PROBE; ++p) {
    // cheap pre-read: most keys find their block already present
    // (a stale EMPTY from the vector cache only costs the CAS below; a non-empty key is final)
    unsigned long long seen = *reinterpret_cast<const volatile unsigned long long*>(&slots[h].key);
    if (seen == WCN_EMPTY_KEY) {
      seen = atomicCAS(&slots[h].key, WCN_EMPTY_KEY, key);
      if (seen == WCN_EMPTY_KEY) seen = key;  // this thread claimed the slot
    }
    if (seen == key) {
      // the result of the atomic is not used, so it is issued without waiting for a reply;
      // repeated keys show up later as fewer set bits than keys
      uint32_t* half = reinterpret_cast<uint32_t*>(&slots[h].mask) + (bit_index >> 5);
      atomicOr(half, bit);
      placed = (int32_t)h;
      break;
    }
    h = (h + 1) & cap_mask;
  }
  if (placed < 0) atomicOr(&hdr->status, WCN_DEV_OVERFLOW);
  slot_of[i] = placed;
}

// base of every occupied slot = running sum of block populations.  A 1024-thread workgroup owns
// BASE_CHUNKS x 1024 consecutive slots, scans them and takes its share of the running sum with a
// single atomic (the atomics of all workgroups serialise on one word, so there should be few).
constexpr int BASE_CHUNKS = 8;
__global__ void __launch_bounds__(1024) table_base(WcnTableHeader* __restrict__ hdr,
                                                   WcnSlot* __restrict__ slots, int64_t capacity) {
  __shared__ int s_wave[BASE_CHUNKS][16];
  __shared__ int s_occ[16];
  __shared__ int s_group_base;
  const int64_t j0 = (int64_t)blockIdx.x * (BASE_CHUNKS * 1024) + threadIdx.x;
  const int lane = wcn_lane(), wave = threadIdx.x >> 6;
  int cnt[BASE_CHUNKS], incl[BASE_CHUNKS], occ = 0;
#pragma unroll
  for (int t = 0; t < BASE_CHUNKS; ++t) {
    const int64_t j = j0 + (int64_t)t * 1024;
    cnt[t] = j < capacity ? __popcll(slots[j].mask) : 0;
  }
#pragma unroll
  for (int t = 0; t < BASE_CHUNKS; ++t) {
    incl[t] = wcn_wave_inclusive_sum(cnt[t]);
    occ += __popcll(__ballot(cnt[t] > 0));
    if (lane == 63) s_wave[t][wave] = incl[t];
  }
  if (lane == 0) s_occ[wave] = occ;
  __syncthreads();
  if (threadIdx.x == 0) {
    int total = 0, blocks = 0;
    for (int t = 0; t < BASE_CHUNKS; ++t)
      for (int w = 0; w < 16; ++w) {
        const int v = s_wave[t][w];
        s_wave[t][w] = total;  // exclusive prefix over (chunk, wave)
        total += v;
      }
    for (int w = 0; w < 16; ++w) blocks += s_occ[w];
    s_group_base = total ? atomicAdd(&hdr->total, total) : 0;
    if (blocks) atomicAdd(&hdr->num_blocks, blocks);
  }
  __syncthreads();
#pragma unroll
  for (int t = 0; t < BASE_CHUNKS; ++t)
    if (cnt[t] > 0) slots[j0 + (int64_t)t * 1024].base = s_group_base + s_wave[t][wave] + incl[t] - cnt[t];
}

__global__ void __launch_bounds__(256) table_perm(const int4* __restrict__ keys, int64_t n_keys,
                                                  const WcnTableHeader* __restrict__ hdr,
                                                  const WcnSlot* __restrict__ slots,
                                                  const int32_t* __restrict__ slot_of,
                                                  int32_t* __restrict__ perm) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_keys) return;
  const int32_t h = slot_of[i];
  if (h < 0) return;
  const WcnLayout L = wcn_make_layout(hdr);
  const int4 c = keys[i];
  uint32_t r[4];
  wcn_relative(L, c.x, c.y, c.z, c.w, r);
  const ulonglong2 km = *reinterpret_cast<const ulonglong2*>(&slots[h]);
  const int32_t pos = slots[h].base + wcn_rank_below(km.y, wcn_block_bit(r));
  if (pos < 0 || pos >= n_keys) return;
  // without duplicate keys every position has exactly one writer
  if (WCN_HAS_DUPLICATES(hdr)) atomicMin(&perm[pos], (int32_t)i); else perm[pos] = (int32_t)i;
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

// Enqueue the five build kernels.  Shared with the strided-coordinate path.
int wcn_table_build_impl(const int32_t* keys, int64_t n_keys, const WcnTableView& v,
                         hipStream_t s) {
  const uint32_t cap_mask = (uint32_t)(v.capacity - 1);
  const int64_t clear_items = 2 * v.capacity > n_keys ? 2 * v.capacity : n_keys;
  hipLaunchKernelGGL(table_clear, dim3(grid_for(clear_items, 256, 4096)), dim3(256), 0, s, v.hdr,
                     v.slots, v.capacity, v.perm, n_keys);
  if (n_keys > 0) {
    hipLaunchKernelGGL(table_bbox, dim3(grid_for(n_keys, 1024 * 8, 128)), dim3(1024), 0, s,
                       (const int4*)keys, n_keys, v.hdr);
    hipLaunchKernelGGL(table_insert, dim3(grid_for(n_keys, 256)), dim3(256), 0, s,
                       (const int4*)keys, n_keys, v.hdr, v.slots, cap_mask, v.slot_of);
    hipLaunchKernelGGL(table_base, dim3(grid_for(v.capacity, 1024 * BASE_CHUNKS)), dim3(1024), 0, s, v.hdr,
                       v.slots, v.capacity);
    hipLaunchKernelGGL(table_perm, dim3(grid_for(n_keys, 256)), dim3(256), 0, s,
                       (const int4*)keys, n_keys, v.hdr, v.slots, v.slot_of, v.perm);
  }
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
  return wcn_table_build_impl(keys, n_keys, v, (hipStream_t)stream);
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
  if (wcn_read_small(&h, table, sizeof(h), (hipStream_t)stream) != WCN_OK) return WCN_ERR_LAUNCH;
  if (host_num_blocks) *host_num_blocks = h.num_blocks;
  return wcn_table_status_from_bits(h.status);
}

}  // extern "C"
