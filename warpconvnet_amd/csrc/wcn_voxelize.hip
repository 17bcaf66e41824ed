// Voxelisation front-end of libwcn_hip.so (gfx950): points -> integer voxel rows, and the
// sorted-unique / CSR grouping of integer rows that the point-to-voxel pooling reduces over.
//
// The reference does this with torch ops: floor(points / voxel_size).int() + a batch column
// (warpconvnet/geometry/coords/ops/voxel.py:92-95), then torch.unique(dim=0, sorted,
// return_inverse, return_counts) + a stable argsort of the inverse + a cumulative sum + a scatter
// (warpconvnet/utils/unique.py:57-109).  Here every row is packed into one 64-bit key whose numeric
// order is the rows' lexicographic order (fields relative to the bounding box, first column most
// significant), the (key, row index) pairs go through one stable radix sort over just the bits in
// use, and one pass over the sorted pairs writes all five results.  The radix sort and the prefix
// sum are rocPRIM's (plain library primitives); everything else is written here.
#include "wcn_common.h"

#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_scan.hpp>
#include <rocprim/iterator/counting_iterator.hpp>
#include <rocprim/iterator/transform_iterator.hpp>

namespace {

struct UniqueHeader {  // first 256 bytes of the workspace
  int32_t mn[4];
  int32_t mx[4];
  int32_t count;   // number of distinct rows
  int32_t pad[55];
};
static_assert(sizeof(UniqueHeader) == 256, "header is 256 bytes");

struct UniqueView {
  UniqueHeader* hdr;
  unsigned long long* keys_a;
  unsigned long long* keys_b;
  uint32_t* idx_a;
  uint32_t* idx_b;
  uint32_t* rank;  // inclusive count of segment heads
  void* temp;      // rocPRIM scratch
  size_t temp_bytes;
};

struct HeadFlag {  // 1 where a sorted key differs from its predecessor
  const unsigned long long* keys;
  __device__ uint32_t operator()(uint32_t i) const {
    return (i == 0 || keys[i] != keys[i - 1]) ? 1u : 0u;
  }
};
using HeadIterator = rocprim::transform_iterator<rocprim::counting_iterator<uint32_t>, HeadFlag, uint32_t>;

size_t prim_temp_bytes(int64_t n) {
  size_t sort_bytes = 0, scan_bytes = 0;
  unsigned long long* k = nullptr;
  uint32_t* v = nullptr;
  (void)rocprim::radix_sort_pairs(nullptr, sort_bytes, k, k, v, v, (size_t)n, 0u, 64u, (hipStream_t)0);
  HeadIterator heads(rocprim::counting_iterator<uint32_t>(0), HeadFlag{nullptr});
  (void)rocprim::inclusive_scan(nullptr, scan_bytes, heads, v, (size_t)n, rocprim::plus<uint32_t>(),
                                (hipStream_t)0);
  return sort_bytes > scan_bytes ? sort_bytes : scan_bytes;
}

size_t unique_layout(void* base, int64_t n, UniqueView* v) {
  char* p = (char*)base;
  size_t off = 0;
  auto take = [&](size_t bytes) {
    char* at = p + off;
    off += wcn_align256(bytes);
    return at;
  };
  const size_t rows = (size_t)(n > 0 ? n : 1);
  char* hdr = take(256);
  char* ka = take(8 * rows);
  char* kb = take(8 * rows);
  char* ia = take(4 * rows);
  char* ib = take(4 * rows);
  char* rk = take(4 * rows);
  const size_t tb = prim_temp_bytes(n > 0 ? n : 1);
  char* tp = take(tb > 0 ? tb : 256);
  if (v) {
    v->hdr = (UniqueHeader*)hdr;
    v->keys_a = (unsigned long long*)ka;
    v->keys_b = (unsigned long long*)kb;
    v->idx_a = (uint32_t*)ia;
    v->idx_b = (uint32_t*)ib;
    v->rank = (uint32_t*)rk;
    v->temp = tp;
    v->temp_bytes = tb;
  }
  return off;
}

// ---- points -> [batch, floor(p * inv)] ----------------------------------------------------------
// torch divides a float tensor by a host scalar as a multiplication with the scalar's reciprocal
// (taken in double, rounded to float); the product is floored and converted to int32 the same way.
// One thread per point; three consecutive points of a thread would make wider loads but the rows
// are 12 bytes, so lanes read adjacent 4-byte words and the 16-byte output rows are full vectors.
struct BatchStarts {
  int64_t start[WCN_VOXEL_MAX_BATCH + 1];
};

__global__ void __launch_bounds__(256) voxel_rows(const float* __restrict__ points, int64_t n,
                                                  float inv, BatchStarts starts, int batch_size,
                                                  const int64_t* __restrict__ device_starts,
                                                  int4* __restrict__ rows) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float x = points[3 * i], y = points[3 * i + 1], z = points[3 * i + 2];
  // batch item = number of starts (beyond the first) that are <= i
  int lo = 0, hi = batch_size;  // answer in [lo, hi)
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    const int64_t s = device_starts ? device_starts[mid] : starts.start[mid];
    if (s <= i) lo = mid; else hi = mid;
  }
  int4 r;
  r.x = lo;
  r.y = (int)floorf(x * inv);
  r.z = (int)floorf(y * inv);
  r.w = (int)floorf(z * inv);
  rows[i] = r;
}

// ---- bounding box of (n, columns) int32 rows ---------------------------------------------------
__global__ void unique_init(UniqueHeader* __restrict__ h) {
  const int t = threadIdx.x;
  if (t < 4) {
    h->mn[t] = INT32_MAX;
    h->mx[t] = INT32_MIN;
  }
  if (t == 4) h->count = 0;
}

__global__ void __launch_bounds__(256) unique_bbox(const int32_t* __restrict__ rows, int64_t n,
                                                   int columns, UniqueHeader* __restrict__ h) {
  int mn[4] = {INT32_MAX, INT32_MAX, INT32_MAX, INT32_MAX};
  int mx[4] = {INT32_MIN, INT32_MIN, INT32_MIN, INT32_MIN};
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    if (columns == 4) {
      const int4 r = reinterpret_cast<const int4*>(rows)[i];
      const int v[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        mn[d] = min(mn[d], v[d]);
        mx[d] = max(mx[d], v[d]);
      }
    } else {
      for (int d = 0; d < columns; ++d) {
        const int v = rows[i * columns + d];
        mn[d] = min(mn[d], v);
        mx[d] = max(mx[d], v);
      }
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
  __shared__ int smn[4][4], smx[4][4];
  const int wave = threadIdx.x >> 6;
  if (wcn_lane() == 0) {
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      smn[wave][d] = mn[d];
      smx[wave][d] = mx[d];
    }
  }
  __syncthreads();
  if (threadIdx.x < (unsigned)columns) {
    const int d = threadIdx.x;
    int a = smn[0][d], b = smx[0][d];
    for (int w = 1; w < 4; ++w) {
      a = min(a, smn[w][d]);
      b = max(b, smx[w][d]);
    }
    atomicMin(&h->mn[d], a);
    atomicMax(&h->mx[d], b);
  }
}

// Field widths of the packed key: column d takes bits(mx - mn); the first column is the most
// significant.  The host computes the same from its copy of the box.
struct KeyLayout {
  uint32_t mn[4];
  uint32_t shift[4];
  uint32_t bits[4];
  uint32_t total;
};

__host__ __device__ inline KeyLayout key_layout(const int32_t* mn, const int32_t* mx, int columns) {
  KeyLayout L;
  for (int d = 0; d < 4; ++d) {
    L.mn[d] = 0;
    L.bits[d] = 0;
    L.shift[d] = 0;
  }
  for (int d = 0; d < columns; ++d) {
    const uint32_t span = (uint32_t)mx[d] - (uint32_t)mn[d];
    const uint32_t b = span == 0 ? 0u : 32u - (uint32_t)__builtin_clz(span);
    L.mn[d] = (uint32_t)mn[d];
    L.bits[d] = b;
  }
  uint32_t at = 0;
  for (int d = columns - 1; d >= 0; --d) {
    L.shift[d] = at;
    at += L.bits[d];
  }
  L.total = at;
  return L;
}

__global__ void __launch_bounds__(256) unique_pack(const int32_t* __restrict__ rows, int64_t n,
                                                   int columns, const UniqueHeader* __restrict__ h,
                                                   unsigned long long* __restrict__ keys,
                                                   uint32_t* __restrict__ idx) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const KeyLayout L = key_layout(h->mn, h->mx, columns);
  int v[4] = {0, 0, 0, 0};
  if (columns == 4) {
    const int4 r = reinterpret_cast<const int4*>(rows)[i];
    v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w;
  } else {
    for (int d = 0; d < columns; ++d) v[d] = rows[i * columns + d];
  }
  unsigned long long key = 0;
#pragma unroll
  for (int d = 0; d < 4; ++d)
    if (d < columns && L.bits[d] > 0)  // a shift by 64 (a single 64-bit field at shift 0 never is) stays out
      key |= (unsigned long long)((uint32_t)v[d] - L.mn[d]) << L.shift[d];
  keys[i] = key;
  idx[i] = (uint32_t)i;
}

// One pass over the sorted (key, row) pairs.  rank[i] = number of segment heads in [0, i].
__global__ void __launch_bounds__(256) unique_emit(
    const unsigned long long* __restrict__ keys, const uint32_t* __restrict__ idx,
    const uint32_t* __restrict__ rank, int64_t n, int columns, UniqueHeader* __restrict__ h,
    int32_t* __restrict__ unique_rows, int64_t* __restrict__ to_orig, int64_t* __restrict__ csr_indices,
    int64_t* __restrict__ csr_offsets, int64_t* __restrict__ to_unique) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const unsigned long long key = keys[i];
  const uint32_t row = idx[i];
  const int64_t u = (int64_t)rank[i] - 1;
  const bool head = i == 0 || keys[i - 1] != key;
  if (csr_indices) csr_indices[i] = row;
  if (to_orig) to_orig[row] = u;
  if (head) {
    if (csr_offsets) csr_offsets[u] = i;
    // the sort is stable, so the head of a segment is the lowest row of its key
    if (to_unique) to_unique[u] = row;
    if (unique_rows) {
      const KeyLayout L = key_layout(h->mn, h->mx, columns);
      for (int d = 0; d < columns; ++d) {
        const uint32_t field =
            L.bits[d] == 0 ? 0u : (uint32_t)((key >> L.shift[d]) & ((1ull << L.bits[d]) - 1ull));
        unique_rows[u * columns + d] = (int32_t)(field + L.mn[d]);
      }
    }
  }
  if (i == n - 1) {
    if (csr_offsets) csr_offsets[u + 1] = n;
    h->count = (int32_t)(u + 1);
  }
}

}  // namespace

extern "C" {

int wcn_voxel_rows(const float* points, int64_t num_points, const int64_t* host_batch_offsets,
                   const int64_t* device_batch_offsets_or_null, int32_t batch_size, double voxel_size,
                   int32_t* rows, void* stream) {
  if (num_points < 0 || num_points >= (1ll << 31) || batch_size < 1 || !host_batch_offsets ||
      !(voxel_size > 0.0))
    return WCN_ERR_INVALID_ARGUMENT;
  if (host_batch_offsets[0] != 0 || host_batch_offsets[batch_size] != num_points)
    return WCN_ERR_INVALID_ARGUMENT;
  for (int b = 0; b < batch_size; ++b)
    if (host_batch_offsets[b + 1] < host_batch_offsets[b]) return WCN_ERR_INVALID_ARGUMENT;
  if (batch_size > WCN_VOXEL_MAX_BATCH && !device_batch_offsets_or_null) return WCN_ERR_INVALID_ARGUMENT;
  if (num_points == 0) return WCN_OK;
  if (!points || !rows) return WCN_ERR_INVALID_ARGUMENT;
  BatchStarts starts;
  for (int b = 0; b <= WCN_VOXEL_MAX_BATCH; ++b)
    starts.start[b] = b <= batch_size && batch_size <= WCN_VOXEL_MAX_BATCH ? host_batch_offsets[b] : 0;
  const float inv = (float)(1.0 / voxel_size);
  hipLaunchKernelGGL(voxel_rows, dim3((unsigned)((num_points + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, points, num_points, inv, starts, batch_size,
                     batch_size > WCN_VOXEL_MAX_BATCH ? device_batch_offsets_or_null : nullptr,
                     (int4*)rows);
  WCN_LAUNCH_CHECK();
  return WCN_OK;
}

size_t wcn_unique_rows_workspace_bytes(int64_t num_rows) {
  if (num_rows < 0 || num_rows >= (1ll << 31)) return 0;
  return unique_layout(nullptr, num_rows, nullptr);
}

int wcn_unique_rows_csr(const int32_t* rows, int64_t num_rows, int32_t columns, void* workspace,
                        size_t workspace_bytes, int32_t* unique_rows, int64_t* to_orig,
                        int64_t* csr_indices, int64_t* csr_offsets, int64_t* to_unique,
                        int64_t* num_unique, void* stream) {
  if (num_rows < 0 || num_rows >= (1ll << 31) || columns < 1 || columns > 4 || !num_unique)
    return WCN_ERR_INVALID_ARGUMENT;
  *num_unique = 0;
  hipStream_t s = (hipStream_t)stream;
  if (num_rows == 0) {
    if (csr_offsets) {
      if (hipMemsetAsync(csr_offsets, 0, sizeof(int64_t), s) != hipSuccess) return WCN_ERR_LAUNCH;
    }
    return WCN_OK;
  }
  if (!rows || !workspace) return WCN_ERR_INVALID_ARGUMENT;
  if (workspace_bytes < wcn_unique_rows_workspace_bytes(num_rows)) return WCN_ERR_WORKSPACE;
  UniqueView v;
  unique_layout(workspace, num_rows, &v);
  const unsigned blocks = (unsigned)((num_rows + 255) / 256);

  hipLaunchKernelGGL(unique_init, dim3(1), dim3(64), 0, s, v.hdr);
  WCN_LAUNCH_CHECK();
  // one workgroup per compute unit: the closing atomics of all workgroups land on the same eight
  // words and are served one after the other
  const unsigned box_blocks = blocks < 256u ? blocks : 256u;
  hipLaunchKernelGGL(unique_bbox, dim3(box_blocks), dim3(256), 0, s, rows, num_rows, (int)columns, v.hdr);
  WCN_LAUNCH_CHECK();
  // The sort needs the number of key bits on the host: one small read, while the keys are packed.
  if (wcn_read_early_begin(v.hdr, 32, s) != WCN_OK) return WCN_ERR_LAUNCH;
  hipLaunchKernelGGL(unique_pack, dim3(blocks), dim3(256), 0, s, rows, num_rows, (int)columns,
                     (const UniqueHeader*)v.hdr, v.keys_a, v.idx_a);
  WCN_LAUNCH_CHECK();
  int32_t box[8];
  if (wcn_read_early_end(box, v.hdr, 32, s) != WCN_OK) return WCN_ERR_LAUNCH;
  const KeyLayout L = key_layout(box, box + 4, columns);
  if (L.total > 64u) return WCN_ERR_COORD_RANGE;

  size_t temp_bytes = v.temp_bytes;
  if (L.total > 0) {
    if (rocprim::radix_sort_pairs(v.temp, temp_bytes, v.keys_a, v.keys_b, v.idx_a, v.idx_b,
                                  (size_t)num_rows, 0u, L.total, s) != hipSuccess)
      return WCN_ERR_LAUNCH;
  }
  const unsigned long long* keys = L.total > 0 ? v.keys_b : v.keys_a;  // all rows equal: nothing to sort
  const uint32_t* idx = L.total > 0 ? v.idx_b : v.idx_a;
  HeadIterator heads(rocprim::counting_iterator<uint32_t>(0), HeadFlag{keys});
  temp_bytes = v.temp_bytes;
  if (rocprim::inclusive_scan(v.temp, temp_bytes, heads, v.rank, (size_t)num_rows,
                              rocprim::plus<uint32_t>(), s) != hipSuccess)
    return WCN_ERR_LAUNCH;
  hipLaunchKernelGGL(unique_emit, dim3(blocks), dim3(256), 0, s, keys, idx, (const uint32_t*)v.rank,
                     num_rows, (int)columns, v.hdr, unique_rows, to_orig, csr_indices, csr_offsets,
                     to_unique);
  WCN_LAUNCH_CHECK();
  int32_t count = 0;
  if (wcn_read_small(&count, &v.hdr->count, sizeof(count), s) != WCN_OK) return WCN_ERR_LAUNCH;
  *num_unique = count;
  return WCN_OK;
}

}  // extern "C"
