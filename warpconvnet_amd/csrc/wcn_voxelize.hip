// Voxelisation front-end of libwcn_hip.so (gfx950): points -> integer voxel rows, and the
// sorted-unique / CSR grouping of integer rows that the point-to-voxel pooling reduces over.
//
// The reference does this with torch ops: floor(points / voxel_size).int() + a batch column
// (warpconvnet/geometry/coords/ops/voxel.py:92-95), then torch.unique(dim=0, sorted,
// return_inverse, return_counts) + a stable argsort of the inverse + a cumulative sum + a scatter
// (warpconvnet/utils/unique.py:57-109).  Here every row is packed into one 64-bit key whose numeric
// order is the rows' lexicographic order (fields relative to the bounding box, first column most
// significant), the (key, row index) pairs go through one stable radix sort over just the bits in
// use (as 32-bit words when they fit), and one pass over the sorted pairs writes all five results.
// For points the rows are never stored: the box and the keys are computed from the points directly.
// The radix sort and the prefix sum are rocPRIM's (plain library primitives); everything else is
// written here.
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

template <typename KeyT>
struct HeadFlag {  // 1 where a sorted key differs from its predecessor
  const KeyT* keys;
  __device__ uint32_t operator()(uint32_t i) const {
    return (i == 0 || keys[i] != keys[i - 1]) ? 1u : 0u;
  }
};
template <typename KeyT>
using HeadIterator =
    rocprim::transform_iterator<rocprim::counting_iterator<uint32_t>, HeadFlag<KeyT>, uint32_t>;

// rocPRIM's default switches to a comparison merge sort below a million items, which ignores how
// few key bits are in use (160 us for a million 28-bit keys against four radix passes of ~10 us).
using SortConfig = rocprim::radix_sort_config<rocprim::default_config, rocprim::default_config,
                                              rocprim::default_config, 32768>;

template <typename KeyT>
size_t prim_temp_bytes_for(int64_t n) {
  size_t sort_bytes = 0, scan_bytes = 0;
  KeyT* k = nullptr;
  uint32_t* v = nullptr;
  (void)rocprim::radix_sort_pairs<SortConfig>(nullptr, sort_bytes, k, k, v, v, (size_t)n, 0u,
                                  (unsigned)(8 * sizeof(KeyT)), (hipStream_t)0);
  HeadIterator<KeyT> heads(rocprim::counting_iterator<uint32_t>(0), HeadFlag<KeyT>{nullptr});
  (void)rocprim::inclusive_scan(nullptr, scan_bytes, heads, v, (size_t)n, rocprim::plus<uint32_t>(),
                                (hipStream_t)0);
  return sort_bytes > scan_bytes ? sort_bytes : scan_bytes;
}

size_t prim_temp_bytes(int64_t n) {
  const size_t a = prim_temp_bytes_for<unsigned long long>(n), b = prim_temp_bytes_for<uint32_t>(n);
  return a > b ? a : b;
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

// ---- where the rows come from -------------------------------------------------------------------
// torch divides a float tensor by a host scalar as a multiplication with the scalar's reciprocal
// (taken in double, rounded to float); the product is floored and converted to int32 the same way.
struct BatchStarts {
  int64_t start[WCN_VOXEL_MAX_BATCH + 1];
};

struct PointRows {  // row i = [batch item of point i, floor(p * inv)]
  const float* points;
  float inv;
  BatchStarts starts;
  int batch_size;
  const int64_t* device_starts;  // used instead of `starts` when there are too many batch items
  __device__ __forceinline__ void load(int64_t i, int v[4]) const {
    const float x = points[3 * i], y = points[3 * i + 1], z = points[3 * i + 2];
    int lo = 0, hi = batch_size;  // the item lies in [lo, hi)
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      const int64_t s = device_starts ? device_starts[mid] : starts.start[mid];
      if (s <= i) lo = mid; else hi = mid;
    }
    v[0] = lo;
    v[1] = (int)floorf(x * inv);
    v[2] = (int)floorf(y * inv);
    v[3] = (int)floorf(z * inv);
  }
  __device__ __forceinline__ int columns() const { return 4; }
};

struct IntRows {  // (n, columns) int32, row-major
  const int32_t* rows;
  int ncol;
  __device__ __forceinline__ void load(int64_t i, int v[4]) const {
    if (ncol == 4) {
      const int4 r = reinterpret_cast<const int4*>(rows)[i];
      v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w;
    } else {
      v[0] = v[1] = v[2] = v[3] = 0;
      for (int d = 0; d < ncol; ++d) v[d] = rows[i * ncol + d];
    }
  }
  __device__ __forceinline__ int columns() const { return ncol; }
};

// One thread per point: 12 bytes read (lanes read adjacent words), one 16-byte row written.
__global__ void __launch_bounds__(256) voxel_rows(PointRows src, int64_t n, int4* __restrict__ rows) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  int v[4];
  src.load(i, v);
  rows[i] = make_int4(v[0], v[1], v[2], v[3]);
}

// ---- bounding box of the rows --------------------------------------------------------------------
// The batch column put in front of integer coordinates: row i = [batch item of row i, c[i][0..dims)].
// One thread per row; with three spatial columns the row goes out as one 16-byte store.
__global__ void __launch_bounds__(256) batch_indexed_rows(const int32_t* __restrict__ coords, int64_t n,
                                                          int dims, BatchStarts starts, int batch_size,
                                                          int32_t* __restrict__ rows) {
  // the offsets arrive with the launch (scalar registers); lanes search them at different places,
  // so they are put into LDS first
  __shared__ int64_t s_start[WCN_VOXEL_MAX_BATCH + 1];
  if (threadIdx.x <= WCN_VOXEL_MAX_BATCH) s_start[threadIdx.x] = starts.start[threadIdx.x];
  __syncthreads();
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  int lo = 0, hi = batch_size;  // the item lies in [lo, hi)
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (s_start[mid] <= i) lo = mid; else hi = mid;
  }
  if (dims == 3) {
    const int32_t* c = coords + 3 * i;
    reinterpret_cast<int4*>(rows)[i] = make_int4(lo, c[0], c[1], c[2]);
  } else {
    int32_t* r = rows + i * (dims + 1);
    r[0] = lo;
    for (int d = 0; d < dims; ++d) r[d + 1] = coords[i * dims + d];
  }
}

__global__ void unique_init(UniqueHeader* __restrict__ h) {
  const int t = threadIdx.x;
  if (t < 4) {
    h->mn[t] = INT32_MAX;
    h->mx[t] = INT32_MIN;
  }
  if (t == 4) h->count = 0;
}

// A few large workgroups: the closing atomics of all workgroups land on the same eight words and
// are served one after the other, so there is one workgroup per compute unit.
template <class Src>
__global__ void __launch_bounds__(1024) unique_bbox(Src src, int64_t n, UniqueHeader* __restrict__ h) {
  int mn[4] = {INT32_MAX, INT32_MAX, INT32_MAX, INT32_MAX};
  int mx[4] = {INT32_MIN, INT32_MIN, INT32_MIN, INT32_MIN};
  const int columns = src.columns();
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    int v[4];
    src.load(i, v);
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      mn[d] = min(mn[d], v[d]);
      mx[d] = max(mx[d], v[d]);
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
  __shared__ int smn[16][4], smx[16][4];
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
    const int waves = (int)(blockDim.x >> 6);
    int a = smn[0][d], b = smx[0][d];
    for (int w = 1; w < waves; ++w) {
      a = min(a, smn[w][d]);
      b = max(b, smx[w][d]);
    }
    atomicMin(&h->mn[d], a);
    atomicMax(&h->mx[d], b);
  }
}

// Field widths of the packed key: column d takes bits(mx - mn); the first column is the most
// significant.  The host computes the same from its copy of the box.  Keys of at most 32 bits are
// stored, sorted and compared as 32-bit words (half the sort's key traffic).
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

template <class Src>
__global__ void __launch_bounds__(256) unique_pack(Src src, int64_t n, const UniqueHeader* __restrict__ h,
                                                   void* __restrict__ keys, uint32_t* __restrict__ idx) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int columns = src.columns();
  const KeyLayout L = key_layout(h->mn, h->mx, columns);
  int v[4];
  src.load(i, v);
  unsigned long long key = 0;
#pragma unroll
  for (int d = 0; d < 4; ++d)
    if (d < columns && L.bits[d] > 0)  // fields of width 0 stay out (their shift may be 64)
      key |= (unsigned long long)((uint32_t)v[d] - L.mn[d]) << L.shift[d];
  if (L.total <= 32u)
    reinterpret_cast<uint32_t*>(keys)[i] = (uint32_t)key;
  else
    reinterpret_cast<unsigned long long*>(keys)[i] = key;
  idx[i] = (uint32_t)i;
}

// One pass over the sorted (key, row) pairs.  rank[i] = number of segment heads in [0, i].
template <typename KeyT>
__global__ void __launch_bounds__(256) unique_emit(
    const KeyT* __restrict__ keys, const uint32_t* __restrict__ idx, const uint32_t* __restrict__ rank,
    int64_t n, int columns, UniqueHeader* __restrict__ h, int32_t* __restrict__ unique_rows,
    int64_t* __restrict__ to_orig, int64_t* __restrict__ csr_indices, int64_t* __restrict__ csr_offsets,
    int64_t* __restrict__ to_unique) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const KeyLayout L = key_layout(h->mn, h->mx, columns);  // the same for every thread: scalar work
  const KeyT key = keys[i];
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
      int32_t field[4];
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const uint32_t f =
            L.bits[d] == 0 ? 0u
                           : (uint32_t)(((unsigned long long)key >> L.shift[d]) & ((1ull << L.bits[d]) - 1ull));
        field[d] = (int32_t)(f + L.mn[d]);
      }
      if (columns == 4) {
        reinterpret_cast<int4*>(unique_rows)[u] = make_int4(field[0], field[1], field[2], field[3]);
      } else {
        for (int d = 0; d < columns; ++d) unique_rows[u * columns + d] = field[d];
      }
    }
  }
  if (i == n - 1) {
    if (csr_offsets) csr_offsets[u + 1] = n;
    h->count = (int32_t)(u + 1);
  }
}

// Sort, rank and emit for one key width.
template <typename KeyT>
int unique_finish(const UniqueView& v, int64_t n, int columns, unsigned key_bits, int32_t* unique_rows,
                  int64_t* to_orig, int64_t* csr_indices, int64_t* csr_offsets, int64_t* to_unique,
                  hipStream_t s) {
  KeyT* keys_a = reinterpret_cast<KeyT*>(v.keys_a);
  KeyT* keys_b = reinterpret_cast<KeyT*>(v.keys_b);
  size_t temp_bytes = v.temp_bytes;
  if (key_bits > 0) {
    if (rocprim::radix_sort_pairs<SortConfig>(v.temp, temp_bytes, keys_a, keys_b, v.idx_a, v.idx_b, (size_t)n, 0u,
                                  key_bits, s) != hipSuccess)
      return WCN_ERR_LAUNCH;
  }
  const KeyT* keys = key_bits > 0 ? keys_b : keys_a;  // all rows equal: nothing to sort
  const uint32_t* idx = key_bits > 0 ? v.idx_b : v.idx_a;
  HeadIterator<KeyT> heads(rocprim::counting_iterator<uint32_t>(0), HeadFlag<KeyT>{keys});
  temp_bytes = v.temp_bytes;
  if (rocprim::inclusive_scan(v.temp, temp_bytes, heads, v.rank, (size_t)n, rocprim::plus<uint32_t>(), s) !=
      hipSuccess)
    return WCN_ERR_LAUNCH;
  hipLaunchKernelGGL(unique_emit<KeyT>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, keys, idx,
                     (const uint32_t*)v.rank, n, columns, v.hdr, unique_rows, to_orig, csr_indices,
                     csr_offsets, to_unique);
  WCN_LAUNCH_CHECK();
  return WCN_OK;
}

// The whole pipeline over a row source.
template <class Src>
int unique_run(const Src& src, int64_t n, int columns, void* workspace, size_t workspace_bytes,
               int32_t* unique_rows, int64_t* to_orig, int64_t* csr_indices, int64_t* csr_offsets,
               int64_t* to_unique, int64_t* num_unique, hipStream_t s) {
  if (workspace_bytes < unique_layout(nullptr, n, nullptr)) return WCN_ERR_WORKSPACE;
  UniqueView v;
  unique_layout(workspace, n, &v);
  const unsigned blocks = (unsigned)((n + 255) / 256);
  hipLaunchKernelGGL(unique_init, dim3(1), dim3(64), 0, s, v.hdr);
  WCN_LAUNCH_CHECK();
  const unsigned big_blocks = (unsigned)((n + 1023) / 1024);
  hipLaunchKernelGGL(unique_bbox<Src>, dim3(big_blocks < 256u ? big_blocks : 256u), dim3(1024), 0, s, src, n,
                     v.hdr);
  WCN_LAUNCH_CHECK();
  // The sort needs the number of key bits on the host: one small read, while the keys are packed.
  if (wcn_read_early_begin(v.hdr, 32, s) != WCN_OK) return WCN_ERR_LAUNCH;
  hipLaunchKernelGGL(unique_pack<Src>, dim3(blocks), dim3(256), 0, s, src, n, (const UniqueHeader*)v.hdr,
                     (void*)v.keys_a, v.idx_a);
  WCN_LAUNCH_CHECK();
  int32_t box[8];
  if (wcn_read_early_end(box, v.hdr, 32, s) != WCN_OK) return WCN_ERR_LAUNCH;
  const KeyLayout L = key_layout(box, box + 4, columns);
  if (L.total > 64u) return WCN_ERR_COORD_RANGE;
  const int rc = L.total <= 32u
                     ? unique_finish<uint32_t>(v, n, columns, L.total, unique_rows, to_orig, csr_indices,
                                               csr_offsets, to_unique, s)
                     : unique_finish<unsigned long long>(v, n, columns, L.total, unique_rows, to_orig,
                                                         csr_indices, csr_offsets, to_unique, s);
  if (rc != WCN_OK) return rc;
  int32_t count = 0;
  if (wcn_read_small(&count, &v.hdr->count, sizeof(count), s) != WCN_OK) return WCN_ERR_LAUNCH;
  *num_unique = count;
  return WCN_OK;
}

// Checks the batch offsets and fills the by-value copy the kernels take.
int make_point_rows(const float* points, int64_t num_points, const int64_t* host_batch_offsets,
                    const int64_t* device_batch_offsets_or_null, int32_t batch_size, double voxel_size,
                    PointRows* src) {
  if (num_points < 0 || num_points >= (1ll << 31) || batch_size < 1 || !host_batch_offsets ||
      !(voxel_size > 0.0))
    return WCN_ERR_INVALID_ARGUMENT;
  if (host_batch_offsets[0] != 0 || host_batch_offsets[batch_size] != num_points)
    return WCN_ERR_INVALID_ARGUMENT;
  for (int b = 0; b < batch_size; ++b)
    if (host_batch_offsets[b + 1] < host_batch_offsets[b]) return WCN_ERR_INVALID_ARGUMENT;
  if (batch_size > WCN_VOXEL_MAX_BATCH && !device_batch_offsets_or_null) return WCN_ERR_INVALID_ARGUMENT;
  if (num_points > 0 && !points) return WCN_ERR_INVALID_ARGUMENT;
  src->points = points;
  src->inv = (float)(1.0 / voxel_size);
  src->batch_size = batch_size;
  src->device_starts = batch_size > WCN_VOXEL_MAX_BATCH ? device_batch_offsets_or_null : nullptr;
  for (int b = 0; b <= WCN_VOXEL_MAX_BATCH; ++b)
    src->starts.start[b] = b <= batch_size && batch_size <= WCN_VOXEL_MAX_BATCH ? host_batch_offsets[b] : 0;
  return WCN_OK;
}

int empty_result(int64_t* csr_offsets, hipStream_t s) {
  if (csr_offsets && hipMemsetAsync(csr_offsets, 0, sizeof(int64_t), s) != hipSuccess) return WCN_ERR_LAUNCH;
  return WCN_OK;
}

}  // namespace

extern "C" {

int wcn_voxel_rows(const float* points, int64_t num_points, const int64_t* host_batch_offsets,
                   const int64_t* device_batch_offsets_or_null, int32_t batch_size, double voxel_size,
                   int32_t* rows, void* stream) {
  PointRows src;
  const int rc = make_point_rows(points, num_points, host_batch_offsets, device_batch_offsets_or_null,
                                 batch_size, voxel_size, &src);
  if (rc != WCN_OK) return rc;
  if (num_points == 0) return WCN_OK;
  if (!rows) return WCN_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(voxel_rows, dim3((unsigned)((num_points + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, src, num_points, (int4*)rows);
  WCN_LAUNCH_CHECK();
  return WCN_OK;
}

int wcn_batch_indexed_rows(const int32_t* coords, int64_t num_rows, int32_t dims,
                           const int64_t* host_batch_offsets, int32_t batch_size, int32_t* rows,
                           void* stream) {
  if (num_rows < 0 || dims < 1 || batch_size < 1 || batch_size > WCN_VOXEL_MAX_BATCH ||
      !host_batch_offsets)
    return WCN_ERR_INVALID_ARGUMENT;
  BatchStarts starts;
  for (int b = 0; b <= batch_size; ++b) {
    starts.start[b] = host_batch_offsets[b];
    if (b > 0 && starts.start[b] < starts.start[b - 1]) return WCN_ERR_INVALID_ARGUMENT;
  }
  for (int b = batch_size + 1; b <= WCN_VOXEL_MAX_BATCH; ++b) starts.start[b] = num_rows;
  if (starts.start[0] != 0 || starts.start[batch_size] != num_rows) return WCN_ERR_INVALID_ARGUMENT;
  if (num_rows == 0) return WCN_OK;
  if (!coords || !rows) return WCN_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(batch_indexed_rows, dim3((unsigned)((num_rows + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, coords, num_rows, (int)dims, starts, (int)batch_size, rows);
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
  if (num_rows == 0) return empty_result(csr_offsets, (hipStream_t)stream);
  if (!rows || !workspace) return WCN_ERR_INVALID_ARGUMENT;
  const IntRows src{rows, (int)columns};
  return unique_run(src, num_rows, (int)columns, workspace, workspace_bytes, unique_rows, to_orig,
                    csr_indices, csr_offsets, to_unique, num_unique, (hipStream_t)stream);
}

int wcn_voxelize_points_csr(const float* points, int64_t num_points, const int64_t* host_batch_offsets,
                            const int64_t* device_batch_offsets_or_null, int32_t batch_size,
                            double voxel_size, void* workspace, size_t workspace_bytes,
                            int32_t* unique_rows, int64_t* to_orig, int64_t* csr_indices,
                            int64_t* csr_offsets, int64_t* to_unique, int64_t* num_unique, void* stream) {
  if (!num_unique) return WCN_ERR_INVALID_ARGUMENT;
  *num_unique = 0;
  PointRows src;
  const int rc = make_point_rows(points, num_points, host_batch_offsets, device_batch_offsets_or_null,
                                 batch_size, voxel_size, &src);
  if (rc != WCN_OK) return rc;
  if (num_points == 0) return empty_result(csr_offsets, (hipStream_t)stream);
  if (!workspace) return WCN_ERR_INVALID_ARGUMENT;
  return unique_run(src, num_points, 4, workspace, workspace_bytes, unique_rows, to_orig, csr_indices,
                    csr_offsets, to_unique, num_unique, (hipStream_t)stream);
}

}  // extern "C"
