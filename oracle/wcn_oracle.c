/*
 * CPU oracle for the sparse-convolution forward path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain scalar C, the algorithms of the reference
 * (kenomo/WarpConvNet v0.3.6) for the path
 *     coordinate hash table -> kernel map -> explicit gather-GEMM-scatter.
 * It is the checker the HIP kernels are compared with.  Nothing in the
 * product (the warpconvnet_amd package, its HIP library) may link, import or
 * call it: only tests/, the smoke check and the cpu_baseline leg of the
 * benchmark do.
 *
 * Each function cites the reference file:line it follows (paths relative to
 * the reference checkout root).  How each function is pinned independently
 * of this restatement is listed in oracle/README.md; tests/test_oracle_*.py
 * holds the pins.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>

#define WCN_HASH_FNV1A 0
#define WCN_HASH_CITY 1
#define WCN_HASH_MURMUR 2

/* ---- hash functions: warpconvnet/csrc/hashmap_kernels.cu:8-118 ---------------------------- */

static uint32_t murmur_scramble(uint32_t k) {
  k *= 0xCC9E2D51u;
  k = (k << 15) | (k >> 17);
  k *= 0x1B873593u;
  return k;
}

/* Raw 32-bit hash of an integer vector, before the reduction to a slot. */
uint32_t wcn_oracle_hash32(const int32_t* key, int key_dim, int method) {
  uint32_t h;
  int i;
  if (method == WCN_HASH_FNV1A) { /* hashmap_kernels.cu:32-36,54-62 */
    h = 2166136261u;
    for (i = 0; i < key_dim; ++i) {
      h ^= (uint32_t)key[i];
      h *= 16777619u;
    }
  } else if (method == WCN_HASH_CITY) { /* hashmap_kernels.cu:38-46,64-71 */
    h = 0;
    for (i = 0; i < key_dim; ++i) {
      h += (uint32_t)key[i] * 0x9E3779B9u;
      h ^= h >> 16;
      h *= 0x85EBCA6Bu;
      h ^= h >> 13;
      h *= 0xC2B2AE35u;
      h ^= h >> 16;
    }
  } else { /* murmur3-32: hashmap_kernels.cu:8-30,73-83 */
    h = 0x9747B28Cu;
    for (i = 0; i < key_dim; ++i) {
      h ^= murmur_scramble((uint32_t)key[i]);
      h = (h << 13) | (h >> 19);
      h = h * 5u + 0xE6546B64u;
    }
    h ^= (uint32_t)(key_dim * 4);
    h ^= h >> 16;
    h *= 0x85EBCA6Bu;
    h ^= h >> 13;
    h *= 0xC2B2AE35u;
    h ^= h >> 16;
  }
  return h;
}

/* Signed modulo reduction used for every hash: hashmap_kernels.cu:60-61. */
int wcn_oracle_hash_slot(const int32_t* key, int key_dim, int capacity, int method) {
  int32_t s = (int32_t)wcn_oracle_hash32(key, key_dim, method);
  return ((s % capacity) + capacity) % capacity;
}

/* ---- open-addressing table (capacity, 2) int32: hashmap_kernels.cu:182-234 ---------------- */

void wcn_oracle_table_init(int32_t* kvs, int capacity) { /* :182-188 */
  int i;
  for (i = 0; i < 2 * capacity; ++i) kvs[i] = -1;
}

/*
 * Insert keys 0..n-1 in ascending index order (hashmap_kernels.cu:191-234).  The reference runs
 * one GPU thread per key and the claim of a slot is an atomicCAS race; serial ascending order is
 * one legal outcome of that race (the lowest index probes first).  As in the reference there is no
 * key-equality test on insert, so duplicate keys occupy separate slots.  Returns the number of
 * keys dropped because no slot was free (the reference drops them silently).
 */
int wcn_oracle_table_insert(int32_t* kvs, int capacity, const int32_t* keys, int n, int key_dim,
                            int method) {
  int dropped = 0, idx;
  for (idx = 0; idx < n; ++idx) {
    int slot = wcn_oracle_hash_slot(keys + (size_t)idx * key_dim, key_dim, capacity, method);
    int initial = slot, attempts = 0, placed = 0;
    while (attempts < capacity) {
      if (kvs[2 * slot] == -1) {
        kvs[2 * slot] = slot;
        kvs[2 * slot + 1] = idx;
        placed = 1;
        break;
      }
      slot = (slot + 1) % capacity;
      if (slot == initial) break;
      attempts++;
    }
    if (!placed) dropped++;
  }
  return dropped;
}

/* One probe sequence: hashmap_kernels.cu:133-177. */
static int table_search_one(const int32_t* kvs, int capacity, const int32_t* vector_keys,
                            const int32_t* q, int key_dim, int method) {
  int slot = wcn_oracle_hash_slot(q, key_dim, capacity, method);
  int initial = slot, attempts = 0;
  while (attempts < capacity) {
    int32_t marker = kvs[2 * slot];
    if (marker == -1) return -1;
    int32_t vi = kvs[2 * slot + 1];
    if (vi != -1 && memcmp(vector_keys + (size_t)vi * key_dim, q, sizeof(int32_t) * key_dim) == 0)
      return vi;
    slot = (slot + 1) % capacity;
    if (slot == initial) return -1;
    attempts++;
  }
  return -1;
}

/* search_kernel_*: hashmap_kernels.cu:237-253. */
void wcn_oracle_table_search(const int32_t* kvs, int capacity, const int32_t* vector_keys,
                             int key_dim, const int32_t* queries, int64_t num_queries, int method,
                             int32_t* results) {
  int64_t i;
  for (i = 0; i < num_queries; ++i)
    results[i] =
        table_search_one(kvs, capacity, vector_keys, queries + i * key_dim, key_dim, method);
}

/* ---- kernel offsets: geometry/coords/search/torch_discrete.py:44-77 ------------------------ */
/* (K,4) table: batch column 0, last spatial dimension fastest, centre (s-1)/2 if odd else 0.   */
void wcn_oracle_kernel_offsets(const int32_t ksize[3], const int32_t dilation[3],
                               int32_t* offsets /* K*4 */) {
  int i, j, k, r = 0;
  int cx = (ksize[0] % 2) ? (ksize[0] - 1) / 2 : 0;
  int cy = (ksize[1] % 2) ? (ksize[1] - 1) / 2 : 0;
  int cz = (ksize[2] % 2) ? (ksize[2] - 1) / 2 : 0;
  for (i = 0; i < ksize[0]; ++i)
    for (j = 0; j < ksize[1]; ++j)
      for (k = 0; k < ksize[2]; ++k, ++r) {
        offsets[4 * r + 0] = 0;
        offsets[4 * r + 1] = (i - cx) * dilation[0];
        offsets[4 * r + 2] = (j - cy) * dilation[1];
        offsets[4 * r + 3] = (k - cz) * dilation[2];
      }
}

/* ---- kernel map: torch_discrete.py:365-466,244-337 + csrc/discrete_kernels.cu:264-334 ------ */
/*
 * found[k*M + m] = index of (out[m] * [1,s] + offset_k) among the input coordinates, or -1.
 * Builds the reference's own table (capacity max(16, 2N): torch_hashmap.py:219) with the chosen
 * hash and probes it the way kernel_map_size_4d_* does: k decoded z-fastest
 * (discrete_kernels.cu:302-304), centre = size/2 if odd else 0 (:291-294), batch column unchanged
 * (:309).  Returns 0, or -1 if memory could not be obtained.
 */
int wcn_oracle_kernel_map_found(const int32_t* in_coords, int n_in, const int32_t* out_coords,
                                int64_t n_out, const int32_t ksize[3], const int32_t stride[3],
                                int method, int32_t* found /* K * n_out */) {
  int capacity = n_in * 2 > 16 ? n_in * 2 : 16;
  int32_t* kvs = (int32_t*)malloc(sizeof(int32_t) * 2 * (size_t)capacity);
  int K = ksize[0] * ksize[1] * ksize[2], kk;
  int64_t m;
  int cx, cy, cz;
  if (!kvs) return -1;
  wcn_oracle_table_init(kvs, capacity);
  wcn_oracle_table_insert(kvs, capacity, in_coords, n_in, 4, method);
  cx = (ksize[0] % 2) ? ksize[0] / 2 : 0;
  cy = (ksize[1] % 2) ? ksize[1] / 2 : 0;
  cz = (ksize[2] % 2) ? ksize[2] / 2 : 0;
  for (kk = 0; kk < K; ++kk) {
    int k = kk % ksize[2];
    int j = (kk / ksize[2]) % ksize[1];
    int i = kk / (ksize[2] * ksize[1]);
    for (m = 0; m < n_out; ++m) {
      int32_t q[4];
      /* torch_discrete.py:407-416: out coords are multiplied by [1, sx, sy, sz] first */
      q[0] = out_coords[4 * m + 0];
      q[1] = out_coords[4 * m + 1] * stride[0] + i - cx;
      q[2] = out_coords[4 * m + 2] * stride[1] + j - cy;
      q[3] = out_coords[4 * m + 3] * stride[2] + k - cz;
      found[(int64_t)kk * n_out + m] = table_search_one(kvs, capacity, in_coords, q, 4, method);
    }
  }
  free(kvs);
  return 0;
}

/*
 * The method="offset" probe: torch_discrete.py:428-444 (offsets from kernel_offsets_from_size :44-77)
 * + _kernel_map_from_offsets :160-241 + discrete_kernels.cu:129-180: found[k*M + m] = index of
 * (out[m] * [1,s] + offsets[k]) among the input coordinates, or -1; `offsets` is (K, 4) with a zero
 * batch column.  The reference's own call of this path is broken (its wrapper passes an argument
 * the callee does not take), so this restates the intent its kernel and offset table spell out.
 */
int wcn_oracle_kernel_map_offsets(const int32_t* in_coords, int n_in, const int32_t* out_coords,
                                  int64_t n_out, const int32_t* offsets, int K,
                                  const int32_t stride[3], int method, int32_t* found /* K * n_out */) {
  int capacity = n_in * 2 > 16 ? n_in * 2 : 16;
  int32_t* kvs = (int32_t*)malloc(sizeof(int32_t) * 2 * (size_t)capacity);
  int kk;
  int64_t m;
  if (!kvs) return -1;
  wcn_oracle_table_init(kvs, capacity);
  wcn_oracle_table_insert(kvs, capacity, in_coords, n_in, 4, method);
  for (kk = 0; kk < K; ++kk) {
    for (m = 0; m < n_out; ++m) {
      int32_t q[4];
      q[0] = out_coords[4 * m + 0] + offsets[4 * kk + 0];
      q[1] = out_coords[4 * m + 1] * stride[0] + offsets[4 * kk + 1];
      q[2] = out_coords[4 * m + 2] * stride[1] + offsets[4 * kk + 2];
      q[3] = out_coords[4 * m + 3] * stride[2] + offsets[4 * kk + 3];
      found[(int64_t)kk * n_out + m] = table_search_one(kvs, capacity, in_coords, q, 4, method);
    }
  }
  free(kvs);
  return 0;
}

/*
 * Row-wise stream compaction: torch_discrete.py:80-157 + discrete_kernels.cu:183-213.
 * offsets[K+1] (exclusive prefix of hits per offset row), and for every hit in row k at column m,
 * in ascending m: in_maps[pos] = found, out_maps[pos] = m.  Pass in_maps == NULL to get only the
 * offsets.  Returns the total number of pairs.
 */
int64_t wcn_oracle_compact_found(const int32_t* found, int K, int64_t M, int64_t* offsets,
                                 int32_t* in_maps, int32_t* out_maps) {
  int k;
  int64_t m, pos = 0;
  offsets[0] = 0;
  for (k = 0; k < K; ++k) {
    for (m = 0; m < M; ++m) {
      int32_t f = found[(int64_t)k * M + m];
      if (f >= 0) {
        if (in_maps) {
          in_maps[pos] = f;
          out_maps[pos] = (int32_t)m;
        }
        pos++;
      }
    }
    offsets[k + 1] = pos;
  }
  return pos;
}

/* ---- strided output coordinates: geometry/coords/ops/stride.py:17-54 ----------------------- */
/*
 * out = unique rows of floor(coords / [1,sx,sy,sz]); the division is a float32 true division
 * followed by floor and a cast back to int32 (stride.py:41), which is what is restated here (it
 * equals integer floor division for |coord| < 2^24).  Uniqueness follows utils/unique.py:125-144
 * (table of capacity 2N, torch_hashmap.py:302-322): the representative of a group of equal rows
 * is the row found by the table search, which under serial ascending insertion is the lowest
 * index; representatives are listed in ascending index order (torch.unique sorts them) and then
 * ordered by batch index (stride.py:44-48; the reference's argsort is not stable, this oracle's
 * is, so ties keep ascending index order).  first_index[r] receives the representative's row in
 * `coords`.  offsets[B+1] is the bincount-cumsum of the batch column
 * (geometry/coords/ops/batch_index.py:143-161).  Returns M, or -1 on allocation failure.
 */
int64_t wcn_oracle_stride_coords(const int32_t* coords, int n, const int32_t stride[3],
                                 int num_batches, int32_t* out_coords /* up to n*4 */,
                                 int32_t* first_index /* up to n */,
                                 int64_t* offsets /* num_batches+1 */) {
  int32_t* disc = (int32_t*)malloc(sizeof(int32_t) * 4 * (size_t)(n > 0 ? n : 1));
  int capacity = 2 * n > 1 ? 2 * n : 1;
  int32_t* kvs = (int32_t*)malloc(sizeof(int32_t) * 2 * (size_t)capacity);
  int32_t* rep = (int32_t*)malloc(sizeof(int32_t) * (size_t)(n > 0 ? n : 1));
  unsigned char* is_rep = (unsigned char*)calloc((size_t)(n > 0 ? n : 1), 1);
  int i, b;
  int64_t M = 0;
  if (!disc || !kvs || !rep || !is_rep) return -1;
  for (i = 0; i < n; ++i) {
    disc[4 * i + 0] = (int32_t)floorf((float)coords[4 * i + 0] / 1.0f);
    disc[4 * i + 1] = (int32_t)floorf((float)coords[4 * i + 1] / (float)stride[0]);
    disc[4 * i + 2] = (int32_t)floorf((float)coords[4 * i + 2] / (float)stride[1]);
    disc[4 * i + 3] = (int32_t)floorf((float)coords[4 * i + 3] / (float)stride[2]);
  }
  wcn_oracle_table_init(kvs, capacity);
  wcn_oracle_table_insert(kvs, capacity, disc, n, 4, WCN_HASH_CITY);
  wcn_oracle_table_search(kvs, capacity, disc, 4, disc, n, WCN_HASH_CITY, rep);
  for (i = 0; i < n; ++i)
    if (rep[i] >= 0) is_rep[rep[i]] = 1;
  /* ascending representative index, then a stable partition by batch index */
  for (b = 0; b <= num_batches; ++b) offsets[b] = 0;
  for (i = 0; i < n; ++i)
    if (is_rep[i]) {
      int bb = disc[4 * i];
      if (bb >= 0 && bb < num_batches) offsets[bb + 1]++;
    }
  for (b = 0; b < num_batches; ++b) offsets[b + 1] += offsets[b];
  {
    int64_t* cursor = (int64_t*)malloc(sizeof(int64_t) * (size_t)(num_batches + 1));
    if (!cursor) return -1;
    memcpy(cursor, offsets, sizeof(int64_t) * (size_t)(num_batches + 1));
    for (i = 0; i < n; ++i)
      if (is_rep[i]) {
        int bb = disc[4 * i];
        if (bb >= 0 && bb < num_batches) {
          int64_t p = cursor[bb]++;
          memcpy(out_coords + 4 * p, disc + 4 * i, sizeof(int32_t) * 4);
          first_index[p] = i;
          M++;
        }
      }
    free(cursor);
  }
  free(disc);
  free(kvs);
  free(rep);
  free(is_rep);
  return M;
}

/* ---- explicit gather-GEMM-scatter forward: nn/functional/sparse_conv.py:281-311 ------------- */
/*
 * out = X @ W[iden] if iden >= 0 else zeros(M, Cout); then for every non-empty offset k != iden,
 * in k order: out[out_map_k] += X[in_map_k] @ W[k].  All arithmetic in double so that it serves as
 * the high-precision yardstick; the per-offset rounding of the reference's low-precision runs is
 * reproduced by the torch restatement in oracle/explicit_conv.py instead.
 * X: (N, Cin), W: (K, Cin, Cout), out: (M, Cout), all row-major doubles.
 */
void wcn_oracle_explicit_conv_f64(const double* X, int64_t N, const double* W, int K, int Cin,
                                  int Cout, const int32_t* in_maps, const int32_t* out_maps,
                                  const int64_t* offsets, int iden, int64_t M, double* out) {
  int64_t m, p;
  int k, c, d;
  memset(out, 0, sizeof(double) * (size_t)M * Cout);
  if (iden >= 0) {
    const double* Wk = W + (size_t)iden * Cin * Cout;
    int64_t rows = N < M ? N : M;
    for (m = 0; m < rows; ++m)
      for (c = 0; c < Cin; ++c) {
        double x = X[m * Cin + c];
        for (d = 0; d < Cout; ++d) out[m * Cout + d] += x * Wk[c * Cout + d];
      }
  }
  for (k = 0; k < K; ++k) {
    const double* Wk = W + (size_t)k * Cin * Cout;
    if (k == iden) continue;
    for (p = offsets[k]; p < offsets[k + 1]; ++p) {
      const double* x = X + (int64_t)in_maps[p] * Cin;
      double* o = out + (int64_t)out_maps[p] * Cout;
      for (c = 0; c < Cin; ++c) {
        double xv = x[c];
        for (d = 0; d < Cout; ++d) o[d] += xv * Wk[c * Cout + d];
      }
    }
  }
}
