/*
 * C ABI of libwcn_hip.so: the MI355X (gfx950) sparse-convolution forward path.
 *
 * Conventions shared by every entry point
 *   - every pointer argument is a DEVICE pointer owned by the caller unless its name starts with
 *     `host_`; no DEVICE memory is allocated or freed by the library: scratch memory is passed in
 *     as a workspace whose size comes from the matching *_bytes() query.  What the library does
 *     keep, per host thread that calls a *_read_* function, is up to three pinned host buffers of
 *     16 KiB and three events (staging of the few bytes those calls bring to the host), created on
 *     first use and held until wcn_thread_release() or the end of the process; and, per process,
 *     the device-resident array behind wcn_sparse_conv_fwd_static;
 *   - per-thread state crosses calls in three places, all named where they are declared:
 *     wcn_kmap_count arms the result mailbox that the same thread's wcn_kmap_read_result collects,
 *     wcn_kmap_last_table_flags reports on that thread's last read, and
 *     wcn_conv_set_timing_events arms the thread's next contraction call;
 *   - a call that waits for the device (the *_read_* functions) polls with an upper bound of
 *     WCN_WAIT_LIMIT_MS milliseconds (environment variable, default 60000) and returns
 *     WCN_ERR_LAUNCH when the stream has not got there by then;
 *   - `stream` is a hipStream_t passed as void*; all work is enqueued on it and, unless stated,
 *     the call returns without waiting for the device;
 *   - the return value is a status: 0 = success, negative = error (wcn_status_string());
 *   - conditions only the device can see (probe limit of the coordinate table exceeded,
 *     coordinate range too wide to pack, more than 2^31-1 pairs) are recorded in the table
 *     header / result block and surface through wcn_kmap_read_result(), wcn_table_read_status();
 *   - coordinates are rows [batch, x, y, z] of int32; index outputs are int32, bit-exact with the
 *     reference's own results.
 *
 * Reference interfaces replaced (paths relative to the kenomo/WarpConvNet checkout):
 *   hash table     warpconvnet/geometry/coords/search/torch_hashmap.py:102-322 and the CuPy
 *                  RawKernels of warpconvnet/csrc/hashmap_kernels.cu:182-301
 *   kernel map     warpconvnet/geometry/coords/search/torch_discrete.py:80-157,244-337 and
 *                  warpconvnet/csrc/discrete_kernels.cu:183-213,264-370
 *   strided coords warpconvnet/geometry/coords/ops/stride.py:17-54, warpconvnet/utils/unique.py:125-144
 *   contraction    warpconvnet/csrc/warpconvnet_pybind.cpp:1174-1247 (_C.gemm.implicit_gemm,
 *                  _C.gemm.cutlass_gemm_AD_gather_scatter) together with the per-offset Python
 *                  loop of warpconvnet/nn/functional/sparse_conv.py:281-311,358-415,495-544
 */
#ifndef WCN_HIP_H_
#define WCN_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define WCN_OK 0
#define WCN_ERR_INVALID_ARGUMENT (-1)  /* null pointer, bad size, unsupported dtype ...        */
#define WCN_ERR_LAUNCH (-2)            /* the HIP runtime refused a launch or a copy           */
#define WCN_ERR_TABLE_OVERFLOW (-3)    /* probe limit exceeded: rebuild with a larger capacity */
#define WCN_ERR_COORD_RANGE (-4)       /* bounding box of the keys cannot be packed in 63 bits */
#define WCN_ERR_TOO_MANY_PAIRS (-5)    /* kernel map would hold more than 2^31-1 pairs         */
#define WCN_ERR_WORKSPACE (-6)         /* workspace smaller than the *_bytes() query demands   */

#define WCN_DTYPE_F32 0
#define WCN_DTYPE_F16 1
#define WCN_DTYPE_BF16 2

/* Library version (major*10000 + minor*100 + patch). */
int wcn_version(void);

/* Frees the calling thread's pinned staging buffers and events (see the conventions above); they
 * come back on the thread's next *_read_* call.  No counterpart in the reference. */
int wcn_thread_release(void);

/* Text for a status code; replaces gemm_status_to_string (warpconvnet_pybind.cpp:1207-1226). */
const char* wcn_status_string(int status);

/* ---------------------------------------------------------------------------------------------
 * Coordinate table.  Replaces TorchHashTable.insert/search (torch_hashmap.py:102-170,225-300;
 * hashmap_kernels.cu:182-253).  Same observable results: search returns the row index of a key
 * among the inserted keys or -1; among duplicate keys the LOWEST row index is returned (the
 * reference returns whichever thread won a race).
 * ------------------------------------------------------------------------------------------- */

/* Slot count the library would pick for n_keys keys (a power of two). */
int64_t wcn_table_default_capacity(int64_t n_keys);

/* Bytes of workspace a table of n_keys keys and `capacity` slots needs. */
size_t wcn_table_bytes(int64_t n_keys, int64_t capacity);

/* Build the table over keys (n_keys, 4) int32.  `capacity` must be a power of two >= 64. */
int wcn_table_build(const int32_t* keys, int64_t n_keys, void* table, int64_t capacity,
                    void* stream);

/* results[i] = row index of queries[i] (num_queries, 4) among the keys, or -1. */
int wcn_table_query(const void* table, int64_t n_keys, int64_t capacity, const int32_t* queries,
                    int64_t num_queries, int32_t* results, void* stream);

/* Waits for the stream, then returns WCN_OK or the error the build kernels recorded;
 * host_num_blocks (may be NULL) receives the number of occupied slots. */
int wcn_table_read_status(const void* table, int32_t* host_num_blocks, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Kernel map.  Replaces generate_kernel_map's device work (torch_discrete.py:244-337,80-157;
 * discrete_kernels.cu:264-334,183-213) with two calls and one host read in between:
 *
 *   wcn_kmap_count  -> probes the table once; per-offset pair counts, their prefix sums and the
 *                      found rows stay in the workspace (device)
 *   wcn_kmap_read_result (waits; host learns offsets[K+1], allocates in_maps/out_maps of L)
 *   wcn_kmap_fill   -> in_maps[L], out_maps[L] in the reference's order: offsets concatenated
 *                      in k order (k = (i*ky + j)*kz + kk), pairs ascending in output index.
 *                      Reads only the workspace wcn_kmap_count filled for the same arguments.
 *
 * Query coordinate of output m and offset k: out[m] * [1, sx, sy, sz] + (0, i-cx, j-cy, kk-cz)
 * with c = size/2 for odd sizes and 0 for even ones (discrete_kernels.cu:291-314).
 * ------------------------------------------------------------------------------------------- */

size_t wcn_kmap_workspace_bytes(int64_t num_out, int32_t num_offsets);

int wcn_kmap_count(const void* table, int64_t n_keys, int64_t capacity, const int32_t* out_coords,
                   int64_t num_out, const int32_t host_kernel_size[3],
                   const int32_t host_stride[3], void* workspace, void* stream);

/* wcn_kmap_count for dilated and re-centred kernels: replaces the method="offset" branch of
 * generate_kernel_map (torch_discrete.py:428-444: kernel_offsets_from_size :44-77 followed by the
 * offset-table probe _kernel_map_from_offsets :160-241, discrete_kernels.cu:129-180).  Query
 * coordinate of output m and offset (i, j, kk): out[m] * [1, sx, sy, sz] +
 * (0, (i - c0) d0, (j - c1) d1, (kk - c2) d2) with d = host_dilation (>= 1) and c = host_centre
 * (the reference's default: (size - 1) / 2 for odd sizes, 0 for even ones).  The other kernel-map
 * calls (read_result, fill, group_start) are used as for wcn_kmap_count. */
int wcn_kmap_count_dilated(const void* table, int64_t n_keys, int64_t capacity,
                           const int32_t* out_coords, int64_t num_out,
                           const int32_t host_kernel_size[3], const int32_t host_stride[3],
                           const int32_t host_dilation[3], const int32_t host_centre[3],
                           void* workspace, void* stream);

/* Waits for the stream.  host_offsets[K+1] receives the exclusive prefix sums of the per-offset
 * pair counts (host_offsets[K] = L).  Returns the table status or WCN_ERR_TOO_MANY_PAIRS. */
int wcn_kmap_read_result(const void* workspace, int64_t num_out, int32_t num_offsets,
                         int64_t* host_offsets, void* stream);

/* Flags of the table behind the last wcn_kmap_read_result call of this host thread (no device
 * access).  Bit 0: some key was inserted more than once.  Without duplicates, a stride-1 map of
 * a coordinate set onto itself with odd kernel sizes is symmetric (the pairs of offset k with in
 * and out exchanged are the pairs of offset K - 1 - k), which wcn_sparse_conv_dgrad exploits.
 * No counterpart in the reference. */
int32_t wcn_kmap_last_table_flags(void);

/* in_maps / out_maps have room for pair_capacity pairs.  The pass reads the pair count and the
 * table status from the workspace itself and writes nothing if there are more pairs than that or
 * the table reported a problem, so it may be enqueued into buffers of assumed size right after
 * wcn_kmap_count, before wcn_kmap_read_result has told the host the count (the result's copy to
 * the host is enqueued by wcn_kmap_count and therefore runs ahead of this pass); the caller then
 * checks host_offsets[K] <= pair_capacity and calls again with larger buffers if not. */
int wcn_kmap_fill(const void* table, int64_t n_keys, int64_t capacity, const int32_t* out_coords,
                  int64_t num_out, const int32_t host_kernel_size[3], const int32_t host_stride[3],
                  const void* workspace, int64_t pair_capacity, int32_t* in_maps,
                  int32_t* out_maps, void* stream);

/* The map of a coordinate set onto itself (the stride-1 convolution: out_coords are the table's own
 * keys, in the same rows): the same results as wcn_kmap_count / wcn_kmap_fill with out_coords =
 * keys and stride 1, from a probe pass that walks the keys in the table's block order, where
 * neighbours in the list are neighbours in space (the reference probes in row order,
 * discrete_kernels.cu:264-334).  Kernel sizes 3x3x3 and 5x5x5 (wcn_kmap_self_supported says whether
 * a size and key count are taken); the workspace is that of wcn_kmap_workspace_bytes(n_keys, K);
 * wcn_kmap_read_result and wcn_kmap_group_start serve both kinds of call. */
int wcn_kmap_self_supported(const int32_t host_kernel_size[3], int64_t n_keys);
int wcn_kmap_count_self(const void* table, int64_t n_keys, int64_t capacity,
                        const int32_t host_kernel_size[3], void* workspace, void* stream);
int wcn_kmap_fill_self(int64_t n_keys, const int32_t host_kernel_size[3], const void* workspace,
                       int64_t pair_capacity, int32_t* in_maps, int32_t* out_maps, void* stream);

/* Device address, inside a kmap workspace, of the (K, ceil(num_out/64)+1) int32 table
 * group_start[k][g] = number of pairs of offset k whose output row is below 64*g (valid after
 * wcn_kmap_count).  The contraction accepts it to skip its own search. */
const int32_t* wcn_kmap_group_start(const void* workspace, int64_t num_out, int32_t num_offsets);

/* ---------------------------------------------------------------------------------------------
 * Strided output coordinates.  Replaces stride_coords / unique_hashmap (stride.py:17-54,
 * unique.py:125-144): rows of floor(coords / [1,sx,sy,sz]) made unique; the representative of
 * equal rows is the lowest source row; output rows ascend in representative index (which keeps
 * a batch-sorted input batch-sorted).  Division is exact integer floor division.
 * ------------------------------------------------------------------------------------------- */

size_t wcn_stride_unique_workspace_bytes(int64_t n, int64_t capacity);

/* `capacity` is the slot count of the internal coordinate table (wcn_table_default_capacity(n),
 * or larger after WCN_ERR_TABLE_OVERFLOW).  out_coords (>= n rows, 4) and first_index (>= n)
 * are written for the first M rows; M is returned through wcn_stride_unique_read_count. */
int wcn_stride_unique(const int32_t* coords, int64_t n, const int32_t host_stride[3],
                      void* workspace, int64_t capacity, int32_t* out_coords,
                      int32_t* first_index, void* stream);

/* The same result for strides of 1, 2 or 4 per dimension through a table that already exists: the
 * wcn_table_build of `coords` itself (the one the kernel maps of that resolution use).  Such a
 * coarse cell is a sub-box of one 4x4x4 block, so its voxels are bits of one slot and the lowest
 * of their rows represents the cell: one slot look-up and a few loads per row, no table over the
 * coarse rows (which wcn_stride_unique builds from n rows that repeat up to 64-fold).  `workspace`:
 * wcn_stride_unique_cells_workspace_bytes(n_keys) bytes; the result is read with
 * wcn_stride_unique_read_count / _read_bounds as after wcn_stride_unique (same n and capacity).
 * Replaces the same reference path (geometry/coords/ops/stride.py:17-54 + utils/unique.py:125-144). */
size_t wcn_stride_unique_cells_workspace_bytes(int64_t n);

int wcn_stride_unique_cells(const void* table, int64_t n_keys, int64_t capacity, const int32_t* coords,
                            const int32_t host_stride[3], void* workspace, int32_t* out_coords,
                            int32_t* first_index, void* stream);

/* Waits for the stream; host_count receives M.  Returns the table status. */
int wcn_stride_unique_read_count(const void* workspace, int64_t n, int64_t capacity,
                                 int64_t* host_count, void* stream);

/* wcn_stride_unique_read_count plus, in the same read, where the rows of every batch item begin:
 * host_bounds[b], b = 0 .. 1024, is the first of the M output rows whose batch id is at least b.
 * Meaningful for inputs whose batch column does not descend (the rows of a Voxels object), whose
 * output rows then do not descend either.  Replaces the reference's offsets_from_batch_index over
 * the strided rows (geometry/coords/ops/batch_index.py:143-161: a bincount and its own wait). */
int wcn_stride_unique_read_bounds(const void* workspace, int64_t n, int64_t capacity,
                                  int64_t* host_count, int64_t* host_bounds, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Feature contraction.  Replaces, in one launch sequence, the whole per-offset loop of the
 * reference forward (sparse_conv.py:281-311 / :358-415 / :495-544) and the native calls it
 * makes (_C.gemm.implicit_gemm, _C.gemm.cutlass_gemm_AD_gather_scatter):
 *
 *   out[m, :] = bias + sum_k sum_{pairs p of offset k with out_maps[p] == m} X[in_maps[p], :] @ W[k]
 *
 * with fp32 accumulation and ONE rounding to the feature dtype at the end.  `out` is fully
 * written (rows without pairs become bias or zero), never accumulated into.
 * If identity_offset >= 0 that offset is applied as out[m] += X[m] @ W[identity_offset] for
 * every m < min(N, M) and its pairs in the map are ignored, as the reference does
 * (sparse_conv.py:292-302).
 * The map is the reference's: in_maps, out_maps, host_offsets[K+1]; the pairs of one offset must
 * name distinct output rows.  out_maps_ascend = 1 promises that out_maps ascends inside every
 * offset (true for every map wcn_kmap_fill or the reference's generate_kernel_map builds);
 * with 0 (the in/out-swapped map of a transposed convolution) the pairs are re-ordered inside
 * the workspace first.  group_start_or_null: the table wcn_kmap_group_start returns for this
 * map, or NULL to have it derived here (only meaningful with out_maps_ascend = 1).
 * ------------------------------------------------------------------------------------------- */

size_t wcn_conv_workspace_bytes(int64_t num_out, int32_t num_offsets, int32_t c_in, int32_t c_out,
                                int32_t dtype, int64_t num_pairs, int32_t out_maps_ascend);

int wcn_sparse_conv_fwd(const void* features, int64_t num_in, int32_t c_in, int32_t dtype,
                        const void* weight, int32_t weight_dtype, int32_t num_offsets,
                        int32_t c_out, const void* bias_or_null, const int32_t* in_maps,
                        const int32_t* out_maps, const int64_t* host_offsets,
                        int32_t identity_offset, int32_t out_maps_ascend,
                        const int32_t* group_start_or_null, void* out, int64_t num_out,
                        void* workspace, size_t workspace_bytes, void* stream);

/* wcn_sparse_conv_fwd with the elementwise work that follows a convolution in a residual network
 * done in the kernel's epilogue, on the fp32 sums before the one rounding:
 *
 *   out[m, :] = act(bias + sum ... + residual[m, :]),   act = max(., 0) if relu != 0
 *
 * residual_or_null: (num_out, c_out) rows of the feature dtype, not the output buffer itself.
 * Replaces the separate elementwise kernels of the reference's modules around a convolution: the
 * addition of a block's shortcut and nn/modules/activations.py:36-52 (ReLU over the features),
 * which read and write the whole output again.  Everything else as wcn_sparse_conv_fwd. */
int wcn_sparse_conv_fwd_fused(const void* features, int64_t num_in, int32_t c_in, int32_t dtype,
                              const void* weight, int32_t weight_dtype, int32_t num_offsets,
                              int32_t c_out, const void* bias_or_null, const int32_t* in_maps,
                              const int32_t* out_maps, const int64_t* host_offsets,
                              int32_t identity_offset, int32_t out_maps_ascend,
                              const int32_t* group_start_or_null, const void* residual_or_null,
                              int32_t relu, void* out, int64_t num_out, void* workspace,
                              size_t workspace_bytes, void* stream);

/* The forward contraction with the weight's tiles made ahead of the call, for weights that stay
 * the same over many calls (inference, the layers of a network between two optimiser steps).
 * wcn_sparse_conv_fwd turns W (K, c_in, c_out) into zero-padded transposed tiles in the kernels'
 * dtype at the start of every call (one more kernel per call: 4 us of a 30 us layer);
 * wcn_conv_prepare_weight does that once into `prepared` (wcn_conv_prepared_weight_bytes bytes of
 * device memory the caller keeps; to be made again whenever W changes), and
 * wcn_sparse_conv_fwd_prepared enqueues the contraction alone.  It takes maps as the map builder
 * leaves them: out_maps ascending inside every offset, `group_start` (wcn_kmap_group_start) and
 * `device_offsets` = the (K + 1) offsets as int64 in device memory (the first K + 1 words of the
 * map builder's workspace; equal to host_offsets).  residual_or_null / relu as in
 * wcn_sparse_conv_fwd_fused; results identical to that entry's bit for bit.  Replaces the same
 * reference path as wcn_sparse_conv_fwd (sparse_conv.py:495-544 + the native GEMMs it calls, which
 * read the caller's weight as it is and need no such step). */
size_t wcn_conv_prepared_weight_bytes(int32_t num_offsets, int32_t c_in, int32_t c_out, int32_t dtype);

/* Workspace of wcn_sparse_conv_fwd_prepared: 0 (workspace may then be null) unless the problem's
 * shape makes the library split the input channels over workgroups (few output rows, wide rows),
 * then the fp32 partial sums of the slices. */
size_t wcn_conv_prepared_workspace_bytes(int64_t num_out, int32_t num_offsets, int32_t c_in, int32_t c_out,
                                         int32_t dtype);

int wcn_conv_prepare_weight(const void* weight, int32_t weight_dtype, int32_t num_offsets, int32_t c_in,
                            int32_t c_out, int32_t dtype, void* prepared, size_t prepared_bytes,
                            void* stream);

int wcn_sparse_conv_fwd_prepared(const void* features, int64_t num_in, int32_t c_in, int32_t dtype,
                                 const void* prepared_weight, size_t prepared_bytes,
                                 int32_t num_offsets, int32_t c_out, const void* bias_or_null,
                                 const int32_t* in_maps, const int32_t* out_maps,
                                 const int64_t* host_offsets, const int64_t* device_offsets,
                                 int32_t identity_offset, const int32_t* group_start,
                                 const void* residual_or_null, int32_t relu, void* out,
                                 int64_t num_out, void* workspace, size_t workspace_bytes,
                                 void* stream);

/* The forward contraction over a map in which EVERY OUTPUT ROW HAS EXACTLY ONE PAIR
 * (host_offsets[num_offsets] == num_out, which is checked, and no output row twice, which the caller
 * vouches for): the transposed convolution that undoes a strided convolution whose kernel is as large
 * as its stride, where every fine voxel has one parent at one offset.  Nothing is accumulated across
 * pairs, so the lists may be in any order inside an offset (a forward map with its lists exchanged is
 * taken as it is, not re-ordered) and need no group-start table:
 *
 *   out[out_maps[p], :] = act(bias + features[in_maps[p], :] @ W[k(p)] + residual[out_maps[p], :])
 *
 * wcn_conv_single_supported says whether a shape is taken (16-bit features, c_in of 32, 64, 96, 128,
 * 192 or 256, c_out a multiple of 8 up to 256, at most 64 offsets).  weight_is_prepared: 0 = W
 * (K, c_in, c_out) as stored, 2 = W (K, c_out, c_in) (the product is then with W[k]^T: the input
 * gradient of a strided convolution with kernel = stride over voxels without repeats is a map of this
 * kind, dX[in_maps] = dY[out_maps] @ W[k]^T, sparse_conv.py:547-627), both with a workspace of
 * wcn_conv_prepared_weight_bytes bytes; 1 = `weight` is the block wcn_conv_prepare_weight made (no
 * workspace).  Replaces the same reference path as wcn_sparse_conv_fwd (sparse_conv.py:495-544 over
 * the map of sparse_conv.py:1916-1939). */
int wcn_conv_single_supported(int32_t dtype, int32_t c_in, int32_t c_out, int32_t num_offsets);

int wcn_sparse_conv_fwd_single(const void* features, int64_t num_in, int32_t c_in, int32_t dtype,
                               const void* weight, int32_t weight_dtype, int32_t weight_is_prepared,
                               int32_t num_offsets, int32_t c_out, const void* bias_or_null,
                               const int32_t* in_maps, const int32_t* out_maps,
                               const int64_t* host_offsets, const void* residual_or_null, int32_t relu,
                               void* out, int64_t num_out, void* workspace, size_t workspace_bytes,
                               void* stream);

/* wcn_sparse_conv_fwd for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 * Same arguments and results as wcn_sparse_conv_fwd, minus the workspace: the scratch memory is a
 * device-resident array of WCN_CONV_STATIC_SCRATCH_BYTES inside the library (each GPU the library
 * runs on holds it until the process ends).  The call enqueues kernels only: no allocation, no
 * free, no copy command.  It returns WCN_ERR_WORKSPACE when
 * wcn_conv_workspace_bytes(num_out, K, c_in, c_out, dtype, L, out_maps_ascend) exceeds that size
 * and WCN_ERR_INVALID_ARGUMENT for more than 127 offsets (they travel in kernel arguments).
 * Every call on a GPU uses that GPU's one array: calls that overlap on the same GPU (different
 * streams or host threads) race.  The first call on a device looks the array's address up and
 * must therefore be made outside graph capture. */
#define WCN_CONV_STATIC_SCRATCH_BYTES (4u << 20)

int wcn_sparse_conv_fwd_static(const void* features, int64_t num_in, int32_t c_in, int32_t dtype,
                               const void* weight, int32_t weight_dtype, int32_t num_offsets,
                               int32_t c_out, const void* bias_or_null, const int32_t* in_maps,
                               const int32_t* out_maps, const int64_t* host_offsets,
                               int32_t identity_offset, int32_t out_maps_ascend,
                               const int32_t* group_start_or_null, void* out, int64_t num_out,
                               void* stream);

/* Re-orders the pair lists of a map so that out_maps ascends inside every offset, and writes the
 * table group_start[k * (G + 1) + g] = number of pairs of offset k with out_maps < 64 g
 * (G = ceil(num_out / 64); (K, G + 1) int32).  This is what wcn_sparse_conv_fwd does inside its
 * workspace on every call with out_maps_ascend = 0; done once here, the results can be kept with
 * the map and passed with out_maps_ascend = 1 and group_start on every later call (the map of a
 * transposed convolution, or a forward map with its lists exchanged for the input gradient).  The
 * reference keeps such a map as it is and pays nothing for its order because its per-offset GEMMs
 * scatter with atomics (sparse_conv.py:1916-1939 builds the exchanged map; :495-544 uses it).
 * Precondition: at most one pair per (offset, output row), which every kernel map satisfies; of
 * several such pairs in a caller's lists only the one with the lowest input row is kept (and the
 * tail of that offset's range in in_sorted / out_sorted is left unwritten, beyond the counts in
 * group_start).  in_sorted / out_sorted have room for host_offsets[K] pairs.  Kernels only. */
size_t wcn_pairs_sort_workspace_bytes(int64_t num_out, int32_t num_offsets, int64_t num_pairs);

int wcn_pairs_sort_by_out(const int32_t* in_maps, const int32_t* out_maps, const int64_t* host_offsets,
                          int32_t num_offsets, int64_t num_out, int32_t* in_sorted,
                          int32_t* out_sorted, int32_t* group_start, void* workspace,
                          size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Gradients of the contraction.  Replace the per-offset loops of the reference backward
 * (sparse_conv.py:314-355 explicit, :418-492 implicit, :547-627 CUTLASS) and the native calls
 * they make (_C.gemm.cutlass_gemm_AD_gather_scatter with the maps exchanged,
 * _C.gemm.cutlass_gemm_trAB_gather, _C.gemm.split_k_implicit_gemm):
 *
 *   grad_in[n, :]  = sum_k sum_{pairs p of offset k with in_maps[p] == n} grad_out[out_maps[p], :] @ W[k]^T
 *   grad_weight[k] = sum_{pairs p of offset k} X[in_maps[p], :]^T (x) grad_out[out_maps[p], :]
 *
 * fp32 accumulation, one rounding; both results are fully written and bitwise reproducible.
 * With identity_offset >= 0 that offset is taken over the rows m < min(N, M) with in = out = m and
 * its pairs in the map are ignored (sparse_conv.py:332-336).
 *
 * wcn_sparse_conv_dgrad is the forward contraction over the map with in and out exchanged; its
 * workspace is wcn_conv_workspace_bytes(num_in, K, c_out, c_in, dtype, num_pairs, ascend) with
 * ascend = map_is_symmetric || in_maps_ascend.  map_is_symmetric = 1 promises that the pairs of
 * offset k with in and out exchanged are exactly the pairs of offset K - 1 - k (a stride-1 map
 * of one coordinate set onto itself): the map is then used as it stands, group_start included.
 * Otherwise in_maps_ascend says whether in_maps ascends inside every offset (true for the map of
 * a transposed convolution, which is a forward map with its lists exchanged); if not the pairs
 * are re-ordered inside the workspace.  `weight` is the forward weight (K, c_in, c_out).
 * ------------------------------------------------------------------------------------------- */

int wcn_sparse_conv_dgrad(const void* grad_out, int64_t num_out, int32_t c_out, int32_t dtype,
                          const void* weight, int32_t weight_dtype, int32_t num_offsets,
                          int32_t c_in, const int32_t* in_maps, const int32_t* out_maps,
                          const int64_t* host_offsets, int32_t identity_offset,
                          int32_t map_is_symmetric, int32_t in_maps_ascend,
                          const int32_t* group_start_or_null, void* grad_in, int64_t num_in,
                          void* workspace, size_t workspace_bytes, void* stream);

/* identity_rows = min(N, M) if identity_offset >= 0, else 0. */
size_t wcn_conv_wgrad_workspace_bytes(int32_t num_offsets, int32_t c_in, int32_t c_out,
                                      int64_t num_pairs, int64_t identity_rows);

/* grad_weight is (K, c_in, c_out) in weight_dtype (the feature dtype or fp32). */
int wcn_sparse_conv_wgrad(const void* features, int64_t num_in, int32_t c_in, const void* grad_out,
                          int64_t num_out, int32_t c_out, int32_t dtype, const int32_t* in_maps,
                          const int32_t* out_maps, const int64_t* host_offsets,
                          int32_t num_offsets, int32_t identity_offset, void* grad_weight,
                          int32_t weight_dtype, void* workspace, size_t workspace_bytes,
                          void* stream);

/* ---------------------------------------------------------------------------------------------
 * Pooling over a kernel map.  Replaces the torch sort + torch_scatter.segment_csr reduction of
 * sparse_reduce (warpconvnet/nn/functional/sparse_pool.py:84-104, ops/reductions.py:38-56) and
 * its autograd:
 *
 *   out[m, :] = reduce over the pairs p with out_maps[p] == m of X[in_maps[p], :]
 *
 * mode 0 = sum, 1 = mean, 2 = max, 3 = min; output rows without pairs become 0.  fp32
 * accumulation, one rounding.  The pairs are first grouped by row: wcn_map_rows_build(gathered_rows = in_maps,
 * grouping_rows = out_maps, ..., num_rows = M) for the forward pass, and with the two lists
 * exchanged (num_rows = N) for the gradient, each into a workspace of
 * wcn_map_rows_workspace_bytes(num_rows, K, L) bytes that the pooling calls then read.
 * For max / min, argmax (M, C) int32 receives the input row that supplied each extremum (-1 where
 * there is none) and must be passed to the gradient.  rows_by_out may be NULL in the gradient of
 * sum, max and min.
 * ------------------------------------------------------------------------------------------- */

size_t wcn_map_rows_workspace_bytes(int64_t num_rows, int32_t num_offsets, int64_t num_pairs);

int wcn_map_rows_build(const int32_t* gathered_rows, const int32_t* grouping_rows,
                       const int64_t* host_offsets, int32_t num_offsets, int64_t num_rows,
                       void* workspace, size_t workspace_bytes, void* stream);

int wcn_sparse_pool_fwd(const void* features, int64_t num_in, int32_t channels, int32_t dtype,
                        const void* rows_by_out, int64_t num_out, int32_t num_offsets,
                        int64_t num_pairs, int32_t mode, void* out, int32_t* argmax_or_null,
                        void* stream);

int wcn_sparse_pool_bwd(const void* grad_out, int64_t num_out, int32_t channels, int32_t dtype,
                        const void* rows_by_in, const void* rows_by_out, int64_t num_in,
                        int32_t num_offsets, int64_t num_pairs, int32_t mode,
                        const int32_t* argmax_or_null, void* grad_in, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Depthwise convolution over a kernel map.  Replaces the per-offset loops of
 * warpconvnet/nn/functional/sparse_conv_depth.py:151-231 (explicit) / :233-345 (implicit, native
 * _C.fma.implicit_fma / implicit_reduction calls):
 *
 *   out[m, c]         = sum_k sum_{pairs p of offset k with out_maps[p] == m} X[in_maps[p], c] * W[k, c]
 *   grad_in[n, c]     = the same over the exchanged map with grad_out in place of X
 *   grad_weight[k, c] = sum_{pairs p of offset k} X[in_maps[p], c] * grad_out[out_maps[p], c]
 *
 * weight is (K, C) in the feature dtype or fp32.  identity_offset >= 0: that offset is taken over
 * the rows m < min(N, M) with in = out = m and its pairs are ignored (sparse_conv_depth.py:163-165).
 * Forward and input gradient read a rows form built by wcn_map_rows_build (by output row, resp.
 * with the lists exchanged, by input row).
 * ------------------------------------------------------------------------------------------- */

int wcn_sparse_depthwise_fwd(const void* features, int64_t num_in, int32_t channels, int32_t dtype,
                             const void* weight, int32_t weight_dtype, const void* rows_by_out,
                             int64_t num_out, int32_t num_offsets, int64_t num_pairs,
                             int32_t identity_offset, void* out, void* stream);

size_t wcn_depthwise_wgrad_workspace_bytes(int32_t num_offsets, int32_t channels, int64_t num_pairs,
                                           int64_t identity_rows);

int wcn_sparse_depthwise_wgrad(const void* features, int64_t num_in, const void* grad_out,
                               int64_t num_out, int32_t channels, int32_t dtype,
                               const int32_t* in_maps, const int32_t* out_maps,
                               const int64_t* host_offsets, int32_t num_offsets,
                               int32_t identity_offset, void* grad_weight, int32_t weight_dtype,
                               void* workspace, size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Morton (Z-order) codes of voxel coordinates.  Replaces the CuPy launch of
 * assign_order_discrete_20bit_kernel_4points (warpconvnet/csrc/morton_code.cu:60-84) behind
 * morton_code() (geometry/coords/ops/serialization.py:181-254):
 *
 *   codes[i] = spread(c[a2] - o[a2]) << 2 | spread(c[a1] - o[a1]) << 1 | spread(c[a0] - o[a0])
 *
 * c = the three spatial columns of row i starting at column first_spatial of a (n, columns) int32
 * array, o = device_origin[3] (the per-column minimum, on the device), (a0, a1, a2) = host_axes
 * (a permutation of 0, 1, 2: the ordering's axis order), spread() = two zero bits between
 * consecutive bits, 21 bits kept.
 * ------------------------------------------------------------------------------------------- */

int wcn_morton_codes(const int32_t* coords, int64_t n, int32_t columns, int32_t first_spatial,
                     const int32_t* device_origin, const int32_t host_axes[3], int64_t* codes,
                     void* stream);

/* ---------------------------------------------------------------------------------------------
 * Voxelisation front-end: points -> voxel rows -> sorted distinct voxels with the CSR grouping of
 * the points, and reductions over those groups.
 *
 * wcn_voxel_rows replaces `torch.floor(batched_points / voxel_size).int()` +
 * `batch_index_from_offset` + `torch.cat` (warpconvnet/geometry/coords/ops/voxel.py:92-95,136-141):
 * rows[i] = [batch item of point i, floor(x * r), floor(y * r), floor(z * r)] with
 * r = (float)(1.0 / voxel_size), which is how torch divides a float tensor by a host scalar on the
 * device.  points (N, 3) fp32; host_batch_offsets (B + 1) int64 on the host; for more than
 * WCN_VOXEL_MAX_BATCH batch items the same offsets must also be given in device memory.
 *
 * wcn_unique_rows_csr replaces unique_torch (warpconvnet/utils/unique.py:57-109), i.e.
 * torch.unique(x, dim=0, sorted=True, return_inverse=True, return_counts=True), the stable argsort
 * of the inverse, the cumulative sum of the counts and the scatter that picks a representative:
 *   unique_rows (M, columns) int32  distinct rows in ascending lexicographic order
 *   to_orig     (N) int64           unique_rows[to_orig[i]] == rows[i]
 *   csr_indices (N) int64           rows grouped by distinct row, ascending row index inside a group
 *   csr_offsets (M + 1) int64       group u is csr_indices[csr_offsets[u] .. csr_offsets[u + 1])
 *   to_unique   (M) int64           lowest row index of each group (the reference's choice is whichever
 *                                   write of a scatter with repeated indices lands last)
 * Every output may be NULL; output buffers must hold N (N + 1 for csr_offsets) entries, the count M
 * is returned through *num_unique.  rows (N, columns) int32, 1 <= columns <= 4; the per-column
 * ranges must pack into 64 bits together (WCN_ERR_COORD_RANGE otherwise).  The call waits for the
 * stream twice (key width, then M).
 *
 * wcn_segment_reduce replaces `row_reduction(features[to_csr_indices], to_csr_offsets, reduction)`
 * (warpconvnet/ops/reductions.py:36-72, torch_scatter.segment_csr; called from
 * warpconvnet/nn/functional/point_pool.py:298-302): out[u] = sum / mean / max / min (mode 0..3, as
 * for wcn_sparse_pool_fwd) over e in [segment_offsets[u], segment_offsets[u + 1]) of
 * features[indices[e]] (features[e] when indices is NULL); num_entries is the length of the entry
 * list (offsets beyond it are cut to it); empty segments give 0.  argmax (M, C)
 * int64 receives the feature row behind each extremum.  wcn_segment_reduce_bwd is its gradient for
 * disjoint segments: segment_of_row (N) names each feature row's segment (out of range = none).
 * ------------------------------------------------------------------------------------------- */

#define WCN_VOXEL_MAX_BATCH 64

int wcn_voxel_rows(const float* points, int64_t num_points, const int64_t* host_batch_offsets,
                   const int64_t* device_batch_offsets_or_null, int32_t batch_size, double voxel_size,
                   int32_t* rows, void* stream);

/* wcn_batch_indexed_rows replaces `torch.cat([batch_index.unsqueeze(1), batched_coords], dim=1)`
 * over `batch_index_from_offset(offsets)` (warpconvnet/geometry/coords/ops/batch_index.py:22-36 and
 * :110-117): rows (n, dims + 1) int32 receives [b, coords[i][0..dims)] with b the batch item whose
 * range [host_batch_offsets[b], host_batch_offsets[b + 1]) holds i.  The offsets (batch_size + 1
 * values, the first 0, the last n, not descending) are read on the host and travel with the launch;
 * batch_size is at most WCN_VOXEL_MAX_BATCH. */
int wcn_batch_indexed_rows(const int32_t* coords, int64_t num_rows, int32_t dims,
                           const int64_t* host_batch_offsets, int32_t batch_size, int32_t* rows,
                           void* stream);

size_t wcn_unique_rows_workspace_bytes(int64_t num_rows);

int wcn_unique_rows_csr(const int32_t* rows, int64_t num_rows, int32_t columns, void* workspace,
                        size_t workspace_bytes, int32_t* unique_rows, int64_t* to_orig,
                        int64_t* csr_indices, int64_t* csr_offsets, int64_t* to_unique,
                        int64_t* num_unique, void* stream);

/* wcn_voxel_rows + wcn_unique_rows_csr over 4-column rows in one call, without storing the rows:
 * the whole of voxel_downsample_csr_mapping (warpconvnet/geometry/coords/ops/voxel.py:51-109) up to
 * its batch offsets.  Same outputs and workspace as wcn_unique_rows_csr (num_rows = num_points). */
int wcn_voxelize_points_csr(const float* points, int64_t num_points, const int64_t* host_batch_offsets,
                            const int64_t* device_batch_offsets_or_null, int32_t batch_size,
                            double voxel_size, void* workspace, size_t workspace_bytes,
                            int32_t* unique_rows, int64_t* to_orig, int64_t* csr_indices,
                            int64_t* csr_offsets, int64_t* to_unique, int64_t* num_unique, void* stream);

int wcn_segment_reduce(const void* features, int64_t num_in, int32_t channels, int32_t dtype,
                       const int64_t* segment_offsets, const int64_t* indices_or_null,
                       int64_t num_entries, int64_t num_segments, int32_t mode, void* out,
                       int64_t* argmax_or_null, void* stream);

int wcn_segment_reduce_bwd(const void* grad_out, int64_t num_segments, int32_t channels, int32_t dtype,
                           const int64_t* segment_offsets, const int64_t* segment_of_row, int64_t num_in,
                           int32_t mode, const int64_t* argmax_or_null, void* grad_in, void* stream);

/* Name of the contraction kernel the last wcn_sparse_conv_fwd / _dgrad call of this host thread
 * enqueued, template arguments included, as a profiler prints it ("" before the first call).  A
 * measurement aid with no counterpart in the reference: the benchmark reports the kernel that ran. */
const char* wcn_conv_last_kernel(void);

/* Measurement hook (no counterpart in the reference, which times whole calls with CUDA events:
 * warpconvnet/utils/timer.py:41-60).  The two hipEvent_t handles are recorded on the call's
 * stream immediately before and after the contraction kernel of the NEXT wcn_sparse_conv_fwd
 * call made by this host thread, so that hipEventElapsedTime gives that kernel's duration
 * alone; the hook then disarms itself.  Pass NULLs to disarm. */
int wcn_conv_set_timing_events(void* start_event, void* stop_event);

/* ---------------------------------------------------------------------------------------------
 * Measurement probe (no counterpart in the reference; not on the product path).  Gathers the rows
 * features[in_maps[p]] (row_bytes = 32, 64 or 128 each; in_maps entries must lie in [0, num_rows))
 * for all num_pairs pairs, 16 rows per wave and request as the contraction does, and does nothing
 * with them: its run time is what the memory system needs for the gather alone.  `sink` is one
 * device word the kernel may write.  Used by `bench.py --gather-floor`.
 * ------------------------------------------------------------------------------------------- */
int wcn_probe_gather_rows(const void* features, int64_t num_rows, int32_t row_bytes,
                          const int32_t* in_maps, int64_t num_pairs, void* sink, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* WCN_HIP_H_ */
