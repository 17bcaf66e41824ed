// Arguments shared by the contraction kernels of wcn_conv.hip and wcn_conv_pack.hip.
#ifndef WCN_CONV_ARGS_H_
#define WCN_CONV_ARGS_H_
#include "wcn_common.h"

#include <type_traits>

struct ConvArgs {
  const void* X;
  const void* Wt;
  const void* zeros;           // 1 KiB of zeros (source of loads that have nothing to fetch)
  const void* bias;            // same dtype as X, or null
  const int32_t* in_maps;      // pair lists; inside every offset out_maps ascends
  const int32_t* out_maps;
  const int64_t* offsets;      // (K + 1), device
  const int32_t* group_start;  // (K, G + 1): pairs of offset k below output row 64 * g
  void* out;
  int64_t num_in, num_out, G;
  int64_t num_pairs;           // all offsets together (known on the host)
  int32_t K, c_in, c_out, c_in_pad, c_out_pad, identity;
  int32_t vec_in;   // feature rows are 16-byte aligned and a whole number of 16-byte vectors
  int32_t vec_out;  // same for output rows
  int32_t flat_in;  // c_in is a multiple of the staged row and the feature matrix is below 4 GiB
  // Few output tiles and several slices of input channels (small maps with wide features): the
  // slices go to different workgroups (blockIdx.z), each writes its fp32 sums to
  // partial[slice][row][c_out_pad] and conv_split_reduce adds them in slice order.
  int32_t split;
  float* partial;
  // What the epilogue does besides bias and rounding (wcn_sparse_conv_fwd_fused): add a row of
  // `residual` (num_out x c_out, the element type of the features) and / or clamp at zero, both
  // on the fp32 sums before the one rounding.
  const void* residual;
  int32_t relu;
  int32_t vec_res;  // rows of `residual` are 16-byte aligned and a whole number of 16-byte vectors
};


// The pair-packed contraction (wcn_conv_pack*.hip): whether it takes a problem, and its launch.
constexpr int WCN_PACK_MAX_BIAS = 1024;  // output channels (padded) whose bias fits the kernel's LDS copy
bool wcn_conv_pack_takes(const ConvArgs& a, int dtype);
int wcn_conv_pack_launch(const ConvArgs& a, int dtype, hipStream_t stream);

// The output-stationary contraction for wide rows (wcn_conv_dense.hip): whether it takes a problem,
// and its launch.
bool wcn_conv_dense_takes(const ConvArgs& a, int dtype);
int wcn_conv_dense_launch(const ConvArgs& a, int dtype, hipStream_t stream);

// The contraction for maps with exactly one pair per output row (wcn_conv_single.hip): whether it
// takes a problem's shape, and its launch over pair lists in any order (`host_offsets`: the K + 1
// offsets; X, Wt, bias, residual, relu, out, the lists and the sizes are read from `a`).
constexpr int WCN_SINGLE_MAX_OFFSETS = 64;
struct WcnSingleTiles {  // tiles of 256 pairs of one offset, in offset order
  int32_t first_tile[WCN_SINGLE_MAX_OFFSETS + 1];
  int32_t first_pair[WCN_SINGLE_MAX_OFFSETS + 1];
  int32_t total;
};
bool wcn_conv_single_takes(int dtype, int c_in, int c_out, int num_offsets);
int wcn_conv_single_launch(const ConvArgs& a, int dtype, const int64_t* host_offsets, hipStream_t stream);

#endif  // WCN_CONV_ARGS_H_

// The contraction for narrow layers (wcn_conv_group.hip): a wave per group of 64 output rows.
bool wcn_conv_group_takes(const ConvArgs& a, int dtype);
int wcn_conv_group_launch(const ConvArgs& a, int dtype, hipStream_t stream);

// The contraction kernel a launcher has just enqueued, as the profiler would print its name
// ("conv_fwd_pack<f16, 512, 11, 4, 2, true, false, false>"): kept per host thread for
// wcn_conv_last_kernel (a measurement aid: reports name what ran, not what was expected to run).
void wcn_conv_note_kernel(const char* format, ...);
template <typename T>
inline const char* wcn_type_text() {
  return sizeof(T) == 4 ? "float" : (std::is_same<T, _Float16>::value ? "f16" : "bf16");
}
