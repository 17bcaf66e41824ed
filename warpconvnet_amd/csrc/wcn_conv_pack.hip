// Pair-packed feature contraction: which problems it takes, and the launch by element type (the
// kernel itself is in wcn_conv_pack_impl.h, instantiated in wcn_conv_pack_{f16,bf16,f32}.hip).
#include "wcn_common.h"
#include "wcn_conv_args.h"

int wcn_conv_pack_launch_f16(const ConvArgs& a, hipStream_t s);
int wcn_conv_pack_launch_bf16(const ConvArgs& a, hipStream_t s);
int wcn_conv_pack_launch_f32(const ConvArgs& a, hipStream_t s);

bool wcn_conv_pack_takes(const ConvArgs& a, int dtype) {
  const int ck = dtype == WCN_DTYPE_F32 ? 32 : 64;
  if (!a.vec_in || a.split || a.c_out_pad > WCN_PACK_MAX_BIAS) return false;
  if (a.c_in_pad == ck) return a.K <= 128;  // rows of one slice
  // rows of up to four slices: a phase per slice and offset, and a step counts the phases it skips in 8 bits
  const int slices = a.c_in_pad / ck;
  return a.c_in_pad % ck == 0 && slices <= 4 && a.c_in > a.c_in_pad - ck && a.K <= 64 && a.K * slices <= 255;
}

int wcn_conv_pack_launch(const ConvArgs& a, int dtype, hipStream_t s) {
  switch (dtype) {
    case WCN_DTYPE_F32: return wcn_conv_pack_launch_f32(a, s);
    case WCN_DTYPE_F16: return wcn_conv_pack_launch_f16(a, s);
    default: return wcn_conv_pack_launch_bf16(a, s);
  }
}
