// The pair-packed contraction for __bf16 features (one translation unit per element type, so that
// the instances compile in parallel).
#include "wcn_conv_pack_impl.h"

int wcn_conv_pack_launch_bf16(const ConvArgs& a, hipStream_t s) { return launch_typed<__bf16>(a, s); }
