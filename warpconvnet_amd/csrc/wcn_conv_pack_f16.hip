// The pair-packed contraction for _Float16 features (one translation unit per element type, so that
// the instances compile in parallel).
#include "wcn_conv_pack_impl.h"

int wcn_conv_pack_launch_f16(const ConvArgs& a, hipStream_t s) { return launch_typed<_Float16>(a, s); }
