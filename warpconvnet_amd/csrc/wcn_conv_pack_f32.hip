// The pair-packed contraction for float features (one translation unit per element type, so that
// the instances compile in parallel).
#include "wcn_conv_pack_impl.h"

int wcn_conv_pack_launch_f32(const ConvArgs& a, hipStream_t s) { return launch_typed<float>(a, s); }
