// 1x1 convolutions that widen the channels, with or without the fused residual add (conv_expand.hip).
#pragma once

#include "conv_shared.h"

namespace hipq {

// true when conv_mfma_expand_kernel serves this launch (a.res set: with the residual add fused in); wherever: every
// layer the kernel can compute, not only those where it measured faster than the kernels it replaces
bool conv_expand_applies(const ConvArgs &a, bool wherever);
void launch_conv_expand(const ConvArgs &a, hipStream_t st);
// chained form: a (with its residual add) followed, in the same kernel, by the 1x1 convolution a2 that reads the sum
// (a2.x is not used: the sum's bytes never come back from memory; a2.y receives a2's output)
bool conv_expand_chain_applies(const ConvArgs &a, const ConvArgs &a2);
void launch_conv_expand_chain(const ConvArgs &a, const ConvArgs &a2, hipStream_t st);

} // namespace hipq
