// A whole identity bottleneck block - 1x1 reduction, 3x3, 1x1 widening, residual add - in one kernel (conv_block.hip).
#pragma once

#include "conv_shared.h"

namespace hipq {

// a1: the 1x1 convolution that reads the block's input x (a1.x), a2: the 3x3 / stride 1 / pad 1 convolution, a3: the
// widening 1x1 convolution with the add's parameters in a3.addq / a3.res_first; the residual is x itself and the sum goes
// to a3.y.  true when conv_bottleneck_kernel computes this chain.
// an != nullptr: the 1x1 convolution that reads the sum, to twice the middle channels (the first layer of the next stage), is
// computed in the kernel as well (output to an->y).
bool conv_block_applies(const ConvArgs &a1, const ConvArgs &a2, const ConvArgs &a3, const ConvArgs *an);
void launch_conv_block(const ConvArgs &a1, const ConvArgs &a2, const ConvArgs &a3, const ConvArgs *an, hipStream_t st);
// true where the one kernel measured faster than the launches it replaces
bool conv_block_preferred(const ConvArgs &a1);

// The chain cut one layer later: a2 (3x3 / stride 1 / pad 1, reads a2.x), a3 (the widening 1x1 with the residual a3.res and
// the add's parameters, sum to a3.y) and - an != nullptr - the 1x1 convolution that reads the sum (output to an->y).
bool conv_block_tail_applies(const ConvArgs &a2, const ConvArgs &a3, const ConvArgs *an);
void launch_conv_block_tail(const ConvArgs &a2, const ConvArgs &a3, const ConvArgs *an, hipStream_t st);
bool conv_block_tail_preferred(const ConvArgs &a2, bool chained);

} // namespace hipq
