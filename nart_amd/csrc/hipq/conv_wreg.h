// 1x1 and 3x3 convolutions over few pixels whose waves load their weight operands straight from memory (conv_wreg.hip).
#pragma once

#include "conv_shared.h"

namespace hipq {

// true when conv_wreg_kernel computes this launch (a.res set: with the residual add in its epilogue)
bool conv_wreg_applies(const ConvArgs &a);
void launch_conv_wreg(const ConvArgs &a, hipStream_t st);
// y = add(a(a.x), b(b.x)): a the widening 1x1 / stride 1 convolution of a block (add parameters in a.addq / a.res_first, a.res any
// non-null pointer, sum to a.y), b its projection shortcut (1x1, stride 1 or 2, twice a's input channels, same output channels)
bool conv_wreg_dual_applies(const ConvArgs &a, const ConvArgs &b);
void launch_conv_wreg_dual(const ConvArgs &a, const ConvArgs &b, hipStream_t st);

} // namespace hipq
