// 1x1 and 3x3 convolutions over few pixels whose waves load their weight operands straight from memory (conv_wreg.hip).
#pragma once

#include "conv_shared.h"

namespace hipq {

// true when conv_wreg_kernel computes this launch (a.res set: with the residual add in its epilogue)
bool conv_wreg_applies(const ConvArgs &a);
void launch_conv_wreg(const ConvArgs &a, hipStream_t st);

} // namespace hipq
