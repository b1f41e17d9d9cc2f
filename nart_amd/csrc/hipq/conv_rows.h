// 3x3 / stride 1 / pad 1 convolutions with 64 input and output channels: input rows resident in LDS, weights in
// registers (conv_rows.hip).
#pragma once

#include "conv_shared.h"

namespace hipq {

bool conv_rows_applies(const ConvArgs &a);
void launch_conv_rows(const ConvArgs &a, hipStream_t st);

} // namespace hipq
