// Depthwise 3x3 convolutions (stride 1 or 2, weight zero point 128): a thread walks down the image and keeps the
// partial sums of the output rows its current input row contributes to (conv_dw.hip).
#pragma once

#include "conv_shared.h"

namespace hipq {

bool conv_dw_slide_applies(const ConvArgs &a);
void launch_conv_dw_slide(const ConvArgs &a, hipStream_t st);

} // namespace hipq
