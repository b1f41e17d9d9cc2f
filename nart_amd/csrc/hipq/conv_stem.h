// The stem convolution fused with its 3x3 / stride 2 / pad 1 max pooling (conv_stem.hip).
#pragma once

#include "conv_shared.h"

namespace hipq {

// true when conv_stem_maxpool_kernel serves this convolution (smallc_rowb: bytes of one kernel row in the small-C k layout)
bool conv_stem_maxpool_applies(const ConvArgs &a, int smallc_rowb);
// yp: pooled output, NHWC with channel stride 64, POH x POW pixels per image
void launch_conv_stem_maxpool(const ConvArgs &a, uint8_t *yp, int POH, int POW, hipStream_t st);

} // namespace hipq
