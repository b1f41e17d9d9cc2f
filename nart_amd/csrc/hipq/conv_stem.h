// The stem convolutions (conv_stem.hip): 5 to 8 taps fused with the 3x3 / stride 2 / pad 1 max pooling behind them; 3x3 / stride 2.
#pragma once

#include "conv_shared.h"

namespace hipq {

// true when conv_stem_maxpool_kernel serves this convolution (smallc_rowb: bytes of one kernel row in the small-C k layout)
bool conv_stem_maxpool_applies(const ConvArgs &a, int smallc_rowb);
// true when the kernel can also compute the 1x1 convolutions `an` and - not null - `an2` on the pooled rows (from the 64
// pooled channels to a multiple of 64 channels each, 320 together at most)
bool conv_stem_next_applies(const ConvArgs &a, int POH, int POW, const ConvArgs &an, const ConvArgs *an2);
// yp: pooled output, NHWC with channel stride 64, POH x POW pixels per image; an, an2 != nullptr: those convolutions,
// outputs to an->y and an2->y
void launch_conv_stem_maxpool(const ConvArgs &a, uint8_t *yp, int POH, int POW, const ConvArgs *an, const ConvArgs *an2, hipStream_t st);

// true when conv_stem3x3_kernel serves this convolution: 3x3 / stride 2 from at most 4 to at most 32 channels, no pooling
bool conv_stem3x3_applies(const ConvArgs &a, int smallc_rowb);
void launch_conv_stem3x3(const ConvArgs &a, hipStream_t st);

} // namespace hipq
