// Host-only pieces of the hipq library: error state, the fixed-point scale decomposition, layout rule.
#include <cmath>
#include <cstdarg>
#include <cstdio>

#include "hipq.h"

namespace hipq {

static thread_local char g_err[512] = "";

int fail(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return 1;
}

void clear_error() { g_err[0] = 0; }

} // namespace hipq

extern "C" int hipq_abi_version(void) { return HIPQ_ABI_VERSION; }

extern "C" const char *hipq_last_error(void) { return hipq::g_err; }

// get_quant_scale / get_quant_scale_int16 / get_quant_scale_int32 of the reference
// (art/modules/quant/include/art/quant/quant_helper.h:60-118): the scale is normalised into [0.5, 1)
// by exact fp32 halving / doubling, the multiplier is its mantissa truncated to bits-1 bits.
extern "C" void hipq_quant_scale(float x, int bits, uint32_t *mult, int *shift)
{
    int s = 0;
    *mult = 0;
    *shift = 0;
    if (std::fabs((double)x) < 1e-10 || !(x > 0.0f) || std::isinf(x))
        return; // zero like the reference; negative / infinite scales never terminate there
    while (x >= 1.0f) {
        x /= 2;
        s -= 1;
    }
    while (x < 0.5f) {
        x *= 2;
        s += 1;
    }
    *mult = (uint32_t)(x * (float)(1ll << (bits - 1)));
    *shift = s + bits - 1;
}

extern "C" int hipq_channel_stride(int C) { return C <= 4 ? 4 : (C + 15) / 16 * 16; }
