// Host-only pieces of the hipq library: error state, the fixed-point scale decomposition, layout rule.
#include <cmath>
#include <cstdarg>
#include <cstdio>

#include <algorithm>

#include "common.h"

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

bool hipq::make_add_params(float ia0, int iz0, float ia1, int iz1, float oa, int oz, int obits, AddParams *p)
{
    int s0, s1;
    hipq_quant_scale(ia0 / oa, 23, &p->m0, &s0); // add.c:119-124
    hipq_quant_scale(ia1 / oa, 23, &p->m1, &s1);
    p->sh = std::min(s0, s1) - 1;
    p->s0 = s0 - p->sh, p->s1 = s1 - p->sh;
    p->z0 = iz0, p->z1 = iz1, p->oz = oz, p->hi = (1 << obits) - 1;
    if (!valid_shift(p->sh) || !valid_shift(p->s0) || !valid_shift(p->s1))
        return false;
    p->fast = p->sh <= 22 && p->s0 <= 30 && p->s1 <= 30 && p->m0 < (1u << 23) && p->m1 < (1u << 23);
    p->c0 = p->c1 = p->cadd = 0;
    if (p->fast) {
        p->c0 = (1 << (p->s0 - 1)) - iz0 * (int32_t)p->m0;
        p->c1 = (1 << (p->s1 - 1)) - iz1 * (int32_t)p->m1;
        p->cadd = (1 << (p->sh - 1)) + (oz << p->sh);
    }
    return true;
}

extern "C" int hipq_channel_stride(int C) { return C <= 4 ? 4 : (C + 15) / 16 * 16; }

// A power of two 2^k: m = 2^(32 - k), s = 0.  Otherwise s = floor(log2 d) and m = ceil(2^(32 + s) / d): m fits 32 bits
// because d > 2^s, and the round-up error e = m * d - 2^(32 + s) is below d < 2^(s + 1), so x * e < 2^(32 + s) for
// x < 2^31, which is the condition for the quotient to be exact.  d == 1 has no such m: m = 0 means "x itself".
extern "C" int hipq_div_magic(uint32_t d, uint32_t *m, int *s)
{
    if (d == 0 || m == nullptr || s == nullptr)
        return -1;
    *m = 0, *s = 0;
    if (d == 1)
        return 0;
    int lg = 31;
    while (!(d >> lg))
        lg--;
    if ((d & (d - 1)) == 0) {
        *m = 1u << (32 - lg);
        return 0;
    }
    *s = lg;
    *m = (uint32_t)(((1ull << (32 + lg)) + d - 1) / d);
    return 0;
}
