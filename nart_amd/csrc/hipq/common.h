// Shared host/device helpers of the hipq kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "hipq.h"

namespace hipq {

// ---- error reporting --------------------------------------------------------------------------
int fail(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
void clear_error();

#define HIPQ_CHECK_HIP(expr)                                                              \
    do {                                                                                  \
        hipError_t e_ = (expr);                                                           \
        if (e_ != hipSuccess)                                                             \
            return ::hipq::fail("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_),    \
                                __FILE__, __LINE__);                                      \
    } while (0)

#define HIPQ_REQUIRE(cond, ...)               \
    do {                                      \
        if (!(cond))                          \
            return ::hipq::fail(__VA_ARGS__); \
    } while (0)

// Every launch is followed by this: a launch that could not be queued is an error, never silent.
static inline int launch_status(const char *what)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess)
        return fail("launch of %s failed: %s", what, hipGetErrorString(e));
    return 0;
}

// ---- fixed-point requantisation (quant_helper.h:31-58 of the reference) -------------------------
struct Requant {
    uint32_t mult;
    int32_t shift; // 1..62
    int32_t zp;
    int32_t hi; // (1 << bits) - 1
};

// floor((x + 2^(s-1)) / 2^s): what the reference's rshift_rn computes for s >= 1.
__host__ __device__ static inline int64_t rshift_rn(int64_t x, int s)
{
    return (x + ((int64_t)1 << (s - 1))) >> s;
}

__host__ __device__ static inline int32_t sat_hi(int32_t v, int32_t hi)
{
    return v > hi ? hi : (v < 0 ? 0 : v);
}

// conv / ip epilogue: int32 accumulator -> saturated output value
__host__ __device__ static inline int32_t requant_acc(int32_t acc, const Requant &q)
{
    int64_t r = rshift_rn((int64_t)acc * (int64_t)q.mult, q.shift) + q.zp;
    return sat_hi((int32_t)r, q.hi);
}

static inline int valid_shift(int s) { return s >= 1 && s <= 62; }

// ---- quantized two-input add (op_quant_add_run, art/modules/quant/src/op/add.c:83-148) ------------------
// Shared by the stand-alone add kernel and by the convolution epilogue that fuses a residual add.
//   t = rrn((int32)(m0*(x0-z0)), s0) + rrn((int32)(m1*(x1-z1)), s1);   y = sat(rrn(t, sh) + oz)
// The operation is symmetric in its inputs (the reference's swap by scale only orders them).
// Fast form, valid when every shift is small enough for 32-bit arithmetic (`fast`): with
// c = 2^(s-1) - z*m the two terms are (x*m + c) >> s (|m*(x-z)| < 2^30, so nothing wraps), and with
// cadd = 2^(sh-1) + oz*2^sh the result is (t + cadd) >> sh before the clamp.
struct AddParams {
    uint32_t m0, m1;    // 22-bit multipliers (get_quant_scale(alpha_i / oalpha, 23))
    int32_t s0, s1, sh; // s0 - sh, s1 - sh, sh
    int32_t z0, z1, oz, hi;
    int32_t c0, c1, cadd;
    int32_t fast;
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ static inline uint32_t add_one_generic(uint32_t x0, uint32_t x1, const AddParams &p)
{
    const int32_t i0 = (int32_t)x0 - p.z0, i1 = (int32_t)x1 - p.z1;
    const int32_t p0 = (int32_t)(p.m0 * (uint32_t)i0), p1 = (int32_t)(p.m1 * (uint32_t)i1);
    const int32_t t = (int32_t)(rshift_rn(p0, p.s0) + rshift_rn(p1, p.s1));
    return (uint32_t)sat_hi((int32_t)(rshift_rn(t, p.sh) + p.oz), p.hi);
}

// (v >> s) saturated to [0, 255] for four values, packed into one dword (v0 in the low byte); s is wave-uniform, 0..31.
// gfx950's v_ashr_pk_u8_i32 shifts two values, saturates them and writes ONE half of its destination - op_sel[3] picks
// the high half - leaving the other half as it was.  It issues at half rate (measured), so the pair costs four issue
// slots against the nine of four shifts, two 16-bit packs, two saturating byte packs and a permute.
__device__ static __forceinline__ uint32_t ashr_sat_u8x4(int32_t v0, int32_t v1, int32_t v2, int32_t v3, int32_t s)
{
    uint32_t o;
    asm("v_ashr_pk_u8_i32 %0, %1, %2, %3" : "=v"(o) : "v"(v0), "v"(v1), "s"(s));
    asm("v_ashr_pk_u8_i32 %0, %1, %2, %3 op_sel:[0,0,0,1]" : "+v"(o) : "v"(v2), "v"(v3), "s"(s));
    return o;
}

template <bool FAST>
__device__ static __forceinline__ uint32_t add_dword(uint32_t a, uint32_t b, const AddParams &p)
{
    if (FAST) {
        // operands fit 24 bits: v_mad_i32_i24 is a full-rate instruction.  The upper clamp moves in front of the last
        // shift ((hi + 1) * 2^sh - 1 is the largest value that shifts to hi; sh <= 22), the lower one is the pack's.
        const int32_t phi = ((p.hi + 1) << p.sh) - 1;
        int32_t v[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const uint32_t x0 = (a >> (8 * e)) & 255, x1 = (b >> (8 * e)) & 255;
            const int32_t t0 = __mul24((int)x0, (int)p.m0) + p.c0, t1 = __mul24((int)x1, (int)p.m1) + p.c1;
            v[e] = min(((t0 >> p.s0) + (t1 >> p.s1)) + p.cadd, phi);
        }
        return ashr_sat_u8x4(v[0], v[1], v[2], v[3], p.sh);
    }
    uint32_t o = 0;
#pragma unroll
    for (int e = 0; e < 4; e++)
        o |= add_one_generic((a >> (8 * e)) & 255, (b >> (8 * e)) & 255, p) << (8 * e);
    return o;
}

template <bool FAST>
__device__ static __forceinline__ u32x4 add_16(u32x4 a, u32x4 b, const AddParams &p)
{
    u32x4 y;
#pragma unroll
    for (int d = 0; d < 4; d++)
        y[d] = add_dword<FAST>(a[d], b[d], p);
    return y;
}

// byte-wise unsigned maximum of two packed dwords: bytes 0 and 2 are compared as the 16-bit halves of x & 0x00ff00ff,
// bytes 1 and 3 in place as the halves of x & 0xff00ff00 (their low bytes are zero on both sides), two v_pk_max_u16
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
__device__ static inline uint32_t max_u8x4(uint32_t a, uint32_t b)
{
    const uint32_t E = 0x00ff00ffu;
    const u16x2 lo = __builtin_elementwise_max(__builtin_bit_cast(u16x2, a & E), __builtin_bit_cast(u16x2, b & E));
    const u16x2 hi = __builtin_elementwise_max(__builtin_bit_cast(u16x2, a & ~E), __builtin_bit_cast(u16x2, b & ~E));
    return __builtin_bit_cast(uint32_t, lo) | __builtin_bit_cast(uint32_t, hi);
}

// Fills *p from the operator's settings; returns false if a scale is outside the fixed-point range.
bool make_add_params(float ia0, int iz0, float ia1, int iz1, float oa, int oz, int obits, AddParams *p);

} // namespace hipq
