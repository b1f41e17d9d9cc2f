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

} // namespace hipq
