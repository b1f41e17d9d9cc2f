// Memory-bound uint8 operators for gfx950: add, n-ary eltwise, relu, pooling, quantize, dequantize,
// layout conversion.  Each is a grid-stride wavefront kernel moving 128 bits per lane per access so that
// a wave touches 1 KiB of contiguous HBM per instruction; the integer arithmetic is the reference's
// fixed-point arithmetic, statement for statement (files under art/modules/quant/src/op/).
#include <algorithm>
#include <cmath>
#include <cstring>

#include "common.h"

namespace hipq {

static inline unsigned grid_for(size_t work_items, int per_block = 256)
{
    const size_t b = (work_items + per_block - 1) / per_block;
    return (unsigned)std::min<size_t>(std::max<size_t>(b, 1), 256 * 16);
}

// ---- add (add.c:83-148); arithmetic in common.h ------------------------------------------------
struct AddArgs {
    const uint8_t *a, *b;
    uint8_t *y;
    size_t count;
    AddParams q;
};

template <bool FAST>
__global__ __launch_bounds__(256) void add_u8_kernel(const AddArgs p)
{
    const size_t nvec = p.count / 16;
    const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x, nthr = (size_t)gridDim.x * blockDim.x;
    for (size_t i = tid; i < nvec; i += nthr) {
        const u32x4 va = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p.a) + i);
        const u32x4 vb = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p.b) + i);
        reinterpret_cast<u32x4 *>(p.y)[i] = add_16<FAST>(va, vb, p.q);
    }
    for (size_t i = nvec * 16 + tid; i < p.count; i += nthr)
        p.y[i] = (uint8_t)add_one_generic(p.a[i], p.b[i], p.q);
}

// ---- n-ary eltwise (eltwise.c:137-271) ---------------------------------------------------------
struct EltArgs {
    const uint8_t *in[HIPQ_MAX_ELTWISE_INPUTS];
    uint32_t mult[HIPQ_MAX_ELTWISE_INPUTS];
    int shift[HIPQ_MAX_ELTWISE_INPUTS]; // shift[n] - s0
    int zp[HIPQ_MAX_ELTWISE_INPUTS];
    int cfast[HIPQ_MAX_ELTWISE_INPUTS]; // fast form: 2^(shift-1) - zp * mult
    int n_in, s0, oz, hi, is_max, fast, cadd;
    uint8_t *y;
    size_t count;
};

// one partial term: input byte x of input n
template <bool FAST>
__device__ static inline int32_t eltwise_term(uint32_t x, int n, const EltArgs &p)
{
    if (FAST) // |mult * (x - zp)| < 2^30 and shift <= 30: 32-bit arithmetic is exact
        return (__mul24((int)x, (int)p.mult[n]) + p.cfast[n]) >> p.shift[n];
    return (int32_t)rshift_rn((int32_t)((uint32_t)((int32_t)x - p.zp[n]) * p.mult[n]), p.shift[n]);
}

template <bool FAST>
__device__ static inline uint32_t eltwise_finish(int32_t t, const EltArgs &p)
{
    if (FAST)
        return (uint32_t)sat_hi((t + p.cadd) >> p.s0, p.hi);
    return (uint32_t)sat_hi((int32_t)(rshift_rn(t, p.s0) + p.oz), p.hi);
}

// NIN inputs and the operation known at compile time (register arrays stay in registers), 16 bytes per thread and input
template <int NIN, bool FAST, bool IS_MAX>
__global__ __launch_bounds__(256) void eltwise_u8_kernel(const EltArgs p)
{
    const size_t nvec = p.count / 16;
    const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x, nthr = (size_t)gridDim.x * blockDim.x;
    for (size_t i = tid; i < nvec; i += nthr) {
        u32x4 v[NIN];
#pragma unroll
        for (int n = 0; n < NIN; n++)
            v[n] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p.in[n]) + i);
        u32x4 o;
#pragma unroll
        for (int d = 0; d < 4; d++) {
            uint32_t w = 0;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                int32_t t = IS_MAX ? -1 : 0; // the reference's running maximum starts at 0xffffffff (eltwise.c:198)
#pragma unroll
                for (int n = 0; n < NIN; n++) {
                    const int32_t r = eltwise_term<FAST>((v[n][d] >> (8 * e)) & 255, n, p);
                    t = IS_MAX ? (t < r ? r : t) : (int32_t)((uint32_t)t + (uint32_t)r);
                }
                w |= eltwise_finish<FAST>(t, p) << (8 * e);
            }
            o[d] = w;
        }
        reinterpret_cast<u32x4 *>(p.y)[i] = o;
    }
    for (size_t i = nvec * 16 + tid; i < p.count; i += nthr) {
        int32_t t = IS_MAX ? -1 : 0;
#pragma unroll
        for (int n = 0; n < NIN; n++) {
            const int32_t r = eltwise_term<false>(p.in[n][i], n, p);
            t = IS_MAX ? (t < r ? r : t) : (int32_t)((uint32_t)t + (uint32_t)r);
        }
        p.y[i] = (uint8_t)eltwise_finish<false>(t, p);
    }
}

// any number of inputs: one byte position at a time per input, no register arrays
__global__ __launch_bounds__(256) void eltwise_u8_generic_kernel(const EltArgs p)
{
    const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x, nthr = (size_t)gridDim.x * blockDim.x;
    for (size_t i = tid; i < p.count; i += nthr) {
        int32_t t = p.is_max ? -1 : 0;
        for (int n = 0; n < p.n_in; n++) {
            const int32_t r = eltwise_term<false>(p.in[n][i], n, p);
            t = p.is_max ? (t < r ? r : t) : (int32_t)((uint32_t)t + (uint32_t)r);
        }
        p.y[i] = (uint8_t)eltwise_finish<false>(t, p);
    }
}

// ---- relu (relu.c:76-115) ----------------------------------------------------------------------
struct ReluArgs {
    const uint8_t *x;
    uint8_t *y;
    size_t count;
    uint32_t mult;
    int shift, iz, oz, hi;
};

__device__ static inline uint32_t relu_one(uint32_t x, const ReluArgs &p)
{
    const int32_t v = (int32_t)x >= p.iz ? (int32_t)x : p.iz;
    const uint32_t pr = (uint32_t)(v - p.iz) * p.mult; // evaluated unsigned, widened without sign
    return (uint32_t)sat_hi((int32_t)(rshift_rn((int64_t)pr, p.shift) + p.oz), p.hi);
}

__global__ __launch_bounds__(256) void relu_u8_kernel(const ReluArgs p)
{
    const size_t nvec = p.count / 16;
    const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x, nthr = (size_t)gridDim.x * blockDim.x;
    for (size_t i = tid; i < nvec; i += nthr) {
        const u32x4 v = reinterpret_cast<const u32x4 *>(p.x)[i];
        u32x4 o;
#pragma unroll
        for (int d = 0; d < 4; d++) {
            uint32_t w = 0;
#pragma unroll
            for (int e = 0; e < 4; e++)
                w |= relu_one((v[d] >> (8 * e)) & 255, p) << (8 * e);
            o[d] = w;
        }
        reinterpret_cast<u32x4 *>(p.y)[i] = o;
    }
    for (size_t i = nvec * 16 + tid; i < p.count; i += nthr)
        p.y[i] = (uint8_t)relu_one(p.x[i], p);
}

// ---- pooling (pool.c:96-249), NHWC: one thread = 4 channels of one output pixel ------------------
struct PoolArgs {
    const uint8_t *x;
    uint8_t *y;
    int N, H, W, OH, OW, cs, kh, kw, ph, pw, sh, sw;
    int is_avg, iz, oz, hi;
    float ia_over_oa; // fp32 ialpha / oalpha, as the reference forms it before dividing by the pool size
    uint32_t mult;    // max pooling: uint16 multiplier
    int shift;
};

// get_quant_scale(x, 16) evaluated on the device with the same fp32 operations (quant_helper.h:98-118)
__device__ static inline void quant_scale16(float x, uint32_t &mult, int &shift)
{
    int s = 0;
    mult = 0;
    shift = 0;
    if (fabs((double)x) < 1e-10)
        return;
    while (x >= 1.0f) {
        x /= 2;
        s -= 1;
    }
    while (x < 0.5f) {
        x *= 2;
        s += 1;
    }
    mult = (uint32_t)(x * 32768.0f);
    shift = s + 15;
}

__global__ __launch_bounds__(256) void pool_u8_kernel(const PoolArgs p)
{
    const int cq = p.cs >> 2;
    const size_t total = (size_t)p.N * p.OH * p.OW * cq;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        const size_t m = idx / cq;
        const int c0 = (int)(idx - m * cq) * 4;
        const int n = (int)(m / ((size_t)p.OH * p.OW)), rem = (int)(m - (size_t)n * p.OH * p.OW);
        const int oh = rem / p.OW, ow = rem - oh * p.OW;
        int hs = oh * p.sh - p.ph, ws = ow * p.sw - p.pw;
        uint32_t o = 0;
        if (!p.is_avg) {
            const int he = min(hs + p.kh, p.H), we = min(ws + p.kw, p.W);
            hs = max(hs, 0), ws = max(ws, 0);
            uint32_t mx[4] = {0, 0, 0, 0};
            for (int i = hs; i < he; i++)
                for (int j = ws; j < we; j++) {
                    const uint32_t v = *reinterpret_cast<const uint32_t *>(
                        p.x + ((size_t)(n * p.H + i) * p.W + j) * p.cs + c0);
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        mx[e] = max(mx[e], (v >> (8 * e)) & 255);
                }
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int32_t pr = (int32_t)p.mult * ((int32_t)mx[e] - p.iz);
                o |= (uint32_t)sat_hi((int32_t)(rshift_rn(pr, p.shift) + p.oz), p.hi) << (8 * e);
            }
        } else {
            int he = min(hs + p.kh, p.H + p.ph), we = min(ws + p.kw, p.W + p.pw);
            const uint32_t pool_size = (uint32_t)((he - hs) * (we - ws)); // padding counts (pool.c:211-213)
            uint32_t mult;
            int shift;
            quant_scale16(p.ia_over_oa / (float)pool_size, mult, shift);
            hs = max(hs, 0), ws = max(ws, 0), he = min(he, p.H), we = min(we, p.W);
            int32_t sum[4] = {0, 0, 0, 0};
            for (int i = hs; i < he; i++)
                for (int j = ws; j < we; j++) {
                    const uint32_t v = *reinterpret_cast<const uint32_t *>(
                        p.x + ((size_t)(n * p.H + i) * p.W + j) * p.cs + c0);
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        sum[e] += (int32_t)((v >> (8 * e)) & 255) - p.iz;
                }
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int32_t pr = (int32_t)(mult * (uint32_t)sum[e]);
                o |= (uint32_t)sat_hi((int32_t)(rshift_rn(pr, shift) + p.oz), p.hi) << (8 * e);
            }
        }
        *reinterpret_cast<uint32_t *>(p.y + m * p.cs + c0) = o;
    }
}

// Max pooling with a channel stride that is a multiple of 16: a thread owns 16 channels of one output pixel (128-bit
// loads, one 128-bit store), 32-bit index arithmetic.  The byte-wise maxima are taken on the packed dwords.
__global__ __launch_bounds__(256) void pool_max16_u8_kernel(const PoolArgs p, double inv_c16, double inv_ow, double inv_oh)
{
    const int c16n = p.cs >> 4;
    const int total = p.N * p.OH * p.OW * c16n; // the host guarantees 31 bits
    const int radd = (1 << (p.shift - 1)) + (p.oz << p.shift);
    const int phi = ((p.hi + 1) << p.shift) - 1; // the largest value that the shift takes to hi
    const bool same = p.mult == (1u << p.shift) && p.iz == p.oz && p.hi == 255;
    // work-groups go to the 8 XCDs in turn: renumbered so that each XCD works on a contiguous eighth of the (image-major)
    // index space, the eighth whose pixels its convolution tiles read (the grid is a multiple of 8)
    const int L = (int)(blockIdx.x & 7) * (int)(gridDim.x >> 3) + (int)(blockIdx.x >> 3);
    for (int idx = L * 256 + threadIdx.x; idx < total; idx += gridDim.x * 256) {
        const int m = (int)((double)idx * inv_c16);
        const int mm = m - (m * c16n > idx) + ((m + 1) * c16n <= idx), c0 = (idx - mm * c16n) * 16;
        int row = (int)((double)mm * inv_ow);
        row += ((row + 1) * p.OW <= mm) - (row * p.OW > mm);
        const int ow = mm - row * p.OW;
        int n = (int)((double)row * inv_oh);
        n += ((n + 1) * p.OH <= row) - (n * p.OH > row);
        const int oh = row - n * p.OH;
        const int hs = max(oh * p.sh - p.ph, 0), ws = max(ow * p.sw - p.pw, 0);
        const int he = min(oh * p.sh - p.ph + p.kh, p.H), we = min(ow * p.sw - p.pw + p.kw, p.W);
        u32x4 mx = {0, 0, 0, 0};
        for (int i = hs; i < he; i++)
            for (int j = ws; j < we; j++) {
                const u32x4 v = *reinterpret_cast<const u32x4 *>(p.x + (size_t)((n * p.H + i) * p.W + j) * p.cs + c0);
#pragma unroll
                for (int d = 0; d < 4; d++)
                    mx[d] = max_u8x4(mx[d], v[d]);
            }
        u32x4 o = mx;
        if (!same) { // else equal scales (a multiplier of exactly 2^shift), equal zero points, 8 bits: the maximum is the result
#pragma unroll
            for (int d = 0; d < 4; d++) {
                int32_t v[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    // mult < 2^16, |max - zp| <= 255: the product fits 24 bits, shift <= 22 (host): 32-bit arithmetic is
                    // exact; the upper clamp in front of the shift, the lower one is the pack's saturation
                    const int32_t pr = __mul24((int)p.mult, (int)((mx[d] >> (8 * e)) & 255) - p.iz);
                    v[e] = min(pr + radd, phi);
                }
                o[d] = ashr_sat_u8x4(v[0], v[1], v[2], v[3], p.shift);
            }
        }
        *reinterpret_cast<u32x4 *>(p.y + (size_t)mm * p.cs + c0) = o;
    }
}

// Global average pooling (one window = the whole image, no padding) with a channel stride that is a multiple of 16.
// A work-group of 256 threads covers 64 groups of 16 channels of one image; the pixels are dealt to 4 thread groups,
// each thread sums its pixels on packed 16-bit lanes (at most 256 pixels per thread), the 4 partial sums meet in LDS.
__global__ __launch_bounds__(256) void pool_gavg16_u8_kernel(const PoolArgs p, uint32_t mult, int shift)
{
    __shared__ int32_t part[3][64][17];
    const int c16n = p.cs >> 4, hw = p.H * p.W;
    const int n = blockIdx.y, chunk = blockIdx.x * 64 + (threadIdx.x & 63), pg = threadIdx.x >> 6;
    const bool live = chunk < c16n;
    uint32_t ev[4] = {0, 0, 0, 0}, od[4] = {0, 0, 0, 0};
    if (live) {
        const uint8_t *src = p.x + (size_t)n * hw * p.cs + chunk * 16;
        for (int i = pg; i < hw; i += 4) {
            const u32x4 v = *reinterpret_cast<const u32x4 *>(src + (size_t)i * p.cs);
#pragma unroll
            for (int d = 0; d < 4; d++) {
                ev[d] += v[d] & 0x00ff00ffu;
                od[d] += (v[d] >> 8) & 0x00ff00ffu;
            }
        }
    }
    int32_t sum[16];
#pragma unroll
    for (int d = 0; d < 4; d++) {
        sum[4 * d + 0] = ev[d] & 0xffff, sum[4 * d + 1] = od[d] & 0xffff;
        sum[4 * d + 2] = ev[d] >> 16, sum[4 * d + 3] = od[d] >> 16;
    }
    if (pg > 0) {
#pragma unroll
        for (int e = 0; e < 16; e++)
            part[pg - 1][threadIdx.x & 63][e] = sum[e];
    }
    __syncthreads();
    if (pg == 0 && live) {
        u32x4 o;
#pragma unroll
        for (int d = 0; d < 4; d++) {
            uint32_t w = 0;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int k = 4 * d + e;
                const int32_t t = sum[k] + part[0][threadIdx.x][k] + part[1][threadIdx.x][k] + part[2][threadIdx.x][k] -
                                  hw * p.iz;
                const int32_t pr = (int32_t)(mult * (uint32_t)t);
                w |= (uint32_t)sat_hi((int32_t)(rshift_rn(pr, shift) + p.oz), p.hi) << (8 * e);
            }
            o[d] = w;
        }
        *reinterpret_cast<u32x4 *>(p.y + (size_t)n * p.cs + chunk * 16) = o;
    }
}

// ---- concat along the channels (op_quant_concat_run, concat.c:82-124) ----------------------------------------------
// Output pixel p, channel c comes from input j with off[j] <= c < off[j+1]; every input has its own rescale
// y = sat(rrn(mult_j * (x - zp_j), shift_j) + oz) with a 16-bit multiplier.  One thread writes one dword (4 channels)
// of the output; when the 4 channels come from one input at a dword-aligned offset they are read as one dword.
struct ConcatArgs {
    const uint8_t *in[HIPQ_MAX_ELTWISE_INPUTS];
    int off[HIPQ_MAX_ELTWISE_INPUTS + 1]; // first output channel of each input; off[n_in] = total channels
    int cs[HIPQ_MAX_ELTWISE_INPUTS];      // channel stride of each input
    uint32_t mult[HIPQ_MAX_ELTWISE_INPUTS];
    int shift[HIPQ_MAX_ELTWISE_INPUTS];
    int zp[HIPQ_MAX_ELTWISE_INPUTS];
    int n_in, oz, hi, cs_out;
    uint8_t *y;
    size_t npix;
};

__device__ static inline uint32_t concat_one(uint32_t x, int j, const ConcatArgs &p)
{
    const int32_t pr = (int32_t)p.mult[j] * ((int32_t)x - p.zp[j]); // 16-bit * 9-bit
    return (uint32_t)sat_hi((int32_t)(rshift_rn(pr, p.shift[j]) + p.oz), p.hi);
}

__global__ __launch_bounds__(256) void concat_u8_kernel(const ConcatArgs p)
{
    const int cq = p.cs_out >> 2;
    const size_t total = p.npix * cq;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
        const size_t pix = idx / cq;
        const int c0 = (int)(idx - pix * cq) * 4;
        uint32_t o = 0;
        int j = 0;
        while (j + 1 < p.n_in && c0 >= p.off[j + 1])
            j++;
        if (c0 + 3 < p.off[j + 1] && ((c0 - p.off[j]) & 3) == 0) {
            const uint32_t v = *reinterpret_cast<const uint32_t *>(p.in[j] + pix * p.cs[j] + (c0 - p.off[j]));
#pragma unroll
            for (int e = 0; e < 4; e++)
                o |= concat_one((v >> (8 * e)) & 255, j, p) << (8 * e);
        } else {
            for (int e = 0; e < 4; e++) {
                const int c = c0 + e;
                if (c >= p.off[p.n_in])
                    break; // pad channels of the output stay zero
                while (c >= p.off[j + 1])
                    j++;
                o |= concat_one(p.in[j][pix * p.cs[j] + (c - p.off[j])], j, p) << (8 * e);
            }
        }
        *reinterpret_cast<uint32_t *>(p.y + pix * p.cs_out + c0) = o;
    }
}

// ---- softmax over the channels (op_quant_softmax_run, softmax.c:89-122) -------------------------------------------
// e(x) = fp32(exp(double(fp32(ialpha * (x - izp))))) takes 256 values: the host tabulates them with the C library's
// exp, the very call the reference makes.  A thread owns a pixel: it sums its channels in fp32 in channel order (the
// reference's order), then y = saturate_float_by_bits(e / sum / oalpha + ozp) with IEEE fp32 divisions.
struct SoftmaxArgs {
    const uint8_t *x;
    uint8_t *y;
    size_t npix;
    int C, cs;
    float oalpha, ozp, hi;
    float table[256];
};

__global__ __launch_bounds__(256) void softmax_u8_kernel(const SoftmaxArgs p)
{
    __shared__ float tab[256];
    tab[threadIdx.x] = p.table[threadIdx.x];
    __syncthreads();
    for (size_t pix = (size_t)blockIdx.x * blockDim.x + threadIdx.x; pix < p.npix; pix += (size_t)gridDim.x * blockDim.x) {
        const uint8_t *xr = p.x + pix * p.cs;
        uint8_t *yr = p.y + pix * p.cs;
        float sum = 0.f;
        for (int c = 0; c < p.C; c++)
            sum = __fadd_rn(sum, tab[xr[c]]);
        for (int c = 0; c < p.C; c++) {
            const float q = __fadd_rn(__fdiv_rn(__fdiv_rn(tab[xr[c]], sum), p.oalpha), p.ozp);
            yr[c] = q > p.hi ? (uint8_t)p.hi : (q < 0 ? (uint8_t)0 : (uint8_t)((double)q + 0.5));
        }
        for (int c = p.C; c < p.cs; c++)
            yr[c] = 0;
    }
}

// ---- quantize (quantize.c:145-157): fp32 NCHW -> uint8 NHWC --------------------------------------
// One thread produces the 4 channels of one dword of the output; reads are coalesced along W per
// channel plane, writes along the pixel index.
struct QuantArgs {
    const float *x;
    uint8_t *y;
    int N, C, H, W, cs;
    float alpha, beta, hi;
    float rcp, xlo, xhi; // uint8 variant: RN(1 / alpha) and the clamp of x - beta, [-alpha, (hi + 1) * alpha]
    int lim; // int8 variant: alpha holds fp32(1 / oalpha), the result is clipped to +-lim
};

// The reference: q = fp32((x - beta) / alpha); q > hi -> hi; q < 0 -> 0 (NaN too: the x86 conversion of NaN is 0 in
// the low byte); else trunc(double(q) + 0.5).  Here, value for value the same byte with a third of the instructions of
// the IEEE division sequence:
//   * x - beta is clamped to [-alpha, (hi + 1) * alpha] first: outside that range the quotient is below 0 or above hi
//     anyway, inside it nothing changes, and no infinity reaches the steps below (a NaN leaves v_med3_f32 as the
//     smallest of the other two operands, i.e. as a negative quotient: 0, like the reference);
//   * the correctly rounded quotient from the correctly rounded reciprocal rcp = RN(1 / alpha) (the host computes it):
//     q0 = RN(a * rcp), then twice r = a - alpha * q (exact in an FMA), q = RN(q + r * rcp).  After the first
//     correction q is within an ulp of a / alpha, and then the second yields RN(a / alpha) (Markstein's theorem on
//     division with a correctly rounded reciprocal; no overflow by the clamp, and an underflowing residual belongs to
//     a quotient far below 0.5, whose byte is 0 whatever its last bits are);
//   * trunc(q + 0.5) for 0 <= q <= hi + 1 without the double: the integer part plus one if the fraction (exact in
//     fp32) is at least a half.
__device__ static inline uint32_t quantize_one(float x, const QuantArgs &p)
{
    float a = __fsub_rn(x, p.beta);
    asm("v_med3_f32 %0, %1, %2, %3" : "=v"(a) : "v"(a), "v"(p.xlo), "v"(p.xhi));
    float q = __fmul_rn(a, p.rcp);
    q = __fmaf_rn(__fmaf_rn(-p.alpha, q, a), p.rcp, q);
    q = __fmaf_rn(__fmaf_rn(-p.alpha, q, a), p.rcp, q);
    q = fmaxf(q, 0.f);
    const uint32_t r = (uint32_t)q + (uint32_t)(__builtin_amdgcn_fractf(q) >= 0.5f);
    return min(r, (uint32_t)p.hi);
}

// op_quantize_run_i8 (quantize.c:159-185): clip(round(x * fp32(1 / oalpha)), -lim, lim).  The product is fp32, round()
// is the C library's on a double (half away from zero), and clip() takes an int: the reference's x86-64 conversion
// turns everything outside int32 (and NaN) into INT32_MIN, which then clips to -lim.
__device__ static inline uint32_t quantize_one_i8(float x, const QuantArgs &p)
{
    const double r = round((double)__fmul_rn(x, p.alpha));
    const int v = (r >= -2147483648.0 && r < 2147483648.0) ? (int)r : INT32_MIN;
    return (uint32_t)min(max(v, -p.lim), p.lim) & 255u;
}

template <bool SIGNED>
__device__ static inline uint32_t quantize_any(float x, const QuantArgs &p)
{
    return SIGNED ? quantize_one_i8(x, p) : quantize_one(x, p);
}

template <bool SIGNED>
__global__ __launch_bounds__(256) void quantize_u8_kernel(const QuantArgs p)
{
    const int cq = p.cs >> 2;
    const size_t hw = (size_t)p.H * p.W, total = (size_t)p.N * hw * cq;
    // pixel index fastest across threads: each channel plane is read with unit stride
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        const size_t pix = idx % hw, rest = idx / hw;
        const int q4 = (int)(rest % cq), n = (int)(rest / cq);
        uint32_t o = 0;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int c = q4 * 4 + e;
            if (c < p.C)
                o |= quantize_any<SIGNED>(p.x[((size_t)n * p.C + c) * hw + pix], p) << (8 * e);
        }
        *reinterpret_cast<uint32_t *>(p.y + ((size_t)n * hw + pix) * p.cs + q4 * 4) = o;
    }
}

// Network inputs (C <= 4, channel stride 4): a thread converts 4 consecutive pixels, i.e. one 128-bit load per
// channel plane and one 128-bit store; blockIdx.y is the image, so no 64-bit index arithmetic is needed.
template <bool SIGNED>
__global__ __launch_bounds__(256) void quantize_u8_c4_kernel(const QuantArgs p)
{
    const int hw = p.H * p.W, hw4 = hw >> 2; // the host checks hw % 4 == 0
    const int n = blockIdx.y;
    const float *xn = p.x + (size_t)n * p.C * hw;
    u32x4 *yn = reinterpret_cast<u32x4 *>(p.y + (size_t)n * hw * 4);
    for (int i = blockIdx.x * 256 + threadIdx.x; i < hw4; i += gridDim.x * 256) {
        u32x4 o = {0, 0, 0, 0};
        for (int c = 0; c < p.C; c++) { // one plane at a time: with every plane's load issued first the kernel is a third slower
            typedef float f32x4 __attribute__((ext_vector_type(4)));
            const f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(xn + (size_t)c * hw) + i);
#pragma unroll
            for (int e = 0; e < 4; e++)
                o[e] |= quantize_any<SIGNED>(v[e], p) << (8 * c);
        }
        yn[i] = o;
    }
}

// ---- dequantize (dequantize.c:111-123): uint8 NHWC -> fp32 NCHW ----------------------------------
struct DequantArgs {
    const uint8_t *x;
    float *y;
    int N, C, H, W, cs;
    float alpha;
    int zp;
    int sgn; // 1: the bytes are int8 and there is no zero point (op_dequantize_run_i8, dequantize.c:125-136)
};

__global__ __launch_bounds__(256) void dequantize_u8_kernel(const DequantArgs p)
{
    const size_t hw = (size_t)p.H * p.W, total = (size_t)p.N * p.C * hw;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        const size_t pix = idx % hw, rest = idx / hw;
        const int c = (int)(rest % p.C), n = (int)(rest / p.C);
        const uint8_t b = p.x[((size_t)n * hw + pix) * p.cs + c];
        const int v = p.sgn ? (int)(int8_t)b : (int)b - p.zp;
        p.y[idx] = __fmul_rn((float)v, p.alpha);
    }
}

// int32 accumulators (NHWC, as hipq_conv2d_run's acc_out writes them) -> fp32 dense NCHW: (float)acc * alpha
struct DequantI32Args {
    const int32_t *x;
    float *y;
    int N, C, H, W, cs;
    float alpha;
};

__global__ __launch_bounds__(256) void dequantize_i32_kernel(const DequantI32Args p)
{
    const size_t hw = (size_t)p.H * p.W, total = (size_t)p.N * p.C * hw;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        const size_t pix = idx % hw, rest = idx / hw;
        const int c = (int)(rest % p.C), n = (int)(rest / p.C);
        p.y[idx] = __fmul_rn(__int2float_rn(p.x[((size_t)n * hw + pix) * p.cs + c]), p.alpha);
    }
}

// ---- layout conversion ---------------------------------------------------------------------------
struct LayoutArgs {
    const uint8_t *src;
    uint8_t *dst;
    int N, C, H, W, cs;
};

__global__ __launch_bounds__(256) void nchw_to_nhwc_kernel(const LayoutArgs p)
{
    const int cq = p.cs >> 2;
    const size_t hw = (size_t)p.H * p.W, total = (size_t)p.N * hw * cq;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        const size_t pix = idx % hw, rest = idx / hw;
        const int q4 = (int)(rest % cq), n = (int)(rest / cq);
        uint32_t o = 0;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int c = q4 * 4 + e;
            if (c < p.C)
                o |= (uint32_t)p.src[((size_t)n * p.C + c) * hw + pix] << (8 * e);
        }
        *reinterpret_cast<uint32_t *>(p.dst + ((size_t)n * hw + pix) * p.cs + q4 * 4) = o;
    }
}

__global__ __launch_bounds__(256) void nhwc_to_nchw_kernel(const LayoutArgs p)
{
    const size_t hw = (size_t)p.H * p.W, total = (size_t)p.N * p.C * hw;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        const size_t pix = idx % hw, rest = idx / hw;
        const int c = (int)(rest % p.C), n = (int)(rest / p.C);
        p.dst[idx] = p.src[((size_t)n * hw + pix) * p.cs + c];
    }
}

__global__ __launch_bounds__(256) void copy_bytes_kernel(const u32x4 *src, u32x4 *dst, size_t nvec)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += (size_t)gridDim.x * blockDim.x)
        dst[i] = src[i];
}

} // namespace hipq

// =================================================================================================
using namespace hipq;

static bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

extern "C" int hipq_add_u8(const void *a, const void *b, void *y, size_t count, float ia0, int iz0, float ia1,
                           int iz1, float oa, int oz, int obits, void *stream)
{
    clear_error();
    HIPQ_REQUIRE(a && b && y, "hipq_add_u8: null pointer");
    HIPQ_REQUIRE(aligned16(a) && aligned16(b) && aligned16(y), "hipq_add_u8: buffers must be 16-byte aligned");
    if (count == 0)
        return 0;
    AddArgs p;
    HIPQ_REQUIRE(make_add_params(ia0, iz0, ia1, iz1, oa, oz, obits, &p.q),
                 "hipq_add_u8: scales out of the fixed-point range");
    p.a = static_cast<const uint8_t *>(a), p.b = static_cast<const uint8_t *>(b), p.y = static_cast<uint8_t *>(y);
    p.count = count;
    const dim3 grid(grid_for(count / 16)), block(256);
    if (p.q.fast)
        hipLaunchKernelGGL(add_u8_kernel<true>, grid, block, 0, static_cast<hipStream_t>(stream), p);
    else
        hipLaunchKernelGGL(add_u8_kernel<false>, grid, block, 0, static_cast<hipStream_t>(stream), p);
    return launch_status("add_u8_kernel");
}

extern "C" int hipq_eltwise_u8(const void *const *in, int n_in, const float *coeff, const float *ialpha,
                               const uint8_t *izp, void *y, size_t count, int operation, float oa, int oz,
                               int obits, void *stream)
{
    clear_error();
    HIPQ_REQUIRE(in && ialpha && izp && y && aligned16(y), "hipq_eltwise_u8: null pointer or output not 16-byte aligned");
    HIPQ_REQUIRE(n_in >= 2 && n_in <= HIPQ_MAX_ELTWISE_INPUTS, "hipq_eltwise_u8: %d inputs (2..%d supported)", n_in,
                 HIPQ_MAX_ELTWISE_INPUTS);
    HIPQ_REQUIRE(operation == HIPQ_ELTWISE_SUM || operation == HIPQ_ELTWISE_MAX,
                 "hipq_eltwise_u8: operation %d is not implemented (PROD is rejected by the reference too)", operation);
    if (count == 0)
        return 0;
    EltArgs p;
    memset(&p, 0, sizeof p);
    int smin = 127, sh[HIPQ_MAX_ELTWISE_INPUTS];
    for (int n = 0; n < n_in; n++) {
        HIPQ_REQUIRE(in[n] && aligned16(in[n]), "hipq_eltwise_u8: input %d is null or not 16-byte aligned", n);
        hipq_quant_scale((coeff ? coeff[n] : 1.0f) * ialpha[n] / oa, 23, &p.mult[n], &sh[n]);
        smin = std::min(smin, sh[n]);
        p.in[n] = static_cast<const uint8_t *>(in[n]);
        p.zp[n] = izp[n];
    }
    p.s0 = smin - 1;
    HIPQ_REQUIRE(valid_shift(p.s0), "hipq_eltwise_u8: scales out of the fixed-point range");
    for (int n = 0; n < n_in; n++) {
        p.shift[n] = sh[n] - p.s0;
        HIPQ_REQUIRE(valid_shift(p.shift[n]), "hipq_eltwise_u8: scales out of the fixed-point range");
    }
    p.n_in = n_in, p.oz = oz, p.hi = (1 << obits) - 1, p.is_max = operation == HIPQ_ELTWISE_MAX;
    p.y = static_cast<uint8_t *>(y), p.count = count;
    // 32-bit form: every product below 2^30 (22-bit multipliers), shifts within a word, the sum of n terms and
    // the folded rounding / zero-point constant without overflow
    p.fast = p.s0 <= 20 && n_in <= 4;
    for (int n = 0; n < n_in; n++) {
        p.fast = p.fast && p.shift[n] <= 30 && p.mult[n] < (1u << 23) && (reinterpret_cast<uintptr_t>(in[n]) & 15) == 0;
        p.cfast[n] = p.fast ? (1 << (p.shift[n] - 1)) - p.zp[n] * (int32_t)p.mult[n] : 0;
    }
    p.fast = p.fast && (reinterpret_cast<uintptr_t>(y) & 15) == 0;
    p.cadd = p.fast ? (1 << (p.s0 - 1)) + (oz << p.s0) : 0;
    const dim3 grid(grid_for(count / 16 + 1)), block(256);
    hipStream_t st = static_cast<hipStream_t>(stream);
#define HIPQ_ELT(NIN)                                                                          \
    if (p.fast && p.is_max)                                                                    \
        hipLaunchKernelGGL((eltwise_u8_kernel<NIN, true, true>), grid, block, 0, st, p);       \
    else if (p.fast)                                                                           \
        hipLaunchKernelGGL((eltwise_u8_kernel<NIN, true, false>), grid, block, 0, st, p);      \
    else if (p.is_max)                                                                         \
        hipLaunchKernelGGL((eltwise_u8_kernel<NIN, false, true>), grid, block, 0, st, p);      \
    else                                                                                       \
        hipLaunchKernelGGL((eltwise_u8_kernel<NIN, false, false>), grid, block, 0, st, p)
    if (n_in == 2) {
        HIPQ_ELT(2);
    } else if (n_in == 3) {
        HIPQ_ELT(3);
    } else if (n_in == 4) {
        HIPQ_ELT(4);
    } else {
        hipLaunchKernelGGL(eltwise_u8_generic_kernel, dim3(grid_for(count)), block, 0, st, p);
    }
#undef HIPQ_ELT
    return launch_status("eltwise_u8_kernel");
}

extern "C" int hipq_relu_u8(const void *x, void *y, size_t count, float ia, int iz, float oa, int oz, int obits,
                            void *stream)
{
    clear_error();
    HIPQ_REQUIRE(x && y && aligned16(x) && aligned16(y), "hipq_relu_u8: null or unaligned pointer");
    if (count == 0)
        return 0;
    ReluArgs p;
    hipq_quant_scale(ia / oa, 24, &p.mult, &p.shift);
    HIPQ_REQUIRE(valid_shift(p.shift), "hipq_relu_u8: scale out of the fixed-point range");
    p.x = static_cast<const uint8_t *>(x), p.y = static_cast<uint8_t *>(y), p.count = count;
    p.iz = iz, p.oz = oz, p.hi = (1 << obits) - 1;
    hipLaunchKernelGGL(relu_u8_kernel, dim3(grid_for(count / 16)), dim3(256), 0, static_cast<hipStream_t>(stream), p);
    return launch_status("relu_u8_kernel");
}

extern "C" int hipq_concat_u8(const void *const *in, int n_in, const int *channels, const float *ialpha, const uint8_t *izp,
                              void *y, size_t npix, float oa, int oz, int obits, void *stream)
{
    clear_error();
    HIPQ_REQUIRE(in && channels && ialpha && izp && y, "hipq_concat_u8: null pointer");
    HIPQ_REQUIRE(n_in >= 2 && n_in <= HIPQ_MAX_ELTWISE_INPUTS, "hipq_concat_u8: %d inputs (2..%d supported)", n_in,
                 HIPQ_MAX_ELTWISE_INPUTS);
    HIPQ_REQUIRE(obits >= 1 && obits <= 8, "hipq_concat_u8: obits must be in 1..8");
    if (npix == 0)
        return 0;
    ConcatArgs p;
    memset(&p, 0, sizeof p);
    for (int j = 0; j < n_in; j++) {
        HIPQ_REQUIRE(in[j] && channels[j] > 0, "hipq_concat_u8: input %d is null or has no channels", j);
        p.in[j] = static_cast<const uint8_t *>(in[j]);
        p.off[j + 1] = p.off[j] + channels[j];
        p.cs[j] = hipq_channel_stride(channels[j]);
        hipq_quant_scale(ialpha[j] / oa, 16, &p.mult[j], &p.shift[j]); // concat.c:104-108
        p.mult[j] &= 0xffff;
        HIPQ_REQUIRE(valid_shift(p.shift[j]), "hipq_concat_u8: scale of input %d out of the fixed-point range", j);
        p.zp[j] = izp[j];
    }
    p.n_in = n_in, p.oz = oz, p.hi = (1 << obits) - 1, p.cs_out = hipq_channel_stride(p.off[n_in]);
    p.y = static_cast<uint8_t *>(y), p.npix = npix;
    hipLaunchKernelGGL(concat_u8_kernel, dim3(grid_for(npix * (p.cs_out / 4))), dim3(256), 0, static_cast<hipStream_t>(stream), p);
    return launch_status("concat_u8_kernel");
}

extern "C" int hipq_softmax_u8(const void *x, void *y, size_t npix, int C, int cs, float ia, int iz, float oa, int oz, int obits,
                               void *stream)
{
    clear_error();
    HIPQ_REQUIRE(x && y && C > 0 && cs >= C, "hipq_softmax_u8: bad argument");
    HIPQ_REQUIRE(obits >= 1 && obits <= 8, "hipq_softmax_u8: obits must be in 1..8");
    if (npix == 0)
        return 0;
    SoftmaxArgs p;
    p.x = static_cast<const uint8_t *>(x), p.y = static_cast<uint8_t *>(y), p.npix = npix, p.C = C, p.cs = cs;
    p.oalpha = oa, p.ozp = (float)oz, p.hi = (float)((1 << obits) - 1);
    for (int v = 0; v < 256; v++) {
        const float arg = ia * (float)(v - iz);        // softmax.c:112: an fp32 product ...
        p.table[v] = (float)std::exp((double)arg);     // ... passed to the double exp, stored as fp32
    }
    hipLaunchKernelGGL(softmax_u8_kernel, dim3(grid_for(npix)), dim3(256), 0, static_cast<hipStream_t>(stream), p);
    return launch_status("softmax_u8_kernel");
}

extern "C" int hipq_pool_u8(const void *x, void *y, int N, int C, int H, int W, int OH, int OW, int cs, int kh, int kw,
                            int ph, int pw, int sh, int sw, int method, float ia, int iz, float oa, int oz, int obits,
                            void *stream)
{
    clear_error();
    HIPQ_REQUIRE(x && y, "hipq_pool_u8: null pointer");
    HIPQ_REQUIRE(N > 0 && C > 0 && H > 0 && W > 0 && OH > 0 && OW > 0 && cs >= C && cs % 4 == 0, "hipq_pool_u8: bad shape");
    HIPQ_REQUIRE(kh > 0 && kw > 0 && sh > 0 && sw > 0 && ph >= 0 && pw >= 0, "hipq_pool_u8: bad window");
    // every window must overlap the padded image, otherwise the reference divides by a pool size <= 0
    HIPQ_REQUIRE((OH - 1) * sh - ph < H + ph && (OW - 1) * sw - pw < W + pw, "hipq_pool_u8: a window lies outside the image");
    PoolArgs p;
    p.x = static_cast<const uint8_t *>(x), p.y = static_cast<uint8_t *>(y);
    p.N = N, p.H = H, p.W = W, p.OH = OH, p.OW = OW, p.cs = cs, p.kh = kh, p.kw = kw, p.ph = ph, p.pw = pw, p.sh = sh, p.sw = sw;
    p.is_avg = method != HIPQ_POOL_MAX, p.iz = iz, p.oz = oz, p.hi = (1 << obits) - 1;
    p.ia_over_oa = ia / oa;
    hipq_quant_scale(ia / oa, 16, &p.mult, &p.shift);
    p.mult &= 0xffff; // get_quant_scale_int16 stores the multiplier in a uint16_t
    HIPQ_REQUIRE(valid_shift(p.shift), "hipq_pool_u8: scale out of the fixed-point range");
    if (!p.is_avg && cs % 16 == 0 && p.shift <= 22 && (long long)N * OH * OW * (cs / 16) < (1ll << 31)
        && (long long)N * H * W * cs < (1ll << 31) && (reinterpret_cast<uintptr_t>(x) & 15) == 0
        && (reinterpret_cast<uintptr_t>(y) & 15) == 0) {
        const size_t total16 = (size_t)N * OH * OW * (cs / 16);
        hipLaunchKernelGGL(pool_max16_u8_kernel, dim3((grid_for(total16) + 7) / 8 * 8), dim3(256), 0, static_cast<hipStream_t>(stream), p,
                           1.0 / (cs / 16), 1.0 / OW, 1.0 / OH);
        return launch_status("pool_max16_u8_kernel");
    }
    if (p.is_avg && OH == 1 && OW == 1 && ph == 0 && pw == 0 && kh >= H && kw >= W && cs % 16 == 0 && H * W <= 1024
        && N <= 65535 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0) {
        uint32_t mult;
        int shift;
        hipq_quant_scale(p.ia_over_oa / (float)(uint32_t)(H * W), 16, &mult, &shift); // pool.c:211-216
        if (valid_shift(shift)) {
            hipLaunchKernelGGL(pool_gavg16_u8_kernel, dim3((cs / 16 + 63) / 64, N), dim3(256), 0,
                               static_cast<hipStream_t>(stream), p, mult, shift);
            return launch_status("pool_gavg16_u8_kernel");
        }
    }
    const size_t total = (size_t)N * OH * OW * (cs / 4);
    hipLaunchKernelGGL(pool_u8_kernel, dim3(grid_for(total)), dim3(256), 0, static_cast<hipStream_t>(stream), p);
    return launch_status("pool_u8_kernel");
}

static int launch_quantize(const char *who, bool sgn, const float *x, void *y, int N, int C, int H, int W, int cs, float oa,
                           int oz, int obits, void *stream)
{
    clear_error();
    HIPQ_REQUIRE(x && y && N > 0 && C > 0 && H > 0 && W > 0 && cs >= C && cs % 4 == 0, "%s: bad argument", who);
    HIPQ_REQUIRE(obits >= 1 && obits <= 8, "%s: obits must be in 1..8", who);
    HIPQ_REQUIRE(oa >= 1e-30f && oa <= 1e30f, "%s: the scale must be a positive number between 1e-30 and 1e30", who);
    QuantArgs p;
    p.x = x, p.y = static_cast<uint8_t *>(y), p.N = N, p.C = C, p.H = H, p.W = W, p.cs = cs;
    p.alpha = sgn ? (float)(1. / (double)oa) : oa; // quantize.c:166: a double division, rounded to fp32
    p.beta = -(oa * (float)oz);                    // quantize.c:152
    p.hi = (float)((1 << obits) - 1);
    p.lim = (1 << (obits - 1)) - 1;
    // RN(1 / alpha): the double quotient rounded to fp32 can be one ulp off the correctly rounded reciprocal (double
    // rounding); alpha * candidate is exact in a double, so the candidate with the smallest |1 - alpha * y| is it
    p.rcp = (float)(1.0 / (double)oa);
    for (float c : {nextafterf(p.rcp, 0.f), nextafterf(p.rcp, INFINITY)})
        if (fabs(1.0 - (double)oa * (double)c) < fabs(1.0 - (double)oa * (double)p.rcp))
            p.rcp = c;
    p.xlo = -oa, p.xhi = (p.hi + 1.f) * oa;
    const hipStream_t st = static_cast<hipStream_t>(stream);
    if (cs == 4 && (H * W) % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0
        && N <= 65535) {
        const unsigned bx = (unsigned)std::min((H * W / 4 + 255) / 256, 1024);
        if (sgn)
            hipLaunchKernelGGL(quantize_u8_c4_kernel<true>, dim3(bx, N), dim3(256), 0, st, p);
        else
            hipLaunchKernelGGL(quantize_u8_c4_kernel<false>, dim3(bx, N), dim3(256), 0, st, p);
        return launch_status(sgn ? "quantize_i8_c4_kernel" : "quantize_u8_c4_kernel");
    }
    const size_t total = (size_t)N * H * W * (cs / 4);
    if (sgn)
        hipLaunchKernelGGL(quantize_u8_kernel<true>, dim3(grid_for(total)), dim3(256), 0, st, p);
    else
        hipLaunchKernelGGL(quantize_u8_kernel<false>, dim3(grid_for(total)), dim3(256), 0, st, p);
    return launch_status(sgn ? "quantize_i8_kernel" : "quantize_u8_kernel");
}

extern "C" int hipq_quantize_u8(const float *x, void *y, int N, int C, int H, int W, int cs, float oa, int oz, int obits,
                                void *stream)
{
    return launch_quantize("hipq_quantize_u8", false, x, y, N, C, H, W, cs, oa, oz, obits, stream);
}

extern "C" int hipq_quantize_i8(const float *x, void *y, int N, int C, int H, int W, int cs, float oa, int obits, void *stream)
{
    return launch_quantize("hipq_quantize_i8", true, x, y, N, C, H, W, cs, oa, 0, obits, stream);
}

static int launch_dequantize(const char *who, int sgn, const void *x, float *y, int N, int C, int H, int W, int cs, float ia,
                             int iz, void *stream)
{
    clear_error();
    HIPQ_REQUIRE(x && y && N > 0 && C > 0 && H > 0 && W > 0 && cs >= C, "%s: bad argument", who);
    DequantArgs p;
    p.x = static_cast<const uint8_t *>(x), p.y = y, p.N = N, p.C = C, p.H = H, p.W = W, p.cs = cs, p.alpha = ia, p.zp = iz;
    p.sgn = sgn;
    hipLaunchKernelGGL(dequantize_u8_kernel, dim3(grid_for((size_t)N * C * H * W)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), p);
    return launch_status(sgn ? "dequantize_i8_kernel" : "dequantize_u8_kernel");
}

extern "C" int hipq_dequantize_u8(const void *x, float *y, int N, int C, int H, int W, int cs, float ia, int iz,
                                  void *stream)
{
    return launch_dequantize("hipq_dequantize_u8", 0, x, y, N, C, H, W, cs, ia, iz, stream);
}

extern "C" int hipq_dequantize_i8(const void *x, float *y, int N, int C, int H, int W, int cs, float ia, void *stream)
{
    return launch_dequantize("hipq_dequantize_i8", 1, x, y, N, C, H, W, cs, ia, 0, stream);
}

extern "C" int hipq_dequantize_i32(const int32_t *x, float *y, int N, int C, int H, int W, int cs, float alpha, void *stream)
{
    clear_error();
    HIPQ_REQUIRE(x && y && N > 0 && C > 0 && H > 0 && W > 0 && cs >= C, "hipq_dequantize_i32: bad argument");
    DequantI32Args p;
    p.x = x, p.y = y, p.N = N, p.C = C, p.H = H, p.W = W, p.cs = cs, p.alpha = alpha;
    hipLaunchKernelGGL(dequantize_i32_kernel, dim3(grid_for((size_t)N * C * H * W)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), p);
    return launch_status("dequantize_i32_kernel");
}

static int layout_args(LayoutArgs &p, const void *src, void *dst, int N, int C, int H, int W, int cs)
{
    HIPQ_REQUIRE(src && dst && N > 0 && C > 0 && H > 0 && W > 0 && cs >= C && cs % 4 == 0, "layout conversion: bad argument");
    p.src = static_cast<const uint8_t *>(src), p.dst = static_cast<uint8_t *>(dst);
    p.N = N, p.C = C, p.H = H, p.W = W, p.cs = cs;
    return 0;
}

extern "C" int hipq_nchw_to_nhwc_u8(const void *src, void *dst, int N, int C, int H, int W, int cs, void *stream)
{
    clear_error();
    LayoutArgs p;
    if (int rc = layout_args(p, src, dst, N, C, H, W, cs))
        return rc;
    hipLaunchKernelGGL(nchw_to_nhwc_kernel, dim3(grid_for((size_t)N * H * W * (cs / 4))), dim3(256), 0,
                       static_cast<hipStream_t>(stream), p);
    return launch_status("nchw_to_nhwc_kernel");
}

extern "C" int hipq_nhwc_to_nchw_u8(const void *src, void *dst, int N, int C, int H, int W, int cs, void *stream)
{
    clear_error();
    LayoutArgs p;
    if (int rc = layout_args(p, src, dst, N, C, H, W, cs))
        return rc;
    hipLaunchKernelGGL(nhwc_to_nchw_kernel, dim3(grid_for((size_t)N * C * H * W)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), p);
    return launch_status("nhwc_to_nchw_kernel");
}

extern "C" int hipq_copy_bytes(const void *src, void *dst, size_t count, void *stream)
{
    clear_error();
    HIPQ_REQUIRE(src && dst && aligned16(src) && aligned16(dst) && count % 16 == 0, "hipq_copy_bytes: need 16-byte granularity");
    hipLaunchKernelGGL(copy_bytes_kernel, dim3(grid_for(count / 16)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const u32x4 *>(src), static_cast<u32x4 *>(dst), count / 16);
    return launch_status("copy_bytes_kernel");
}
