/*
 * CPU oracle — see quant_oracle.h.  TEST INFRASTRUCTURE ONLY; never linked into the product.
 *
 * Build with -ffp-contract=off (no FMA contraction) so that every fp32 expression is evaluated
 * operation by operation, as the reference's x86-64 SSE build evaluates it.
 */
#include "quant_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* quant_helper.h:60-118: normalise x into [0.5, 1) by fp32 halving/doubling; mult = x * 2^(bits-1). */
void orc_quant_scale(float x, int bits, uint32_t *mult, int *shift)
{
    int s = 0;
    *shift = 0;
    *mult = 0;
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
    s += bits - 1;
    /* the reference multiplies the float by an integer power of two (converted to float): exact */
    *mult = (uint32_t)(x * (float)(1ll << (bits - 1)));
    *shift = s;
}

/* quant_helper.h:55-58: floor((x + 2^(bits-1)) / 2^bits), written the way the reference writes it. */
int64_t orc_rshift_rn(int64_t x, int bits)
{
    int64_t t = x >> (bits - 1);
    return (t + ((t & 1) << 1)) >> 1;
}

/* quant_helper.h:33-36 */
uint8_t orc_sat_bits(int32_t x, int bits)
{
    int32_t hi = (1 << bits) - 1;
    return x > hi ? (uint8_t)hi : (x < 0 ? 0 : (uint8_t)x);
}

int orc_conv_out_dim(int in, int pad, int kernel, int stride)
{
    /* op.c:549-555, unsigned arithmetic in the reference; hole == 1 */
    return (int)(((uint32_t)in + (uint32_t)pad * 2u - (uint32_t)kernel) / (uint32_t)stride + 1u);
}

int orc_pool_out_dim(int in, int pad, int kernel, int stride, int ceil_mode, int any_pad)
{
    /* op.c:931-955 */
    double v = ((double)(uint32_t)in + pad * 2.0 - (double)kernel) / (double)stride + 1;
    uint32_t o = (uint32_t)(ceil_mode ? ceil(v) : floor(v));
    if (any_pad) {
        if ((o - 1) * (uint32_t)stride >= (uint32_t)in + (uint32_t)pad)
            o--;
    }
    return (int)o;
}

/* the shared conv/ip epilogue: conv_2d_uint8_impl.c:159-164, ip.cpp:201-208 */
static inline uint8_t requant_acc(int32_t acc, uint32_t mult, int shift, int ozp, int obits)
{
    int64_t r = orc_rshift_rn((int64_t)acc * (int64_t)mult, shift) + ozp;
    return orc_sat_bits((int32_t)r, obits);
}

void orc_conv2d_u8(const uint8_t *x, const uint8_t *w, const int32_t *bias, uint8_t *y,
                   int32_t *acc_out, int N, int C, int H, int W, int K, int R, int S, int pad_h,
                   int pad_w, int stride_h, int stride_w, int group, float ialpha, int izp,
                   float walpha, int wzp, float oalpha, int ozp, int obits)
{
    const int OH = orc_conv_out_dim(H, pad_h, R, stride_h);
    const int OW = orc_conv_out_dim(W, pad_w, S, stride_w);
    const int cg = C / group, kg = K / group;
    uint32_t mult;
    int shift;
    orc_quant_scale(ialpha * walpha / oalpha, 32, &mult, &shift);

    int32_t *row = (int32_t *)malloc(sizeof(int32_t) * (size_t)OW);
    for (int n = 0; n < N; n++)
        for (int k = 0; k < K; k++) {
            const int g = k / kg;
            for (int oh = 0; oh < OH; oh++) {
                /* accumulate one output row; uint32 arithmetic = the wrapping int32 of the reference */
                for (int ow = 0; ow < OW; ow++)
                    row[ow] = bias ? bias[k] : 0;
                for (int c = 0; c < cg; c++)
                    for (int r = 0; r < R; r++) {
                        const int ih = oh * stride_h - pad_h + r;
                        if (ih < 0 || ih >= H)
                            continue;
                        const uint8_t *xr = x + (((size_t)n * C + (size_t)g * cg + c) * H + ih) * W;
                        const uint8_t *wr = w + (((size_t)k * cg + c) * R + r) * S;
                        for (int s = 0; s < S; s++) {
                            const int32_t wv = (int32_t)wr[s] - wzp;
                            if (wv == 0)
                                continue;
                            for (int ow = 0; ow < OW; ow++) {
                                const int iw = ow * stride_w - pad_w + s;
                                if (iw < 0 || iw >= W)
                                    continue;
                                row[ow] = (int32_t)((uint32_t)row[ow]
                                                    + (uint32_t)(((int32_t)xr[iw] - izp) * wv));
                            }
                        }
                    }
                size_t o = (((size_t)n * K + k) * OH + oh) * OW;
                for (int ow = 0; ow < OW; ow++) {
                    if (acc_out)
                        acc_out[o + ow] = row[ow];
                    y[o + ow] = requant_acc(row[ow], mult, shift, ozp, obits);
                }
            }
        }
    free(row);
}

/* ---- reference-shaped conv (timed "port" baseline) ------------------------------------------ */

static void transpose_i16(const int16_t *a, int16_t *t, size_t rows, size_t cols)
{
    for (size_t i = 0; i < rows; i++)
        for (size_t j = 0; j < cols; j++)
            t[j * rows + i] = a[i * cols + j];
}

static void transpose_i32(const int32_t *a, int32_t *t, size_t rows, size_t cols)
{
    for (size_t i = 0; i < rows; i++)
        for (size_t j = 0; j < cols; j++)
            t[j * rows + i] = a[i * cols + j];
}

void orc_conv2d_u8_refshape(const uint8_t *x, const uint8_t *w, const int32_t *bias, uint8_t *y,
                            int N, int C, int H, int W, int K, int R, int S, int pad_h, int pad_w,
                            int stride_h, int stride_w, int group, float ialpha, int izp,
                            float walpha, int wzp, float oalpha, int ozp, int obits)
{
    const int OH = orc_conv_out_dim(H, pad_h, R, stride_h);
    const int OW = orc_conv_out_dim(W, pad_w, S, stride_w);
    const size_t cg = (size_t)(C / group), kg = (size_t)(K / group);
    const size_t ohw = (size_t)OH * OW, kk = cg * R * S;
    const size_t xn = (size_t)C * H * W, wn = (size_t)K * kk;
    uint32_t mult;
    int shift;
    orc_quant_scale(ialpha * walpha / oalpha, 32, &mult, &shift);

    int16_t *x16 = (int16_t *)malloc(sizeof(int16_t) * xn);
    int16_t *w16 = (int16_t *)malloc(sizeof(int16_t) * wn);
    int16_t *col = (int16_t *)malloc(sizeof(int16_t) * ohw * kk);
    int16_t *wt = (int16_t *)malloc(sizeof(int16_t) * kg * kk);
    int32_t *acc = (int32_t *)malloc(sizeof(int32_t) * (size_t)K * ohw);
    int32_t *ct = (int32_t *)malloc(sizeof(int32_t) * kg * ohw);

    for (int n = 0; n < N; n++) { /* the reference handles one image per call */
        /* widening of activations AND weights happens on every run (conv_2d_uint8_impl.c:107-112) */
        for (size_t i = 0; i < xn; i++)
            x16[i] = (int16_t)(x[(size_t)n * xn + i] - izp);
        for (size_t i = 0; i < wn; i++)
            w16[i] = (int16_t)(w[i] - wzp);
        for (size_t k = 0; k < (size_t)K; k++)
            for (size_t p = 0; p < ohw; p++)
                acc[k * ohw + p] = bias ? bias[k] : 0;
        for (int g = 0; g < group; g++) {
            /* im2col: col[pixel][c*R*S + r*S + s] (im2col.cpp:487-855) */
            const int16_t *xg = x16 + (size_t)g * cg * H * W;
            for (int oh = 0; oh < OH; oh++)
                for (int ow = 0; ow < OW; ow++) {
                    int16_t *cp = col + ((size_t)oh * OW + ow) * kk;
                    for (size_t c = 0; c < cg; c++)
                        for (int r = 0; r < R; r++)
                            for (int s = 0; s < S; s++) {
                                int ih = oh * stride_h - pad_h + r, iw = ow * stride_w - pad_w + s;
                                *cp++ = (ih < 0 || ih >= H || iw < 0 || iw >= W)
                                    ? 0
                                    : xg[(c * H + ih) * W + iw];
                            }
                }
            /* gemm_i16xi16 (gemm.c:306-355): transpose C and A, axpy over M with zero skip, transpose back */
            int32_t *cg_acc = acc + (size_t)g * kg * ohw;
            transpose_i32(cg_acc, ct, kg, ohw);
            transpose_i16(w16 + (size_t)g * kg * kk, wt, kg, kk);
            for (size_t p = 0; p < ohw; p++) {
                int32_t *cc = ct + p * kg;
                const int16_t *bp = col + p * kk;
                for (size_t j = 0; j < kk; j++) {
                    const int16_t b = bp[j];
                    if (b == 0)
                        continue;
                    const int16_t *ap = wt + j * kg;
                    for (size_t m = 0; m < kg; m++)
                        cc[m] = (int32_t)((uint32_t)cc[m] + (uint32_t)((int32_t)b * ap[m]));
                }
            }
            transpose_i32(ct, cg_acc, ohw, kg);
        }
        uint8_t *yo = y + (size_t)n * K * ohw;
        for (size_t i = 0; i < (size_t)K * ohw; i++)
            yo[i] = requant_acc(acc[i], mult, shift, ozp, obits);
    }
    free(x16);
    free(w16);
    free(col);
    free(wt);
    free(acc);
    free(ct);
}

void orc_ip_u8(const uint8_t *x, const uint8_t *w, const int32_t *bias, uint8_t *y,
               int32_t *acc_out, int M, int Kdim, int Nout, float ialpha, int izp, float walpha,
               int wzp, float oalpha, int ozp, int obits)
{
    uint32_t mult;
    int shift;
    orc_quant_scale(ialpha * walpha / oalpha, 32, &mult, &shift);
    int16_t *xs = (int16_t *)malloc(sizeof(int16_t) * (size_t)Kdim);
    for (int m = 0; m < M; m++) {
        for (int k = 0; k < Kdim; k++)
            xs[k] = (int16_t)((int)x[(size_t)m * Kdim + k] - izp);
        for (int n = 0; n < Nout; n++) {
            uint32_t acc = bias ? (uint32_t)bias[n] : 0u;
            const uint8_t *wr = w + (size_t)n * Kdim;
            for (int k = 0; k < Kdim; k++)
                acc += (uint32_t)((int32_t)xs[k] * ((int32_t)wr[k] - wzp));
            if (acc_out)
                acc_out[(size_t)m * Nout + n] = (int32_t)acc;
            y[(size_t)m * Nout + n] = requant_acc((int32_t)acc, mult, shift, ozp, obits);
        }
    }
    free(xs);
}

void orc_add_u8(const uint8_t *a, const uint8_t *b, uint8_t *y, size_t count, float ialpha0,
                int izp0, float ialpha1, int izp1, float oalpha, int ozp, int obits)
{
    /* add.c:105-118: order the operands so that alpha0 <= alpha1 */
    if (ialpha0 > ialpha1) {
        float tf = ialpha0;
        ialpha0 = ialpha1;
        ialpha1 = tf;
        int tz = izp0;
        izp0 = izp1;
        izp1 = tz;
        const uint8_t *tp = a;
        a = b;
        b = tp;
    }
    uint32_t m0, m1;
    int s0, s1;
    orc_quant_scale(ialpha0 / oalpha, 23, &m0, &s0);
    orc_quant_scale(ialpha1 / oalpha, 23, &m1, &s1);
    const int sh = (s0 > s1 ? s1 : s0) - 1;
    for (size_t i = 0; i < count; i++) {
        int32_t i0 = (int32_t)a[i] - izp0;
        int32_t i1 = (int32_t)b[i] - izp1;
        /* uint32 * int32 wraps, then reinterpreted as int32 (add.c:138-139) */
        int32_t p0 = (int32_t)(m0 * (uint32_t)i0);
        int32_t p1 = (int32_t)(m1 * (uint32_t)i1);
        int32_t t = (int32_t)(orc_rshift_rn(p0, s0 - sh) + orc_rshift_rn(p1, s1 - sh));
        y[i] = orc_sat_bits((int32_t)(orc_rshift_rn(t, sh) + ozp), obits);
    }
}

void orc_eltwise_u8(const uint8_t *const *in, int n_in, const float *coeff, const float *ialpha,
                    const uint8_t *izp, uint8_t *y, size_t count, int operation, float oalpha,
                    int ozp, int obits)
{
    uint32_t *mult = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)n_in);
    int *shift = (int *)malloc(sizeof(int) * (size_t)n_in);
    int smin = 127; /* eltwise.c:243-251 */
    for (int n = 0; n < n_in; n++) {
        float c = coeff ? coeff[n] : 1.0f;
        orc_quant_scale(c * ialpha[n] / oalpha, 23, &mult[n], &shift[n]);
        if (smin > shift[n])
            smin = shift[n];
    }
    const int s0 = smin - 1; /* eltwise.c:156 */
    for (size_t i = 0; i < count; i++) {
        int32_t t = (operation == 2) ? (int32_t)0xffffffff : 0; /* eltwise.c:198: max starts at -1 */
        for (int n = 0; n < n_in; n++) {
            int32_t p = (int32_t)((uint32_t)((int32_t)in[n][i] - (int32_t)izp[n]) * mult[n]);
            int64_t r = orc_rshift_rn(p, shift[n] - s0);
            if (operation == 2) {
                int32_t ri = (int32_t)r;
                t = t < ri ? ri : t;
            } else {
                t = (int32_t)(t + r);
            }
        }
        y[i] = orc_sat_bits((int32_t)(orc_rshift_rn(t, s0) + ozp), obits);
    }
    free(mult);
    free(shift);
}

void orc_relu_u8(const uint8_t *x, uint8_t *y, size_t count, float ialpha, int izp, float oalpha,
                 int ozp, int obits)
{
    uint32_t mult;
    int shift;
    orc_quant_scale(ialpha / oalpha, 24, &mult, &shift);
    for (size_t i = 0; i < count; i++) {
        int32_t v = x[i] >= izp ? x[i] : izp;
        /* int32 * uint32 is evaluated unsigned and widened without sign (relu.c:104-107) */
        uint32_t p = (uint32_t)(v - izp) * mult;
        y[i] = orc_sat_bits((int32_t)(orc_rshift_rn((int64_t)p, shift) + ozp), obits);
    }
}

void orc_pool_u8(const uint8_t *x, uint8_t *y, int N, int C, int H, int W, int OH, int OW, int kh,
                 int kw, int pad_h, int pad_w, int stride_h, int stride_w, int method, float ialpha,
                 int izp, float oalpha, int ozp, int obits)
{
    if (method == 0) { /* pool.c:96-166 */
        uint32_t m32;
        int shift;
        orc_quant_scale(ialpha / oalpha, 16, &m32, &shift);
        const int32_t mult = (int32_t)(uint16_t)m32;
        for (int n = 0; n < N; n++)
            for (int c = 0; c < C; c++) {
                const uint8_t *xp = x + ((size_t)n * C + c) * H * W;
                for (int oh = 0; oh < OH; oh++)
                    for (int ow = 0; ow < OW; ow++) {
                        int hs = oh * stride_h - pad_h, ws = ow * stride_w - pad_w;
                        int he = hs + kh < H ? hs + kh : H, we = ws + kw < W ? ws + kw : W;
                        hs = hs > 0 ? hs : 0;
                        ws = ws > 0 ? ws : 0;
                        uint8_t mx = 0;
                        for (int i = hs; i < he; i++)
                            for (int j = ws; j < we; j++)
                                if (xp[i * W + j] > mx)
                                    mx = xp[i * W + j];
                        int32_t p = mult * ((int32_t)mx - izp);
                        y[(((size_t)n * C + c) * OH + oh) * OW + ow]
                            = orc_sat_bits((int32_t)(orc_rshift_rn(p, shift) + ozp), obits);
                    }
            }
        return;
    }
    /* pool.c:168-249: the divisor counts padding up to (H + pad), the scale is re-derived per window */
    for (int n = 0; n < N; n++)
        for (int oh = 0; oh < OH; oh++)
            for (int ow = 0; ow < OW; ow++) {
                int hs = oh * stride_h - pad_h, ws = ow * stride_w - pad_w;
                int he = hs + kh < H + pad_h ? hs + kh : H + pad_h;
                int we = ws + kw < W + pad_w ? ws + kw : W + pad_w;
                uint32_t pool_size = (uint32_t)((he - hs) * (we - ws));
                uint32_t mult;
                int shift;
                orc_quant_scale(ialpha / oalpha / pool_size, 16, &mult, &shift);
                hs = hs > 0 ? hs : 0;
                ws = ws > 0 ? ws : 0;
                he = he < H ? he : H;
                we = we < W ? we : W;
                for (int c = 0; c < C; c++) {
                    const uint8_t *xp = x + ((size_t)n * C + c) * H * W;
                    int32_t sum = 0;
                    for (int i = hs; i < he; i++)
                        for (int j = ws; j < we; j++)
                            sum += (int32_t)xp[i * W + j] - izp;
                    int32_t p = (int32_t)((uint32_t)mult * (uint32_t)sum);
                    y[(((size_t)n * C + c) * OH + oh) * OW + ow]
                        = orc_sat_bits((int32_t)(orc_rshift_rn(p, shift) + ozp), obits);
                }
            }
}

void orc_quantize_u8(const float *x, uint8_t *y, size_t count, float oalpha, int ozp, int obits)
{
    const float alpha = oalpha;
    const float beta = -(oalpha * (float)ozp); /* quantize.c:152: float * uint8 in fp32 */
    const float hi = (float)((1 << obits) - 1);
    for (size_t i = 0; i < count; i++) {
        float q = (x[i] - beta) / alpha; /* fp32 subtract, IEEE fp32 divide */
        /* quant_helper.h:38-41: the +0.5 is a double addition, then truncation */
        y[i] = q > hi ? (uint8_t)hi : (q < 0 ? 0 : (uint8_t)((double)q + 0.5));
    }
}

void orc_dequantize_u8(const uint8_t *x, float *y, size_t count, float ialpha, int izp)
{
    for (size_t i = 0; i < count; i++)
        y[i] = (float)((int)x[i] - izp) * ialpha; /* dequantize.c:121 */
}

/* Dequantize of int32 accumulators.  NO counterpart in the reference: op_dequantize_run_u8 / _i8 (dequantize.c:111-136)
 * read bytes only.  An accumulator of a convolution or inner product counts units of ialpha * walpha (the scale its
 * int32 bias is quantised with, python/docs/tutorial/switch/cuda_quant.rst:60), so its real value is the closed form
 * y = (float)acc * alpha with alpha = ialpha * walpha formed in fp32 by the caller: one int32 -> fp32 conversion (round to
 * nearest even beyond 2^24) and one fp32 multiply, like dequantize.c:121.  Pinned by that closed form only (numpy's
 * astype(float32) * float32 in tests/test_oracle.py): parity unpinned against any reference output. */
void orc_dequantize_i32(const int32_t *x, float *y, size_t count, float alpha)
{
    for (size_t i = 0; i < count; i++)
        y[i] = (float)x[i] * alpha;
}

/* op_quant_concat_run — concat.c:82-124: whatever `axis` says, the loop copies image by image and input by input,
 * i.e. it concatenates along dimension 1; every input is rescaled: (mult, shift) = gqs(ialpha_j / oalpha, 16),
 * y = sat(rrn(mult * (x - izp_j), shift) + ozp).  mult is a uint16_t, the product an int. */
void orc_concat_u8(const uint8_t *const *in, int n_in, const size_t *per_image, const float *ialpha,
                   const uint8_t *izp, uint8_t *y, int N, float oalpha, int ozp, int obits)
{
    for (int n = 0; n < N; n++)
        for (int j = 0; j < n_in; j++) {
            uint32_t mult;
            int shift;
            orc_quant_scale(ialpha[j] / oalpha, 16, &mult, &shift);
            mult &= 0xffff;
            const uint8_t *src = in[j] + (size_t)n * per_image[j];
            for (size_t k = 0; k < per_image[j]; k++) {
                const int32_t p = (int32_t)mult * ((int32_t)src[k] - (int32_t)izp[j]);
                *y++ = orc_sat_bits((int32_t)(orc_rshift_rn(p, shift) + ozp), obits);
            }
        }
}

/* op_quant_softmax_run — softmax.c:89-122: e = (float)exp((double)(ialpha * (x - izp))) (the argument is an fp32
 * product, exp is the C library's double routine), the sum runs in fp32 in channel order, and
 * y = saturate_float_by_bits(e / sum / oalpha + ozp) with every operation in fp32. */
void orc_softmax_u8(const uint8_t *x, uint8_t *y, size_t outer, size_t ch, size_t inner, float ialpha, int izp,
                    float oalpha, int ozp, int obits)
{
    const float hi = (float)((1 << obits) - 1);
    float *e = (float *)malloc(sizeof(float) * (ch ? ch : 1));
    for (size_t o = 0; o < outer; o++)
        for (size_t i = 0; i < inner; i++) {
            float sum = 0.f;
            for (size_t c = 0; c < ch; c++) {
                const size_t idx = (o * ch + c) * inner + i;
                e[c] = (float)exp((double)(ialpha * (float)((int)x[idx] - izp)));
                sum += e[c];
            }
            for (size_t c = 0; c < ch; c++) {
                const size_t idx = (o * ch + c) * inner + i;
                const float q = e[c] / sum / oalpha + (float)ozp;
                y[idx] = q > hi ? (uint8_t)hi : (q < 0 ? 0 : (uint8_t)((double)q + 0.5));
            }
        }
    free(e);
}

/* ---- int8 symmetric variants (no zero points) --------------------------------------------------- */

/* ssaturate_int_by_bits — quant_helper.h:43-47: clip to +-(2^bits - 1), then the implicit conversion of the
 * int result to the int8_t return type (two's complement truncation; with bits = 8 values beyond +-127 wrap). */
int8_t orc_ssat_bits(int32_t x, int bits)
{
    const int32_t m = (1 << bits) - 1;
    const int32_t c = x > m ? m : (x < -m ? -m : x);
    return (int8_t)(uint8_t)((uint32_t)c & 255u);
}

static inline int8_t requant_acc_i8(int32_t acc, uint32_t mult, int shift, int obits)
{
    /* conv_2d_int8_impl.c:148-172, ip.cpp:268-272: the int64 result of rshift_rn is passed to an int32_t parameter */
    return orc_ssat_bits((int32_t)orc_rshift_rn((int64_t)acc * (int64_t)mult, shift), obits);
}

/* per-channel weight scales: the epilogues above with (mult, shift) = get_quant_scale_int32(ialpha * walpha[k] / oalpha) */
void orc_requant_per_channel_u8(const int32_t *acc, uint8_t *y, size_t outer, size_t K, size_t inner, float ialpha,
                                const float *walpha, float oalpha, int ozp, int obits)
{
    for (size_t k = 0; k < K; k++) {
        uint32_t mult;
        int shift;
        orc_quant_scale(ialpha * walpha[k] / oalpha, 32, &mult, &shift);
        for (size_t o = 0; o < outer; o++)
            for (size_t i = 0; i < inner; i++) {
                const size_t at = (o * K + k) * inner + i;
                y[at] = requant_acc(acc[at], mult, shift, ozp, obits);
            }
    }
}

void orc_requant_per_channel_i8(const int32_t *acc, int8_t *y, size_t outer, size_t K, size_t inner, float ialpha,
                                const float *walpha, float oalpha, int obits)
{
    for (size_t k = 0; k < K; k++) {
        uint32_t mult;
        int shift;
        orc_quant_scale(ialpha * walpha[k] / oalpha, 32, &mult, &shift);
        for (size_t o = 0; o < outer; o++)
            for (size_t i = 0; i < inner; i++) {
                const size_t at = (o * K + k) * inner + i;
                y[at] = requant_acc_i8(acc[at], mult, shift, obits);
            }
    }
}

/* op_conv_2d_i8xi8_run — conv_2d_int8_impl.c:34-174 with im2col_i8 (utils/im2col.cpp:22-116: out-of-image taps
 * are 0) and the portable branch of gemm_i8xi8 (gemm/default/gemm.c:257-303: int32 += int8 * int8). */
void orc_conv2d_i8(const int8_t *x, const int8_t *w, const int32_t *bias, int8_t *y, int32_t *acc_out, int N,
                   int C, int H, int W, int K, int R, int S, int pad_h, int pad_w, int stride_h, int stride_w,
                   int group, float ialpha, float walpha, float oalpha, int obits)
{
    const int OH = orc_conv_out_dim(H, pad_h, R, stride_h);
    const int OW = orc_conv_out_dim(W, pad_w, S, stride_w);
    const int cg = C / group, kg = K / group;
    uint32_t mult;
    int shift;
    orc_quant_scale(ialpha * walpha / oalpha, 32, &mult, &shift);
    for (int n = 0; n < N; n++)
        for (int k = 0; k < K; k++) {
            const int g = k / kg;
            for (int oh = 0; oh < OH; oh++)
                for (int ow = 0; ow < OW; ow++) {
                    uint32_t acc = bias ? (uint32_t)bias[k] : 0u;
                    for (int c = 0; c < cg; c++)
                        for (int r = 0; r < R; r++) {
                            const int ih = oh * stride_h - pad_h + r;
                            if (ih < 0 || ih >= H)
                                continue;
                            for (int s = 0; s < S; s++) {
                                const int iw = ow * stride_w - pad_w + s;
                                if (iw < 0 || iw >= W)
                                    continue;
                                const int32_t xv = x[(((size_t)n * C + (size_t)g * cg + c) * H + ih) * W + iw];
                                const int32_t wv = w[(((size_t)k * cg + c) * R + r) * S + s];
                                acc += (uint32_t)(xv * wv);
                            }
                        }
                    const size_t o = (((size_t)n * K + k) * OH + oh) * OW + ow;
                    if (acc_out)
                        acc_out[o] = (int32_t)acc;
                    y[o] = requant_acc_i8((int32_t)acc, mult, shift, obits);
                }
        }
}

/* op_quant_ip_i8xi8_run — ip.cpp:211-274. */
void orc_ip_i8(const int8_t *x, const int8_t *w, const int32_t *bias, int8_t *y, int32_t *acc_out, int M,
               int Kdim, int Nout, float ialpha, float walpha, float oalpha, int obits)
{
    uint32_t mult;
    int shift;
    orc_quant_scale(ialpha * walpha / oalpha, 32, &mult, &shift);
    for (int m = 0; m < M; m++)
        for (int n = 0; n < Nout; n++) {
            uint32_t acc = bias ? (uint32_t)bias[n] : 0u;
            for (int k = 0; k < Kdim; k++)
                acc += (uint32_t)((int32_t)x[(size_t)m * Kdim + k] * (int32_t)w[(size_t)n * Kdim + k]);
            if (acc_out)
                acc_out[(size_t)m * Nout + n] = (int32_t)acc;
            y[(size_t)m * Nout + n] = requant_acc_i8((int32_t)acc, mult, shift, obits);
        }
}

/* op_quantize_run_i8 — quantize.c:159-185: alpha = (float)(1.0 / oalpha) (a double division), the product is
 * fp32, round() is the C library's (half away from zero), the double -> int conversion of clip()'s argument is
 * x86-64's cvttsd2si: values outside int32 (and NaN) become INT32_MIN. */
void orc_quantize_i8(const float *x, int8_t *y, size_t count, float oalpha, int obits)
{
    const float alpha = (float)(1. / (double)oalpha);
    const int l = (int)((1l << (obits - 1)) - 1);
    for (size_t i = 0; i < count; i++) {
        const double r = round((double)(x[i] * alpha));
        const int32_t v = (r >= -2147483648.0 && r < 2147483648.0) ? (int32_t)r : INT32_MIN;
        y[i] = (int8_t)(v > l ? l : (v < -l ? -l : v));
    }
}

/* op_dequantize_run_i8 — dequantize.c:125-136. */
void orc_dequantize_i8(const int8_t *x, float *y, size_t count, float ialpha)
{
    for (size_t i = 0; i < count; i++)
        y[i] = (float)x[i] * ialpha;
}

uint64_t orc_fnv1a64(const uint8_t *p, size_t n)
{
    uint64_t h = 1469598103934665603ull;
    for (size_t i = 0; i < n; i++)
        h = (h ^ p[i]) * 1099511628211ull;
    return h;
}

void orc_xorshift_fill(uint64_t *state, uint32_t *out, size_t n)
{
    uint64_t s = *state;
    for (size_t i = 0; i < n; i++) {
        s ^= s << 13;
        s ^= s >> 7;
        s ^= s << 17;
        out[i] = (uint32_t)(s >> 32);
    }
    *state = s;
}
