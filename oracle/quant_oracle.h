/*
 * CPU oracle for NART's quantized-inference operators.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the arithmetic of the reference CPU
 * `quant` module (art/modules/quant), used as the checker in tests, in the smoke run and as the
 * timed CPU baseline of the benchmark.  Nothing on the product path (the HIP library, the `hip`
 * case module, the host core) may call or link it.
 *
 * All tensors are dense NCHW (the reference's layout), uint8 unless stated.  Every function cites
 * the reference function whose results it must reproduce bit for bit.
 *
 * How each function is pinned (none of them is "parity unpinned"):
 *   - against the reference module itself, compiled from its own sources into oracle/_ref by
 *     oracle/Makefile (differential tests on random shapes and parameters),
 *   - against the ten conv known-answer checksums recorded from the reference (tests/golden),
 *   - against committed golden outputs produced by the compiled reference (the .npz files under tests/golden),
 *   - against independent numpy formulations (exact rational rounding, int64 einsum).
 *
 * Parameter domain: requantisation shifts must end up in [1, 62] (the reference shifts an int64 by
 * that amount; outside this range its behaviour is undefined in C and is not restated here).
 */
#ifndef NART_QUANT_ORACLE_H
#define NART_QUANT_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* get_quant_scale / _int16 / _int32 — quant_helper.h:60-118 (bits = 32, 16, 24, 23 are the callers' choices). */
void orc_quant_scale(float x, int bits, uint32_t *mult, int *shift);

/* rshift_rn — quant_helper.h:55-58. */
int64_t orc_rshift_rn(int64_t x, int bits);

/* saturate_int_by_bits — quant_helper.h:33-36. */
uint8_t orc_sat_bits(int32_t x, int bits);

/* Output extent of a convolution — art/src/op.c:549-555 (hole = 1). */
int orc_conv_out_dim(int in, int pad, int kernel, int stride);

/* Output extent of a pooling window sweep — art/src/op.c:931-955.  any_pad: pad_h || pad_w (the
 * "last window starts inside the padded image" correction applies to both axes once either pads). */
int orc_pool_out_dim(int in, int pad, int kernel, int stride, int ceil_mode, int any_pad);

/*
 * op_conv_2d_u8xu8_run — conv_2d_uint8_impl.c:39-165 (+ im2col.cpp:487, gemm.c:306).
 * x [N,C,H,W], w [K,C/group,R,S], bias [K] or NULL (NULL is defined as zero), y [N,K,OH,OW].
 * acc_out (optional) receives the int32 accumulators (bias included) in y's order.
 */
void orc_conv2d_u8(const uint8_t *x, const uint8_t *w, const int32_t *bias, uint8_t *y,
                   int32_t *acc_out, int N, int C, int H, int W, int K, int R, int S, int pad_h,
                   int pad_w, int stride_h, int stride_w, int group, float ialpha, int izp,
                   float walpha, int wzp, float oalpha, int ozp, int obits);

/*
 * The same operator computed the way the reference does it (widen to int16 every run, im2col,
 * transposed GEMM with zero skipping, scalar requantisation), one image at a time.  Only used as
 * the timed "port" CPU baseline when the compiled reference is not available.
 */
void orc_conv2d_u8_refshape(const uint8_t *x, const uint8_t *w, const int32_t *bias, uint8_t *y,
                            int N, int C, int H, int W, int K, int R, int S, int pad_h, int pad_w,
                            int stride_h, int stride_w, int group, float ialpha, int izp,
                            float walpha, int wzp, float oalpha, int ozp, int obits);

/* op_quant_ip_u8xu8_run — ip.cpp:133-209.  x [M,Kdim], w [Nout,Kdim], bias [Nout] or NULL, y [M,Nout]. */
void orc_ip_u8(const uint8_t *x, const uint8_t *w, const int32_t *bias, uint8_t *y,
               int32_t *acc_out, int M, int Kdim, int Nout, float ialpha, int izp, float walpha,
               int wzp, float oalpha, int ozp, int obits);

/* op_quant_add_run — add.c:83-148 (two inputs). */
void orc_add_u8(const uint8_t *a, const uint8_t *b, uint8_t *y, size_t count, float ialpha0,
                int izp0, float ialpha1, int izp1, float oalpha, int ozp, int obits);

/* op_quant_eltwise_accumulate_output_sum / _max + prepare — eltwise.c:137-271.  operation: 1 = SUM, 2 = MAX. */
void orc_eltwise_u8(const uint8_t *const *in, int n_in, const float *coeff, const float *ialpha,
                    const uint8_t *izp, uint8_t *y, size_t count, int operation, float oalpha,
                    int ozp, int obits);

/* op_quant_relu_run — relu.c:76-115. */
void orc_relu_u8(const uint8_t *x, uint8_t *y, size_t count, float ialpha, int izp, float oalpha,
                 int ozp, int obits);

/* op_quant_pool_max_run / op_quant_pool_average_run — pool.c:96-249.  method: 0 = MAX, else AVE. */
void orc_pool_u8(const uint8_t *x, uint8_t *y, int N, int C, int H, int W, int OH, int OW, int kh,
                 int kw, int pad_h, int pad_w, int stride_h, int stride_w, int method, float ialpha,
                 int izp, float oalpha, int ozp, int obits);

/* op_quantize_run_u8 — quantize.c:145-157 with saturate_float_by_bits, quant_helper.h:38-41. */
void orc_quantize_u8(const float *x, uint8_t *y, size_t count, float oalpha, int ozp, int obits);

/* op_dequantize_run_u8 — dequantize.c:111-123. */
void orc_dequantize_u8(const uint8_t *x, float *y, size_t count, float ialpha, int izp);
void orc_dequantize_i32(const int32_t *x, float *y, size_t count, float alpha);

/* op_quant_concat_run — concat.c:82-124.  per_image[j] = elements of input j per image (C_j*H*W). */
void orc_concat_u8(const uint8_t *const *in, int n_in, const size_t *per_image, const float *ialpha,
                   const uint8_t *izp, uint8_t *y, int N, float oalpha, int ozp, int obits);
/* op_quant_softmax_run — softmax.c:89-122 over [outer, ch, inner]. */
void orc_softmax_u8(const uint8_t *x, uint8_t *y, size_t outer, size_t ch, size_t inner, float ialpha, int izp,
                    float oalpha, int ozp, int obits);

/* ---- int8 symmetric variants: no zero points, outputs clipped to +-(2^obits - 1) and truncated to int8 ---- */
/* ssaturate_int_by_bits — quant_helper.h:43-47. */
int8_t orc_ssat_bits(int32_t x, int bits);
/* op_conv_2d_i8xi8_run — conv_2d_int8_impl.c:34-174 (x86-64 branch: gemm_i8xi8, i.e. ibits or wbits == 8). */
void orc_conv2d_i8(const int8_t *x, const int8_t *w, const int32_t *bias, int8_t *y, int32_t *acc_out, int N,
                   int C, int H, int W, int K, int R, int S, int pad_h, int pad_w, int stride_h, int stride_w,
                   int group, float ialpha, float walpha, float oalpha, int obits);
/* op_quant_ip_i8xi8_run — ip.cpp:211-274. */
void orc_ip_i8(const int8_t *x, const int8_t *w, const int32_t *bias, int8_t *y, int32_t *acc_out, int M,
               int Kdim, int Nout, float ialpha, float walpha, float oalpha, int obits);
/* op_quantize_run_i8 — quantize.c:159-185. */
void orc_quantize_i8(const float *x, int8_t *y, size_t count, float oalpha, int obits);
/* op_dequantize_run_i8 — dequantize.c:125-136. */
void orc_dequantize_i8(const int8_t *x, float *y, size_t count, float ialpha);

/* Per-channel weight scales.  The reference CPU module reads walpha[0] only (conv_2d_uint8_impl.c:57-66); its CUDA
 * sibling forms one scale ialpha * walpha[k] / oalpha per output channel (cuda_quant/src/op/conv_2d_quant.cu:751-764).
 * This is the CPU module's epilogue (conv_2d_uint8_impl.c:159-164 / conv_2d_int8_impl.c:148-172) with its (mult, shift)
 * pair derived per channel by get_quant_scale_int32: acc is [outer, K, inner] int32 (NCHW accumulators: outer = N,
 * inner = OH*OW; inner-product accumulators: outer = M, inner = 1).  Pinned by tests/test_oracle.py: equal scales give
 * the per-tensor functions' bytes, and exact rational rounding per channel. */
void orc_requant_per_channel_u8(const int32_t *acc, uint8_t *y, size_t outer, size_t K, size_t inner, float ialpha,
                                const float *walpha, float oalpha, int ozp, int obits);
void orc_requant_per_channel_i8(const int32_t *acc, int8_t *y, size_t outer, size_t K, size_t inner, float ialpha,
                                const float *walpha, float oalpha, int obits);

/* FNV-1a-64 over a byte buffer (the checksum the recorded known answers use). */
uint64_t orc_fnv1a64(const uint8_t *p, size_t n);

/* xorshift64 (13, 7, 17) stream used by the recorded known answers: out[i] = high 32 bits of the state. */
void orc_xorshift_fill(uint64_t *state, uint32_t *out, size_t n);

#ifdef __cplusplus
}
#endif
#endif
