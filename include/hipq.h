/*
 * hipq — C ABI of the MI355X (gfx950) quantized-inference kernels.
 *
 * This is the boundary between host code (the `hip` case module for NART's art runtime, the Python
 * runner, tests, benchmarks) and the hand-written HIP kernels.  Only plain C types cross it: device
 * and host pointers, sizes, scalars, one POD descriptor per operator and opaque plan handles.
 *
 * Each entry point names the function of the reference CPU `quant` module (paths relative to
 * art/modules/quant/) whose results it reproduces BIT-EXACTLY on the same inputs:
 *   - integer operators (conv, ip, add, eltwise, relu, pool): identical int32 accumulators and
 *     identical uint8 outputs, no tolerance;
 *   - quantize: IEEE fp32 subtract and divide followed by the reference's "+0.5 in double, truncate"
 *     rounding, identical bytes; dequantize: one fp32 multiply, identical bits.
 *
 * Device tensor layout.  The reference works on dense NCHW.  On the device, 4-D uint8 activations
 * are kept channels-last ("NHWC") with the channel count padded to a stride `cs`:
 *       element (n, c, h, w) lives at byte ((n*H + h)*W + w)*cs + c,          cs = hipq_channel_stride(C)
 * cs is 4 for C <= 4 (network inputs), otherwise C rounded up to a multiple of 16.  Bytes in the pad
 * channels are unspecified and never influence valid outputs.  2-D activations [M, K] are NHWC with
 * H = W = 1.  hipq_nchw_to_nhwc_u8 / hipq_nhwc_to_nchw_u8 convert at the host boundary.
 *
 * Conventions: every function returns 0 on success and a non-zero code on failure, with a
 * human-readable reason available from hipq_last_error().  `stream` is a hipStream_t passed as
 * void* (NULL = the default stream); all launches are asynchronous on it.  No function falls back to
 * host computation: without a usable GPU every compute entry point fails with an error.
 */
#ifndef HIPQ_H
#define HIPQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 3: per-channel weight scales, the fused stem (convolution + max pooling), the streaming and channel-widening kernels'
 * hooks, hipq_conv2d_plan_kernel_add.
 * 4: whole residual blocks in one launch (hipq_bottleneck_*, hipq_conv2d_run_add2, hipq_conv2d_run_maxpool_conv),
 * hipq_dequantize_i32; the machine probes (hipq_probe_launch) are gone.  Every other entry point of version 3 is unchanged. */
#define HIPQ_ABI_VERSION 4

#define HIPQ_ELTWISE_SUM 1 /* SETTING_ELTWISE_OP_SUM */
#define HIPQ_ELTWISE_MAX 2 /* SETTING_ELTWISE_OP_MAX */
#define HIPQ_POOL_MAX 0    /* SETTING_POOL_MAX */
#define HIPQ_POOL_AVE 1    /* SETTING_POOL_AVE */
#define HIPQ_MAX_ELTWISE_INPUTS 8
#define HIPQ_DTYPE_U8 0
#define HIPQ_DTYPE_I8 1

int hipq_abi_version(void);
const char *hipq_last_error(void);

/* Fixed-point scale decomposition, get_quant_scale* — include/art/quant/quant_helper.h:60-118. */
void hipq_quant_scale(float scale, int bits, uint32_t *mult, int *shift);

/* Channel stride of the device layout for a tensor with C channels. */
int hipq_channel_stride(int C);
/*
 * Host helper (no counterpart in the reference): the reciprocal with which the kernels divide by a run-time constant,
 * floor(x / d) == (uint32_t)(((uint64_t)x * *m) >> 32) >> *s for every 0 <= x < 2^31 (*m == 0: d is 1, the quotient
 * is x).  Returns -1 for d == 0 or a null pointer.
 */
int hipq_div_magic(uint32_t d, uint32_t *m, int *s);

/* ---- layout conversion at the host boundary (no counterpart in the reference, which is NCHW only) */
int hipq_nchw_to_nhwc_u8(const void *src_nchw, void *dst_nhwc, int N, int C, int H, int W, int cs,
                         void *stream);
int hipq_nhwc_to_nchw_u8(const void *src_nhwc, void *dst_nchw, int N, int C, int H, int W, int cs,
                         void *stream);

/* ---- convolution ---------------------------------------------------------------------------- */
typedef struct hipq_conv2d_desc {
    int32_t N, C, H, W;       /* input, logical dims */
    int32_t K, R, S;          /* output channels, kernel height / width */
    int32_t pad_h, pad_w, stride_h, stride_w, group;
    int32_t in_cs, out_cs;    /* channel strides of x and y on the device */
    float ialpha, walpha, oalpha;
    int32_t izp, wzp, ozp;    /* zero points, 0..255 */
    int32_t obits;            /* output saturates to [0, 2^obits - 1] */
    int32_t relu;             /* 1: y = max(y, ozp) after requantisation (== a following quant relu
                                 op with equal in/out scale and zero point, src/op/relu.c:76-115) */
    int32_t dtype;            /* HIPQ_DTYPE_U8 (0): asymmetric uint8 tensors, op_conv_2d_u8xu8_run.
                                 HIPQ_DTYPE_I8: int8 symmetric x, w and y, op_conv_2d_i8xi8_run
                                 (src/op/conv_2d_int8_impl.c:34-174) / op_quant_ip_i8xi8_run (src/op/ip.cpp:211-274):
                                 zero points are ignored, taps outside the image are 0, y is
                                 clip(v, -(2^obits - 1), 2^obits - 1) truncated to int8 (ssaturate_int_by_bits,
                                 quant_helper.h:43-47; obits = 8 wraps beyond +-127 exactly as the reference does) */
} hipq_conv2d_desc;

typedef struct hipq_conv2d_plan hipq_conv2d_plan;

/*
 * Setup: derives (mult, shift) from ialpha*walpha/oalpha, re-packs the weights for the kernel chosen
 * for this shape (int8 MFMA fragments for dense convolutions; tap-major vectors for depthwise) and
 * folds bias and the zero-point terms into one int32 per output channel; uploads both.
 * w: host, uint8 [K, C/group, R, S]; bias: host, int32 [K] or NULL (NULL == zeros).
 * Replaces op_quant_conv_2d_tp_prepare + the per-run widening in op_conv_2d_u8xu8_run
 * (src/op/conv_2d.c:95-147, src/op/conv_2d_uint8_impl.c:107-124).
 */
int hipq_conv2d_plan_create(const hipq_conv2d_desc *desc, const uint8_t *w, const int32_t *bias,
                            hipq_conv2d_plan **plan_out);
/*
 * The same with one weight scale per output channel: walpha is a host array of K floats that replaces desc->walpha, and
 * channel k is requantised with (mult, shift) = get_quant_scale_int32(ialpha * walpha[k] / oalpha)
 * (quant_helper.h:60-118) - the arithmetic of op_conv_2d_u8xu8_run (src/op/conv_2d_uint8_impl.c:57-66, 127-143) with
 * the pair chosen per channel.  The reference CPU module reads walpha[0] only; a per-channel array is what its CUDA
 * sibling accepts (art/modules/cuda_quant/src/op/conv_2d_quant.cu:751-764).  With K equal scales the result is
 * bit-identical to hipq_conv2d_plan_create.  Zero points, output scale, bias and clamps stay per tensor.  Every run entry
 * point works on such a plan (kernel name suffix "_perchannel").  Parity of the per-channel results is UNPINNED against the
 * reference: no reference output or fixture covers them (they are checked against this build's own oracle, exact rational
 * rounding per channel and "K equal scales == per tensor"), and the CUDA sibling named above rescales with float
 * multipliers ialpha * walpha[k] / oalpha rather than fixed-point pairs, so its rounding can differ in the last bit.
 */
int hipq_conv2d_plan_create_per_channel(const hipq_conv2d_desc *desc, const uint8_t *w, const int32_t *bias,
                                        const float *walpha, hipq_conv2d_plan **plan_out);
void hipq_conv2d_plan_destroy(hipq_conv2d_plan *plan);
/* Name of the kernel variant the plan dispatches to (for logs and tests). */
const char *hipq_conv2d_plan_kernel(const hipq_conv2d_plan *plan);
/* Name of the kernel variant that hipq_conv2d_run_add dispatches to for this plan, assuming the 32-bit form of the add
 * ("" for a plan that cannot fuse the add).  The string is valid until the calling thread's next call. */
const char *hipq_conv2d_plan_kernel_add(const hipq_conv2d_plan *plan);

/*
 * Tuning hook (no counterpart in the reference): choose the work-group tile (index: 0 128x128, 1 256x64, 2 128x64,
 * 3 64x128, 4 64x64 pixels x channels; -1 keeps the current one) and the number of load stages (2..4, or 8 for the
 * 64x128 / 64x64 tiles — other tiles then use 4; 0 = the built-in rule) of a plan that runs the DMA-fed MFMA kernel.  Every choice computes identical results; callers that
 * can time a whole network (nart_amd/runner.py) search the choices per layer.  Other plans return an error.
 */
int hipq_conv2d_plan_select(hipq_conv2d_plan *plan, int tile, int stages);
/*
 * Tuning hook (no counterpart in the reference) for the specialised MFMA kernels.  Halo-tile kernel (name
 * "..._halo"): 3x3 / stride 1 / pad 1 convolutions whose input channel stride is a multiple of 64 load each input tile with
 * its halo once and form the nine taps from LDS instead of streaming every tap from memory.  Pointwise kernel (name
 * "..._pointwise"): 1x1 / stride 1 convolutions with at most 64 input and 256 output channels (weight zero point 128)
 * feed the MFMA from global memory wave by wave, without LDS staging or barriers (hipq_conv2d_run only: the fused add
 * of hipq_conv2d_run_add and accumulator dumps take the tile kernel).  Two-group kernel (name "..._k2"): the tile
 * kernel with 512 threads, two groups of four waves that each reduce every other 64-byte slab of k and add their partial
 * accumulators through LDS (convolutions, with or without a fused residual add, with an even number of at least 8 slabs;
 * not with an explicit stage count).
 * Widening kernel (name "..._expand"): 1x1 convolutions without padding from 64, 128 or 256 input channels (stride) to
 * at least twice as many and 256 to 1024 output channels over at least 1024 pixels (weight zero point 128) keep a wave's
 * pixel operands in registers while a work-group walks a contiguous range of 128-pixel x 64-channel output tiles, with
 * the residual add of hipq_conv2d_run_add applied in place on a prefetched residual tile.
 * Rows kernel (name "..._rows3x3"): 3x3 / stride 1 / pad 1 convolutions with an input and output channel stride of 64
 * on rows of at most 64 pixels (weight zero point 128, one-multiply requantisation) keep the input rows of a work-group
 * in LDS and all weights in registers; the residual add of hipq_conv2d_run_add is applied to the bytes on their way out.
 * 3x3 stem kernel (name "..._stem3x3"): 3x3 / stride 2 convolutions of an image with at most 4 channels (channel stride 4,
 * rows of at most 248 pixels, a multiple of 4) to at most 32 channels (stride 32), weight zero point 128: the input rows
 * of a work-group in LDS, two multiplies per 32 pixels, 128-bit stores straight from the accumulators; modes 1 and 2.
 * mode 1 (the default) uses them where they measured faster: the rows kernel wherever it applies, the halo kernel for
 * the other 64-channel inputs up to 63 pixels wide, the pointwise kernel wherever it applies, the two-group kernel for layers with at most one tile per CU (256),
 * the widening kernel at 64 input channels with or without the add (from 150 000 pixels), with it at 128 (from 50 000)
 * and without it at 256 (from 20 000);
 * mode 2 the halo kernel instead of the rows kernel and also for 128, 256 and 512 channels (128-channel tiles, images up to 31 pixels wide), the
 * two-group kernel whatever the number of tiles and the widening kernel wherever it applies; mode 0 none of them.
 * Identical results in every mode.  Plans that do not run the MFMA kernel return an error.
 */
int hipq_conv2d_plan_special(hipq_conv2d_plan *plan, int mode);
/*
 * Tuning hook (no counterpart in the reference) for the streaming kernel (name "..._stream_<rows>x<cols>"): layers over
 * at most 256 output pixels (1024 where a pixel's reduction is at least 512 bytes long) whose input pixels are multiples
 * of 128 bytes (weight zero point 128, or int8) - the fully-connected layers, op_quant_ip_u8xu8_run
 * (src/op/ip.cpp:133-209), whose pixels are the batch, and convolutions of any kernel size, stride and padding over small
 * images (the late stages of a network at batch 1); hipq_conv2d_run_add fuses the residual add into it.  They
 * are bound by the weight stream, so the output is cut into strips of 16 or 32 channels, one work-group each, whose waves
 * split the reduction and stream their shares through LDS stages of their own into the 16x16x64 MFMA.  rows: pixel rows
 * per work-group (16, 32, 64 or 128), cols: 16 or 32 (128 x 32 does not exist), waves: 4; 0, 0, 0 returns to the built-in rule (one strip
 * shape that minimises what a CU pulls through its L1).  hipq_conv2d_plan_special(plan, 0) switches the kernel off, and so
 * does naming a tile with hipq_conv2d_plan_select.
 * Identical results for every choice.  Plans that the kernel does not serve return an error.
 */
int hipq_conv2d_plan_stream(hipq_conv2d_plan *plan, int rows, int cols, int waves);

/*
 * Run: op_conv_2d_u8xu8_run — src/op/conv_2d_uint8_impl.c:39-165 (im2col src/utils/im2col.cpp:487,
 * GEMM src/gemm/default/gemm.c:306).  x, y: device NHWC.  acc_out: optional device int32
 * [N*OH*OW, out_cs] that receives the raw accumulators (bias included), NULL to skip.
 * Unlike the reference (which aborts for N > 1, conv_2d_uint8_impl.c:104) any batch size runs.
 */
int hipq_conv2d_run(const hipq_conv2d_plan *plan, const void *x, void *y, int32_t *acc_out,
                    void *stream);

/*
 * Convolution with a ReLU fused into its epilogue, for a plan created with relu = 0: y = max(conv(x), ozp), which is
 * bit-identical to hipq_conv2d_run followed by hipq_relu_u8 with input and output scale and zero point equal to the
 * plan's oalpha / ozp and the plan's obits (op_conv_2d_u8xu8_run, then op_quant_relu_run — src/op/relu.c:76-115: with
 * equal scales the multiplier is exactly one).  The same as running a plan created with relu = 1; a caller that learns
 * only at run time that a ReLU follows (the art module) does not need a second plan.  uint8 plans only.
 */
int hipq_conv2d_run_relu(const hipq_conv2d_plan *plan, const void *x, void *y, void *stream);

/*
 * A fully-connected layer followed by the dequantize that reads it, in one launch: op_quant_ip_u8xu8_run
 * (art/modules/quant/src/op/ip.cpp:133-209), then op_dequantize_run_u8 (src/op/dequantize.c:111-123) on its bytes -
 * y[n][k] = (byte - ozp) * oalpha as float32, N x K dense; the uint8 output itself is not written.  Serves uint8 plans
 * whose output is one pixel per image and that run the streaming kernel; hipq_conv2d_dequant_fusable returns 1 for
 * those, given the dequantize's own scale and zero point (they must equal the plan's output parameters).
 */
int hipq_conv2d_dequant_fusable(const hipq_conv2d_plan *plan, float alpha, int zp);
int hipq_conv2d_run_dequant(const hipq_conv2d_plan *plan, const void *x, float *y, void *stream);
/*
 * Convolution with the residual add fused into its epilogue: y = add(conv(x), residual), bit-identical to
 * hipq_conv2d_run followed by hipq_add_u8 on the stored bytes (op_conv_2d_u8xu8_run, then op_quant_add_run —
 * src/op/add.c:83-148), but the convolution's own uint8 result never travels to memory.  `residual` has the
 * layout and geometry of y.  The add's inputs are (conv, residual), or (residual, conv) when
 * residual_is_input0 != 0; the convolution's output scale and zero point are the plan's oalpha / ozp, the
 * residual's are res_alpha / res_zp; oalpha / ozp / obits describe the sum.  Only plans that run an MFMA
 * kernel support it (others fail with an error: run the two operators separately).
 */
int hipq_conv2d_run_add(const hipq_conv2d_plan *plan, const void *x, const void *residual, int residual_is_input0,
                        float res_alpha, int res_zp, float oalpha, int ozp, int obits, void *y, void *stream);

/*
 * hipq_conv2d_run_add followed, in the same kernel, by the 1x1 convolution `next` that reads the sum (the last layer of
 * one bottleneck block, its residual add, and the first layer of the next block): y = add(conv(x), residual) and
 * y_next = next(y), bit-identical to hipq_conv2d_run_add followed by hipq_conv2d_run(next, y, y_next).  The sum is
 * written once and never read back.  Serves uint8 plans where `plan` is a 1x1 convolution from 64 or 128 to a multiple
 * of 64 (at most 1024) channels over at least 1024 pixels that the widening kernel computes, and `next` a 1x1 / stride 1
 * convolution of the same pixels to 64 or 128 channels (channel stride equal to that) whose input scale and zero point
 * are the sum's oalpha / ozp, obits 8, weight zero points 128, per-tensor weight scales.
 * hipq_conv2d_add_conv_fusable answers (1 / 0) whether two plans and an add can run this way;
 * hipq_conv2d_run_add_conv fails with an error otherwise.  A ReLU that `next` was created with applies to y_next;
 * next_relu != 0 applies the ReLU clamp of hipq_conv2d_run_relu to y_next whatever `next` was created with.
 */
int hipq_conv2d_add_conv_fusable(const hipq_conv2d_plan *plan, int residual_is_input0, float res_alpha, int res_zp,
                                 float oalpha, int ozp, int obits, const hipq_conv2d_plan *next);
int hipq_conv2d_run_add_conv(const hipq_conv2d_plan *plan, const void *x, const void *residual, int residual_is_input0,
                             float res_alpha, int res_zp, float oalpha, int ozp, int obits, void *y,
                             const hipq_conv2d_plan *next, int next_relu, void *y_next, void *stream);

/*
 * The last layer of a bottleneck block with a projection shortcut, in one launch: y = add(plan(x), shortcut(x_shortcut)),
 * bit-identical to hipq_conv2d_run(shortcut, x_shortcut, r) followed by hipq_conv2d_run_add(plan, x, residual = r, ...) -
 * op_conv_2d_u8xu8_run (src/op/conv_2d_uint8_impl.c:39-165) twice, then op_quant_add_run (src/op/add.c:83-148) - but the
 * shortcut's bytes never travel to memory.  `plan`: a 1x1 / stride 1 convolution from 256 or 512 channels; `shortcut`: a
 * 1x1 convolution, stride 1 or 2, from twice as many channels to the same output pixels and channels (a multiple of 128);
 * uint8 tensors with dense channel strides, weight zero points 128, per-tensor weight scales, no ReLU on the shortcut.
 * The add's inputs are (plan(x), shortcut(...)), or the other way round when shortcut_is_input0 != 0; oalpha / ozp /
 * obits (8) describe the sum.  hipq_conv2d_add2_fusable answers (1 / 0); hipq_conv2d_run_add2 fails with an error
 * otherwise (run the operators separately).
 */
int hipq_conv2d_add2_fusable(const hipq_conv2d_plan *plan, const hipq_conv2d_plan *shortcut, int shortcut_is_input0, float oalpha,
                             int ozp, int obits);
int hipq_conv2d_run_add2(const hipq_conv2d_plan *plan, const void *x, const hipq_conv2d_plan *shortcut, const void *x_shortcut,
                         int shortcut_is_input0, float oalpha, int ozp, int obits, void *y, void *stream);

/*
 * An identity bottleneck block of a residual network in one launch: y = add(widen(mid(reduce(x))), x), bit-identical to
 * hipq_conv2d_run(reduce, x, t1), hipq_conv2d_run(mid, t1, t2) and hipq_conv2d_run_add(widen, t2, residual = x, ...) -
 * op_conv_2d_u8xu8_run (src/op/conv_2d_uint8_impl.c:39-165) three times, then op_quant_add_run (src/op/add.c:83-148) -
 * but t1, t2 and the widening layer's own output never travel to memory.  `reduce`: a 1x1 / stride 1 convolution from
 * CW = 256, 512 or 1024 channels to CM = CW / 4; `mid`: 3x3 / stride 1 / pad 1, CM -> CM; `widen`: 1x1, CM -> CW; all on
 * images whose height and width are multiples of 7, uint8 tensors with dense channel strides, weight zero points 128,
 * per-tensor weight scales, each layer reading its input with the scale and zero point the previous one writes.  The
 * residual is x itself, read with `reduce`'s input scale and zero point; the add's inputs are (widen(...), x), or
 * (x, widen(...)) when residual_is_input0 != 0; oalpha / ozp / obits (8) describe the sum.  y must not be x.
 * hipq_bottleneck_fusable answers (1 / 0) whether three plans and an add can run this way; hipq_bottleneck_run fails
 * with an error otherwise (run the operators separately).
 */
int hipq_bottleneck_fusable(const hipq_conv2d_plan *reduce, const hipq_conv2d_plan *mid, const hipq_conv2d_plan *widen,
                            int residual_is_input0, float oalpha, int ozp, int obits);
int hipq_bottleneck_run(const hipq_conv2d_plan *reduce, const hipq_conv2d_plan *mid, const hipq_conv2d_plan *widen,
                        const void *x, int residual_is_input0, float oalpha, int ozp, int obits, void *y, void *stream);

/* The same with the 1x1 / stride 1 convolution that reads the sum computed in the kernel as well: y_next = next(y), with
 * `next` from CW to 2 CM channels (the first layer of the next stage; execute.c:43-90 runs it as one more operator),
 * reading the sum with the scale and zero point given for it; next_relu as in hipq_conv2d_run_relu.  The sum is written
 * too - the next stage's shortcut reads it.  x, y and y_next are three different tensors.
 * hipq_bottleneck_conv_fusable answers (1 / 0); hipq_bottleneck_run_conv fails with an error where it answers 0. */
int hipq_bottleneck_conv_fusable(const hipq_conv2d_plan *reduce, const hipq_conv2d_plan *mid, const hipq_conv2d_plan *widen,
                                 int residual_is_input0, float oalpha, int ozp, int obits, const hipq_conv2d_plan *next);
int hipq_bottleneck_run_conv(const hipq_conv2d_plan *reduce, const hipq_conv2d_plan *mid, const hipq_conv2d_plan *widen,
                             const void *x, int residual_is_input0, float oalpha, int ozp, int obits, void *y,
                             const hipq_conv2d_plan *next, int next_relu, void *y_next, void *stream);

/*
 * The rest of a bottleneck block in one launch, from its 3x3 convolution on: y = add(widen(mid(x)), residual) and, when
 * `next` is not NULL, y_next = next(y) - bit-identical to hipq_conv2d_run(mid, x, t), hipq_conv2d_run_add(widen, t,
 * residual, ...) and hipq_conv2d_run(next, y, y_next): op_conv_2d_u8xu8_run (src/op/conv_2d_uint8_impl.c:39-165), then
 * op_quant_add_run (src/op/add.c:83-148), then op_conv_2d_u8xu8_run again; t never travels to memory and y is written
 * but not read back.  `mid`: 3x3 / stride 1 / pad 1, CM -> CM with CM = 64, 128 or 256; `widen`: 1x1, CM -> 4 CM;
 * `next`: 1x1 / stride 1, 4 CM -> CM (the first layer of the next block); images of 8 x 8, 4 x 14 or 7 x 7 pixel patches
 * (height and width multiples of 8 and 8, of 4 and 14, or of 7 and 7); uint8 tensors with dense channel strides, weight
 * zero points 128, per-tensor weight scales, each layer reading its input with the scale and zero point it is written
 * with.  The residual (any tensor of y's shape, e.g. a projection shortcut) and the add are described as in
 * hipq_conv2d_run_add; next_relu as in hipq_conv2d_run_add_conv.  hipq_bottleneck_tail_fusable answers (1 / 0);
 * hipq_bottleneck_tail_run fails with an error otherwise (run the operators separately).
 */
int hipq_bottleneck_tail_fusable(const hipq_conv2d_plan *mid, const hipq_conv2d_plan *widen, int residual_is_input0,
                                 float res_alpha, int res_zp, float oalpha, int ozp, int obits, const hipq_conv2d_plan *next);
int hipq_bottleneck_tail_run(const hipq_conv2d_plan *mid, const hipq_conv2d_plan *widen, const void *x, const void *residual,
                             int residual_is_input0, float res_alpha, int res_zp, float oalpha, int ozp, int obits, void *y,
                             const hipq_conv2d_plan *next, int next_relu, void *y_next, void *stream);

/*
 * Convolution with the max pooling that follows it in one kernel: y = maxpool3x3/2/1(conv(x)), bit-identical to
 * hipq_conv2d_run followed by hipq_pool_u8(HIPQ_POOL_MAX, kernel 3, stride 2, pad 1) whose input and output scale and
 * zero point both equal the convolution's output parameters (op_conv_2d_u8xu8_run, then op_quant_pool_max_run -
 * src/op/pool.c:96-160: with equal scales the pooling's rescale is the identity).  Serves the stem of a residual
 * network: uint8 tensors, an input with at most 4 channels (channel stride 4), stride 2, at most 64 output channels,
 * convolution rows of at most 128 pixels, weight zero point 128, a per-tensor weight scale.  The convolution's own output
 * never travels to memory.  hipq_conv2d_maxpool_fusable answers (1 / 0) whether a plan and a pooling operator -
 * described by its settings and its output size OH x OW, as inferred by art/src/op.c:903-967 - can run this way;
 * hipq_conv2d_run_maxpool fails with an error otherwise (run the two operators separately).  y: NHWC [N, OH, OW, 64].
 * relu != 0 also applies the ReLU clamp of hipq_conv2d_run_relu between the two (conv, relu, pool as three operators
 * with equal scales: op_quant_relu_run is then max(x, zero point)).
 */
int hipq_conv2d_maxpool_fusable(const hipq_conv2d_plan *plan, int OH, int OW, int kernel, int stride, int pad, float ialpha,
                                int izp, float oalpha, int ozp, int obits);
int hipq_conv2d_run_maxpool(const hipq_conv2d_plan *plan, const void *x, void *y, int OH, int OW, int relu, void *stream);

/* The same with the 1x1 convolutions that read the pooled tensor computed in the kernel as well (ResNet: the first layer
 * of the first bottleneck block, 64 -> 64 channels, and that block's projection shortcut, 64 -> 256; execute.c:43-90
 * runs convolution, pooling and those convolutions as four operators): every pooled row is multiplied while it is still
 * on the chip.  The pooled tensor is written too.  `next` and `next2` (may be NULL, then next2_relu and y_next2 are
 * ignored) read the pooled tensor with the scale and zero point `plan` writes it with; each has a multiple of 64 output
 * channels, 320 together at most; next_relu as in hipq_conv2d_run_relu; y_next: NHWC [N, OH, OW, K of next], y_next2
 * likewise, all tensors distinct.  hipq_conv2d_maxpool_conv_fusable answers (1 / 0) whether the plans and a 3x3 / stride 2
 * / pad 1 pooling to OH x OW run this way; the run entry point fails with an error otherwise. */
int hipq_conv2d_maxpool_conv_fusable(const hipq_conv2d_plan *plan, int OH, int OW, const hipq_conv2d_plan *next,
                                     const hipq_conv2d_plan *next2);
int hipq_conv2d_run_maxpool_conv(const hipq_conv2d_plan *plan, const void *x, void *y, int OH, int OW, int relu,
                                 const hipq_conv2d_plan *next, int next_relu, void *y_next, const hipq_conv2d_plan *next2,
                                 int next2_relu, void *y_next2, void *stream);

/* ---- inner product: op_quant_ip_u8xu8_run — src/op/ip.cpp:133-209.
 * Expressed as a 1x1 convolution over M "pixels": desc {N=M, C=Kdim, H=W=1, K=Nout, R=S=1}.
 * When the reference's input is [M, C, H, W] with H*W > 1, pass the weights re-ordered from
 * (c, h, w) to (h, w, c-with-stride) — hipq_ip_reorder_weights does that on the host. */
int hipq_ip_reorder_weights(const uint8_t *w, uint8_t *w_out, int Nout, int C, int H, int W, int cs,
                            int wzp);

/* ---- element-wise --------------------------------------------------------------------------- */
/* op_quant_add_run — src/op/add.c:83-148.  count = number of bytes (pad channels included). */
int hipq_add_u8(const void *a, const void *b, void *y, size_t count, float ialpha0, int izp0,
                float ialpha1, int izp1, float oalpha, int ozp, int obits, void *stream);
/* op_quant_eltwise_accumulate_output_sum / _max — src/op/eltwise.c:137-271. */
int hipq_eltwise_u8(const void *const *in, int n_in, const float *coeff, const float *ialpha,
                    const uint8_t *izp, void *y, size_t count, int operation, float oalpha, int ozp,
                    int obits, void *stream);
/* op_quant_relu_run — src/op/relu.c:76-115. */
int hipq_relu_u8(const void *x, void *y, size_t count, float ialpha, int izp, float oalpha, int ozp,
                 int obits, void *stream);

/* op_quant_concat_run — src/op/concat.c:82-124: concatenation along the channels with a per-input rescale.
 * in[j]: NHWC with channels[j] channels (stride hipq_channel_stride(channels[j])); y: NHWC with the summed
 * channel count; npix = N*H*W. */
int hipq_concat_u8(const void *const *in, int n_in, const int *channels, const float *ialpha,
                   const uint8_t *izp, void *y, size_t npix, float oalpha, int ozp, int obits, void *stream);
/* op_quant_softmax_run — src/op/softmax.c:89-122, over the channels of every pixel (axis 1 of NCHW). */
int hipq_softmax_u8(const void *x, void *y, size_t npix, int C, int cs, float ialpha, int izp,
                    float oalpha, int ozp, int obits, void *stream);

/* ---- pooling: op_quant_pool_max_run / op_quant_pool_average_run — src/op/pool.c:96-249.
 * x: NHWC [N,H,W,cs], y: NHWC [N,OH,OW,cs]; OH, OW as inferred by art/src/op.c:903-967. */
int hipq_pool_u8(const void *x, void *y, int N, int C, int H, int W, int OH, int OW, int cs, int kh,
                 int kw, int pad_h, int pad_w, int stride_h, int stride_w, int method, float ialpha,
                 int izp, float oalpha, int ozp, int obits, void *stream);

/* ---- quantize / dequantize -------------------------------------------------------------------
 * op_quantize_run_u8 — src/op/quantize.c:145-157: x fp32 dense NCHW (as the host wrote it), y uint8
 * NHWC with stride cs (pass H = W = 1, cs = C for a flat tensor). */
int hipq_quantize_u8(const float *x_nchw, void *y_nhwc, int N, int C, int H, int W, int cs,
                     float oalpha, int ozp, int obits, void *stream);
/* op_dequantize_run_u8 — src/op/dequantize.c:111-123: x uint8 NHWC, y fp32 dense NCHW. */
int hipq_dequantize_u8(const void *x_nhwc, float *y_nchw, int N, int C, int H, int W, int cs,
                       float ialpha, int izp, void *stream);

/* op_quantize_run_i8 — src/op/quantize.c:159-185 (qtype SYMMETRIC, 2..8 bits): y int8 NHWC,
 * y = clip(round(x * (float)(1.0 / oalpha)), -(2^(obits-1) - 1), 2^(obits-1) - 1). */
int hipq_quantize_i8(const float *x_nchw, void *y_nhwc, int N, int C, int H, int W, int cs,
                     float oalpha, int obits, void *stream);
/* op_dequantize_run_i8 — src/op/dequantize.c:125-136: x int8 NHWC, y = x * ialpha, fp32 dense NCHW. */
int hipq_dequantize_i8(const void *x_nhwc, float *y_nchw, int N, int C, int H, int W, int cs,
                       float ialpha, void *stream);

/* Dequantize of int32 accumulators.  No counterpart in the reference (op_dequantize_run_u8 / _i8, src/op/dequantize.c:111-136,
 * read bytes only): x int32 NHWC [N, H, W, cs] as hipq_conv2d_run's acc_out writes it, y fp32 dense NCHW,
 * y = (float)x * alpha with alpha = ialpha * walpha formed in fp32 by the caller (the unit an accumulator and its int32
 * bias count in): one conversion, round to nearest even, and one fp32 multiply as in dequantize.c:121.  Checked against
 * that closed form only. */
int hipq_dequantize_i32(const int32_t *x_nhwc, float *y_nchw, int N, int C, int H, int W, int cs, float alpha, void *stream);

/* A plain device-to-device copy kernel of known size; the calibration reference for HBM counters. */
int hipq_copy_bytes(const void *src, void *dst, size_t count, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* HIPQ_H */
