// The network stem on gfx950: a strided convolution over an image with at most 4 channels, with the 3x3 / stride 2 /
// pad 1 max pooling that follows it computed in the same kernel.
//
// Reproduces op_conv_2d_u8xu8_run (art/modules/quant/src/op/conv_2d_uint8_impl.c:39-165) followed by
// op_quant_pool_max_run (art/modules/quant/src/op/pool.c:96-160) bit for bit, for a pooling operator whose input and
// output scale and zero point are equal (its rescale is then the identity, and a maximum of bytes is exact).
//
// Why one kernel: the stem writes the largest tensor of the network (64 x 112 x 112 x 64 bytes = 51 MB at batch 64) only
// for the pooling to read it back and keep a quarter.  Here the convolution's rows never leave the CU.
//   * a work-group owns PH = 4 pooled rows of one image, i.e. 9 convolution rows (the first is shared with the
//     work-group above: 12.5 % of the rows are computed twice), i.e. up to 24 input rows.  Those input rows - contiguous
//     in memory, 4 bytes per pixel - go into LDS ONCE with the load unit, one row per instruction, beside pad columns
//     that hold the byte izp; so do the packed weights (16 KB).  After that the kernel reads no global memory;
//   * k = (kernel row, 8 taps, 4 channels): a k-step of 32 bytes is one kernel row, and the pixel operand of
//     v_mfma_i32_32x32x32_i8 - lane (p, h): taps 4h .. 4h + 3 of output pixel p - is 16 CONSECUTIVE bytes of the input
//     row in LDS, at byte 4 (stride p - pad + 4h): closed-form addressing, no per-tap border tests (the borders are the
//     pad columns and pad rows);
//   * a wave computes 32 output pixels x 64 channels of a convolution row, requantises them (ReLU included) and parks the
//     bytes in one of three row buffers in LDS; every second row the 256 threads take the byte-wise maxima of the 3 x 3
//     windows from those buffers and write one pooled row with 128-bit stores.
// Requirements (checked by the host): uint8 tensors, input channel stride 4, at most 64 output channels with stride 64,
// kernel at most 8 x 8, horizontal pad at most 4, convolution rows of at most 128 pixels, image rows of at most 248
// pixels (a multiple of 4), weight zero point 128.
#include "conv_stem.h"

namespace hipq {

constexpr int kStemPH = 4;                    // pooled rows per work-group
constexpr int kStemCR = 2 * kStemPH + 1;      // convolution rows per work-group
constexpr int kStemPitch = 16 + 1024;         // bytes of a patch row: 4 pad pixels, then one 1 KB load
constexpr int kStemMaxPatchRows = 2 * (kStemCR - 1) * 1 + 8; // stride 2: 2 (CR - 1) + R rows, R <= 8

template <bool FAST>
__global__ __launch_bounds__(256) void conv_stem_maxpool_kernel(const ConvArgs a, uint8_t *yp, const int POH, const int POW,
                                                                const int nrb)
{
    constexpr int PITCH = kStemPitch, PR_MAX = kStemMaxPatchRows;
    constexpr int W_BYTES = 4 * 64 * 64;      // up to four slabs of 64 rows x 64 bytes
    constexpr int P_OFF = W_BYTES, R_OFF = P_OFF + PR_MAX * PITCH, ROWBUF = 128 * 64;
    __shared__ __attribute__((aligned(1024))) uint8_t lds[R_OFF + 3 * ROWBUF];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = (int)blockIdx.x / nrb, rb = (int)blockIdx.x % nrb;
    const int ph0 = rb * kStemPH;
    const int cr0 = 2 * ph0 - 1;                              // first convolution row (pool: stride 2, pad 1)
    const int ir0 = cr0 * a.stride_h - a.pad_h;               // first input row
    const int prows = (kStemCR - 1) * a.stride_h + a.R;       // input rows the 9 convolution rows touch

    // ---- everything this work-group will ever read, into LDS ----------------------------------------------
    for (int i = wave; i < a.nslab * 4; i += 4)               // packed weights: rows 0..63 of every slab
        __builtin_amdgcn_global_load_lds((gptr_t)(a.wpack + (size_t)(i >> 2) * a.kout_pad * 64 + (i & 3) * 1024 + lane * 16),
                                         (lptr_t)(lds + i * 1024), 16, 0, 0);
    const int wq = a.W >> 2;                                  // 16-byte pieces of an image row
    for (int j = wave; j < prows; j += 4) {
        const int ir = ir0 + j;
        const bool ok = (unsigned)ir < (unsigned)a.H && lane < wq;
        const uint8_t *src = ok ? a.x + ((size_t)(n * a.H + ir) * a.W) * 4 + lane * 16 : a.padbuf; // beyond the image: the byte izp
        __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(lds + P_OFF + j * PITCH + 16), 16, 0, 0);
    }
    if (tid < prows) {                                        // the four pad pixels left of every row
        const uint32_t pw = a.padword;
        *reinterpret_cast<u32x4 *>(lds + P_OFF + tid * PITCH) = u32x4{pw, pw, pw, pw};
    }
    __builtin_amdgcn_s_waitcnt(0); // vmcnt(0), lgkmcnt(0)
    __builtin_amdgcn_s_barrier();

    const int half = lane >> 5, p = lane & 31, swz = (lane >> 2) & 3;
    const int px = wave * 32 + p;                             // this lane's pixel of the convolution row
    const int owc = min(px, a.OW - 1);                        // lanes beyond the row compute a copy that is never stored
    const int boff = P_OFF + 16 + (owc * a.stride_w - a.pad_w + 4 * half) * 4; // + patch row * PITCH
    const int foff0 = p * 64 + (((0 + half) ^ swz) << 4), foff1 = p * 64 + (((2 + half) ^ swz) << 4);
    v4i bias[2][4];
#pragma unroll
    for (int tn = 0; tn < 2; tn++)
#pragma unroll
        for (int g = 0; g < 4; g++)
            bias[tn][g] = *reinterpret_cast<const v4i *>(a.bias2 + tn * 32 + g * 8 + half * 4);

    for (int i = 0; i < kStemCR; i++) {
        const int cr = cr0 + i;
        uint8_t *rowbuf = lds + R_OFF + (i % 3) * ROWBUF;
        if ((unsigned)cr < (unsigned)a.OH) {
            v16i acc[2];
#pragma unroll
            for (int tn = 0; tn < 2; tn++)
#pragma unroll
                for (int g = 0; g < 4; g++)
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        acc[tn][g * 4 + e] = bias[tn][g][e];
            const uint8_t *prow = lds + boff + (i * a.stride_h) * PITCH;
            for (int ks = 0; ks < a.R; ks++) {                // one kernel row = one k-step of 32 bytes
                const uint32_t *bp = reinterpret_cast<const uint32_t *>(prow + ks * PITCH);
                v4i bf = {(int)bp[0], (int)bp[1], (int)bp[2], (int)bp[3]};
                bf ^= (int)a.xmask;
                const uint8_t *wp = lds + (ks >> 1) * 4096 + ((ks & 1) ? foff1 : foff0);
                const v4i af0 = *reinterpret_cast<const v4i *>(wp), af1 = *reinterpret_cast<const v4i *>(wp + 2048);
                acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af0, bf, acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af1, bf, acc[1], 0, 0, 0);
            }
            if (px < a.OW) {
#pragma unroll
                for (int tn = 0; tn < 2; tn++)
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        int32_t rq[4];
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            rq[e] = conv_requant<FAST>(a, acc[tn][g * 4 + e]);
                        const int ch = tn * 32 + g * 8 + half * 4;
                        // 16-byte piece c of pixel px sits at piece c ^ (px & 3): spreads a wave's dword stores over the banks
                        *reinterpret_cast<uint32_t *>(rowbuf + px * 64 + (((ch >> 4) ^ (px & 3)) << 4) + (ch & 15))
                            = pack_low_bytes(rq[0], rq[1], rq[2], rq[3]);
                    }
            }
        }
        __syncthreads();
        if (i >= 2 && !(i & 1)) {
            const int ph = ph0 + ((i - 2) >> 1);
            const int pwi = tid >> 2, c16 = tid & 3;         // pooled pixel, group of 16 channels
            if (ph < POH && pwi < POW) {
                u32x4 mx = {0, 0, 0, 0};
#pragma unroll
                for (int r = 0; r < 3; r++) {
                    const int row = i - 2 + r;                // index among this work-group's convolution rows
                    if ((unsigned)(cr0 + row) >= (unsigned)a.OH)
                        continue;                             // pooling pads with nothing: the row does not take part
                    const uint8_t *rbuf = lds + R_OFF + (row % 3) * ROWBUF;
#pragma unroll
                    for (int c = 0; c < 3; c++) {
                        const int col = 2 * pwi - 1 + c;
                        if ((unsigned)col >= (unsigned)a.OW)
                            continue;
                        const u32x4 v = *reinterpret_cast<const u32x4 *>(rbuf + col * 64 + ((c16 ^ (col & 3)) << 4));
#pragma unroll
                        for (int d = 0; d < 4; d++)
                            mx[d] = max_u8x4(mx[d], v[d]);
                    }
                }
                *reinterpret_cast<u32x4 *>(yp + ((size_t)(n * POH + ph) * POW + pwi) * 64 + c16 * 16) = mx;
            }
            __syncthreads(); // the two older row buffers are free again
        }
    }
}

bool conv_stem_maxpool_applies(const ConvArgs &a, int smallc_rowb)
{
    return a.in_cs == 4 && a.out_cs == 64 && a.K <= 64 && a.R <= 8 && a.S <= 8 && smallc_rowb == 32 && a.stride_h == 2
        && a.stride_w == 2 && a.pad_w <= 4 && a.OW <= 128 && a.W % 4 == 0 && a.W <= 248 && a.nslab <= 4 && a.qmult == nullptr
        && a.group == 1 && (a.OW - 1) * 2 - a.pad_w + 7 < 252 && a.xmask != 0 && a.bwz == 0;
}

void launch_conv_stem_maxpool(const ConvArgs &a, uint8_t *yp, int POH, int POW, hipStream_t st)
{
    const int nrb = (POH + kStemPH - 1) / kStemPH;
    const dim3 grid(a.N * nrb), block(256);
    if (a.fastq)
        hipLaunchKernelGGL(conv_stem_maxpool_kernel<true>, grid, block, 0, st, a, yp, POH, POW, nrb);
    else
        hipLaunchKernelGGL(conv_stem_maxpool_kernel<false>, grid, block, 0, st, a, yp, POH, POW, nrb);
}

} // namespace hipq
