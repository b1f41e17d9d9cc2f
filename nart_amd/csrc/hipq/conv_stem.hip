// The network stem on gfx950: a strided convolution over an image with at most 4 channels, with the 3x3 / stride 2 /
// pad 1 max pooling that follows it computed in the same kernel.
//
// Reproduces op_conv_2d_u8xu8_run (art/modules/quant/src/op/conv_2d_uint8_impl.c:39-165) followed by
// op_quant_pool_max_run (art/modules/quant/src/op/pool.c:96-160) bit for bit, for a pooling operator whose input and
// output scale and zero point are equal (its rescale is then the identity, and a maximum of bytes is exact).
//
// Why one kernel: the stem writes the largest tensor of the network (64 x 112 x 112 x 64 bytes = 51 MB at batch 64) only
// for the pooling to read it back and keep a quarter.  Here the convolution's rows never leave the CU.
//   * a work-group owns `ph` pooled rows of one image (the host picks ph so that the grid fills the chip in whole
//     rounds), i.e. 2 ph + 1 convolution rows (the first is shared with the work-group above), i.e. 4 ph + R input
//     rows.  Those input rows - contiguous in memory, 4 bytes per pixel - go into LDS ONCE with the load unit, one row
//     per instruction, beside pad columns that hold the byte izp.  After that the kernel reads no global memory;
//   * k = (kernel row, 8 taps, 4 channels): a k-step of 32 bytes is one kernel row, and the pixel operand of
//     v_mfma_i32_32x32x32_i8 - lane (p, h): taps 4h .. 4h + 3 of output pixel p - is 16 CONSECUTIVE bytes of the input
//     row in LDS, at byte 4 (stride p - pad + 4h): closed-form addressing, no per-tap border tests (the borders are the
//     pad columns and pad rows).  The weight operands of all R k-steps (2 R x 4 registers) are loaded once and stay in
//     registers for every row;
//   * a wave computes 32 output pixels x 64 channels of a convolution row.  The vertical half of the pooling runs on
//     the int32 accumulators in registers (the same lane owns the same pixel column in every row, and a maximum
//     commutes with the monotonic requantisation): only one row in 2.25 is requantised.  Its bytes go to a row buffer
//     in LDS, from which the 256 threads take the horizontal 3-maxima and write one pooled row with 128-bit stores.
//   * NEXT (1 or 2): the 1x1 convolutions that read the 64 pooled channels (the first layer of the first bottleneck
//     block, 64 -> 64, and its projection shortcut, 64 -> 256) are computed on every pooled row while it is still in
//     LDS: their weights (fragment order, ConvArgs::wfrag) and folded biases wait in LDS, a wave takes one of the two
//     pixel tiles and every second 32-channel tile, two multiplies per tile.  The pooled row is written as well.
// Requirements (checked by the host): uint8 tensors, input channel stride 4, at most 64 output channels with stride 64,
// kernel rows of 5 to 8 taps, 5 to 8 kernel rows, stride 2, horizontal pad at most 4, convolution rows of at most 128
// pixels, image rows of at most 248 pixels (a multiple of 4), weight zero point 128.
#include <type_traits>

#include "conv_stem.h"
#include "conv_frag.h"

namespace hipq {

constexpr int kStemMaxPH = 7;                     // pooled rows per work-group, at most
constexpr int kStemPitch = 16 + 1024;             // bytes of a patch row: 4 pad pixels, then one 1 KB load
constexpr int kStemMaxPatchRows = 4 * kStemMaxPH + 8; // stride 2: 2 (2 ph) + R rows, R <= 8
constexpr int kStemRowBuf = 128 * 64;             // one requantised row: 128 pixels x 64 channels
constexpr int kStemPoolBuf = 64 * 64;             // NEXT: one pooled row, 64 pixel slots x 64 channels
constexpr int kStemNextCh = 320;                  // NEXT: output channels of the chained layers together, at most

template <int R, bool FAST, int NEXT>
__global__ __launch_bounds__(256, 2) void conv_stem_maxpool_kernel(const ConvArgs a, uint8_t *yp, const int POH, const int POW,
                                                                const int nrb, const int ph_per_wg, const ConvArgs an,
                                                                const ConvArgs an2)
{
    constexpr int PITCH = kStemPitch;
    constexpr int R_OFF = kStemMaxPatchRows * PITCH;
    constexpr int P_OFF = R_OFF + 2 * kStemRowBuf;
    constexpr int W_OFF = P_OFF + kStemPoolBuf;   // NEXT: the chained layers' weights, 64 bytes a channel, then their biases
    constexpr int B_OFF = W_OFF + kStemNextCh * 64;
    __shared__ __attribute__((aligned(1024))) uint8_t lds[NEXT ? B_OFF + kStemNextCh * 4 : P_OFF];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = (int)blockIdx.x / nrb, rb = (int)blockIdx.x % nrb;
    const int ph0 = rb * ph_per_wg;
    const int nph = min(ph_per_wg, POH - ph0);                // pooled rows of this work-group
    const int cr0 = 2 * ph0 - 1;                              // first convolution row (pool: stride 2, pad 1)
    const int ir0 = cr0 * 2 - a.pad_h;                        // first input row (convolution: stride 2)
    const int prows = 4 * nph + R;                            // input rows the 2 nph + 1 convolution rows touch

    // ---- the input rows this work-group will ever read, into LDS --------------------------------------------
    const int wq = a.W >> 2;                                  // 16-byte pieces of an image row
    for (int j = wave; j < prows; j += 4) {
        const int ir = ir0 + j;
        const bool ok = (unsigned)ir < (unsigned)a.H && lane < wq;
        const uint8_t *src = ok ? a.x + ((size_t)(n * a.H + ir) * a.W) * 4 + lane * 16 : a.padbuf; // beyond the image: the byte izp
        __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(lds + j * PITCH + 16), 16, 0, 0);
    }
    if (tid < prows) {                                        // the four pad pixels left of every row
        const uint32_t pw = a.padword;
        *reinterpret_cast<u32x4 *>(lds + tid * PITCH) = u32x4{pw, pw, pw, pw};
    }

    // ---- this lane's weight operands (rows p and 32 + p of the packed slabs, which hold two kernel rows each) and
    // its 32 folded biases, for the whole kernel
    const int half = lane >> 5, p = lane & 31, swz = (lane >> 2) & 3;
    v4i wreg[R][2];
#pragma unroll
    for (int ks = 0; ks < R; ks++)
#pragma unroll
        for (int tn = 0; tn < 2; tn++)
            wreg[ks][tn] = ldg128(a.wpack + (size_t)(ks >> 1) * a.kout_pad * 64 + (tn * 32 + p) * 64
                                  + (((2 * (ks & 1) + half) ^ swz) << 4));
    v16i bias[2];
#pragma unroll
    for (int tn = 0; tn < 2; tn++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const v4i b = *reinterpret_cast<const v4i *>(a.bias2 + tn * 32 + g * 8 + half * 4);
#pragma unroll
            for (int e = 0; e < 4; e++)
                bias[tn][g * 4 + e] = b[e];
        }
    // NEXT: the chained layers' weights (one slab: the 64 bytes of a channel's 64 inputs, tiles of 32 channels in
    // fragment order) and folded biases -> LDS, layer after layer
    if (NEXT) {
        const int k1 = an.K, k2 = NEXT == 2 ? an2.K : 0;
        for (int i = tid; i < (k1 + k2) * 4; i += 256) { // 16-byte pieces
            const uint8_t *src = i < k1 * 4 ? an.wfrag + (size_t)i * 16 : an2.wfrag + (size_t)(i - k1 * 4) * 16;
            *reinterpret_cast<v4i *>(lds + W_OFF + i * 16) = ldg128(src);
        }
        for (int i = tid; i < k1 + k2; i += 256)
            *reinterpret_cast<int32_t *>(lds + B_OFF + i * 4) = i < k1 ? an.bias2[i] : an2.bias2[i - k1];
        if (tid < kStemPoolBuf / 16) // pixel slots beyond the row are multiplied too: give them defined bytes
            *reinterpret_cast<u32x4 *>(lds + P_OFF + tid * 16) = u32x4{0, 0, 0, 0};
    }
    __builtin_amdgcn_s_waitcnt(0); // vmcnt(0), lgkmcnt(0)
    __builtin_amdgcn_s_barrier();

    const int px = wave * 32 + p;                             // this lane's pixel of the convolution row
    const int owc = min(px, a.OW - 1);                        // lanes beyond the row compute a copy that is never stored
    const uint8_t *bbase = lds + 16 + (owc * 2 - a.pad_w + 4 * half) * 4; // + patch row * PITCH
    constexpr int32_t kNone = -2147483647 - 1;                // a row outside the image takes no part in the maximum
    const bool sat = a.lo == 0 && a.q.hi == 255;              // the clamp is the saturation of the pack

    // convolution row i of this work-group: 32 pixels x 64 channels per wave, accumulators start from the bias
    auto conv_row = [&](int i, v16i(&acc)[2]) {
        if ((unsigned)(cr0 + i) >= (unsigned)a.OH) {
#pragma unroll
            for (int tn = 0; tn < 2; tn++)
#pragma unroll
                for (int e = 0; e < 16; e++)
                    acc[tn][e] = kNone;
            return;
        }
        const uint8_t *prow = bbase + (2 * i) * PITCH;
        v4i bf[R];
#pragma unroll
        for (int ks = 0; ks < R; ks++) {
            const uint32_t *bp = reinterpret_cast<const uint32_t *>(prow + ks * PITCH);
            bf[ks] = v4i{(int)bp[0], (int)bp[1], (int)bp[2], (int)bp[3]} ^ (int)a.xmask;
        }
        acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wreg[0][0], bf[0], bias[0], 0, 0, 0);
        acc[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wreg[0][1], bf[0], bias[1], 0, 0, 0);
#pragma unroll
        for (int ks = 1; ks < R; ks++) {
            acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wreg[ks][0], bf[ks], acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wreg[ks][1], bf[ks], acc[1], 0, 0, 0);
        }
    };

    v16i vm[2], acc[2];
    conv_row(0, vm);
    for (int j = 0; j < nph; j++) {
        conv_row(2 * j + 1, acc);
#pragma unroll
        for (int tn = 0; tn < 2; tn++)
#pragma unroll
            for (int e = 0; e < 16; e++)
                vm[tn][e] = max(vm[tn][e], acc[tn][e]);
        conv_row(2 * j + 2, acc);
        // the vertical maxima of pooled row j, requantised, into the row buffer; the last row starts the next maximum
        uint8_t *rowbuf = lds + R_OFF + (j & 1) * kStemRowBuf;
        if (px < a.OW) {
            // sat_c: the clamp range is exactly [0, 255] and the pack's saturation is the clamp (one test per row, not per dword)
            auto emit = [&](auto sat_c) {
#pragma unroll
                for (int tn = 0; tn < 2; tn++)
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        int32_t rq[4];
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            rq[e] = max(vm[tn][g * 4 + e], acc[tn][g * 4 + e]);
                        uint32_t packed;
                        if (FAST && decltype(sat_c)::value) {
                            packed = conv_requant4<true>(a, rq[0], rq[1], rq[2], rq[3]);
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; e++)
                                rq[e] = conv_requant<FAST>(a, rq[e]);
                            packed = pack_low_bytes(rq[0], rq[1], rq[2], rq[3]);
                        }
                        const int ch = tn * 32 + g * 8 + half * 4;
                        // 16-byte piece c of pixel px sits at piece c ^ (px & 3): spreads a wave's dword stores over the banks
                        *reinterpret_cast<uint32_t *>(rowbuf + px * 64 + (((ch >> 4) ^ (px & 3)) << 4) + (ch & 15)) = packed;
                    }
            };
            if (sat)
                emit(std::true_type{});
            else
                emit(std::false_type{});
        }
#pragma unroll
        for (int tn = 0; tn < 2; tn++)
            vm[tn] = acc[tn];
        // One barrier per pooled row: the buffers alternate, and a thread writes buffer (j & 1) again only after the
        // barrier of row j + 1, which every thread reaches after its reads of row j.
        __syncthreads();
        const int pwi = tid >> 2, c16 = tid & 3;              // pooled pixel, group of 16 channels
        if (pwi < POW) {
            u32x4 mx = {0, 0, 0, 0};
#pragma unroll
            for (int c = 0; c < 3; c++) {
                const int col = 2 * pwi - 1 + c;
                if ((unsigned)col >= (unsigned)a.OW)
                    continue;                                 // pooling pads with nothing: the column does not take part
                const u32x4 v = *reinterpret_cast<const u32x4 *>(rowbuf + col * 64 + ((c16 ^ (col & 3)) << 4));
#pragma unroll
                for (int d = 0; d < 4; d++)
                    mx[d] = max_u8x4(mx[d], v[d]);
            }
            *reinterpret_cast<u32x4 *>(yp + ((size_t)(n * POH + ph0 + j) * POW + pwi) * 64 + c16 * 16) = mx;
            if (NEXT) // 16-byte piece c of pooled pixel q at piece c ^ (q & 3)
                *reinterpret_cast<u32x4 *>(lds + P_OFF + pwi * 64 + ((c16 ^ (pwi & 3)) << 4)) = mx;
        }
        if (NEXT) {
            // every thread passes the next row's barrier only after its reads below: one buffer is enough
            __syncthreads();
            // wave w: pixel tile w & 1, pairs of neighbouring 32-channel tiles of each layer in turn with wave w ^ 2
            const int q = 32 * (wave & 1) + p;
            v4i b[2];
#pragma unroll
            for (int kk = 0; kk < 2; kk++) // both layers read the pooled bytes with the same zero point (the host checks)
                b[kk] = *reinterpret_cast<const v4i *>(lds + P_OFF + q * 64 + (((2 * kk + half) ^ (q & 3)) << 4)) ^ (int)an.xmask;
            const size_t pixn = (size_t)(n * POH + ph0 + j) * POW + q;
            // ch0: the layer's first channel among all chained channels; U neighbouring tiles at a time, so that one tile's
            // LDS reads and multiplies run under another's requantisation and a lane's two stores are 64 consecutive bytes
            auto tiles = [&](const ConvArgs &al, const int ch0, const int nt0, auto U) {
                v16i accn[U.value];
#pragma unroll
                for (int u = 0; u < U.value; u++) {
                    const int c = ch0 + 32 * (nt0 + u);
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const v4i bv = *reinterpret_cast<const v4i *>(lds + B_OFF + (c + 16 * half + 4 * g) * 4);
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            accn[u][4 * g + e] = bv[e];
                    }
                }
#pragma unroll
                for (int kk = 0; kk < 2; kk++)
#pragma unroll
                    for (int u = 0; u < U.value; u++) {
                        const uint8_t *wp = lds + W_OFF + (ch0 + 32 * (nt0 + u)) * 64 + lane * 16;
                        accn[u] = __builtin_amdgcn_mfma_i32_32x32x32_i8(*reinterpret_cast<const v4i *>(wp + kk * 1024), b[kk], accn[u], 0, 0, 0);
                    }
#pragma unroll
                for (int u = 0; u < U.value; u++) {
                    const v4i o = frag::requant16(al, accn[u], 0);
                    if (q < POW)
                        *reinterpret_cast<v4i *>(al.y + pixn * al.K + 32 * (nt0 + u) + 16 * half) = o;
                }
            };
            auto layer = [&](const ConvArgs &al, const int ch0) {
                const int ntl = al.K / 32; // a multiple of 2; the waves of a pixel tile (wave >> 1 = 0, 1) take pairs of tiles in turn
                if (ntl == 2) {
                    tiles(al, ch0, wave >> 1, std::integral_constant<int, 1>());
                    return;
                }
                for (int nt = 2 * (wave >> 1); nt < ntl; nt += 4)
                    tiles(al, ch0, nt, std::integral_constant<int, 2>());
            };
            layer(an, 0);
            if (NEXT == 2)
                layer(an2, an.K);
        }
    }
}

bool conv_stem_maxpool_applies(const ConvArgs &a, int smallc_rowb)
{
    return a.in_cs == 4 && a.out_cs == 64 && a.K <= 64 && a.R >= 5 && a.R <= 8 && a.S <= 8 && smallc_rowb == 32
        && a.stride_h == 2 && a.stride_w == 2 && a.pad_w <= 4 && a.OW <= 128 && a.W % 4 == 0 && a.W <= 248 && a.nslab <= 4
        && a.qmult == nullptr && a.group == 1 && (a.OW - 1) * 2 - a.pad_w + 7 < 252 && a.xmask != 0 && a.bwz == 0;
}

// Pooled rows per work-group: two work-groups fit a CU (their LDS), so the grid runs in rounds of 512; the cost of a choice
// is its number of rounds times the convolution rows a work-group computes.
static int stem_rows_per_wg(int N, int POH)
{
    int best = 1;
    long best_cost = 0;
    for (int ph = 1; ph <= kStemMaxPH; ph++) {
        const long wgs = (long)N * ((POH + ph - 1) / ph);
        const long cost = ((wgs + 511) / 512) * (2 * ph + 1 + 3); // + 3: the fixed part of a work-group (loads, weights)
        if (ph == 1 || cost < best_cost) {
            best = ph;
            best_cost = cost;
        }
    }
    return best;
}

template <int R>
static void launch_stem_r(const ConvArgs &a, uint8_t *yp, int POH, int POW, const ConvArgs *an, const ConvArgs *an2, hipStream_t st)
{
    const int ph = stem_rows_per_wg(a.N, POH), nrb = (POH + ph - 1) / ph;
    const dim3 grid(a.N * nrb), block(256);
    if (an && an2) // conv_stem_next_applies: the one-multiply requantisation
        hipLaunchKernelGGL((conv_stem_maxpool_kernel<R, true, 2>), grid, block, 0, st, a, yp, POH, POW, nrb, ph, *an, *an2);
    else if (an)
        hipLaunchKernelGGL((conv_stem_maxpool_kernel<R, true, 1>), grid, block, 0, st, a, yp, POH, POW, nrb, ph, *an, *an);
    else if (a.fastq)
        hipLaunchKernelGGL((conv_stem_maxpool_kernel<R, true, 0>), grid, block, 0, st, a, yp, POH, POW, nrb, ph, a, a);
    else
        hipLaunchKernelGGL((conv_stem_maxpool_kernel<R, false, 0>), grid, block, 0, st, a, yp, POH, POW, nrb, ph, a, a);
}

// the 1x1 convolutions that the stem's kernel computes on its pooled rows: from the 64 pooled channels to a multiple of 64
// channels, stride 1, on POH x POW pixels; an2 may be null; together at most kStemNextCh channels
bool conv_stem_next_applies(const ConvArgs &a, int POH, int POW, const ConvArgs &an, const ConvArgs *an2)
{
    auto ok = [&](const ConvArgs &l) {
        return l.R == 1 && l.S == 1 && l.pad_h == 0 && l.pad_w == 0 && l.stride_h == 1 && l.stride_w == 1 && l.group == 1 && l.C == 64
            && l.in_cs == 64 && l.K >= 64 && l.K % 64 == 0 && l.out_cs == l.K && l.nslab == 1 && l.kout_pad >= l.K && l.N == a.N
            && l.H == POH && l.W == POW && l.OH == POH && l.OW == POW && l.bwz == 0 && l.xmask == an.xmask && l.xmask != 0 && l.lo >= 0 && l.fastq
            && l.qmult == nullptr && l.acc_out == nullptr && l.deq_out == nullptr && l.res == nullptr && l.wfrag != nullptr;
    };
    return a.fastq && POW <= 64 && ok(an) && (!an2 || ok(*an2)) && an.K + (an2 ? an2->K : 0) <= kStemNextCh;
}

void launch_conv_stem_maxpool(const ConvArgs &a, uint8_t *yp, int POH, int POW, const ConvArgs *an, const ConvArgs *an2, hipStream_t st)
{
    switch (a.R) {
    case 5: launch_stem_r<5>(a, yp, POH, POW, an, an2, st); break;
    case 6: launch_stem_r<6>(a, yp, POH, POW, an, an2, st); break;
    case 7: launch_stem_r<7>(a, yp, POH, POW, an, an2, st); break;
    default: launch_stem_r<8>(a, yp, POH, POW, an, an2, st); break; // conv_stem_maxpool_applies: 5 <= R <= 8
    }
}


// ---------------------------------------------------------------------------------------------------------------------
// A 3x3 / stride 2 stem with no pooling behind it (MobileNet-style: RGB to 32 channels): the same idea, smaller.  Such a
// layer is all memory traffic (27 multiplies per output byte) and the register-staged tile kernel spends its time
// gathering taps with per-dword border tests.  Here a work-group owns `rb` output rows of one image; the 2 rb + 1 input
// rows go into LDS once (one row per load-unit instruction, pad columns and rows outside the image holding the byte
// izp); k = (kernel row, 4 taps, 4 channels) as the plan packs it for 3-tap rows, so a k-step of 32 bytes is TWO kernel
// rows - lane (p, h) reads 16 consecutive bytes of input row 2 oh - pad + 2 step + h - and the whole reduction is two
// multiplies (the fourth kernel row and every fourth tap carry weight zero: whatever bytes stand there count for
// nothing).  MFMA row i computes channel 16 ((i >> 2) & 1) + 4 (i >> 3) + (i & 3), so the 16 accumulators of a lane are
// 16 consecutive channels of its pixel and leave as one 128-bit store, a wave writing 1 KB of consecutive bytes.
// Requirements (checked by the host): uint8 tensors, input channel stride 4, output channel stride 32, 3 x 3, stride 2,
// horizontal pad at most 4, output rows of at most 128 pixels, image rows of at most 248 pixels (a multiple of 4),
// weight zero point 128, one scale for all channels.
constexpr int kStem3MaxRB = 8;                    // output rows per work-group, at most
constexpr int kStem3PatchRows = 2 * kStem3MaxRB + 2; // + 1 row of the last window, + 1 that only zero weights ever meet

template <bool FAST, bool SAT>
__global__ __launch_bounds__(256) void conv_stem3x3_kernel(const ConvArgs a, const int nrb, const int rb)
{
    constexpr int PITCH = kStemPitch;
    __shared__ __attribute__((aligned(1024))) uint8_t lds[kStem3PatchRows * PITCH];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = (int)blockIdx.x / nrb, oh0 = ((int)blockIdx.x % nrb) * rb;
    const int nrows = min(rb, a.OH - oh0);
    const int ir0 = oh0 * 2 - a.pad_h;
    const int prows = 2 * nrows + 1;

    const int wq = a.W >> 2;
    for (int j = wave; j < prows; j += 4) {
        const int ir = ir0 + j;
        const bool ok = (unsigned)ir < (unsigned)a.H && lane < wq;
        const uint8_t *src = ok ? a.x + ((size_t)(n * a.H + ir) * a.W) * 4 + lane * 16 : a.padbuf;
        __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(lds + j * PITCH + 16), 16, 0, 0);
    }
    if (tid < prows) {
        const uint32_t pw = a.padword;
        *reinterpret_cast<u32x4 *>(lds + tid * PITCH) = u32x4{pw, pw, pw, pw};
    }

    const int half = lane >> 5, p = lane & 31;
    const int ch = 16 * ((p >> 2) & 1) + 4 * (p >> 3) + (p & 3); // the channel MFMA row p computes
    v4i wreg[2];
#pragma unroll
    for (int ks = 0; ks < 2; ks++)
        wreg[ks] = ldg128(a.wpack + ch * 64 + (((2 * ks + half) ^ ((ch >> 2) & 3)) << 4));
    v16i bias;
#pragma unroll
    for (int g = 0; g < 4; g++) {
        const v4i b = *reinterpret_cast<const v4i *>(a.bias2 + 16 * half + 4 * g);
#pragma unroll
        for (int e = 0; e < 4; e++)
            bias[g * 4 + e] = b[e];
    }
    __builtin_amdgcn_s_waitcnt(0); // vmcnt(0), lgkmcnt(0)
    __builtin_amdgcn_s_barrier();

    const int px = wave * 32 + p;
    const int owc = min(px, a.OW - 1); // lanes beyond the row compute a copy that is never stored
    const uint8_t *bbase = lds + 16 + (owc * 2 - a.pad_w) * 4 + half * PITCH;
    uint8_t *yrow = a.y + ((size_t)(n * a.OH + oh0) * a.OW + px) * 32 + 16 * half;
    for (int i = 0; i < nrows; i++) {
        const uint32_t *b0 = reinterpret_cast<const uint32_t *>(bbase + (2 * i) * PITCH);
        const uint32_t *b1 = reinterpret_cast<const uint32_t *>(bbase + (2 * i + 2) * PITCH);
        const v4i bf0 = v4i{(int)b0[0], (int)b0[1], (int)b0[2], (int)b0[3]} ^ (int)a.xmask;
        const v4i bf1 = v4i{(int)b1[0], (int)b1[1], (int)b1[2], (int)b1[3]} ^ (int)a.xmask;
        v16i acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(wreg[0], bf0, bias, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(wreg[1], bf1, acc, 0, 0, 0);
        u32x4 out;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            if (SAT) { // clamp range exactly [0, 255]: saturating packs instead of clamps
                out[g] = conv_requant4<true>(a, acc[g * 4], acc[g * 4 + 1], acc[g * 4 + 2], acc[g * 4 + 3]);
            } else {
                out[g] = pack_low_bytes(conv_requant<FAST>(a, acc[g * 4]), conv_requant<FAST>(a, acc[g * 4 + 1]),
                                        conv_requant<FAST>(a, acc[g * 4 + 2]), conv_requant<FAST>(a, acc[g * 4 + 3]));
            }
        }
        if (px < a.OW)
            *reinterpret_cast<u32x4 *>(yrow + (size_t)i * a.OW * 32) = out;
    }
}

bool conv_stem3x3_applies(const ConvArgs &a, int smallc_rowb)
{
    return a.in_cs == 4 && a.out_cs == 32 && a.K <= 32 && a.R == 3 && a.S == 3 && smallc_rowb == 16 && a.stride_h == 2
        && a.stride_w == 2 && a.pad_w <= 4 && a.OW <= 128 && a.OW >= 1 && a.W % 4 == 0 && a.W <= 248 && a.nslab == 1
        && a.qmult == nullptr && a.group == 1 && (a.OW - 1) * 2 - a.pad_w + 3 < 256 && a.xmask != 0 && a.bwz == 0
        && a.res == nullptr && !plain_epilogue(a);
}

// Output rows per work-group: four work-groups fit a CU, so the grid runs in rounds of 1024; the cost of a choice is its
// number of rounds times the rows a work-group loads and computes.
static int stem3_rows_per_wg(int N, int OH)
{
    int best = 1;
    long best_cost = 0;
    for (int rb = 1; rb <= kStem3MaxRB; rb++) {
        const long wgs = (long)N * ((OH + rb - 1) / rb);
        const long cost = ((wgs + 1023) / 1024) * (rb + 2); // + 2: the fixed part of a work-group (loads, weights)
        if (rb == 1 || cost < best_cost) {
            best = rb;
            best_cost = cost;
        }
    }
    return best;
}

void launch_conv_stem3x3(const ConvArgs &a, hipStream_t st)
{
    const int rb = stem3_rows_per_wg(a.N, a.OH), nrb = (a.OH + rb - 1) / rb;
    const dim3 grid(a.N * nrb), block(256);
    if (a.fastq && a.lo == 0 && a.q.hi == 255)
        hipLaunchKernelGGL((conv_stem3x3_kernel<true, true>), grid, block, 0, st, a, nrb, rb);
    else if (a.fastq)
        hipLaunchKernelGGL((conv_stem3x3_kernel<true, false>), grid, block, 0, st, a, nrb, rb);
    else
        hipLaunchKernelGGL((conv_stem3x3_kernel<false, false>), grid, block, 0, st, a, nrb, rb);
}

} // namespace hipq
