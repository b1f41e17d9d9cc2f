// An identity bottleneck block of a residual network in ONE kernel: the 1x1 convolution that reduces the channels, the
// 3x3 convolution, the 1x1 convolution that widens them again and the residual add with the block's input.  gfx950 only.
//
// Reproduces, bit for bit, op_conv_2d_u8xu8_run (art/modules/quant/src/op/conv_2d_uint8_impl.c:39-165) three times and
// op_quant_add_run (art/modules/quant/src/op/add.c:83-148) on their bytes: every intermediate value is requantised,
// clamped and re-read exactly as if it had travelled through memory.
//
// Why: at 14x14 (and 28x28, 56x56) pixels per image and batch 64 the three layers are three launches that each find a
// few microseconds of matrix work per CU behind a launch, a cold start and a drain, and that hand 3 to 13 MB to one
// another through memory.  Here a work-group owns a 7x7 patch of ONE image through the whole block:
//   * x: the patch with a one-pixel border (at most 9x9 pixels, clipped to the image), all CW channels, is fetched once
//     into LDS by the load unit; it is the pixel operand of the first layer and, later, the residual;
//   * layer 1 (CW -> CM, CM = CW / 4) is computed for every pixel of that region - the border pixels are computed again by
//     the neighbouring patches' work-groups, which is the price of never synchronising work-groups - and its bytes go to
//     a 9x9 grid of pixel rows in LDS whose out-of-image positions hold the 3x3 layer's pad byte;
//   * layer 2 (3x3) reads its nine taps as nine shifted windows of that grid: output index m = 9 * row + column over
//     7 rows of 9 (two columns of each row are computed and dropped), so tap (dr, ds) of output m is grid row
//     m + 9 (dr + 1) + (ds + 1) - closed-form addressing, consecutive lanes on consecutive LDS rows; its bytes go to LDS;
//   * layer 3 (CM -> CW) reads them as its pixel operand, requantises, adds the residual from the x tile in LDS with
//     the reference's arithmetic and stores the sum.
// Weights never pass through LDS: the waves of a work-group split the OUTPUT CHANNELS, so no two waves want the same
// weight bytes, and a wave loads its MFMA weight operands straight from global memory (L2) into registers, a ring of
// slabs ahead of its multiplies; LDS bandwidth is left to the pixel operands.  The work-group has one wave per 32 middle
// channels: in layers 1 and 2 a wave owns a 32-channel tile for all pixels and the whole reduction, so the waves
// exchange nothing (splitting the reduction between two waves instead read every pixel operand once, not twice, but the
// exchange of partial sums through LDS and its barriers cost more than the reads: 28 -> 25.6 us per block at 14x14).  In
// layer 3 every wave owns 128 output channels, keeps its pixel operands for the whole reduction in registers and works
// through 4 chunks of 32 channels: multiplies of one wave run under the other's vector arithmetic of the add.
// MFMA rows are permuted (row i computes channel 16 ((i >> 2) & 1) + 4 (i >> 3) + (i & 3) of its 32) so that a lane's 16
// accumulators are 16 consecutive channels of one pixel: one 128-bit LDS or global store, no transpose.
// Requirements (checked by the host): uint8 tensors, weight zero points 128, per-tensor scales, one-multiply
// requantisation in all three layers, 32-bit form of the add to 8 bits, CM of 64, 128 or 256, image height and width
// multiples of 7.
#include "conv_block.h"
#include "conv_frag.h"

#include <algorithm>

namespace hipq {

using namespace frag;

namespace {

constexpr int kPatch = 7;          // a work-group's output pixels: kPatch x kPatch of one image
constexpr int kGridW = kPatch + 2; // the patch with its border: kGridW x kGridW pixel rows in LDS
constexpr int kGridRows = 96;      // rows held for that grid (81 positions; the row-padded output index reaches row 83)

// LDS tiles whose rows are the CM bytes of a pixel (the grid, layer 2's bytes): rows of 128 bytes or more lie 16 bytes
// further apart than their length, so that the lanes of a wave, which read the same 16-byte chunk of consecutive rows,
// fall on different bank groups, and a tap's shift on the grid is a constant added to the address (no swizzle to redo
// per tap); 64-byte rows read without conflicts as they are.
template <int CM>
constexpr int kRowStride = CM >= 128 ? CM + 16 : CM;
template <int CM>
__device__ static inline int row_off(int row, int chunk) { return row * kRowStride<CM> + (chunk << 4); }

struct BlockGeom {
    int H, W, PY, PX, npatch;
    int IH, IW; // the tail kernel's input image where its 3x3 layer has stride 2 (H, W: the output image)
};

} // namespace

// G = CM / 64 (1, 2, 4): 2 G waves.  MT1: pixel tiles of layer 1 (2: regions of at most 64 pixels, i.e. images of at
// most 2 x 2 patches; 3: up to 9 x 9 = 81).
// NX: 0, or 2 - the 1x1 convolution that reads the sum (CW -> 2 CM channels, the first layer of the next stage) is computed
// as well: the sum tile takes the x tile's place in LDS, row = output index m, and is that layer's pixel operand.
template <int G, int MT1, int NX>
__global__ __launch_bounds__(128 * G, 2) void conv_bottleneck_kernel(const ConvArgs a1, const ConvArgs a2, const ConvArgs a3,
                                                                    const ConvArgs an, const BlockGeom geo)
{
    constexpr int NW = 2 * G, NT = 128 * G, CM = 64 * G, CW = 256 * G;
    constexpr int X_BYTES = 32 * MT1 * CW;                  // the region's pixel rows, CW bytes each
    constexpr int G_OFF = X_BYTES, G_BYTES = kGridRows * kRowStride<CM>; // layer 1's bytes on the 9 x 9 grid, CM bytes a row; later layer 2's
    constexpr int D1 = MT1 == 2 ? 10 : 8, D2 = 10;          // slabs of weights a wave holds ahead, layers 1 and 2
    __shared__ __attribute__((aligned(1024))) uint8_t lds[G_OFF + G_BYTES];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int p = lane & 31, h = lane >> 5;

    // work-groups go to the 8 XCDs in turn: XCD x takes the x-th contiguous eighth of the patches, so the patches of an
    // image - which share border pixels - and all weights are read through one L2
    const int gid = (int)(blockIdx.x % 8) * (int)(gridDim.x / 8) + (int)(blockIdx.x / 8);
    if (gid >= geo.npatch)
        return;
    const int ppi = geo.PY * geo.PX;
    const int n = gid / ppi, pr = gid - n * ppi, pi = pr / geo.PX, pj = pr - pi * geo.PX;
    const int y0 = pi * kPatch, x0 = pj * kPatch;
    const int ry0 = max(y0 - 1, 0), rx0 = max(x0 - 1, 0);
    const int RW = min(x0 + kPatch, geo.W - 1) - rx0 + 1, RH = min(y0 + kPatch, geo.H - 1) - ry0 + 1;
    const int M1 = RW * RH;          // pixels of the region: at most 81 (64 when MT1 == 2: the host checks)
    const int rwinv = 65536 / RW + 1; // j / RW == (j * rwinv) >> 16 for 0 <= j < 128, 7 <= RW <= 9

    // ---- x region -> LDS: region pixel j at row j, its 16-byte piece c at piece c ^ (j & 15) of every 256 bytes ----
    {
        constexpr int LPR = CW / 16 >= 64 ? 64 : CW / 16, RPI = 64 / LPR; // lanes per pixel row, rows per wave instruction
        constexpr int NINST = X_BYTES / 1024;
        static_assert(CW <= 1024 && NINST % NW == 0, "a pixel row is at most one wave instruction");
        const int pos = lane % LPR;
#pragma unroll
        for (int q = 0; q < NINST / NW; q++) {
            const int i = wave + NW * q;
            const int j = i * RPI + lane / LPR;
            const int jj = min(j, M1 - 1); // rows beyond the region repeat its last pixel: computed, never used
            const int jy = (jj * rwinv) >> 16, jx = jj - jy * RW;
            const uint8_t *src = a1.x + (size_t)((n * geo.H + ry0 + jy) * geo.W + rx0 + jx) * CW + ((pos ^ (j & 15)) << 4);
            __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(lds + i * 1024), 16, 0, 0);
        }
    }
    // ---- the grid starts as the 3x3 layer's pad byte everywhere (re-centred like every byte kept there) ----
    {
        const int padw = (int)(a2.padword ^ a2.xmask);
        const v4i pv = {padw, padw, padw, padw};
#pragma unroll
        for (int o = tid * 16; o < G_BYTES; o += NT * 16)
            *reinterpret_cast<v4i *>(lds + G_OFF + o) = pv;
    }

    // Weight operands come in fragment order (ConvArgs::wfrag): the 1 KB a wave's load instruction fetches for slab s,
    // 32-channel tile T, k-step kk is contiguous at ((s * tiles + T) * 2 + kk) * 1024, lane l's 16 bytes at 16 l.
    // layers 1 and 2: a wave owns 32 of the CM channels and the whole reduction, so the waves exchange nothing
    const int ct0 = 32 * wave;
    const size_t wslab1 = (size_t)a1.kout_pad * 64, wslab2 = (size_t)a2.kout_pad * 64, wslab3 = (size_t)a3.kout_pad * 64;
    const uint8_t *w10 = a1.wfrag + (size_t)ct0 * 64 + lane * 16;
    const uint8_t *w20 = a2.wfrag + (size_t)ct0 * 64 + lane * 16;
    auto ldw1 = [&](int s, int kk) { return ldg128(w10 + (size_t)s * wslab1 + kk * 1024); };
    auto ldw2 = [&](int s, int kk) { return ldg128(w20 + (size_t)s * wslab2 + kk * 1024); };
    // layer 1, slab s: pieces 4 s .. 4 s + 3 of every pixel row of the x tile
    auto ldb1 = [&](int s, int kk, int t) {
        const int j = 32 * t + p, hs = h ^ (j & 15);
        return *reinterpret_cast<const v4i *>(lds + j * CW + (s >> 2) * 256 + (((4 * (s & 3) + 2 * kk) ^ hs) << 4));
    };
    // layer 2, slab s: channels 64 cb .. + 63 of tap (tap / 3, tap % 3), read at the tap's shift on the grid
    auto ldb2 = [&](int s, int kk, int t) {
        const int tap = s / G, cb = s % G, tr = (tap * 11) >> 5, off = tr * kGridW + (tap - 3 * tr);
        const int gr = 32 * t + p + off;
        return *reinterpret_cast<const v4i *>(lds + G_OFF + row_off<CM>(gr, 4 * cb + 2 * kk + h));
    };

    // ================= layer 1: CW -> CM on the region's pixels =================
    v16i acc1[MT1];
#pragma unroll
    for (int t = 0; t < MT1; t++)
        init_acc(acc1[t], a1.bias2 + ct0 + 16 * h, false);
    WeightRing1<D1> r1;
    ring_fill1<4 * G, D1>(r1, ldw1);
    // the region's bytes have landed (and this wave's pad bytes are written) before anyone reads LDS
    wait_vmcnt<0>();
    __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    reduce_all<4 * G, MT1, D1>(acc1, r1, (int)a1.xmask, ldw1, ldb1);
    // layer 2's first weights and folded biases travel while layer 1 is finished
    WeightRing1<D2> r2;
    ring_fill1<9 * G, D2>(r2, ldw2);
    v16i acc2[2];
#pragma unroll
    for (int t = 0; t < 2; t++)
        init_acc(acc2[t], a2.bias2 + ct0 + 16 * h, false);
    // channels ct0 + 16 h .. + 15 of region pixel j -> the grid position of that pixel
#pragma unroll
    for (int t = 0; t < MT1; t++) {
        const int j = 32 * t + p;
        if (j < M1) {
            const int jy = (j * rwinv) >> 16, jx = j - jy * RW;
            const int g = (ry0 + jy - y0 + 1) * kGridW + (rx0 + jx - x0 + 1);
            const v4i o = requant16(a1, acc1[t], a2.xmask);
            *reinterpret_cast<v4i *>(lds + G_OFF + row_off<CM>(g, (ct0 >> 4) + h)) = o;
        }
    }
    __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();

    // ================= layer 2: 3x3, CM -> CM, output index m = 9 * row + column =================
    reduce_all<9 * G, 2, D2>(acc2, r2, 0, ldw2, ldb2);
    // layer 3: this wave's 128 output channels in 4 chunks of 32; the first chunk's weights and biases travel now
    const uint8_t *w3 = a3.wfrag + (size_t)(128 * wave) * 64 + lane * 16;
    v4i wf[2 * G], b3[4];
    auto load_chunk = [&](int cc) {
#pragma unroll
        for (int ks = 0; ks < 2 * G; ks++)
            wf[ks] = ldg128(w3 + (size_t)(ks >> 1) * wslab3 + (size_t)cc * 2048 + (ks & 1) * 1024);
#pragma unroll
        for (int g = 0; g < 4; g++)
            b3[g] = *reinterpret_cast<const v4i *>(a3.bias2 + 128 * wave + 32 * cc + 16 * h + 4 * g);
    };
    load_chunk(0);
    v4i o2[2];
#pragma unroll
    for (int t = 0; t < 2; t++)
        o2[t] = requant16(a2, acc2[t], a3.xmask);
    __builtin_amdgcn_s_barrier(); // every wave is done reading the grid: layer 2's bytes go there, row m
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int m = 32 * t + p;
        const v4i o = o2[t];
        *reinterpret_cast<v4i *>(lds + G_OFF + row_off<CM>(m, (ct0 >> 4) + h)) = o;
    }
    __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();

    // ================= layer 3: CM -> CW and the residual add =================
    {
        v4i bf[2][2 * G]; // pixel operands of the whole reduction
        int jres[2];      // the output pixel's row in the x tile
        size_t yoff[2];
        bool valid[2];
        int pixo[2];
#pragma unroll
        for (int t = 0; t < 2; t++) {
            const int m = 32 * t + p;
#pragma unroll
            for (int ks = 0; ks < 2 * G; ks++)
                bf[t][ks] = *reinterpret_cast<const v4i *>(lds + G_OFF + row_off<CM>(m, 2 * ks + h));
            const int py = (m * 57) >> 9, px = m - py * kGridW; // m / 9 for m < 64
            valid[t] = py < kPatch && px < kPatch;
            jres[t] = valid[t] ? (y0 + py - ry0) * RW + (x0 + px - rx0) : 0;
            pixo[t] = (n * geo.H + y0 + py) * geo.W + x0 + px;
            yoff[t] = (size_t)pixo[t] * CW;
        }
        for (int cc = 0; cc < 4; cc++) {
            const int ch = 128 * wave + 32 * cc; // first of the chunk's 32 channels
            v16i acc[2];
#pragma unroll
            for (int g = 0; g < 4; g++)
#pragma unroll
                for (int e = 0; e < 4; e++)
                    acc[0][4 * g + e] = b3[g][e];
            acc[1] = acc[0];
#pragma unroll
            for (int ks = 0; ks < 2 * G; ks++)
#pragma unroll
                for (int t = 0; t < 2; t++)
                    acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[ks], bf[t][ks], acc[t], 0, 0, 0);
            if (cc + 1 < 4)
                load_chunk(cc + 1); // into the registers the multiplies above have read: they arrive during the arithmetic below
            const int c16 = (ch >> 4) + h; // the 16-byte piece of the pixel's CW bytes
            v4i res[2];
#pragma unroll
            for (int t = 0; t < 2; t++)
                res[t] = *reinterpret_cast<const v4i *>(lds + jres[t] * CW + (c16 & ~15) * 16 + (((c16 & 15) ^ (jres[t] & 15)) << 4));
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const v4i o = requant_add16(a3, acc[t], res[t]);
                if (valid[t])
                    *reinterpret_cast<v4i *>(a3.y + yoff[t] + ch + 16 * h) = o;
                if (NX) {
                    // the sum tile over the x tile: only this wave ever touches these 16-byte pieces (its own channels), and
                    // every lane has read its residuals of this chunk above
                    const int m = 32 * t + p;
                    *reinterpret_cast<v4i *>(lds + m * CW + (c16 & ~15) * 16 + (((c16 & 15) ^ (m & 15)) << 4)) = o;
                }
            }
        }
        if (!NX)
            return;
        // ================= the next stage's first layer: CW -> NX * CM on the sum tile =================
        // a wave owns the 32-channel tiles wave, wave + NW, ... one after the other
        const size_t wslabn = (size_t)an.kout_pad * 64;
#pragma unroll
        for (int jx = 0; jx < (NX ? NX : 1); jx++) {
            const int cn = 32 * (wave + NW * jx);
            const uint8_t *wn0 = an.wfrag + (size_t)cn * 64 + lane * 16;
            auto ldwn = [&](int s, int kk) { return ldg128(wn0 + (size_t)s * wslabn + kk * 1024); };
            WeightRing1<D1> rr;
            ring_fill1<4 * G, D1>(rr, ldwn);
            v16i accn[2];
#pragma unroll
            for (int t = 0; t < 2; t++)
                init_acc(accn[t], an.bias2 + cn + 16 * h, false);
            if (jx == 0) {
                __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): this wave's part of the sum tile is written
                __builtin_amdgcn_s_barrier();
            }
            reduce_all<4 * G, 2, D1>(accn, rr, (int)an.xmask, ldwn, ldb1);
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const v4i o = requant16(an, accn[t], 0);
                if (valid[t])
                    *reinterpret_cast<v4i *>(an.y + (size_t)pixo[t] * (NX * CM) + cn + 16 * h) = o;
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// The same machinery cut one layer later: the 3x3 convolution of a bottleneck block, its widening 1x1 convolution with
// the residual add, and - CHAIN - the 1x1 convolution that reads the sum (the first layer of the NEXT block), for the
// stages with many pixels per image (56x56, 28x28).  Cutting the chain at the narrowest tensor means that a work-group
// re-reads a border of 64 G bytes per pixel instead of recomputing a layer on it, needs no x tile in LDS (the residual
// may be any tensor, e.g. a projection shortcut, and comes straight from memory a chunk ahead of its use), and - the
// next layer being 1x1 - can finish that layer for exactly its own pixels.  A work-group owns a PH x PW patch of one
// image (8x8, 4x14 or 7x7: 64, 56 or 49 of its 64 pixel slots do useful vector arithmetic):
//   * the patch of the 3x3 layer's input with its border, (PH + 2) x (PW + 2) pixel rows of CM bytes, goes to LDS
//     (out-of-image positions hold the pad byte);
//   * layer 2 (3x3) as above, on the compact pixel index q = PW * row + column, its bytes to LDS;
//   * layer 3 + add as above, the sum stored and - CHAIN - kept in LDS, 64 pixel rows of CW bytes;
//   * CHAIN: the next layer (CW -> CM, or CW -> 2 CM where the next stage begins) reads that tile as its pixel operand.
// ST: the 3x3 layer's stride (1, or 2 - the first block of a stage: the grid then holds (2 PH + 1) x (2 PW + 1) input pixels).
template <int G, int PH, int PW, int NX, int ST>
__global__ __launch_bounds__(128 * G, (G == 1 ? (NX ? 4 : 3) : G == 2 ? (NX && ST == 1 && (NX == 1 || PH == 4) ? 4 : 3) : 2)) void conv_bottleneck_tail_kernel(const ConvArgs a2, const ConvArgs a3, const ConvArgs an,
                                                                         const BlockGeom geo)
{
    constexpr int NW = 2 * G, NT = 128 * G, CM = 64 * G, CW = 256 * G;
    constexpr bool CHAIN = NX != 0; // the next layer has NX * CM output channels
    constexpr int GW = ST * (PW - 1) + 3, GH = ST * (PH - 1) + 3, NPIX = PH * PW, GROWS = (GH * GW + 7) / 8 * 8;
    constexpr int G_OFF = 0, G_BYTES = GROWS * kRowStride<CM>;            // layer 2's input on the bordered grid
    constexpr int M_OFF = G_OFF + G_BYTES, M_BYTES = 64 * kRowStride<CM>; // layer 2's bytes, row = pixel
    // the sum tile takes the place of the grid and of layer 2's bytes once every wave holds its operands of layer 3
    constexpr int S_OFF = 0, S_BYTES = CHAIN ? 64 * CW : 0;
    // LDSB: layer 3's folded biases wait in LDS instead of in registers a chunk ahead - 16 registers less at the add's
    // arithmetic, which is what lets the 128-channel chained form keep four waves per SIMD (896 work-groups at 28x28 and
    // batch 64: one round of 1024 slots instead of 768 and a nearly empty second round)
    constexpr bool LDSB = G == 2 && CHAIN && ST == 1;
    constexpr int B3_OFF = (M_OFF + M_BYTES > S_BYTES ? M_OFF + M_BYTES : S_BYTES), B3_BYTES = LDSB ? 4 * CW : 0;
    constexpr int D2 = G == 1 ? 4 : G == 2 ? 6 : 10, DN = D2; // slabs of weights a wave holds ahead (four or three waves per SIMD: fewer registers)
    static_assert(NPIX <= 64, "pixel slots");
    __shared__ __attribute__((aligned(1024))) uint8_t lds[B3_OFF + B3_BYTES];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int p = lane & 31, h = lane >> 5;
    const int gid = (int)(blockIdx.x % 8) * (int)(gridDim.x / 8) + (int)(blockIdx.x / 8); // XCD x: the x-th eighth of the patches
    if (gid >= geo.npatch)
        return;
    const int ppi = geo.PY * geo.PX;
    const int n = gid / ppi, pr = gid - n * ppi, pi = pr / geo.PX, pj = pr - pi * geo.PX;
    const int y0 = pi * PH, x0 = pj * PW;

    // ---- the 3x3 layer's input patch with its border -> LDS, re-centred; out-of-image positions read the pad source ----
    {
        constexpr int CPR = CM / 16, ITEMS = GROWS * CPR;
#pragma unroll
        for (int k = 0; k < (ITEMS + NT - 1) / NT; k++) {
            const int it = tid + k * NT;
            if (ITEMS % NT == 0 || it < ITEMS) {
                const int g = it / CPR, c = it % CPR;
                const int gy = g / GW, gx = g - gy * GW;
                const int iy = ST * y0 - 1 + gy, ix = ST * x0 - 1 + gx;
                const int ih = ST == 1 ? geo.H : geo.IH, iw = ST == 1 ? geo.W : geo.IW;
                const bool in = g < GH * GW && (unsigned)iy < (unsigned)ih && (unsigned)ix < (unsigned)iw;
                const uint8_t *src = in ? a2.x + (size_t)((n * ih + iy) * iw + ix) * CM + c * 16 : a2.padbuf;
                *reinterpret_cast<v4i *>(lds + G_OFF + row_off<CM>(g, c)) = ldg128(src) ^ (int)a2.xmask;
            }
        }
    }
    if (LDSB) {
        for (int i = tid * 4; i < CW; i += NT * 4)
            *reinterpret_cast<v4i *>(lds + B3_OFF + i * 4) = *reinterpret_cast<const v4i *>(a3.bias2 + i);
    }
    const int ct0 = 32 * wave; // layers 2 and next: a wave owns 32 of the CM channels and the whole reduction
    const size_t wslab2 = (size_t)a2.kout_pad * 64, wslab3 = (size_t)a3.kout_pad * 64, wslabn = (size_t)an.kout_pad * 64;
    const uint8_t *w20 = a2.wfrag + (size_t)ct0 * 64 + lane * 16;
    auto ldw2 = [&](int s, int kk) { return ldg128(w20 + (size_t)s * wslab2 + kk * 1024); };
    // the lane's pixels q = 32 t + p (slots beyond the patch repeat its last pixel and are never stored)
    int grow[2];
    size_t pix[2];
    bool valid[2];
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int q = 32 * t + p, qq = min(q, NPIX - 1), py = qq / PW, px = qq - py * PW;
        valid[t] = q < NPIX;
        grow[t] = (ST * py + 1) * GW + ST * px + 1; // the centre tap's grid row
        pix[t] = (size_t)((n * geo.H + y0 + py) * geo.W + x0 + px);
    }
    auto ldb2 = [&](int s, int kk, int t) {
        const int tap = s / G, cb = s % G, tr = (tap * 11) >> 5;
        const int gr = grow[t] + (tr - 1) * GW + (tap - 3 * tr - 1);
        return *reinterpret_cast<const v4i *>(lds + G_OFF + row_off<CM>(gr, 4 * cb + 2 * kk + h));
    };

    // ================= layer 2: 3x3, CM -> CM =================
    WeightRing1<D2> r2;
    ring_fill1<9 * G, D2>(r2, ldw2);
    v16i acc2[2];
#pragma unroll
    for (int t = 0; t < 2; t++)
        init_acc(acc2[t], a2.bias2 + ct0 + 16 * h, false);
    __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): this thread's part of the grid is written
    __builtin_amdgcn_s_barrier();
    reduce_all<9 * G, 2, D2>(acc2, r2, 0, ldw2, ldb2);
    // layer 3: this wave's 128 output channels in 4 chunks of 32; the first chunk's weights, biases and residual travel now
    const uint8_t *w3 = a3.wfrag + (size_t)(128 * wave) * 64 + lane * 16;
    v4i wf[2 * G], b3[4], rn[2];
    auto load_chunk = [&](int cc) {
#pragma unroll
        for (int ks = 0; ks < 2 * G; ks++)
            wf[ks] = ldg128(w3 + (size_t)(ks >> 1) * wslab3 + (size_t)cc * 2048 + (ks & 1) * 1024);
        if (!LDSB) {
#pragma unroll
            for (int g = 0; g < 4; g++)
                b3[g] = *reinterpret_cast<const v4i *>(a3.bias2 + 128 * wave + 32 * cc + 16 * h + 4 * g);
        }
#pragma unroll
        for (int t = 0; t < 2; t++)
            rn[t] = ldg128(a3.res + pix[t] * CW + 128 * wave + 32 * cc + 16 * h);
    };
    load_chunk(0);
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int q = 32 * t + p;
        const v4i o = requant16(a2, acc2[t], a3.xmask);
        *reinterpret_cast<v4i *>(lds + M_OFF + row_off<CM>(q, (ct0 >> 4) + h)) = o;
    }
    __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();

    // ================= layer 3: CM -> CW and the residual add =================
    {
        v4i bf[2][2 * G];
#pragma unroll
        for (int t = 0; t < 2; t++) {
            const int q = 32 * t + p;
#pragma unroll
            for (int ks = 0; ks < 2 * G; ks++)
                bf[t][ks] = *reinterpret_cast<const v4i *>(lds + M_OFF + row_off<CM>(q, 2 * ks + h));
        }
        if (CHAIN) { // the sum tile lies over what the waves have just read
            __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
            __builtin_amdgcn_s_barrier();
        }
        for (int cc = 0; cc < 4; cc++) {
            const int ch = 128 * wave + 32 * cc;
            v16i acc[2];
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const v4i bv = LDSB ? *reinterpret_cast<const v4i *>(lds + B3_OFF + (ch + 16 * h + 4 * g) * 4) : b3[g];
#pragma unroll
                for (int e = 0; e < 4; e++)
                    acc[0][4 * g + e] = bv[e];
            }
            acc[1] = acc[0];
#pragma unroll
            for (int ks = 0; ks < 2 * G; ks++)
#pragma unroll
                for (int t = 0; t < 2; t++)
                    acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[ks], bf[t][ks], acc[t], 0, 0, 0);
            const v4i rc[2] = {rn[0], rn[1]};
            if (cc + 1 < 4)
                load_chunk(cc + 1); // the next chunk's operands arrive during the arithmetic below
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const v4i o = requant_add16(a3, acc[t], rc[t]);
                if (!CHAIN && valid[t]) // 16 bytes of each of 32 pixels per instruction; the chained form stores whole rows below
                    *reinterpret_cast<v4i *>(a3.y + pix[t] * CW + ch + 16 * h) = o;
                if (CHAIN) { // the sum tile: pixel row q, 16-byte piece c at piece c ^ (q & 15) of every 256 bytes
                    const int q = 32 * t + p, c16 = (ch >> 4) + h;
                    *reinterpret_cast<v4i *>(lds + S_OFF + q * CW + (c16 & ~15) * 16 + (((c16 & 15) ^ (q & 15)) << 4)) = o;
                }
            }
        }
    }
    if (!CHAIN)
        return;

    // ================= the next block's first layer: CW -> NX * CM on the sum tile =================
    // a wave owns the 32-channel tiles wave, wave + NW, ... one after the other (the sum tile is read once per tile)
#pragma unroll
    for (int jx = 0; jx < (NX ? NX : 1); jx++) {
        const int cn = 32 * (wave + NW * jx);
        const uint8_t *wn0 = an.wfrag + (size_t)cn * 64 + lane * 16;
        auto ldwn = [&](int s, int kk) { return ldg128(wn0 + (size_t)s * wslabn + kk * 1024); };
        auto ldbn = [&](int s, int kk, int t) {
            const int j = 32 * t + p, hs = h ^ (j & 15);
            return *reinterpret_cast<const v4i *>(lds + S_OFF + j * CW + (s >> 2) * 256 + (((4 * (s & 3) + 2 * kk) ^ hs) << 4));
        };
        WeightRing1<DN> rr;
        ring_fill1<4 * G, DN>(rr, ldwn);
        v16i accn[2];
#pragma unroll
        for (int t = 0; t < 2; t++)
            init_acc(accn[t], an.bias2 + cn + 16 * h, false);
        if (jx == 0) {
            __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): this wave's part of the sum tile is written
            __builtin_amdgcn_s_barrier();
            // The sum leaves from the tile as whole pixel rows: a wave instruction writes 1 KB of consecutive bytes, where a
            // store per chunk writes 32 bytes of each of 32 rows.  Lines written in pieces cost the kernel that reads the sum
            // dearly (the ResNet-50 pass: 0.724 -> 0.698 ms); the stores drain under the multiplies below.  (The same in the
            // whole-block kernel and in the unchained form, where nothing follows to hide the drain, measured 1 % slower.)
            constexpr int PPR = CW / 16; // 16-byte pieces per pixel row
#pragma unroll
            for (int k = 0; k < 64 * PPR / NT; k++) {
                const int item = tid + k * NT, q = item / PPR, c16 = item % PPR;
                const int py = q / PW, px = q - py * PW;
                const v4i o = *reinterpret_cast<const v4i *>(lds + S_OFF + q * CW + (c16 & ~15) * 16 + (((c16 & 15) ^ (q & 15)) << 4));
                if (q < NPIX)
                    *reinterpret_cast<v4i *>(a3.y + (size_t)((n * geo.H + y0 + py) * geo.W + x0 + px) * CW + c16 * 16) = o;
            }
        }
        reduce_all<4 * G, 2, DN>(accn, rr, (int)an.xmask, ldwn, ldbn);
#pragma unroll
        for (int t = 0; t < 2; t++) {
            const v4i o = requant16(an, accn[t], 0);
            if (valid[t])
                *reinterpret_cast<v4i *>(an.y + pix[t] * (NX * CM) + cn + 16 * h) = o;
        }
    }
}

// the patch shape of the tail kernel for an H x W image: 8x8 fills every pixel slot, 4x14 seven in eight, 7x7 three in four
static bool tail_patch(int H, int W, int *ph, int *pw)
{
    if (H % 8 == 0 && W % 8 == 0)
        *ph = 8, *pw = 8;
    else if (H % 4 == 0 && W % 14 == 0)
        *ph = 4, *pw = 14;
    else if (H % 7 == 0 && W % 7 == 0)
        *ph = 7, *pw = 7;
    else
        return false;
    return true;
}

bool conv_block_tail_applies(const ConvArgs &a2, const ConvArgs &a3, const ConvArgs *an)
{
    const int cm = a2.in_cs, cw = a3.out_cs;
    auto plain = [](const ConvArgs &a) {
        return a.group == 1 && a.bwz == 0 && a.xmask != 0 && a.lo >= 0 && a.fastq && a.qmult == nullptr && a.acc_out == nullptr && a.deq_out == nullptr && a.wfrag != nullptr;
    };
    auto one = [](const ConvArgs &a) {
        return a.R == 1 && a.S == 1 && a.pad_h == 0 && a.pad_w == 0 && a.stride_h == 1 && a.stride_w == 1;
    };
    // the layers after the 3x3 one work on its output image
    auto same_image = [&](const ConvArgs &a) { return a.N == a2.N && a.H == a2.OH && a.W == a2.OW && a.OH == a2.OH && a.OW == a2.OW; };
    const int st = a2.stride_h;
    int ph, pw;
    if (!(plain(a2) && plain(a3) && (cm == 64 || cm == 128 || cm == 256) && cw == 4 * cm
          && a2.R == 3 && a2.S == 3 && a2.pad_h == 1 && a2.pad_w == 1 && a2.stride_w == st && (st == 1 || (st == 2 && cm == 128))
          && a2.OH == (a2.H - 1) / st + 1 && a2.OW == (a2.W - 1) / st + 1 && a2.C == cm
          && a2.K == cm && a2.out_cs == cm && a2.nslab == 9 * cm / 64 && a2.kout_pad >= cm && a2.res == nullptr
          && one(a3) && a3.C == cm && a3.in_cs == cm && a3.K == cw && a3.nslab == cm / 64 && a3.kout_pad >= cw && same_image(a3)
          && a3.res != nullptr && a3.addq.fast && a3.addq.hi == 255 && tail_patch(a2.OH, a2.OW, &ph, &pw)
          && (long long)a2.N * a2.H * a2.W * cw < (1ll << 31)))
        return false;
    if (an == nullptr)
        return true;
    return plain(*an) && one(*an) && an->C == cw && an->in_cs == cw && (an->K == cm || an->K == 2 * cm) && an->out_cs == an->K
        && an->nslab == cw / 64 && an->kout_pad >= an->K && an->res == nullptr && same_image(*an);
}

template <int G, int PH, int PW, int ST>
static void launch_tail_gp(const ConvArgs &a2, const ConvArgs &a3, const ConvArgs *an, hipStream_t st)
{
    BlockGeom geo;
    geo.H = a2.OH, geo.W = a2.OW, geo.PY = a2.OH / PH, geo.PX = a2.OW / PW;
    geo.IH = a2.H, geo.IW = a2.W;
    geo.npatch = a2.N * geo.PY * geo.PX;
    const dim3 grid((unsigned)((geo.npatch + 7) / 8 * 8)), block(128 * G);
    if (an && an->K == 2 * a2.in_cs)
        hipLaunchKernelGGL((conv_bottleneck_tail_kernel<G, PH, PW, 2, ST>), grid, block, 0, st, a2, a3, *an, geo);
    else if (an)
        hipLaunchKernelGGL((conv_bottleneck_tail_kernel<G, PH, PW, 1, ST>), grid, block, 0, st, a2, a3, *an, geo);
    else
        hipLaunchKernelGGL((conv_bottleneck_tail_kernel<G, PH, PW, 0, ST>), grid, block, 0, st, a2, a3, a3, geo);
}

template <int G, int ST>
static void launch_tail_g(const ConvArgs &a2, const ConvArgs &a3, const ConvArgs *an, hipStream_t st)
{
    int ph = 0, pw = 0;
    tail_patch(a2.OH, a2.OW, &ph, &pw);
    if (ph == 8)
        launch_tail_gp<G, 8, 8, ST>(a2, a3, an, st);
    else if (ph == 4)
        launch_tail_gp<G, 4, 14, ST>(a2, a3, an, st);
    else
        launch_tail_gp<G, 7, 7, ST>(a2, a3, an, st);
}

void launch_conv_block_tail(const ConvArgs &a2, const ConvArgs &a3, const ConvArgs *an, hipStream_t st)
{
    if (a2.stride_h == 2) // conv_block_tail_applies: 128 middle channels only
        return launch_tail_g<2, 2>(a2, a3, an, st);
    switch (a2.in_cs) {
    case 64: launch_tail_g<1, 1>(a2, a3, an, st); break;
    case 128: launch_tail_g<2, 1>(a2, a3, an, st); break;
    default: launch_tail_g<4, 1>(a2, a3, an, st); break; // conv_block_tail_applies: 64, 128 or 256 middle channels
    }
}

// Measured at batch 64: blocks of 256 middle channels (14x14 images) 25.6 us against 8.0 + 13.2 + 14.5 and two launch
// gaps; 128 channels (28x28) 40.6 against 49.0, where the tail form below does better still; 64 channels lose.
bool conv_block_preferred(const ConvArgs &a1) { return a1.out_cs == 256; }

// Measured at batch 64: 128 middle channels (28x28 images) 32 us with the next layer, 27 without, against 14.0 + 28.6
// and a launch gap; 64 channels (56x56) 43 to 48 with the next layer against 13.8 + 37.3 and the gap, but 58 without
// (the sum's pixel tile is what that form saves); 256 channels belong to the whole-block kernel.
bool conv_block_tail_preferred(const ConvArgs &a2, bool chained) { return a2.in_cs == 128 || (a2.in_cs == 64 && chained); }

bool conv_block_applies(const ConvArgs &a1, const ConvArgs &a2, const ConvArgs &a3, const ConvArgs *an)
{
    const int cm = a1.out_cs, cw = a1.in_cs;
    auto plain = [](const ConvArgs &a) {
        return a.group == 1 && a.bwz == 0 && a.xmask != 0 && a.lo >= 0 && a.fastq && a.qmult == nullptr && a.acc_out == nullptr && a.deq_out == nullptr && a.wfrag != nullptr;
    };
    auto one = [](const ConvArgs &a) {
        return a.R == 1 && a.S == 1 && a.pad_h == 0 && a.pad_w == 0 && a.stride_h == 1 && a.stride_w == 1;
    };
    auto same_image = [&](const ConvArgs &a) { return a.N == a1.N && a.H == a1.H && a.W == a1.W && a.OH == a1.H && a.OW == a1.W; };
    if (an && !(plain(*an) && one(*an) && an->C == cw && an->in_cs == cw && an->K == 2 * cm && an->out_cs == an->K
                && an->nslab == cw / 64 && an->kout_pad >= an->K && an->res == nullptr && same_image(*an)))
        return false;
    return plain(a1) && plain(a2) && plain(a3) && (cm == 64 || cm == 128 || cm == 256) && cw == 4 * cm
        && one(a1) && a1.C == cw && a1.K == cm && a1.nslab == cw / 64 && a1.kout_pad >= cm && a1.res == nullptr && same_image(a1)
        && a2.R == 3 && a2.S == 3 && a2.pad_h == 1 && a2.pad_w == 1 && a2.stride_h == 1 && a2.stride_w == 1 && a2.C == cm
        && a2.in_cs == cm && a2.K == cm && a2.out_cs == cm && a2.nslab == 9 * cm / 64 && a2.kout_pad >= cm && a2.res == nullptr
        && same_image(a2)
        && one(a3) && a3.C == cm && a3.in_cs == cm && a3.K == cw && a3.out_cs == cw && a3.nslab == cm / 64 && a3.kout_pad >= cw
        && same_image(a3) && a3.res != nullptr && a3.addq.fast && a3.addq.hi == 255
        && a1.H % kPatch == 0 && a1.W % kPatch == 0 && (long long)a1.N * a1.H * a1.W * cw < (1ll << 31);
}

template <int G>
static void launch_block_g(const ConvArgs &a1, const ConvArgs &a2, const ConvArgs &a3, const ConvArgs *an, hipStream_t st)
{
    BlockGeom geo;
    geo.H = a1.H, geo.W = a1.W, geo.PY = a1.H / kPatch, geo.PX = a1.W / kPatch;
    geo.npatch = a1.N * geo.PY * geo.PX;
    const dim3 grid((unsigned)((geo.npatch + 7) / 8 * 8)), block(128 * G);
    const bool small = geo.PY <= 2 && geo.PX <= 2; // every region is at most 8 x 8 pixels
    if (small && an)
        hipLaunchKernelGGL((conv_bottleneck_kernel<G, 2, 2>), grid, block, 0, st, a1, a2, a3, *an, geo);
    else if (small)
        hipLaunchKernelGGL((conv_bottleneck_kernel<G, 2, 0>), grid, block, 0, st, a1, a2, a3, a3, geo);
    else if (an)
        hipLaunchKernelGGL((conv_bottleneck_kernel<G, 3, 2>), grid, block, 0, st, a1, a2, a3, *an, geo);
    else
        hipLaunchKernelGGL((conv_bottleneck_kernel<G, 3, 0>), grid, block, 0, st, a1, a2, a3, a3, geo);
}

void launch_conv_block(const ConvArgs &a1, const ConvArgs &a2, const ConvArgs &a3, const ConvArgs *an, hipStream_t st)
{
    switch (a1.out_cs) {
    case 64: launch_block_g<1>(a1, a2, a3, an, st); break;
    case 128: launch_block_g<2>(a1, a2, a3, an, st); break;
    default: launch_block_g<4>(a1, a2, a3, an, st); break; // conv_block_applies: 64, 128 or 256 middle channels
    }
}

} // namespace hipq
