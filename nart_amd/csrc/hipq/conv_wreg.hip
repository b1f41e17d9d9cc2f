// Convolutions over few pixels per launch (the 14x14 and 7x7 stages of a network): 1x1 and 3x3 layers, stride 1 or 2, as
// implicit GEMM whose weight operands never pass through LDS.  gfx950 only.
//
// Reproduces op_conv_2d_u8xu8_run (art/modules/quant/src/op/conv_2d_uint8_impl.c:39-165) and, with a residual,
// op_quant_add_run (art/modules/quant/src/op/add.c:83-148) bit for bit, like the tile kernels of conv.hip.
//
// The tile kernels stream both operands through LDS in 64-byte steps of the reduction, a barrier per step; on these
// layers a work-group has one or two tiles' worth of work and every step is a round trip of its own.  Here a work-group
// owns 64 output pixels x 128 output channels and the WHOLE reduction:
//   * its pixel operand goes to LDS once, by the load unit: for a 1x1 layer the 64 pixels' channels (stride 2: every
//     other pixel of every other row), for a 3x3 layer the 7x7 output patch's input region with its border (9x9 pixel rows,
//     15x15 at stride 2; out-of-image positions read the pad bytes), tap (r, s) of output pixel (y, x) being grid row
//     (S y + r) * GW + S x + s;
//   * each of the four waves owns 32 of the 128 channels for all 64 pixels and the whole reduction, and loads its MFMA
//     weight operands straight from memory in fragment order (ConvArgs::wfrag), eight slabs ahead of the multiplies - no
//     two waves want the same weight bytes, so LDS bandwidth is left to the pixel operands, the loop has no barrier and
//     the waves exchange nothing (splitting the reduction between two waves read every pixel operand once instead of
//     twice, but the exchange of partial sums through LDS cost more: 0.644 -> 0.639 ms per ResNet-50 pass);
//   * a lane holds 16 consecutive channels of a pixel: it requantises them, adds the residual where there is one, and
//     stores 16 bytes.
// Requirements (checked by the host): uint8 tensors, weight zero point 128, per-tensor scale, one-multiply
// requantisation, dense channel strides, input channels a multiple of 64 (1x1: 256, 512, 1024 or 2048; 3x3: 128, 256 or
// 512), output channels a multiple of 128; 3x3: pad 1, output height and width multiples of 7.
#include "conv_wreg.h"

#include <algorithm>

#include "conv_frag.h"

namespace hipq {

using namespace frag;

namespace {

constexpr int kWregPatch = 7; // 3x3 layers: a work-group's output pixels are a 7 x 7 patch of one image

struct WregGeom {
    int npg, nnb; // pixel groups, channel groups (a work-group's share: nbpw blocks of 128 output channels)
    int PY, PX;   // 3x3: patches per image
    int nbpw;     // blocks of 128 output channels a work-group walks with one load of its pixel operands (1: conv_wreg_kernel)
};

} // namespace

// CPT: 64-byte slabs per tap (input channels / 64); TAPS: 1 or 9; S: stride; ADD: residual add in the epilogue
template <int CPT, int TAPS, int S, bool ADD>
__global__ __launch_bounds__(256, 2) void conv_wreg_kernel(const ConvArgs a, const WregGeom geo)
{
    constexpr int RB = 64 * CPT;                                  // bytes of a pixel row
    constexpr int GW = TAPS == 9 ? S * (kWregPatch - 1) + 3 : 0;  // 3x3: the input region of a patch is GW x GW pixels
    constexpr int ROWS0 = TAPS == 9 ? GW * GW : 64;
    constexpr int X_BYTES = (ROWS0 * RB + 4095) / 4096 * 4096;    // whole instructions of the four waves
    constexpr int STOT = TAPS * CPT, D = 8;
    static_assert(TAPS == 9 || CPT >= 4, "1x1 layers: pixel rows of at least 256 bytes");
    __shared__ __attribute__((aligned(1024))) uint8_t lds[X_BYTES];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int p = lane & 31, h = lane >> 5;
    // work-groups go to the 8 XCDs in turn: XCD x takes the x-th contiguous eighth of the list, in which the channel
    // blocks of one pixel group are neighbours (they read the same pixels)
    const int gid = (int)(blockIdx.x % 8) * (int)(gridDim.x / 8) + (int)(blockIdx.x / 8);
    if (gid >= geo.npg * geo.nnb)
        return;
    const int pg = gid / geo.nnb, nb = gid - pg * geo.nnb;
    int n = 0, y0 = 0, x0 = 0; // 3x3: image and first output pixel of the patch
    if (TAPS == 9) {
        const int ppi = geo.PY * geo.PX, pr = pg % ppi, pi = pr / geo.PX;
        n = pg / ppi, y0 = pi * kWregPatch, x0 = (pr - pi * geo.PX) * kWregPatch;
    }

    // ---- the pixel operand -> LDS: 16-byte piece c of row r at piece c ^ swz(r) ----
    {
        constexpr int CPR = RB / 16;
#pragma unroll
        for (int k = 0; k < X_BYTES / 4096; k++) {
            const int id = (k * 4 + wave) * 64 + lane, row = id / CPR, c = (id % CPR) ^ swz<RB>(row);
            const uint8_t *src;
            if (TAPS == 9) {
                const int gy = row / GW, gx = row - gy * GW, iy = S * y0 - 1 + gy, ix = S * x0 - 1 + gx;
                const bool in = row < GW * GW && (unsigned)iy < (unsigned)a.H && (unsigned)ix < (unsigned)a.W;
                src = in ? a.x + (size_t)((n * a.H + iy) * a.W + ix) * RB + c * 16 : a.padbuf + (c & 3) * 16;
            } else {
                const int m = min(pg * 64 + row, a.P - 1); // rows beyond the tensor repeat its last pixel: never stored
                if (S == 1) {
                    src = a.x + (size_t)m * RB + c * 16;
                } else {
                    const int ohw = a.OH * a.OW, ni = fast_div(m, ohw, a.inv_ohw), rem = m - ni * ohw;
                    const int oy = fast_div(rem, a.OW, a.inv_ow), ox = rem - oy * a.OW;
                    src = a.x + (size_t)((ni * a.H + oy * S) * a.W + ox * S) * RB + c * 16;
                }
            }
            __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(lds + (k * 4 + wave) * 1024), 16, 0, 0);
        }
    }

    // the wave's channel tile: 32 of the block's 128 channels, for all 64 pixels and the whole reduction
    const int ct0 = 128 * nb + 32 * wave;
    const size_t wslab = (size_t)a.kout_pad * 64;
    const uint8_t *w0 = a.wfrag + (size_t)ct0 * 64 + lane * 16;
    auto ldw = [&](int s, int kk) { return ldg128(w0 + (size_t)s * wslab + kk * 1024); };
    // the lane's output pixels q = 32 t + p
    int prow[2];    // 1x1: the pixel's row in LDS; 3x3: the grid row of its first tap
    size_t pix[2];  // the output pixel's index in y
    bool valid[2];
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int q = 32 * t + p;
        if (TAPS == 9) {
            const int qq = min(q, kWregPatch * kWregPatch - 1), py = (qq * 37) >> 8, px = qq - py * kWregPatch; // qq / 7 for qq < 49
            valid[t] = q < kWregPatch * kWregPatch;
            prow[t] = S * py * GW + S * px;
            pix[t] = (size_t)((n * a.OH + y0 + py) * a.OW + x0 + px);
        } else {
            valid[t] = pg * 64 + q < a.P;
            prow[t] = q;
            pix[t] = (size_t)min(pg * 64 + q, a.P - 1);
        }
    }
    auto ldb = [&](int s, int kk, int t) {
        if (TAPS == 9) {
            const int tap = s / CPT, cb = s % CPT, tr = (tap * 11) >> 5;
            const int gr = prow[t] + tr * GW + (tap - 3 * tr), hs = h ^ swz<RB>(gr);
            return *reinterpret_cast<const v4i *>(lds + gr * RB + (((4 * cb + 2 * kk) ^ hs) << 4));
        }
        const int j = prow[t], hs = h ^ (j & 15); // slab s: pieces 4 s .. 4 s + 3 of the pixel's row
        return *reinterpret_cast<const v4i *>(lds + j * RB + (s >> 2) * 256 + (((4 * (s & 3) + 2 * kk) ^ hs) << 4));
    };

    v16i acc[2];
#pragma unroll
    for (int t = 0; t < 2; t++)
        init_acc(acc[t], a.bias2 + ct0 + 16 * h, false);
    WeightRing1<D> ring;
    ring_fill1<STOT, D>(ring, ldw);
    v4i res[2];
    if (ADD) {
#pragma unroll
        for (int t = 0; t < 2; t++)
            res[t] = ldg128(a.res + pix[t] * a.out_cs + ct0 + 16 * h);
    }
    // every wave's share of the pixel operand has landed before anyone reads it
    wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
    reduce_all<STOT, 2, D>(acc, ring, (int)a.xmask, ldw, ldb);
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const v4i o = ADD ? requant_add16(a, acc[t], res[t]) : requant16(a, acc[t], 0);
        if (valid[t])
            *reinterpret_cast<v4i *>(a.y + pix[t] * a.out_cs + ct0 + 16 * h) = o;
    }
}

// The last layer of a bottleneck block with a projection shortcut: y = add(a(x), b(xb)) with both convolutions in the
// same kernel - a: 1x1 / stride 1 from 64 CPT channels (its add parameters in a.addq / a.res_first, the sum to a.y), b:
// 1x1 / stride S2 from 64 CPT2 channels to the same output channels, whose requantised bytes are the add's other operand
// and never travel to memory (a launch, and a write and a read of the widest tensor of the block, disappear).  Both pixel
// operands go to LDS at the start; b is reduced first and its 16 bytes per lane and pixel tile wait in registers while a is
// reduced into the same accumulators.
template <int CPT, int CPT2, int S2>
__global__ __launch_bounds__(256, (4096 * (CPT + CPT2) <= 53248 ? 3 : 4096 * (CPT + CPT2) <= 81920 ? 2 : 1)) void conv_wreg_dual_kernel(const ConvArgs a, const ConvArgs b, const WregGeom geo)
{
    constexpr int RB = 64 * CPT, RB2 = 64 * CPT2, X_BYTES = 64 * RB, X2_BYTES = 64 * RB2;
    constexpr int D = 6;
    static_assert(CPT >= 4 && CPT2 >= 4, "pixel rows of at least 256 bytes");
    __shared__ __attribute__((aligned(1024))) uint8_t lds[X_BYTES + X2_BYTES];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int p = lane & 31, h = lane >> 5;
    const int gid = (int)(blockIdx.x % 8) * (int)(gridDim.x / 8) + (int)(blockIdx.x / 8); // XCD x: the x-th eighth of the list
    if (gid >= geo.npg * geo.nnb)
        return;
    const int pg = gid / geo.nnb, nb = gid - pg * geo.nnb;

    // ---- both pixel operands -> LDS: 16-byte piece c of row r at piece c ^ (r & 15) of every 256 bytes ----
#pragma unroll
    for (int k = 0; k < (X_BYTES + X2_BYTES) / 4096; k++) {
        const bool second = k >= X_BYTES / 4096;
        const int id = ((second ? k - X_BYTES / 4096 : k) * 4 + wave) * 64 + lane;
        const int cpr = second ? RB2 / 16 : RB / 16, row = id / cpr, c = (id % cpr) ^ (row & 15);
        const int m = min(pg * 64 + row, a.P - 1); // rows beyond the tensor repeat its last pixel: never stored
        const uint8_t *src;
        if (!second) {
            src = a.x + (size_t)m * RB + c * 16;
        } else if (S2 == 1) {
            src = b.x + (size_t)m * RB2 + c * 16;
        } else {
            const int ohw = a.OH * a.OW, ni = fast_div(m, ohw, a.inv_ohw), rem = m - ni * ohw;
            const int oy = fast_div(rem, a.OW, a.inv_ow), ox = rem - oy * a.OW;
            src = b.x + (size_t)((ni * b.H + oy * S2) * b.W + ox * S2) * RB2 + c * 16;
        }
        __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(lds + (k * 4 + wave) * 1024), 16, 0, 0);
    }

    // The work-group walks geo.nbpw blocks of 128 output channels with the pixel operands it has loaded once; per block a
    // wave owns 32 channels for all 64 pixels and both reductions.
    const size_t wslab = (size_t)a.kout_pad * 64, wslab2 = (size_t)b.kout_pad * 64;
    int ct0 = 128 * nb * geo.nbpw + 32 * wave;
    const uint8_t *w0, *v0;
    auto ldw = [&](int s, int kk) { return ldg128(w0 + (size_t)s * wslab + kk * 1024); };
    auto ldw2 = [&](int s, int kk) { return ldg128(v0 + (size_t)s * wslab2 + kk * 1024); };
    auto ldb = [&](int s, int kk, int t) {
        const int j = 32 * t + p, hs = h ^ (j & 15);
        return *reinterpret_cast<const v4i *>(lds + j * RB + (s >> 2) * 256 + (((4 * (s & 3) + 2 * kk) ^ hs) << 4));
    };
    auto ldb2 = [&](int s, int kk, int t) {
        const int j = 32 * t + p, hs = h ^ (j & 15);
        return *reinterpret_cast<const v4i *>(lds + X_BYTES + j * RB2 + (s >> 2) * 256 + (((4 * (s & 3) + 2 * kk) ^ hs) << 4));
    };
    size_t pix[2];
    bool valid[2];
#pragma unroll
    for (int t = 0; t < 2; t++) {
        valid[t] = pg * 64 + 32 * t + p < a.P;
        pix[t] = (size_t)min(pg * 64 + 32 * t + p, a.P - 1);
    }
    WeightRing1<D> ring, ringa;
    v0 = b.wfrag + (size_t)ct0 * 64 + lane * 16;
    ring_fill1<CPT2, D>(ring, ldw2);
    wait_vmcnt<0>(); // every wave's share of both pixel operands has landed before anyone reads them
    __builtin_amdgcn_s_barrier();
    for (int bi = 0; bi < geo.nbpw; bi++) {
        // ---- the shortcut b: its bytes for this wave's 32 channels of the 64 pixels stay in registers ----
        v16i acc[2];
#pragma unroll
        for (int t = 0; t < 2; t++)
            init_acc(acc[t], b.bias2 + ct0 + 16 * h, false);
        w0 = a.wfrag + (size_t)ct0 * 64 + lane * 16;
        ring_fill1<CPT, D>(ringa, ldw); // a's first weights travel while b is reduced
        reduce_all<CPT2, 2, D>(acc, ring, (int)b.xmask, ldw2, ldb2);
        v4i res[2];
#pragma unroll
        for (int t = 0; t < 2; t++)
            res[t] = requant16(b, acc[t], 0);
        // ---- a, then the add ----
#pragma unroll
        for (int t = 0; t < 2; t++)
            init_acc(acc[t], a.bias2 + ct0 + 16 * h, false);
        const int st0 = ct0; // this block's channels; the next block's shortcut weights travel during a's reduction and the add
        ct0 += 128;
        if (bi + 1 < geo.nbpw) {
            v0 = b.wfrag + (size_t)ct0 * 64 + lane * 16;
            ring_fill1<CPT2, D>(ring, ldw2);
        }
        reduce_all<CPT, 2, D>(acc, ringa, (int)a.xmask, ldw, ldb);
#pragma unroll
        for (int t = 0; t < 2; t++) {
            const v4i o = requant_add16(a, acc[t], res[t]);
            if (valid[t])
                *reinterpret_cast<v4i *>(a.y + pix[t] * a.out_cs + st0 + 16 * h) = o;
        }
    }
}

// a: the widening 1x1 convolution (stride 1, add parameters set, a.res any non-null pointer), b: the shortcut
bool conv_wreg_dual_applies(const ConvArgs &a, const ConvArgs &b)
{
    auto plain1x1 = [](const ConvArgs &c) {
        return c.group == 1 && c.bwz == 0 && c.xmask != 0 && c.lo >= 0 && c.fastq && c.qmult == nullptr && c.acc_out == nullptr && c.deq_out == nullptr
            && c.wfrag != nullptr && c.C == c.in_cs && c.in_cs % 64 == 0 && c.K == c.out_cs && c.out_cs % 128 == 0 && c.R == 1 && c.S == 1
            && c.pad_h == 0 && c.pad_w == 0 && c.stride_h == c.stride_w && c.nslab == c.in_cs / 64;
    };
    if (!(plain1x1(a) && plain1x1(b) && a.stride_h == 1 && (b.stride_h == 1 || b.stride_h == 2) && a.res != nullptr && a.addq.fast
          && a.addq.hi == 255 && b.res == nullptr && b.q.hi == 255 && a.out_cs == b.out_cs && a.N == b.N && a.OH == b.OH
          && a.OW == b.OW && a.P == b.P && (long long)b.N * b.H * b.W * b.in_cs < (1ll << 31)))
        return false;
    const int c1 = a.in_cs / 64, c2 = b.in_cs / 64;
    return (c1 == 4 || c1 == 8) && c2 == 2 * c1;
}

void launch_conv_wreg_dual(const ConvArgs &a, const ConvArgs &b, hipStream_t st)
{
    WregGeom geo;
    geo.PY = geo.PX = 0, geo.npg = (a.P + 63) / 64;
    // channel blocks per work-group: as many as still leave about two work-groups per CU (each reuses its pixel operands
    // in LDS and pays the start of the kernel once), in whole divisors of the block count
    const int nblk = a.out_cs / 128;
    geo.nbpw = 1;
    for (int k = 2; k <= 8; k++)
        if (nblk % k == 0 && (long long)geo.npg * (nblk / k) >= 384)
            geo.nbpw = k;
    geo.nnb = nblk / geo.nbpw;
    const dim3 grid((unsigned)((geo.npg * geo.nnb + 7) / 8 * 8)), block(256);
    const int c1 = a.in_cs / 64;
    if (c1 == 4 && b.stride_h == 1)
        hipLaunchKernelGGL((conv_wreg_dual_kernel<4, 8, 1>), grid, block, 0, st, a, b, geo);
    else if (c1 == 4)
        hipLaunchKernelGGL((conv_wreg_dual_kernel<4, 8, 2>), grid, block, 0, st, a, b, geo);
    else if (b.stride_h == 1)
        hipLaunchKernelGGL((conv_wreg_dual_kernel<8, 16, 1>), grid, block, 0, st, a, b, geo);
    else
        hipLaunchKernelGGL((conv_wreg_dual_kernel<8, 16, 2>), grid, block, 0, st, a, b, geo);
}

bool conv_wreg_applies(const ConvArgs &a)
{
    if (!(a.group == 1 && a.bwz == 0 && a.xmask != 0 && a.lo >= 0 && a.fastq && a.qmult == nullptr && a.acc_out == nullptr && a.deq_out == nullptr
          && a.wfrag != nullptr && a.C == a.in_cs && a.in_cs % 64 == 0 && a.K == a.out_cs && a.out_cs % 128 == 0
          && a.stride_h == a.stride_w && (a.stride_h == 1 || a.stride_h == 2) && a.nslab == a.R * a.S * a.in_cs / 64
          && (a.res == nullptr || (a.addq.fast && a.addq.hi == 255))))
        return false;
    const int cpt = a.in_cs / 64;
    if (a.R == 1 && a.S == 1)
        return a.pad_h == 0 && a.pad_w == 0 && (cpt == 4 || cpt == 8 || cpt == 16 || cpt == 32);
    return a.R == 3 && a.S == 3 && a.pad_h == 1 && a.pad_w == 1 && (cpt == 2 || cpt == 4 || cpt == 8) && a.res == nullptr
        && a.OH % kWregPatch == 0 && a.OW % kWregPatch == 0;
}

template <int CPT, int TAPS, int S>
static void launch_wreg(const ConvArgs &a, hipStream_t st)
{
    WregGeom geo;
    geo.nnb = a.out_cs / 128, geo.nbpw = 1;
    geo.PY = a.OH / kWregPatch, geo.PX = a.OW / kWregPatch;
    geo.npg = TAPS == 9 ? a.N * geo.PY * geo.PX : (a.P + 63) / 64;
    const dim3 grid((unsigned)((geo.npg * geo.nnb + 7) / 8 * 8)), block(256);
    if constexpr (TAPS == 1) {
        if (a.res != nullptr) {
            hipLaunchKernelGGL((conv_wreg_kernel<CPT, TAPS, S, true>), grid, block, 0, st, a, geo);
            return;
        }
    }
    hipLaunchKernelGGL((conv_wreg_kernel<CPT, TAPS, S, false>), grid, block, 0, st, a, geo);
}

void launch_conv_wreg(const ConvArgs &a, hipStream_t st)
{
    const int cpt = a.in_cs / 64, key = (a.R == 3 ? 1000 : 0) + cpt * 10 + a.stride_h;
    switch (key) {
#define HIPQ_WREG_CASE(CPT_, TAPS_, S_) \
    case (TAPS_ == 9 ? 1000 : 0) + CPT_ * 10 + S_: launch_wreg<CPT_, TAPS_, S_>(a, st); break;
        HIPQ_WREG_CASE(4, 1, 1)
        HIPQ_WREG_CASE(8, 1, 1)
        HIPQ_WREG_CASE(16, 1, 1)
        HIPQ_WREG_CASE(32, 1, 1)
        HIPQ_WREG_CASE(4, 1, 2)
        HIPQ_WREG_CASE(8, 1, 2)
        HIPQ_WREG_CASE(16, 1, 2)
        HIPQ_WREG_CASE(32, 1, 2)
        HIPQ_WREG_CASE(2, 9, 1)
        HIPQ_WREG_CASE(4, 9, 1)
        HIPQ_WREG_CASE(8, 9, 1)
        HIPQ_WREG_CASE(2, 9, 2)
        HIPQ_WREG_CASE(4, 9, 2)
        HIPQ_WREG_CASE(8, 9, 2)
#undef HIPQ_WREG_CASE
    default: break; // conv_wreg_applies admits nothing else
    }
}

} // namespace hipq
