// Quantized uint8 convolution for gfx950: implicit GEMM on the int8 MFMA units.
//
// Computes, bit for bit, what the reference CPU module computes in op_conv_2d_u8xu8_run
// (art/modules/quant/src/op/conv_2d_uint8_impl.c:39-165):
//     acc[n,k,oh,ow] = bias[k] + sum_{c,r,s} (x[n,c,ih,iw] - izp) * (w[k,c,r,s] - wzp)     (int32, wrapping)
//     y = sat( (int32)( floor((acc * mult + 2^(shift-1)) / 2^shift) + ozp ) )
//
// Mapping to the hardware
//   * GEMM view: D[kout][pixel] = sum_k A[kout][k] * B[k][pixel], k = (r, s, c) with c fastest, so that
//     16 consecutive k are 16 consecutive channels = one 128-bit load from the NHWC activation tensor.
//   * v_mfma_i32_32x32x32_i8 multiplies SIGNED bytes.  Activations and weights are unsigned with zero
//     points, so both are re-centred: xs = x - 128 (a byte-wise XOR with 0x80), ws = w - 128, and with
//     a = 128 - izp, b = 128 - wzp
//         sum (x - izp)(w - wzp) = sum xs*ws + b * sum xs + a * sum ws + Kp*a*b.
//     The last two terms are per-output-channel constants folded, with the bias, into `bias2` at setup.
//     The second term is per pixel and non-zero only for wzp != 128; it is accumulated with v_dot4 from
//     the very bytes that feed the MFMA (template flag HAS_WZP).  Taps that fall outside the image read
//     the byte izp (xs = -a), which makes their (x - izp) exactly zero; k slots that exist only because
//     of padding (pad channels, tail of the last 64-byte slab) carry the weight wzp (ws = -b), which
//     makes their contribution zero whatever activation byte happens to sit there.
//   * A (weights) is pre-packed at setup in MFMA fragment order, so a wave fetches a 32x32 fragment with
//     one fully coalesced 1 KiB global load (L2/L1 resident; it never touches LDS).
//     B (activations) is gathered from global memory 16 bytes per thread, XOR-ed, staged in LDS
//     (row stride 80 bytes: conflict-free 128-bit reads) and double buffered.
//   * A work-group of 4 waves computes a (WM*64 pixels) x (WN*64 channels) tile; each wave owns a
//     64x64 sub-tile = 2x2 MFMA tiles = 64 int32 accumulators per lane.
//   * Epilogue: each lane holds 4 consecutive output channels of one pixel per accumulator quad, so the
//     requantised bytes are packed into one dword and stored straight into the NHWC output.
//   * Work-groups are renumbered so that each of the 8 XCDs (round-robin dispatch) gets a contiguous
//     range of pixel tiles: neighbouring tiles share input halos and weight fragments in that XCD's L2.
#include <cstring>
#include <string>
#include <vector>

#include "common.h"

namespace hipq {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

struct ConvArgs {
    const uint8_t *x;
    uint8_t *y;
    int32_t *acc_out;
    const uint8_t *wpack; // MFMA: A fragments; depthwise: [tap][cs] int8 (w - wzp may not fit: stored as int16)
    const int32_t *bias2; // per output channel, padded
    int N, C, H, W, K, OH, OW;
    int in_cs, out_cs;
    int R, S, pad_h, pad_w, stride_h, stride_w, group;
    int P;     // N*OH*OW output pixels
    int rowb;  // bytes of one k "row": in_cs (generic) or 4*round_up(S,4) (small-C mode)
    int Ktot;  // generic: R*S*in_cs; small-C: R*rowb
    int nslab; // ceil(Ktot / 64)
    int nbm, nbn;
    int bwz;          // b = 128 - wzp
    int izp, wzp;     // for the non-MFMA kernels
    uint32_t padword; // byte izp in all four lanes
    Requant q;
    int lo; // lower clamp: ozp when ReLU is fused, else 0
};

__device__ static inline v4i ldg128(const uint8_t *p) { return *reinterpret_cast<const v4i *>(p); }

// ------------------------------------------------------------------------------------------------
// MFMA implicit-GEMM kernel.  SMALLC: input has channel stride 4 (C <= 4, e.g. the RGB stem); then one
// 16-byte piece is 4 horizontally adjacent taps x 4 channels and k = (r, s padded to 4, c4).
template <int WM, int WN, bool HAS_WZP, bool SMALLC>
__global__ __launch_bounds__(256) void conv_mfma_kernel(const ConvArgs a)
{
    constexpr int BM = WM * 64, BN = WN * 64, NPT = BM / 64, LSTR = 80;
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * BM * LSTR];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave % WM, wn = wave / WM;

    // XCD-aware renumbering: hardware block b runs on XCD b % 8; give each XCD a contiguous range.
    const int nblk = a.nbm * a.nbn;
    const int L = (int)(blockIdx.x % 8) * (int)(gridDim.x / 8) + (int)(blockIdx.x / 8);
    if (L >= nblk)
        return;
    const int bm = L / a.nbn, bn = L % a.nbn;

    // ---- loader state: this thread fetches piece (tid & 3) of pixels (tid >> 2) + 64 * j ----------
    int lp_pix[NPT], lp_ih0[NPT], lp_iw0[NPT];
    bool lp_ok[NPT];
    const int ohw = a.OH * a.OW;
#pragma unroll
    for (int j = 0; j < NPT; j++) {
        const int m = bm * BM + (tid >> 2) + 64 * j;
        lp_ok[j] = m < a.P;
        const int mm = lp_ok[j] ? m : 0;
        const int n = mm / ohw, rem = mm - n * ohw;
        const int oh = rem / a.OW, ow = rem - oh * a.OW;
        lp_ih0[j] = oh * a.stride_h - a.pad_h;
        lp_iw0[j] = ow * a.stride_w - a.pad_w;
        lp_pix[j] = n * a.H * a.W;
    }
    // position of this thread's piece in k space: row kr (a tap, or a kernel row in small-C mode),
    // column ks (generic mode only) and byte offset kc inside the row
    int kc = (tid & 3) * 16, kr = 0, ks = 0;
    auto normalise = [&]() {
        while (kc >= a.rowb) {
            kc -= a.rowb;
            if (SMALLC) {
                kr++;
            } else if (++ks == a.S) {
                ks = 0;
                kr++;
            }
        }
    };
    normalise();

    v4i breg[NPT];
    auto load_b = [&]() {
#pragma unroll
        for (int j = 0; j < NPT; j++) {
            const int ih = lp_ih0[j] + kr;
            const bool row_ok = lp_ok[j] && kr < a.R && (unsigned)ih < (unsigned)a.H;
            v4i v = {(int)a.padword, (int)a.padword, (int)a.padword, (int)a.padword};
            if (SMALLC) {
                const int s0 = kc >> 2;
                const int iw = lp_iw0[j] + s0;
                if (row_ok) {
                    const uint32_t *p = reinterpret_cast<const uint32_t *>(a.x) + (lp_pix[j] + ih * a.W + iw);
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (s0 + e < a.S && (unsigned)(iw + e) < (unsigned)a.W)
                            v[e] = (int)p[e];
                }
            } else {
                const int iw = lp_iw0[j] + ks;
                if (row_ok && (unsigned)iw < (unsigned)a.W)
                    v = ldg128(a.x + (size_t)(lp_pix[j] + ih * a.W + iw) * a.in_cs + kc);
            }
            breg[j] = v ^ (int)0x80808080;
        }
        kc += 64;
        normalise();
    };
    auto store_b = [&](uint8_t *buf) {
#pragma unroll
        for (int j = 0; j < NPT; j++)
            *reinterpret_cast<v4i *>(buf + ((tid >> 2) + 64 * j) * LSTR + (tid & 3) * 16) = breg[j];
    };

    // ---- A fragments: [kout tile][slab][half][lane] x 16 bytes -------------------------------------
    const int T0 = (bn * BN + wn * 64) >> 5;
    const uint8_t *wbase = a.wpack + (size_t)lane * 16;
    auto load_a = [&](v4i(&dst)[2][2], int slab) {
#pragma unroll
        for (int tn = 0; tn < 2; tn++)
#pragma unroll
            for (int kk = 0; kk < 2; kk++)
                dst[kk][tn] = ldg128(wbase + ((((size_t)(T0 + tn) * a.nslab + slab) * 2 + kk) << 10));
    };

    v16i acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++)
                acc[i][j][e] = 0;
    int colsum[2] = {0, 0};

    v4i acur[2][2], anext[2][2];
    load_b();
    load_a(acur, 0);
    store_b(lds);
    __syncthreads();

    const int brow = (wm * 64 + (lane & 31)) * LSTR + (lane >> 5) * 16;
    int cur = 0;
    for (int i = 0; i < a.nslab; i++) {
        const bool more = i + 1 < a.nslab;
        if (more) {
            load_b();
            load_a(anext, i + 1);
        }
        const uint8_t *buf = lds + cur * (BM * LSTR);
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
            const v4i b0 = *reinterpret_cast<const v4i *>(buf + brow + kk * 32);
            const v4i b1 = *reinterpret_cast<const v4i *>(buf + brow + 32 * LSTR + kk * 32);
            acc[0][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(acur[kk][0], b0, acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(acur[kk][0], b1, acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(acur[kk][1], b0, acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(acur[kk][1], b1, acc[1][1], 0, 0, 0);
            if (HAS_WZP) {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    colsum[0] = __builtin_amdgcn_sdot4(b0[e], 0x01010101, colsum[0], false);
                    colsum[1] = __builtin_amdgcn_sdot4(b1[e], 0x01010101, colsum[1], false);
                }
            }
        }
        if (more)
            store_b(lds + (cur ^ 1) * (BM * LSTR));
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 2; kk++)
#pragma unroll
            for (int tn = 0; tn < 2; tn++)
                acur[kk][tn] = anext[kk][tn];
        cur ^= 1;
    }

    // ---- epilogue ------------------------------------------------------------------------------
    if (HAS_WZP) {
        // a lane's B fragment covers half of the k range of its pixel; lanes l and l^32 share the pixel
        colsum[0] += __shfl_xor(colsum[0], 32);
        colsum[1] += __shfl_xor(colsum[1], 32);
    }
#pragma unroll
    for (int tm = 0; tm < 2; tm++) {
        const int m = bm * BM + wm * 64 + tm * 32 + (lane & 31);
        if (m >= a.P)
            continue;
        const int corr = HAS_WZP ? a.bwz * colsum[tm] : 0;
#pragma unroll
        for (int tn = 0; tn < 2; tn++) {
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int ko = bn * BN + wn * 64 + tn * 32 + g * 8 + (lane >> 5) * 4;
                if (ko >= a.out_cs)
                    continue;
                const v4i bias = *reinterpret_cast<const v4i *>(a.bias2 + ko);
                uint32_t packed = 0;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int32_t v = (int32_t)((uint32_t)acc[tn][tm][g * 4 + e] + (uint32_t)bias[e] + (uint32_t)corr);
                    if (a.acc_out)
                        a.acc_out[(size_t)m * a.out_cs + ko + e] = v;
                    int32_t r = requant_acc(v, a.q);
                    r = r < a.lo ? a.lo : r;
                    packed |= (uint32_t)r << (8 * e);
                }
                *reinterpret_cast<uint32_t *>(a.y + (size_t)m * a.out_cs + ko) = packed;
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Depthwise (group == C == K): memory-bound; one thread = 4 channels of one output pixel.
// Weights are stored tap-major as int16 (w - wzp needs 9 bits): wpack[tap][cs].
__global__ __launch_bounds__(256) void conv_depthwise_kernel(const ConvArgs a)
{
    const int cq = a.in_cs >> 2; // channel quads per pixel
    const size_t total = (size_t)a.P * cq;
    const int16_t *wq = reinterpret_cast<const int16_t *>(a.wpack);
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        const int m = (int)(idx / cq), c0 = (int)(idx - (size_t)m * cq) * 4;
        const int n = m / (a.OH * a.OW), rem = m - n * (a.OH * a.OW);
        const int oh = rem / a.OW, ow = rem - oh * a.OW;
        int32_t acc[4];
#pragma unroll
        for (int e = 0; e < 4; e++)
            acc[e] = a.bias2[c0 + e];
        for (int r = 0; r < a.R; r++) {
            const int ih = oh * a.stride_h - a.pad_h + r;
            if ((unsigned)ih >= (unsigned)a.H)
                continue;
            for (int s = 0; s < a.S; s++) {
                const int iw = ow * a.stride_w - a.pad_w + s;
                if ((unsigned)iw >= (unsigned)a.W)
                    continue;
                const uint32_t xv = *reinterpret_cast<const uint32_t *>(
                    a.x + ((size_t)(n * a.H + ih) * a.W + iw) * a.in_cs + c0);
                const int16_t *wp = wq + (size_t)(r * a.S + s) * a.in_cs + c0;
#pragma unroll
                for (int e = 0; e < 4; e++)
                    acc[e] += ((int)((xv >> (8 * e)) & 255) - a.izp) * (int)wp[e];
            }
        }
        uint32_t packed = 0;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            if (a.acc_out)
                a.acc_out[(size_t)m * a.out_cs + c0 + e] = acc[e];
            int32_t r = requant_acc(acc[e], a.q);
            r = r < a.lo ? a.lo : r;
            packed |= (uint32_t)r << (8 * e);
        }
        *reinterpret_cast<uint32_t *>(a.y + (size_t)m * a.out_cs + c0) = packed;
    }
}

// ------------------------------------------------------------------------------------------------
// Direct kernel for everything else (grouped convolutions with 1 < group < C): one thread per output
// element.  Correct for every parameter combination; not tuned.  wpack = the original uint8 [K,C/g,R,S].
__global__ __launch_bounds__(256) void conv_direct_kernel(const ConvArgs a)
{
    const size_t total = (size_t)a.P * a.K;
    const int cg = a.C / a.group, kg = a.K / a.group;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        const int m = (int)(idx / a.K), k = (int)(idx - (size_t)m * a.K);
        const int n = m / (a.OH * a.OW), rem = m - n * (a.OH * a.OW);
        const int oh = rem / a.OW, ow = rem - oh * a.OW;
        const int g = k / kg;
        uint32_t acc = (uint32_t)a.bias2[k];
        for (int r = 0; r < a.R; r++) {
            const int ih = oh * a.stride_h - a.pad_h + r;
            if ((unsigned)ih >= (unsigned)a.H)
                continue;
            for (int s = 0; s < a.S; s++) {
                const int iw = ow * a.stride_w - a.pad_w + s;
                if ((unsigned)iw >= (unsigned)a.W)
                    continue;
                const uint8_t *xp = a.x + ((size_t)(n * a.H + ih) * a.W + iw) * a.in_cs + g * cg;
                const uint8_t *wp = a.wpack + ((size_t)k * cg * a.R + r) * a.S + s;
                for (int c = 0; c < cg; c++)
                    acc += (uint32_t)(((int)xp[c] - a.izp) * ((int)wp[(size_t)c * a.R * a.S] - a.wzp));
            }
        }
        if (a.acc_out)
            a.acc_out[(size_t)m * a.out_cs + k] = (int32_t)acc;
        int32_t r = requant_acc((int32_t)acc, a.q);
        r = r < a.lo ? a.lo : r;
        a.y[(size_t)m * a.out_cs + k] = (uint8_t)r;
    }
}

} // namespace hipq

// =================================================================================================
// host side
using namespace hipq;

enum ConvVariant { kMfma, kMfmaSmallC, kDepthwise, kDirect };

struct hipq_conv2d_plan {
    hipq_conv2d_desc d;
    ConvArgs args;
    ConvVariant variant;
    int wm, wn;
    bool has_wzp;
    void *d_w = nullptr, *d_bias = nullptr;
    std::string name;
};

static int conv_out_dim(int in, int pad, int k, int stride)
{
    // art/src/op.c:549-555 (unsigned arithmetic, hole == 1)
    return (int)(((uint32_t)in + 2u * (uint32_t)pad - (uint32_t)k) / (uint32_t)stride + 1u);
}

extern "C" int hipq_conv2d_plan_create(const hipq_conv2d_desc *dp, const uint8_t *w, const int32_t *bias,
                                       hipq_conv2d_plan **plan_out)
{
    clear_error();
    HIPQ_REQUIRE(dp && w && plan_out, "hipq_conv2d_plan_create: null argument");
    const hipq_conv2d_desc &d = *dp;
    HIPQ_REQUIRE(d.N > 0 && d.C > 0 && d.H > 0 && d.W > 0 && d.K > 0 && d.R > 0 && d.S > 0, "conv: empty dimension");
    HIPQ_REQUIRE(d.stride_h > 0 && d.stride_w > 0 && d.pad_h >= 0 && d.pad_w >= 0, "conv: bad stride/pad");
    HIPQ_REQUIRE(d.group > 0 && d.C % d.group == 0 && d.K % d.group == 0, "conv: channels not divisible by group");
    HIPQ_REQUIRE(d.H + 2 * d.pad_h >= d.R && d.W + 2 * d.pad_w >= d.S, "conv: kernel larger than padded input");
    HIPQ_REQUIRE(d.in_cs >= d.C && d.out_cs >= d.K && d.in_cs % 4 == 0 && d.out_cs % 4 == 0,
                 "conv: channel strides must be multiples of 4 and cover C / K");
    HIPQ_REQUIRE(d.izp >= 0 && d.izp <= 255 && d.wzp >= 0 && d.wzp <= 255 && d.ozp >= 0 && d.ozp <= 255,
                 "conv: zero points must be in 0..255");
    HIPQ_REQUIRE(d.obits >= 1 && d.obits <= 8, "conv: obits must be in 1..8");

    auto *p = new hipq_conv2d_plan();
    p->d = d;
    ConvArgs &a = p->args;
    memset(&a, 0, sizeof(a));
    a.N = d.N, a.C = d.C, a.H = d.H, a.W = d.W, a.K = d.K, a.R = d.R, a.S = d.S;
    a.pad_h = d.pad_h, a.pad_w = d.pad_w, a.stride_h = d.stride_h, a.stride_w = d.stride_w, a.group = d.group;
    a.in_cs = d.in_cs, a.out_cs = d.out_cs;
    a.OH = conv_out_dim(d.H, d.pad_h, d.R, d.stride_h);
    a.OW = conv_out_dim(d.W, d.pad_w, d.S, d.stride_w);
    a.izp = d.izp, a.wzp = d.wzp;
    const long long P = (long long)d.N * a.OH * a.OW;
    if (P <= 0 || P * (long long)d.out_cs >= (1ll << 31) || (long long)d.N * d.H * d.W * d.in_cs >= (1ll << 31)) {
        delete p;
        return fail("conv: tensor too large for 32-bit indexing (or empty output)");
    }
    a.P = (int)P;
    hipq_quant_scale(d.ialpha * d.walpha / d.oalpha, 32, &a.q.mult, &a.q.shift);
    a.q.zp = d.ozp;
    a.q.hi = (1 << d.obits) - 1;
    a.lo = d.relu ? d.ozp : 0;
    if (!valid_shift(a.q.shift)) {
        delete p;
        return fail("conv: requantisation shift %d outside 1..62 (scale %g)", a.q.shift,
                    (double)(d.ialpha * d.walpha / d.oalpha));
    }
    a.padword = 0x01010101u * (uint32_t)d.izp;
    const int aoff = 128 - d.izp, boff = 128 - d.wzp;
    a.bwz = boff;

    const int cg = d.C / d.group;
    std::vector<uint8_t> wbuf;
    std::vector<int32_t> bbuf;
    if (d.group == 1 && (d.in_cs % 16 == 0 || d.in_cs == 4)) {
        const bool smallc = d.in_cs == 4;
        p->variant = smallc ? kMfmaSmallC : kMfma;
        p->wn = d.K <= 64 ? 1 : 2;
        p->wm = 4 / p->wn;
        const int BM = p->wm * 64, BN = p->wn * 64;
        a.nbm = (a.P + BM - 1) / BM;
        a.nbn = (d.out_cs + BN - 1) / BN;
        a.rowb = smallc ? 4 * ((d.S + 3) / 4 * 4) : d.in_cs;
        a.Ktot = smallc ? d.R * a.rowb : d.R * d.S * d.in_cs;
        a.nslab = (a.Ktot + 63) / 64;
        p->has_wzp = boff != 0;
        const int NT = a.nbn * BN / 32;
        wbuf.assign((size_t)NT * a.nslab * 2048, 0);
        bbuf.assign((size_t)NT * 32, 0);
        for (int T = 0; T < NT; T++)
            for (int l = 0; l < 32; l++) {
                const int ko = T * 32 + l;
                if (ko >= d.K)
                    continue; // rows of pad output channels stay zero; their outputs are don't-care
                long long wsum = 0;
                for (int kp = 0; kp < a.nslab * 64; kp++) {
                    int ws = -boff; // a padding slot: (ws + b) == 0
                    if (kp < a.Ktot) {
                        int r, s, c;
                        if (smallc) {
                            r = kp / a.rowb, s = (kp % a.rowb) / 4, c = kp % 4;
                        } else {
                            const int tap = kp / d.in_cs;
                            c = kp % d.in_cs, r = tap / d.S, s = tap % d.S;
                        }
                        if (s < d.S && c < d.C)
                            ws = (int)w[(((size_t)ko * d.C + c) * d.R + r) * d.S + s] - 128;
                    }
                    wsum += ws;
                    const int slab = kp >> 6, kk = (kp >> 5) & 1, half = (kp >> 4) & 1, i = kp & 15;
                    wbuf[((((size_t)T * a.nslab + slab) * 2 + kk) * 64 + half * 32 + l) * 16 + i] = (uint8_t)(int8_t)ws;
                }
                const long long c0 = (bias ? (long long)bias[ko] : 0) + (long long)aoff * wsum
                    + (long long)a.nslab * 64 * aoff * boff;
                bbuf[ko] = (int32_t)(uint32_t)(unsigned long long)c0;
            }
        char nm[96];
        snprintf(nm, sizeof nm, "conv_mfma_i8_%dx%d%s%s", BM, BN, smallc ? "_c4" : "", p->has_wzp ? "_wzp" : "");
        p->name = nm;
    } else if (d.group == d.C && d.K == d.C && d.in_cs == d.out_cs) {
        p->variant = kDepthwise;
        wbuf.assign((size_t)d.R * d.S * d.in_cs * 2, 0);
        int16_t *wq = reinterpret_cast<int16_t *>(wbuf.data());
        for (int c = 0; c < d.C; c++)
            for (int t = 0; t < d.R * d.S; t++)
                wq[(size_t)t * d.in_cs + c] = (int16_t)((int)w[(size_t)c * d.R * d.S + t] - d.wzp);
        bbuf.assign(d.in_cs, 0);
        for (int c = 0; c < d.C; c++)
            bbuf[c] = bias ? bias[c] : 0;
        p->name = "conv_depthwise_u8";
    } else {
        p->variant = kDirect;
        wbuf.assign(w, w + (size_t)d.K * cg * d.R * d.S);
        bbuf.assign(d.K, 0);
        for (int k = 0; k < d.K; k++)
            bbuf[k] = bias ? bias[k] : 0;
        p->name = "conv_direct_u8";
    }

    hipError_t e = hipMalloc(&p->d_w, wbuf.size());
    if (e == hipSuccess)
        e = hipMalloc(&p->d_bias, bbuf.size() * sizeof(int32_t));
    if (e == hipSuccess)
        e = hipMemcpy(p->d_w, wbuf.data(), wbuf.size(), hipMemcpyHostToDevice);
    if (e == hipSuccess)
        e = hipMemcpy(p->d_bias, bbuf.data(), bbuf.size() * sizeof(int32_t), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        hipq_conv2d_plan_destroy(p);
        return fail("conv: uploading packed weights failed: %s", hipGetErrorString(e));
    }
    a.wpack = static_cast<const uint8_t *>(p->d_w);
    a.bias2 = static_cast<const int32_t *>(p->d_bias);
    *plan_out = p;
    return 0;
}

extern "C" void hipq_conv2d_plan_destroy(hipq_conv2d_plan *p)
{
    if (!p)
        return;
    if (p->d_w)
        (void)hipFree(p->d_w);
    if (p->d_bias)
        (void)hipFree(p->d_bias);
    delete p;
}

extern "C" const char *hipq_conv2d_plan_kernel(const hipq_conv2d_plan *p) { return p ? p->name.c_str() : ""; }

template <int WM, int WN>
static void launch_mfma(const hipq_conv2d_plan *p, const ConvArgs &a, hipStream_t st)
{
    const int nblk = a.nbm * a.nbn;
    const dim3 grid((nblk + 7) / 8 * 8), block(256);
    if (p->variant == kMfmaSmallC) {
        if (p->has_wzp)
            hipLaunchKernelGGL((conv_mfma_kernel<WM, WN, true, true>), grid, block, 0, st, a);
        else
            hipLaunchKernelGGL((conv_mfma_kernel<WM, WN, false, true>), grid, block, 0, st, a);
    } else {
        if (p->has_wzp)
            hipLaunchKernelGGL((conv_mfma_kernel<WM, WN, true, false>), grid, block, 0, st, a);
        else
            hipLaunchKernelGGL((conv_mfma_kernel<WM, WN, false, false>), grid, block, 0, st, a);
    }
}

extern "C" int hipq_conv2d_run(const hipq_conv2d_plan *p, const void *x, void *y, int32_t *acc_out, void *stream)
{
    clear_error();
    HIPQ_REQUIRE(p && x && y, "hipq_conv2d_run: null argument");
    ConvArgs a = p->args;
    a.x = static_cast<const uint8_t *>(x);
    a.y = static_cast<uint8_t *>(y);
    a.acc_out = acc_out;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (p->variant) {
    case kMfma:
    case kMfmaSmallC:
        if (p->wn == 1)
            launch_mfma<4, 1>(p, a, st);
        else
            launch_mfma<2, 2>(p, a, st);
        break;
    case kDepthwise: {
        const size_t total = (size_t)a.P * (a.in_cs / 4);
        const unsigned blocks = (unsigned)std::min<size_t>((total + 255) / 256, 256 * 32);
        hipLaunchKernelGGL(conv_depthwise_kernel, dim3(blocks), dim3(256), 0, st, a);
        break;
    }
    case kDirect: {
        const size_t total = (size_t)a.P * a.K;
        const unsigned blocks = (unsigned)std::min<size_t>((total + 255) / 256, 256 * 32);
        hipLaunchKernelGGL(conv_direct_kernel, dim3(blocks), dim3(256), 0, st, a);
        break;
    }
    }
    return launch_status(p->name.c_str());
}

extern "C" int hipq_ip_reorder_weights(const uint8_t *w, uint8_t *w_out, int Nout, int C, int H, int W, int cs, int wzp)
{
    clear_error();
    HIPQ_REQUIRE(w && w_out && Nout > 0 && C > 0 && H > 0 && W > 0 && cs >= C, "hipq_ip_reorder_weights: bad argument");
    const size_t kin = (size_t)C * H * W, kout = (size_t)H * W * cs;
    for (int n = 0; n < Nout; n++)
        for (int h = 0; h < H; h++)
            for (int x = 0; x < W; x++)
                for (int c = 0; c < cs; c++)
                    w_out[n * kout + ((size_t)h * W + x) * cs + c]
                        = c < C ? w[n * kin + ((size_t)c * H + h) * W + x] : (uint8_t)wzp;
    return 0;
}
