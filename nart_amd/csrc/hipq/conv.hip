// Quantized convolution for gfx950: implicit GEMM on the int8 MFMA units (uint8 asymmetric and int8 symmetric tensors).
//
// Computes, bit for bit, what the reference CPU module computes in op_conv_2d_u8xu8_run
// (art/modules/quant/src/op/conv_2d_uint8_impl.c:39-165):
//     acc[n,k,oh,ow] = bias[k] + sum_{c,r,s} (x[n,c,ih,iw] - izp) * (w[k,c,r,s] - wzp)     (int32, wrapping)
//     y = sat( (int32)( floor((acc * mult + 2^(shift-1)) / 2^shift) + ozp ) )
// and, for int8 tensors, op_conv_2d_i8xi8_run (conv_2d_int8_impl.c:34-174): no zero points, the result clipped to
// +-(2^obits - 1) and truncated to a byte.
//
// Mapping to the hardware
//   * GEMM view: D[kout][pixel] = sum_k A[kout][k] * B[k][pixel], k = (r, s, c) with c fastest, so that
//     16 consecutive k are 16 consecutive channels = one 128-bit load from the NHWC activation tensor.
//   * v_mfma_i32_32x32x32_i8 multiplies SIGNED bytes.  uint8 activations and weights have zero points, so both
//     are re-centred: xs = x - 128 (a byte-wise XOR with 0x80), ws = w - 128, and with a = 128 - izp, b = 128 - wzp
//         sum (x - izp)(w - wzp) = sum xs*ws + b * sum xs + a * sum ws + Kp*a*b.
//     The last two terms are per-output-channel constants folded, with the bias, into `bias2` at setup;
//     the accumulators START at bias2, so the epilogue adds nothing.  The second term is per pixel and
//     non-zero only for wzp != 128; it is accumulated with v_dot4 from the very bytes that feed the MFMA
//     (template flag HAS_WZP).  Taps that fall outside the image read the byte izp (xs = -a), which makes
//     their (x - izp) exactly zero; k slots that exist only because of padding (pad channels, tail of the
//     last 64-byte slab) carry the weight wzp (ws = -b), which makes their contribution zero whatever
//     activation byte happens to sit there.  int8 tensors need none of this: the XOR mask is 0, a = b = 0.
//   * A work-group of 4 waves computes a BM pixels x BN channels tile, 64 bytes of k ("slab") at a time.
//     Both operands go through LDS and are put there by the load unit itself (global_load_lds_dwordx4: no VGPR
//     staging, no LDS store instructions): the weight slab [BN][64] is a straight copy of the pre-packed
//     weights, the activation slab [BM][64] is gathered 16 bytes per lane.  Rows are 64 bytes without padding;
//     the four 16-byte chunks of a row sit at chunk ^ ((row >> 2) & 3), which keeps the MFMA fragment reads
//     bank-conflict free; the weights are packed in that order on the host.  Two stages for short reductions
//     (more work-groups per CU, whose load, multiply and store phases overlap), three or four for long ones.
//   * Epilogue.  mult = m * 2^7 with m < 2^24, and for 33 <= shift <= 52 (every realistic scale)
//         floor((acc*mult + 2^(shift-1)) / 2^shift) + zp == (mulhi(acc, mult) + 2^(t-1) + zp*2^t) >> t,  t = shift-32
//     because the low 32 bits of the product cannot carry across the floor.  That is one v_mul_hi_i32, one
//     add, one shift and a saturating pack per output instead of a 64-bit multiply-add-shift.  Other shifts take
//     the 64-bit path.  Each lane then holds 4 consecutive channels of one pixel per accumulator quad;
//     the packed dwords are transposed through LDS so that every pixel's channels leave as 128-bit stores.
//     A residual add can run here as well (hipq_conv2d_run_add): in the accumulator layout, against a residual
//     tile that the load unit fetched into LDS while the reduction ran.
//   * Work-groups are renumbered so that each of the 8 XCDs (round-robin dispatch) gets a contiguous
//     range of pixel tiles: neighbouring tiles share input halos and weight slabs in that XCD's L2.
//   * 3x3 / stride 1 / pad 1 layers with 64 input channels run conv_mfma_halo_kernel: the input tile is loaded once
//     with its halo and the nine taps are read from LDS at shifted rows, instead of one slab per tap from memory.
//   * 1x1 / stride 1 layers with at most 64 input and 256 output channels run conv_mfma_pointwise_kernel: a wave per
//     strip of 32 pixels, pixel fragments straight from global memory, no LDS staging of activations, no barriers.
//   * Other shapes: C <= 4 inputs (the RGB stem) use a register-staged variant of the same tile computation,
//     depthwise 3x3 a dot-product kernel, remaining depthwise / grouped shapes plain per-output kernels.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <string>
#include <type_traits>
#include <vector>

#include "common.h"
#include "conv_shared.h"
#include "conv_stem.h"
#include "conv_block.h"
#include "conv_expand.h"
#include "conv_dw.h"
#include "conv_rows.h"
#include "conv_wreg.h"

namespace hipq {

// ------------------------------------------------------------------------------------------------
// MFMA implicit-GEMM kernel.  SMALLC: input has channel stride 4 (C <= 4, e.g. the RGB stem); then one
// 16-byte piece is 4 horizontally adjacent taps x 4 channels and k = (r, s padded to 4, c4).
template <int BM, int BN, int WM, int WN, bool HAS_WZP, bool SMALLC>
__global__ __launch_bounds__(256) void conv_mfma_kernel(const ConvArgs a)
{
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32; // MFMA tiles per wave: pixels x channels
    constexpr int NPB = BM / 64, NPA = BN / 64;         // 16-byte pieces per thread and slab
    constexpr int STAGE = (BM + BN) * 64;
    constexpr int OSTR = BN + 16; // row stride of the output staging tile
    constexpr int LDS_BYTES = 2 * STAGE > BM * OSTR ? 2 * STAGE : BM * OSTR;
    static_assert(WM * WN == 4 && TM >= 1 && TN >= 1 && NPB >= 1 && NPA >= 1, "tile shape");
    __shared__ __attribute__((aligned(16))) uint8_t lds[LDS_BYTES];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave % WM, wn = wave / WM;

    // XCD-aware renumbering: hardware block b runs on XCD b % 8; give each XCD a contiguous range.
    const int nblk = a.nbm * a.nbn;
    const int L = (int)(blockIdx.x % 8) * (int)(gridDim.x / 8) + (int)(blockIdx.x / 8);
    if (L >= nblk)
        return;
    const int bm = L / a.nbn, bn = L % a.nbn;

    // ---- activation loader: this thread fetches piece (tid & 3) of pixels (tid >> 2) + 64 * j -------
    int lp_pix[NPB], lp_ih0[NPB], lp_iw0[NPB];
    bool lp_ok[NPB];
    const int ohw = a.OH * a.OW;
#pragma unroll
    for (int j = 0; j < NPB; j++) {
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

    v4i breg[NPB], areg[NPA];
    auto load_b = [&]() {
#pragma unroll
        for (int j = 0; j < NPB; j++) {
            const int ih = lp_ih0[j] + kr;
            const bool row_ok = lp_ok[j] && kr < a.R && (unsigned)ih < (unsigned)a.H;
            v4i v = {(int)a.padword, (int)a.padword, (int)a.padword, (int)a.padword};
            if (SMALLC) {
                const int s0 = kc >> 2;
                const int iw = lp_iw0[j] + s0;
                if (row_ok) {
                    const uint32_t *p = reinterpret_cast<const uint32_t *>(a.x) + (lp_pix[j] + ih * a.W + iw);
                    if (iw >= 0 && iw + 3 < a.W) { // weights of taps beyond S are "zero": any byte will do
                        v = reinterpret_cast<const v4i_a4 *>(p)->v;
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            if ((unsigned)(iw + e) < (unsigned)a.W)
                                v[e] = (int)p[e];
                    }
                }
            } else {
                const int iw = lp_iw0[j] + ks;
                if (row_ok && (unsigned)iw < (unsigned)a.W)
                    v = ldg128(a.x + (size_t)(lp_pix[j] + ih * a.W + iw) * a.in_cs + kc);
            }
            breg[j] = v;
        }
        kc += 64;
        normalise();
    };
    const uint8_t *wsrc = a.wpack + (size_t)bn * BN * 64 + tid * 16;
    auto load_a = [&](int slab) {
#pragma unroll
        for (int j = 0; j < NPA; j++)
            areg[j] = ldg128(wsrc + (size_t)slab * a.kout_pad * 64 + j * 4096);
    };
    // chunk (tid & 3) of row (tid >> 2) + 64 j lands at chunk ^ ((row >> 2) & 3)
    const int bst = BN * 64 + (tid >> 2) * 64 + (((tid & 3) ^ ((tid >> 4) & 3)) << 4);
    auto store_ab = [&](uint8_t *stage) {
#pragma unroll
        for (int j = 0; j < NPA; j++)
            *reinterpret_cast<v4i *>(stage + tid * 16 + j * 4096) = areg[j];
#pragma unroll
        for (int j = 0; j < NPB; j++)
            *reinterpret_cast<v4i *>(stage + bst + j * 4096) = breg[j];
    };

    // ---- accumulators start at the folded per-channel constant ---------------------------------
    const int ch0 = bn * BN + wn * (TN * 32); // first channel of this wave
    v16i acc[TN][TM];
#pragma unroll
    for (int tn = 0; tn < TN; tn++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const v4i bias = *reinterpret_cast<const v4i *>(a.bias2 + ch0 + tn * 32 + g * 8 + (lane >> 5) * 4);
#pragma unroll
            for (int tm = 0; tm < TM; tm++)
#pragma unroll
                for (int e = 0; e < 4; e++)
                    acc[tn][tm][g * 4 + e] = bias[e];
        }
    int colsum[TM];
#pragma unroll
    for (int tm = 0; tm < TM; tm++)
        colsum[tm] = 0;

    // fragment addresses: row (lane & 31) of a 32-row tile, k bytes [32 kk + 16 (lane >> 5), +16)
    const int swz = (lane >> 2) & 3, half = lane >> 5;
    const int foff0 = (lane & 31) * 64 + (((0 + half) ^ swz) << 4);
    const int foff1 = (lane & 31) * 64 + (((2 + half) ^ swz) << 4);
    const int arow = wn * (TN * 32) * 64, brow = BN * 64 + wm * (TM * 32) * 64;

    load_a(0);
    load_b();
    store_ab(lds);
    __syncthreads();

    for (int i = 0; i < a.nslab; i++) {
        const bool more = i + 1 < a.nslab;
        if (more) {
            load_a(i + 1);
            load_b();
        }
        const uint8_t *buf = lds + (i & 1) * STAGE;
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
            const int fo = kk ? foff1 : foff0;
            v4i af[TN], bf[TM];
#pragma unroll
            for (int tn = 0; tn < TN; tn++)
                af[tn] = *reinterpret_cast<const v4i *>(buf + arow + tn * 2048 + fo);
#pragma unroll
            for (int tm = 0; tm < TM; tm++)
                bf[tm] = *reinterpret_cast<const v4i *>(buf + brow + tm * 2048 + fo) ^ (int)a.xmask;
#pragma unroll
            for (int tn = 0; tn < TN; tn++)
#pragma unroll
                for (int tm = 0; tm < TM; tm++)
                    acc[tn][tm] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[tn], bf[tm], acc[tn][tm], 0, 0, 0);
            if (HAS_WZP) {
#pragma unroll
                for (int tm = 0; tm < TM; tm++)
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        colsum[tm] = __builtin_amdgcn_sdot4(bf[tm][e], 0x01010101, colsum[tm], false);
            }
        }
        if (more)
            store_ab(lds + ((i + 1) & 1) * STAGE);
        __syncthreads();
    }

    // ---- epilogue ------------------------------------------------------------------------------
    if (HAS_WZP) {
        // a lane's B fragment covers half of the k range of its pixel; lanes l and l^32 share the pixel
#pragma unroll
        for (int tm = 0; tm < TM; tm++)
            colsum[tm] = a.bwz * (colsum[tm] + __shfl_xor(colsum[tm], 32));
    }
    // the last barrier of the main loop has retired every read of the stages
    if (a.fastq && a.lo == 0 && a.q.hi == 255)
        conv_epilogue<BM, BN, WM, WN, HAS_WZP, true, true, TM, TN>(a, acc, colsum, lds, bm, bn, wm, wn);
    else if (a.fastq)
        conv_epilogue<BM, BN, WM, WN, HAS_WZP, true, false, TM, TN>(a, acc, colsum, lds, bm, bn, wm, wn);
    else
        conv_epilogue<BM, BN, WM, WN, HAS_WZP, false, false, TM, TN>(a, acc, colsum, lds, bm, bn, wm, wn);
}

// ------------------------------------------------------------------------------------------------
// The same tile computation with the operands streamed global -> LDS by the load unit itself
// (global_load_lds_dwordx4: every lane names a 16-byte global source, the wave's 64 pieces land
// contiguously at the LDS address in M0), NS stages deep.  HBM latency on this chip is of the order of a
// microsecond, a slab of MFMA work a tenth of that: only several slabs in flight per work-group keep
// the matrix cores fed.  No VGPR staging, no LDS store instructions.  Out-of-image taps read 16 bytes of
// the byte izp from `padbuf`, so every lane always issues a load and the counts below are uniform.
// Synchronisation: vmcnt counts this wave's loads in issue order; after waiting until at most the
// younger slabs are outstanding, one barrier per slab makes the stage visible to all waves and at the
// same time retires every read of the stage that is about to be refilled.

// ALIGNED: a slab never straddles two taps (in_cs a multiple of 64, or a 1x1 kernel with any in_cs, whose last slab
// may be partial); the source addresses then advance by a wave-uniform offset and the bounds tests are redone only
// when the tap changes.
// FUSED: the residual add runs in the accumulator layout on a residual tile prefetched into LDS (see
// conv_epilogue_fused_add); only instantiated for ALIGNED && !HAS_WZP.
template <int BM, int BN, int WM, int WN, int NS, bool HAS_WZP, bool ALIGNED, bool FUSED = false>
__global__ __launch_bounds__(256) void conv_mfma_dma_kernel(const ConvArgs a)
{
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    constexpr int NPB = BM / 64, NPA = BN / 64, LPS = NPA + NPB; // loads per thread and stage
    constexpr int STAGE = (BM + BN) * 64;
    constexpr int OSTR = BN + 16;
    constexpr int STAGES_BYTES = NS * STAGE > BM * OSTR ? NS * STAGE : BM * OSTR;
    constexpr int LDS_BYTES = STAGES_BYTES + (FUSED ? BM * BN : 0); // the residual tile follows the stages
    static_assert(WM * WN == 4 && TM >= 1 && TN >= 1 && NPB >= 1 && NPA >= 1 && NS >= 2, "tile shape");
    static_assert((NS - 2) * LPS <= 63, "vmcnt range");
    __shared__ __attribute__((aligned(1024))) uint8_t lds[LDS_BYTES];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave % WM, wn = wave / WM;
    const int nblk = a.nbm * a.nbn;
    const int L = (int)(blockIdx.x % 8) * (int)(gridDim.x / 8) + (int)(blockIdx.x / 8);
    if (L >= nblk)
        return;
    const int bm = L / a.nbn, bn = L % a.nbn;

    // ---- activation source: LDS slot tid (+256 j) = phys chunk (tid & 3) of row (tid >> 2) + 64 j holds the
    // logical chunk (tid & 3) ^ ((row >> 2) & 3) of that pixel's 64-byte k slab
    int lp_pix[NPB], lp_ih0[NPB], lp_iw0[NPB];
    bool lp_ok[NPB];
    const int ohw = a.OH * a.OW;
#pragma unroll
    for (int j = 0; j < NPB; j++) {
        const int m = bm * BM + (tid >> 2) + 64 * j;
        lp_ok[j] = m < a.P;
        const int mm = lp_ok[j] ? m : 0;
        const int n = fast_div(mm, ohw, a.inv_ohw), rem = mm - n * ohw;
        const int oh = fast_div(rem, a.OW, a.inv_ow), ow = rem - oh * a.OW;
        lp_ih0[j] = oh * a.stride_h - a.pad_h;
        lp_iw0[j] = ow * a.stride_w - a.pad_w;
        lp_pix[j] = n * a.H * a.W;
    }
    const int chunk16 = ((tid & 3) ^ ((tid >> 4) & 3)) * 16;
    int kc = chunk16, kr = 0, ks = 0; // generic mode: this thread's position in k space
    auto normalise = [&]() {
        while (kc >= a.rowb) {
            kc -= a.rowb;
            if (++ks == a.S) {
                ks = 0;
                kr++;
            }
        }
    };
    // aligned mode: per-pixel base pointers (possibly outside the tensor for border pixels: never dereferenced
    // unless the tap is inside the image) + a uniform byte offset of the current (tap, channel slab)
    const uint8_t *lp_ptr[NPB];
    bool lp_in[NPB];
    int tap_r = 0, tap_s = 0, tap_c = 0, tap_off = 0;
    auto set_tap = [&]() {
#pragma unroll
        for (int j = 0; j < NPB; j++)
            lp_in[j] = lp_ok[j] && (unsigned)(lp_ih0[j] + tap_r) < (unsigned)a.H && (unsigned)(lp_iw0[j] + tap_s) < (unsigned)a.W;
        tap_off = (tap_r * a.W + tap_s) * a.in_cs;
    };
    if (ALIGNED) {
#pragma unroll
        for (int j = 0; j < NPB; j++)
            lp_ptr[j] = a.x + (ptrdiff_t)(lp_pix[j] + lp_ih0[j] * a.W + lp_iw0[j]) * a.in_cs + chunk16;
        set_tap();
    } else {
        normalise();
    }
    const uint8_t *wsrc = a.wpack + (size_t)bn * BN * 64 + tid * 16;
    const int wave_off = __builtin_amdgcn_readfirstlane(wave) * 1024;
    const size_t wslab = (size_t)a.kout_pad * 64;
    const bool pad_last = ALIGNED && chunk16 + 64 * (a.nslab - 1) >= a.in_cs * a.R * a.S; // only ever true for 1x1 kernels

    int st_issue = 0; // stage the next issue() fills; stages are used round-robin
    auto issue = [&](int slab) {
        uint8_t *st = lds + st_issue * STAGE + wave_off;
        st_issue = st_issue + 1 == NS ? 0 : st_issue + 1;
        const uint8_t *ws = wsrc + slab * wslab;
#pragma unroll
        for (int j = 0; j < NPA; j++)
            __builtin_amdgcn_global_load_lds((gptr_t)(ws + j * 4096), (lptr_t)(st + j * 4096), 16, 0, 0);
        if (ALIGNED) {
            const int off = tap_off + tap_c;
            // 1x1 kernels whose channel stride is not a multiple of 64: the chunks of the last slab that lie beyond the
            // pixel's own bytes (their weights are pad slots) come from the pad buffer, not from the next pixel
            const bool skip = pad_last && slab == a.nslab - 1;
#pragma unroll
            for (int j = 0; j < NPB; j++) {
                const uint8_t *src = lp_in[j] && !skip ? lp_ptr[j] + off : a.padbuf;
                __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(st + BN * 64 + j * 4096), 16, 0, 0);
            }
            tap_c += 64;
            if (tap_c == a.in_cs) {
                tap_c = 0;
                if (++tap_s == a.S) {
                    tap_s = 0;
                    ++tap_r;
                }
                set_tap();
            }
        } else {
#pragma unroll
            for (int j = 0; j < NPB; j++) {
                const int ih = lp_ih0[j] + kr, iw = lp_iw0[j] + ks;
                const bool ok = lp_ok[j] && kr < a.R && (unsigned)ih < (unsigned)a.H && (unsigned)iw < (unsigned)a.W;
                const uint8_t *src = ok ? a.x + (size_t)(lp_pix[j] + ih * a.W + iw) * a.in_cs + kc : a.padbuf;
                __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(st + BN * 64 + j * 4096), 16, 0, 0);
            }
            kc += 64;
            normalise();
        }
    };

    const int swz = (lane >> 2) & 3, half = lane >> 5;
    const int foff0 = (lane & 31) * 64 + (((0 + half) ^ swz) << 4);
    const int foff1 = (lane & 31) * 64 + (((2 + half) ^ swz) << 4);
    const int arow = wn * (TN * 32) * 64, brow = BN * 64 + wm * (TM * 32) * 64;

    // first the stage loads, then the (ordinary) loads of the folded bias: the bias loads are YOUNGER than the
    // first NS-1 slabs, which makes the very first wait below conservative (it also waits for slabs 1..NS-2) and
    // every later one exact; in exchange the bias latency overlaps with the activations' on their way from HBM
    if (FUSED) {
        // the residual tile first: these loads are the oldest, so every counted wait below covers them as well
        constexpr int NPR = BM * BN / 4096, CPR = BN / 16;
#pragma unroll
        for (int j = 0; j < NPR; j++) {
            const int sl = tid + 256 * j, r = sl / CPR, c = (sl % CPR) ^ ((r >> 1) & (CPR - 1));
            const int m = bm * BM + r;
            const uint8_t *src = (m < a.P && bn * BN + c * 16 < a.out_cs) ? a.res + (size_t)m * a.out_cs + bn * BN + c * 16 : a.padbuf;
            __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(lds + STAGES_BYTES + wave_off + j * 4096), 16, 0, 0);
        }
    }
    for (int s = 0; s < NS - 1 && s < a.nslab; s++)
        issue(s);

    const int ch0 = bn * BN + wn * (TN * 32);
    v16i acc[TN][TM];
#pragma unroll
    for (int tn = 0; tn < TN; tn++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const v4i bias = *reinterpret_cast<const v4i *>(a.bias2 + ch0 + tn * 32 + g * 8 + (lane >> 5) * 4);
#pragma unroll
            for (int tm = 0; tm < TM; tm++)
#pragma unroll
                for (int e = 0; e < 4; e++)
                    acc[tn][tm][g * 4 + e] = bias[e];
        }
    int colsum[TM];
#pragma unroll
    for (int tm = 0; tm < TM; tm++)
        colsum[tm] = 0;


    // Fragment reads run one k-step (32 bytes of k) ahead of the MFMAs that consume them, so the LDS latency
    // hides behind the matrix pipe.  make_ready(i) = slab i has landed for every wave, and every wave's reads of the
    // stage that slab i+NS-1 will occupy (the stage of slab i-1) have returned their data.
    int st_comp = 0;
    auto make_ready = [&](int i) {
        if (i + NS - 2 <= a.nslab - 1)
            wait_vmcnt<(NS - 2) * LPS>(); // slabs i+1 .. i+NS-2 may still be in flight
        else
            wait_vmcnt<0>();
        // This wave's fragment reads of slab i-1 must have RETURNED, not merely been issued, before the barrier lets any
        // wave refill that stage: the load unit's LDS writes are not ordered against another wave's pending ds_reads.
        // (The reads were issued a whole multiply() ago, so the wait is normally free.)
        __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0), vmcnt / expcnt untouched
        __builtin_amdgcn_s_barrier();
        if (i + NS - 1 < a.nslab)
            issue(i + NS - 1);
    };
    auto read_frags = [&](v4i(&af)[TN], v4i(&bf)[TM], const uint8_t *buf, int fo) {
#pragma unroll
        for (int tn = 0; tn < TN; tn++)
            af[tn] = *reinterpret_cast<const v4i *>(buf + arow + tn * 2048 + fo);
#pragma unroll
        for (int tm = 0; tm < TM; tm++)
            bf[tm] = *reinterpret_cast<const v4i *>(buf + brow + tm * 2048 + fo);
    };
    auto multiply = [&](v4i(&af)[TN], v4i(&bf)[TM]) {
#pragma unroll
        for (int tm = 0; tm < TM; tm++)
            bf[tm] ^= (int)a.xmask;
#pragma unroll
        for (int tn = 0; tn < TN; tn++)
#pragma unroll
            for (int tm = 0; tm < TM; tm++)
                acc[tn][tm] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[tn], bf[tm], acc[tn][tm], 0, 0, 0);
        if (HAS_WZP) {
#pragma unroll
            for (int tm = 0; tm < TM; tm++)
#pragma unroll
                for (int e = 0; e < 4; e++)
                    colsum[tm] = __builtin_amdgcn_sdot4(bf[tm][e], 0x01010101, colsum[tm], false);
        }
    };

    v4i af0[TN], bf0[TM], af1[TN], bf1[TM];
    make_ready(0);
    read_frags(af0, bf0, lds, foff0);
    for (int i = 0; i + 1 < a.nslab; i++) { // the last slab is peeled off: no conditional reads inside the loop
        const uint8_t *buf = lds + st_comp * STAGE;
        st_comp = st_comp + 1 == NS ? 0 : st_comp + 1;
        read_frags(af1, bf1, buf, foff1);
        multiply(af0, bf0);
        make_ready(i + 1);
        read_frags(af0, bf0, lds + st_comp * STAGE, foff0);
        multiply(af1, bf1);
    }
    read_frags(af1, bf1, lds + st_comp * STAGE, foff1);
    multiply(af0, bf0);
    multiply(af1, bf1);

    // ---- epilogue -----------------------------------------------------------------------------------------
    if (HAS_WZP) {
#pragma unroll
        for (int tm = 0; tm < TM; tm++)
            colsum[tm] = a.bwz * (colsum[tm] + __shfl_xor(colsum[tm], 32));
    }
    __syncthreads(); // every wave has finished reading the last stage; no load is in flight any more
    if (FUSED) {
        conv_epilogue_fused_add<BM, BN, WM, WN, TM, TN>(a, acc, lds, lds + STAGES_BYTES, bm, bn, wm, wn);
        return;
    }
    if (a.fastq && a.lo == 0 && a.q.hi == 255)
        conv_epilogue<BM, BN, WM, WN, HAS_WZP, true, true, TM, TN>(a, acc, colsum, lds, bm, bn, wm, wn);
    else if (a.fastq)
        conv_epilogue<BM, BN, WM, WN, HAS_WZP, true, false, TM, TN>(a, acc, colsum, lds, bm, bn, wm, wn);
    else
        conv_epilogue<BM, BN, WM, WN, HAS_WZP, false, false, TM, TN>(a, acc, colsum, lds, bm, bn, wm, wn);
}

// ------------------------------------------------------------------------------------------------
// The same tile with the reduction shared by TWO groups of four waves (512 threads): group g streams and multiplies the
// slabs g, g + 2, g + 4, ... through NS stages of its own, and the two partial accumulators are added through LDS before
// the epilogue.  A layer with few tiles (a 14x14 or 7x7 image at a moderate batch) leaves most CUs with a single
// work-group, i.e. one wave per SIMD, whose load issue, fragment reads and multiplies then run strictly one after the
// other; a second wave per SIMD working on the other half of the reduction overlaps them without adding a byte of
// global traffic (unlike smaller tiles) and without a reduction through memory (unlike a split across work-groups).
// Aligned addressing, weight zero point 128 (or int8), an even number of slabs, no fused residual: the host checks.
template <int BM, int BN, int WM, int WN, int NS>
__global__ __launch_bounds__(512) void conv_mfma_dma_k2_kernel(const ConvArgs a)
{
    constexpr bool HAS_WZP = false;
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    constexpr int NPB = BM / 64, NPA = BN / 64, LPS = NPA + NPB; // loads per thread and stage
    constexpr int STAGE = (BM + BN) * 64;
    constexpr int OSTR = BN + 16;
    constexpr int GROUP_BYTES = NS * STAGE; // the stages of one group
    constexpr int LDS_BYTES = 2 * GROUP_BYTES;
    static_assert(LDS_BYTES >= BM * BN * 4 && LDS_BYTES >= BM * OSTR, "the stages double as reduction and staging buffers");
    static_assert(WM * WN == 4 && TM >= 1 && TN >= 1 && NPB >= 1 && NPA >= 1 && NS >= 2, "tile shape");
    static_assert((NS - 2) * LPS <= 63, "vmcnt range");
    __shared__ __attribute__((aligned(1024))) uint8_t lds[LDS_BYTES];

    const int grp = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 8); // wave-uniform
    const int tid = threadIdx.x & 255, lane = tid & 63, wave = tid >> 6;  // position inside the group
    const int wm = wave % WM, wn = wave / WM;
    uint8_t *const glds = lds + grp * GROUP_BYTES;
    const int ng = a.nslab >> 1; // slabs per group
    const int nblk = a.nbm * a.nbn;
    const int L = (int)(blockIdx.x % 8) * (int)(gridDim.x / 8) + (int)(blockIdx.x / 8);
    if (L >= nblk)
        return;
    const int bm = L / a.nbn, bn = L % a.nbn;

    // ---- activation source: LDS slot tid (+256 j) = phys chunk (tid & 3) of row (tid >> 2) + 64 j holds the
    // logical chunk (tid & 3) ^ ((row >> 2) & 3) of that pixel's 64-byte k slab
    int lp_pix[NPB], lp_ih0[NPB], lp_iw0[NPB];
    bool lp_ok[NPB];
    const int ohw = a.OH * a.OW;
#pragma unroll
    for (int j = 0; j < NPB; j++) {
        const int m = bm * BM + (tid >> 2) + 64 * j;
        lp_ok[j] = m < a.P;
        const int mm = lp_ok[j] ? m : 0;
        const int n = fast_div(mm, ohw, a.inv_ohw), rem = mm - n * ohw;
        const int oh = fast_div(rem, a.OW, a.inv_ow), ow = rem - oh * a.OW;
        lp_ih0[j] = oh * a.stride_h - a.pad_h;
        lp_iw0[j] = ow * a.stride_w - a.pad_w;
        lp_pix[j] = n * a.H * a.W;
    }
    const int chunk16 = ((tid & 3) ^ ((tid >> 4) & 3)) * 16;
    // per-pixel base pointers (possibly outside the tensor for border pixels: never dereferenced
    // unless the tap is inside the image) + a uniform byte offset of the current (tap, channel slab)
    const uint8_t *lp_ptr[NPB];
    bool lp_in[NPB];
    int tap_r = 0, tap_s = 0, tap_c = 0, tap_off = 0;
    auto set_tap = [&]() {
#pragma unroll
        for (int j = 0; j < NPB; j++)
            lp_in[j] = lp_ok[j] && (unsigned)(lp_ih0[j] + tap_r) < (unsigned)a.H && (unsigned)(lp_iw0[j] + tap_s) < (unsigned)a.W;
        tap_off = (tap_r * a.W + tap_s) * a.in_cs;
    };
#pragma unroll
    for (int j = 0; j < NPB; j++)
        lp_ptr[j] = a.x + (ptrdiff_t)(lp_pix[j] + lp_ih0[j] * a.W + lp_iw0[j]) * a.in_cs + chunk16;
    set_tap();
    const uint8_t *wsrc = a.wpack + (size_t)bn * BN * 64 + tid * 16;
    const int wave_off = __builtin_amdgcn_readfirstlane(wave) * 1024;
    const size_t wslab = (size_t)a.kout_pad * 64;
    const bool pad_last = chunk16 + 64 * (a.nslab - 1) >= a.in_cs * a.R * a.S; // only ever true for 1x1 kernels

    auto advance = [&]() { // step the (tap, channel slab) position by one slab
        tap_c += 64;
        if (tap_c == a.in_cs) {
            tap_c = 0;
            if (++tap_s == a.S) {
                tap_s = 0;
                ++tap_r;
            }
            set_tap();
        }
    };
    if (grp)
        advance(); // group 1 starts at slab 1
    int st_issue = 0; // stage the next issue() fills; stages are used round-robin
    auto issue = [&](int slab) { // slab: index in the whole reduction
        uint8_t *st = glds + st_issue * STAGE + wave_off;
        st_issue = st_issue + 1 == NS ? 0 : st_issue + 1;
        const uint8_t *ws = wsrc + slab * wslab;
#pragma unroll
        for (int j = 0; j < NPA; j++)
            __builtin_amdgcn_global_load_lds((gptr_t)(ws + j * 4096), (lptr_t)(st + j * 4096), 16, 0, 0);
        const int off = tap_off + tap_c;
        // 1x1 kernels whose channel stride is not a multiple of 64: the chunks of the last slab that lie beyond the
        // pixel's own bytes (their weights are pad slots) come from the pad buffer, not from the next pixel
        const bool skip = pad_last && slab == a.nslab - 1;
#pragma unroll
        for (int j = 0; j < NPB; j++) {
            const uint8_t *src = lp_in[j] && !skip ? lp_ptr[j] + off : a.padbuf;
            __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(st + BN * 64 + j * 4096), 16, 0, 0);
        }
        advance();
        advance(); // the slab in between belongs to the other group
    };

    const int swz = (lane >> 2) & 3, half = lane >> 5;
    const int foff0 = (lane & 31) * 64 + (((0 + half) ^ swz) << 4);
    const int foff1 = (lane & 31) * 64 + (((2 + half) ^ swz) << 4);
    const int arow = wn * (TN * 32) * 64, brow = BN * 64 + wm * (TM * 32) * 64;

    // first the stage loads, then the (ordinary) loads of the folded bias (see conv_mfma_dma_kernel)
    for (int s = 0; s < NS - 1 && s < ng; s++)
        issue(2 * s + grp);

    const int ch0 = bn * BN + wn * (TN * 32);
    v16i acc[TN][TM];
#pragma unroll
    for (int tn = 0; tn < TN; tn++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const v4i bias = *reinterpret_cast<const v4i *>(a.bias2 + ch0 + tn * 32 + g * 8 + (lane >> 5) * 4);
#pragma unroll
            for (int tm = 0; tm < TM; tm++)
#pragma unroll
                for (int e = 0; e < 4; e++)
                    acc[tn][tm][g * 4 + e] = grp ? 0 : bias[e];
        }
    int colsum[TM];
#pragma unroll
    for (int tm = 0; tm < TM; tm++)
        colsum[tm] = 0;


    // Fragment reads run one k-step (32 bytes of k) ahead of the MFMAs that consume them, so the LDS latency
    // hides behind the matrix pipe.  make_ready(i) = slab i has landed for every wave, and every wave's reads of the
    // stage that slab i+NS-1 will occupy (the stage of slab i-1) have returned their data.
    int st_comp = 0;
    auto make_ready = [&](int i) {
        if (i + NS - 2 <= ng - 1)
            wait_vmcnt<(NS - 2) * LPS>(); // this group's slabs i+1 .. i+NS-2 may still be in flight
        else
            wait_vmcnt<0>();
        // This wave's fragment reads of slab i-1 must have RETURNED, not merely been issued, before the barrier lets any
        // wave refill that stage: the load unit's LDS writes are not ordered against another wave's pending ds_reads.
        // (The reads were issued a whole multiply() ago, so the wait is normally free.)
        __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0), vmcnt / expcnt untouched
        __builtin_amdgcn_s_barrier();
        if (i + NS - 1 < ng)
            issue(2 * (i + NS - 1) + grp);
    };
    auto read_frags = [&](v4i(&af)[TN], v4i(&bf)[TM], const uint8_t *buf, int fo) {
#pragma unroll
        for (int tn = 0; tn < TN; tn++)
            af[tn] = *reinterpret_cast<const v4i *>(buf + arow + tn * 2048 + fo);
#pragma unroll
        for (int tm = 0; tm < TM; tm++)
            bf[tm] = *reinterpret_cast<const v4i *>(buf + brow + tm * 2048 + fo);
    };
    auto multiply = [&](v4i(&af)[TN], v4i(&bf)[TM]) {
#pragma unroll
        for (int tm = 0; tm < TM; tm++)
            bf[tm] ^= (int)a.xmask;
#pragma unroll
        for (int tn = 0; tn < TN; tn++)
#pragma unroll
            for (int tm = 0; tm < TM; tm++)
                acc[tn][tm] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[tn], bf[tm], acc[tn][tm], 0, 0, 0);
        if (HAS_WZP) {
#pragma unroll
            for (int tm = 0; tm < TM; tm++)
#pragma unroll
                for (int e = 0; e < 4; e++)
                    colsum[tm] = __builtin_amdgcn_sdot4(bf[tm][e], 0x01010101, colsum[tm], false);
        }
    };

    v4i af0[TN], bf0[TM], af1[TN], bf1[TM];
    make_ready(0);
    read_frags(af0, bf0, glds, foff0);
    for (int i = 0; i + 1 < ng; i++) { // the last slab is peeled off: no conditional reads inside the loop
        const uint8_t *buf = glds + st_comp * STAGE;
        st_comp = st_comp + 1 == NS ? 0 : st_comp + 1;
        read_frags(af1, bf1, buf, foff1);
        multiply(af0, bf0);
        make_ready(i + 1);
        read_frags(af0, bf0, glds + st_comp * STAGE, foff0);
        multiply(af1, bf1);
    }
    read_frags(af1, bf1, glds + st_comp * STAGE, foff1);
    multiply(af0, bf0);
    multiply(af1, bf1);

    // ---- the two partial sums meet in LDS, then group 0 runs the usual epilogue ---------------------------------
    __syncthreads(); // every wave has finished reading the last stages; no load is in flight any more
    int32_t *red = reinterpret_cast<int32_t *>(lds) + wave * (TN * TM * 16 * 64) + lane; // [wave][register][lane]
    if (grp) {
#pragma unroll
        for (int tn = 0; tn < TN; tn++)
#pragma unroll
            for (int tm = 0; tm < TM; tm++)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    red[((tn * TM + tm) * 16 + r) * 64] = acc[tn][tm][r];
    }
    __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    if (!grp) {
#pragma unroll
        for (int tn = 0; tn < TN; tn++)
#pragma unroll
            for (int tm = 0; tm < TM; tm++)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    acc[tn][tm][r] = (int32_t)((uint32_t)acc[tn][tm][r] + (uint32_t)red[((tn * TM + tm) * 16 + r) * 64]);
    }
    __builtin_amdgcn_s_waitcnt(0xC07F); // the sums are in registers before the staging tile overwrites the buffer
    __builtin_amdgcn_s_barrier();
    if (grp) {
        // group 1 only keeps the barrier count of conv_epilogue's staged path (one barrier; the plain path has none)
        if (!plain_epilogue(a)) {
            __builtin_amdgcn_s_barrier();
        }
        return;
    }
    if (a.fastq && a.lo == 0 && a.q.hi == 255)
        conv_epilogue<BM, BN, WM, WN, HAS_WZP, true, true, TM, TN>(a, acc, colsum, lds, bm, bn, wm, wn);
    else if (a.fastq)
        conv_epilogue<BM, BN, WM, WN, HAS_WZP, true, false, TM, TN>(a, acc, colsum, lds, bm, bn, wm, wn);
    else
        conv_epilogue<BM, BN, WM, WN, HAS_WZP, false, false, TM, TN>(a, acc, colsum, lds, bm, bn, wm, wn);
}

// ------------------------------------------------------------------------------------------------
// 3x3, stride 1, pad 1 convolutions (in_cs a multiple of 64).  The nine taps of an output pixel read nine shifted copies
// of the same input bytes, so instead of streaming one 64-byte slab per pixel and tap, the work-group loads, per
// 64-channel slab, the pixels [m0 - W - 1, m0 + BM + W] of the flattened (n, h, w) index space ONCE (a "halo tile" of
// BM + 2W + 2 rows of 64 bytes) and forms the pixel fragments of tap (dr, ds) by reading row r + W + 1 + dr*W + ds of it.
// A tap outside the image would find a wrong neighbour there (the flat index runs on into the previous row or image):
// such lanes read a row of pad bytes instead, chosen by a 9-bit mask computed once per lane.  Weight slabs are streamed as
// in conv_mfma_dma_kernel, in the order (channel slab, tap) - slab tap * (in_cs / 64) + channel slab of the packed
// weights; int32 accumulation does not depend on the order.  The LDS fill per k-step drops from (BM + BN) * 64 bytes to
// BN * 64 + (BM + 2W + 2) * 64 / 9, and all bytes a tile touches first are requested at once.
// The halo tiles of ALL channel slabs are requested when the work-group starts (NAB = in_cs / 64 buffers): a halo that
// arrives from HBM in the middle of the weight stream would hold up every younger weight slab behind it, because a wave's
// loads complete in order.  NPH: halo rows / 64 (>= BM + 2W + 2 rows, the host checks).
template <int BM, int BN, int WM, int WN, int NS, int NPH, int NAB>
__global__ __launch_bounds__(256) void conv_mfma_halo_kernel(const ConvArgs a)
{
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    constexpr int NPA = BN / 64; // weight loads per thread and slab
    constexpr int WSTAGE = BN * 64;
    constexpr int ABUF = NPH * 64 * 64;
    constexpr int A_OFF = NS * WSTAGE;
    constexpr int PAD_OFF = A_OFF + NAB * ABUF; // 64 pad bytes
    constexpr int OSTR = BN + 16;
    constexpr int LDS_BYTES = PAD_OFF + 64 > BM * OSTR ? PAD_OFF + 64 : BM * OSTR;
    static_assert(WM * WN == 4 && TM >= 1 && TN >= 1 && NS >= 2 && NS <= 9, "tile shape");
    static_assert((NS - 2) * NPA <= 63, "vmcnt range");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS");
    __shared__ __attribute__((aligned(1024))) uint8_t lds[LDS_BYTES];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave % WM, wn = wave / WM;
    const int nblk = a.nbm * a.nbn;
    const int L = (int)(blockIdx.x % 8) * (int)(gridDim.x / 8) + (int)(blockIdx.x / 8);
    if (L >= nblk)
        return;
    const int bm = L / a.nbn, bn = L % a.nbn;
    const int nc = a.in_cs >> 6;
    const int m0 = bm * BM;

    // ---- halo source: LDS slot tid (+256 j) = phys chunk (tid & 3) of halo row (tid >> 2) + 64 j
    const int chunk16 = ((tid & 3) ^ ((tid >> 4) & 3)) * 16;
    if (tid < 16)
        *reinterpret_cast<uint32_t *>(lds + PAD_OFF + tid * 4) = a.padword; // visible after the first barrier
    const int hrows = BM + 2 * a.W + 2;
    const uint8_t *hp[NPH];
#pragma unroll
    for (int j = 0; j < NPH; j++) {
        const int row = (tid >> 2) + 64 * j, q = m0 - a.W - 1 + row;
        hp[j] = (row < hrows && q >= 0 && q < a.P) ? a.x + (size_t)q * a.in_cs + chunk16 : nullptr;
    }
    const int wave_off = __builtin_amdgcn_readfirstlane(wave) * 1024;
    auto issue_halo = [&](int cs) {
        uint8_t *dst = lds + A_OFF + cs * ABUF + wave_off;
#pragma unroll
        for (int j = 0; j < NPH; j++) {
            const uint8_t *src = hp[j] ? hp[j] + cs * 64 : a.padbuf;
            __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(dst + j * 4096), 16, 0, 0);
        }
    };
    const uint8_t *wsrc = a.wpack + (size_t)bn * BN * 64 + tid * 16;
    const size_t wslab = (size_t)a.kout_pad * 64;
    int st_issue = 0, wi_t = 0, wi_cs = 0; // next weight slab to issue: (channel slab, tap), and its stage
    auto issue_w = [&]() {
        uint8_t *st = lds + st_issue * WSTAGE + wave_off;
        st_issue = st_issue + 1 == NS ? 0 : st_issue + 1;
        const uint8_t *ws = wsrc + (size_t)(wi_t * nc + wi_cs) * wslab;
#pragma unroll
        for (int j = 0; j < NPA; j++)
            __builtin_amdgcn_global_load_lds((gptr_t)(ws + j * 4096), (lptr_t)(st + j * 4096), 16, 0, 0);
        if (++wi_t == 9) {
            wi_t = 0;
            ++wi_cs;
        }
    };

    // ---- this lane's pixel rows and their tap masks
    const int half = lane >> 5;
    int hr0[TM], vm[TM];
    const int hw = a.H * a.W;
#pragma unroll
    for (int tm = 0; tm < TM; tm++) {
        const int r = wm * (TM * 32) + tm * 32 + (lane & 31), m = m0 + r;
        hr0[tm] = r + a.W + 1;
        int mask = 0;
        if (m < a.P) {
            const int n = fast_div(m, hw, a.inv_ohw), rem = m - n * hw;
            const int oh = fast_div(rem, a.W, a.inv_ow), ow = rem - oh * a.W;
#pragma unroll
            for (int t = 0; t < 9; t++) {
                const int ih = oh + t / 3 - 1, iw = ow + t % 3 - 1;
                mask |= ((unsigned)ih < (unsigned)a.H && (unsigned)iw < (unsigned)a.W) ? 1 << t : 0;
            }
        }
        vm[tm] = mask;
    }

#pragma unroll
    for (int cs = 0; cs < NAB; cs++)
        issue_halo(cs);
    for (int s = 0; s < NS - 1 && s < a.nslab; s++)
        issue_w();

    const int ch0 = bn * BN + wn * (TN * 32);
    v16i acc[TN][TM];
#pragma unroll
    for (int tn = 0; tn < TN; tn++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const v4i bias = *reinterpret_cast<const v4i *>(a.bias2 + ch0 + tn * 32 + g * 8 + (lane >> 5) * 4);
#pragma unroll
            for (int tm = 0; tm < TM; tm++)
#pragma unroll
                for (int e = 0; e < 4; e++)
                    acc[tn][tm][g * 4 + e] = bias[e];
        }
    int colsum[TM];
#pragma unroll
    for (int tm = 0; tm < TM; tm++)
        colsum[tm] = 0;

    // ready(i): weight slab i has landed (and with it every halo, which are older), every wave's reads of step i-1 have
    // returned; then the freed weight stage is refilled.
    auto make_ready = [&](int i) {
        if (i + NS - 2 <= a.nslab - 1)
            wait_vmcnt<(NS - 2) * NPA>();
        else
            wait_vmcnt<0>();
        __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): this wave's fragment reads (and the pad row's store) are done
        __builtin_amdgcn_s_barrier();
        if (i + NS - 1 < a.nslab)
            issue_w();
    };

    const int swz = (lane >> 2) & 3;
    const int foff0 = (lane & 31) * 64 + (((0 + half) ^ swz) << 4);
    const int foff1 = (lane & 31) * 64 + (((2 + half) ^ swz) << 4);
    const int arow = wn * (TN * 32) * 64;
    int rt = 0, rs = 0, shift = -a.W - 1, a_off = A_OFF; // tap being read, its column, its row shift, its halo buffer
    // LDS address of this lane's bytes [16 half, 16 half + 16) of the current tap's halo row, or of the pad row where the
    // tap lies outside the image (branch-free: the mask is 0 / -1); bytes [32 + 16 half, ...) are at that address ^ 32.
    const int padc = PAD_OFF + (half << 4);
    int adr[TM];
    auto tap_addresses = [&]() {
#pragma unroll
        for (int tm = 0; tm < TM; tm++) {
            const int hr = hr0[tm] + shift;
            const int x = a_off + (hr << 6) + ((((hr >> 2) ^ half) & 3) << 4);
            const int inside = __builtin_amdgcn_sbfe(vm[tm], rt, 1);
            adr[tm] = padc ^ ((x ^ padc) & inside);
        }
    };
    auto read_frags = [&](v4i(&af)[TN], v4i(&bf)[TM], const uint8_t *wbuf, int kk) {
#pragma unroll
        for (int tn = 0; tn < TN; tn++)
            af[tn] = *reinterpret_cast<const v4i *>(wbuf + arow + tn * 2048 + (kk ? foff1 : foff0));
        if (kk == 0)
            tap_addresses();
#pragma unroll
        for (int tm = 0; tm < TM; tm++)
            bf[tm] = *reinterpret_cast<const v4i *>(lds + (adr[tm] ^ (kk << 4)));
    };
    auto next_tap = [&]() {
        ++shift;
        if (++rs == 3) {
            rs = 0;
            shift += a.W - 3;
        }
        if (++rt == 9) {
            rt = 0;
            shift = -a.W - 1;
            a_off += ABUF;
        }
    };
    auto multiply = [&](v4i(&af)[TN], v4i(&bf)[TM]) {
#pragma unroll
        for (int tm = 0; tm < TM; tm++)
            bf[tm] ^= (int)a.xmask;
#pragma unroll
        for (int tn = 0; tn < TN; tn++)
#pragma unroll
            for (int tm = 0; tm < TM; tm++)
                acc[tn][tm] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[tn], bf[tm], acc[tn][tm], 0, 0, 0);
    };

    int st_comp = 0;
    v4i af0[TN], bf0[TM], af1[TN], bf1[TM];
    make_ready(0);
    read_frags(af0, bf0, lds, 0);
    for (int i = 0; i + 1 < a.nslab; i++) {
        const uint8_t *buf = lds + st_comp * WSTAGE;
        st_comp = st_comp + 1 == NS ? 0 : st_comp + 1;
        read_frags(af1, bf1, buf, 2);
        next_tap();
        multiply(af0, bf0);
        make_ready(i + 1);
        read_frags(af0, bf0, lds + st_comp * WSTAGE, 0);
        multiply(af1, bf1);
    }
    read_frags(af1, bf1, lds + st_comp * WSTAGE, 2);
    multiply(af0, bf0);
    multiply(af1, bf1);

    __syncthreads(); // every wave has finished reading; no load is in flight any more
    if (a.fastq && a.lo == 0 && a.q.hi == 255)
        conv_epilogue<BM, BN, WM, WN, false, true, true, TM, TN>(a, acc, colsum, lds, bm, bn, wm, wn);
    else if (a.fastq)
        conv_epilogue<BM, BN, WM, WN, false, true, false, TM, TN>(a, acc, colsum, lds, bm, bn, wm, wn);
    else
        conv_epilogue<BM, BN, WM, WN, false, false, false, TM, TN>(a, acc, colsum, lds, bm, bn, wm, wn);
}

// ------------------------------------------------------------------------------------------------
// Pointwise (1x1, stride 1) convolutions with at most 64 input and 256 output channels.  Such layers are memory-bound
// (an expansion writes 4 to 16 bytes per byte it reads), and the tile machinery above - LDS staging of the activations,
// a barrier per slab, a transposing epilogue - is pure overhead for them.  Here a WAVE owns a strip of 32 pixels:
//   * its pixel fragments come straight from global memory: lane (p, h) loads bytes [32 s + 16 h, +16) of pixel p for
//     k-step s - a pixel's channels are contiguous, so that IS the MFMA operand;
//   * the weights (at most 16 KB, in the packed order of the tile kernels) and the folded bias sit in LDS for the life of
//     the work-group, which loops over strips;
//   * the rows of each 32-channel block are permuted: MFMA row i computes channel 16 ((i >> 2) & 1) + 4 (i >> 3) + (i & 3)
//     of the block, so the 16 accumulators of lane (p, h) are the 16 CONSECUTIVE channels 16 h .. 16 h + 15 of the block
//     and leave as one 128-bit store: no transpose, no barrier;
// The fused residual add stays with the tile kernels: applied to packed bytes in this layout it costs more vector
// arithmetic than their accumulator-layout form, and the layer becomes VALU-bound (measured 49 against 31 us).
// NKS: k-steps of 32 bytes (1: up to 32 input channels, 2: up to 64).  PLAIN_SAT: clamp range exactly [0, 255].
// Requires the one-multiply requantisation (the host checks).
template <int NKS, bool PLAIN_SAT>
__device__ static inline void pointwise_strips(const ConvArgs &a, const uint8_t *lds)
{
    constexpr int MAXB = 8; // 32-channel blocks
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, p = lane & 31;
    const int nb = (a.out_cs + 31) >> 5, nstrips = (a.P + 31) >> 5;
    const int prow = 16 * ((p >> 2) & 1) + 4 * (p >> 3) + (p & 3); // the channel (within a block) MFMA row p stands for
    const int32_t *lbias = reinterpret_cast<const int32_t *>(lds + 256 * 64);
    // work-groups go to the 8 XCDs in turn: XCD x takes the x-th contiguous eighth of the strips (the pixels its tile
    // kernels read and write), its work-groups interleaved inside that eighth (the grid is a multiple of 8)
    const int xcd = blockIdx.x & 7, s8 = (nstrips + 7) >> 3, s_end = min((xcd + 1) * s8, nstrips);
    for (int strip = xcd * s8 + (int)(blockIdx.x >> 3) * 4 + wave; strip < s_end; strip += (int)(gridDim.x >> 3) * 4) {
        const int m = strip * 32 + p;
        const bool ok = m < a.P;
        v4i bf[NKS];
#pragma unroll
        for (int s = 0; s < NKS; s++) {
            const int kb = 32 * s + 16 * half;
            bf[s] = v4i{0, 0, 0, 0}; // k slots beyond the input channels carry zero weights
            if (ok && kb < a.in_cs)
                bf[s] = *reinterpret_cast<const v4i *>(a.x + (size_t)m * a.in_cs + kb) ^ (int)a.xmask;
        }
        const size_t orow = (size_t)m * a.out_cs + 16 * half;
#pragma unroll
        for (int b = 0; b < MAXB; b++) {
            if (b >= nb)
                break;
            v16i acc;
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const v4i bv = *reinterpret_cast<const v4i *>(lbias + b * 32 + 16 * half + 4 * g);
#pragma unroll
                for (int e = 0; e < 4; e++)
                    acc[g * 4 + e] = bv[e];
            }
            const int ko = b * 32 + prow;
#pragma unroll
            for (int s = 0; s < NKS; s++) {
                const v4i af = *reinterpret_cast<const v4i *>(lds + ko * 64 + (((2 * s + half) ^ ((ko >> 2) & 3)) << 4));
                acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, bf[s], acc, 0, 0, 0);
            }
            u32x4 cv;
#pragma unroll
            for (int g = 0; g < 4; g++) {
                if (PLAIN_SAT) {
                    cv[g] = conv_requant4<true>(a, acc[g * 4], acc[g * 4 + 1], acc[g * 4 + 2], acc[g * 4 + 3]);
                } else {
                    int32_t rq[4];
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        rq[e] = conv_requant<true>(a, acc[g * 4 + e]);
                    cv[g] = pack_low_bytes(rq[0], rq[1], rq[2], rq[3]);
                }
            }
            if (ok && b * 32 + 16 * half < a.out_cs)
                *reinterpret_cast<u32x4 *>(a.y + orow + b * 32) = cv;
        }
    }
}

template <int NKS>
__global__ __launch_bounds__(256) void conv_mfma_pointwise_kernel(const ConvArgs a)
{
    __shared__ __attribute__((aligned(1024))) uint8_t lds[256 * 64 + 256 * 4]; // weights [kout_pad <= 256][64], folded bias
    const int tid = threadIdx.x;
    for (int i = tid * 16; i < a.kout_pad * 64; i += 256 * 16)
        *reinterpret_cast<v4i *>(lds + i) = *reinterpret_cast<const v4i *>(a.wpack + i);
    for (int i = tid; i < a.kout_pad; i += 256)
        reinterpret_cast<int32_t *>(lds + 256 * 64)[i] = a.bias2[i];
    __syncthreads();
    if (a.lo == 0 && a.q.hi == 255)
        pointwise_strips<NKS, true>(a, lds);
    else
        pointwise_strips<NKS, false>(a, lds);
}

// ------------------------------------------------------------------------------------------------
// Fully-connected layers and other 1x1 / stride 1 layers over a few hundred pixels at most (op_quant_ip_u8xu8_run,
// art/modules/quant/src/op/ip.cpp:133-209, with the batch as the pixels).  Such a layer is a weight stream: every weight
// byte is used once per pixel row and the weights are many times larger than the activations, so the time is the time
// it takes to pull the weights out of HBM, and that takes every CU.  The tile kernels cannot give every CU a share (a
// 128-row by 4096-column problem has 32 of their tiles); this kernel cuts the output into narrow column strips instead:
//   * a work-group owns 16*NB output channels of 16*MB pixel rows and the whole reduction, on v_mfma_i32_16x16x64_i8:
//     a weight fragment (16 rows of a 64-byte slab, 1 KB of the packed weights) is used by MB multiplies, a pixel
//     fragment by NB, all of one wave;
//   * the NW waves split the reduction in chunks of 128 bytes of k (two slabs: whole cache lines of the pixel rows), and
//     each wave streams ITS chunks through LDS stages of its own, R deep, with the load unit (global_load_lds_dwordx4,
//     eight lanes per 128-byte line: loading the MFMA operand straight into registers would make neighbouring lanes ask
//     for 16 bytes of sixteen different rows, a quarter of the L1 rate).  No barrier in the loop: a wave waits for its
//     own loads (vmcnt) and refills a stage once its own reads of it have returned (lgkmcnt);
//   * 16-byte piece c of pixel row r sits at piece c ^ (r & 7) of its 128-byte LDS row, the blocks of eight rows are
//     spaced so that rows r and r + 8 start in different halves of the banks, the weights keep their packed order: the
//     fragment reads are free of bank conflicts;
//   * the waves' partial sums meet once, in LDS, and the waves share the epilogue.
// Requires in_cs % 128 == 0, weight zero point 128 (or int8), no fused residual: the host checks.
template <int MB, int NB>
struct StreamCfg {
    static constexpr int ROWS = 16 * MB;
    static constexpr int XI = ROWS / 8;            // pixel loads per chunk: 8 rows of 128 bytes each
    static constexpr int PER = XI + 2 * NB;        // loads per chunk
    // block j of 8 pixel rows sits at j * 1024 + ((j + 1) >> 1) * 128: the two blocks of a 16-row fragment start in
    // different halves of the banks
    static constexpr int XBYTES = XI * 1024 + (XI / 2 + 1) * 128;
    static constexpr int STAGE = XBYTES + 2 * NB * 1024;
    static constexpr int R0 = (160 * 1024) / (4 * STAGE);
    static constexpr int R = R0 > 4 ? 4 : R0;      // stages per wave (four waves)
    static_assert(R >= 2 && (R - 1) * PER <= 63, "stage count / vmcnt range");
};

// CONVX: any kernel size, stride and padding (a convolution over few pixels - the last stages of a network at batch 1 -
// is the same weight stream): chunk c of a pixel's reduction is 128 bytes of the channels of ONE tap, read from the
// neighbouring pixel that tap points at, or from the pad source where it points outside the image.
template <int MB, int NB, bool CONVX>
__global__ __launch_bounds__(256) void conv_mfma_stream_kernel(const ConvArgs a, const int mtiles)
{
    using Cfg = StreamCfg<MB, NB>;
    constexpr int NW = 4, NT = MB * NB, R = Cfg::R, STAGE = Cfg::STAGE, PER = Cfg::PER, XI = Cfg::XI;
    constexpr int WOFF = Cfg::XBYTES; // the weight slabs follow the pixel rows in a stage
    static_assert(NW * R * STAGE >= NW * NT * 1024, "the stages double as the reduction buffer");
    __shared__ __attribute__((aligned(1024))) uint8_t lds[NW * R * STAGE];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, q = lane >> 4;
    // Work-groups go to the 8 XCDs in turn; the m-tiles of one column strip get consecutive numbers inside one XCD, so
    // that the second reader of a strip's weights finds them in that XCD's L2.
    const int idx = (int)blockIdx.x >> 3;
    const int nt = (idx / mtiles) * 8 + ((int)blockIdx.x & 7), mt = idx % mtiles;
    const int n0 = nt * (16 * NB), m0 = mt * (16 * MB);
    if (n0 >= a.out_cs)
        return;

    const int nch = a.nslab >> 1;                                // chunks of two slabs
    const int cnt = wave < nch ? (nch - wave + NW - 1) / NW : 0; // chunks of this wave
    // Every work-group reads the same pixel rows: each starts the reduction at a different chunk, so that they do not
    // all ask for the same lines at the same time (the order of an exact integer sum is free).
    const int rot = (nt * 7 + mt * 3) % nch;
    auto chunk_of = [&](int t) {
        int c = wave + NW * t + rot;
        return c >= nch ? c - nch : c;
    };
    uint8_t *const wl = lds + wave * (R * STAGE);
    // load lane l of pixel instruction j: row 8 j + (l >> 3), LDS piece l & 7 = logical piece (l & 7) ^ (row & 7)
    const int xrow = lane >> 3, xoff = ((lane & 7) ^ xrow) << 4;
    const uint8_t *wsrc = a.wpack + (size_t)n0 * 64 + lane * 16;
    const size_t wslab = (size_t)a.kout_pad * 64;
    // CONVX: this lane's pixel of load j - first input row and column of its window, pixel index of its image's origin
    int wih[CONVX ? XI : 1], wiw[CONVX ? XI : 1], wpix[CONVX ? XI : 1];
    if (CONVX) {
        const int ohw = a.OH * a.OW;
#pragma unroll
        for (int j = 0; j < XI; j++) {
            const int m = min(m0 + 8 * j + xrow, a.P - 1);
            const int n = fast_div(m, ohw, a.inv_ohw), rem = m - n * ohw;
            const int oh = fast_div(rem, a.OW, a.inv_ow), ow = rem - oh * a.OW;
            wih[j] = oh * a.stride_h - a.pad_h, wiw[j] = ow * a.stride_w - a.pad_w, wpix[j] = n * a.H * a.W;
        }
    }
    const int cpt = a.in_cs >> 7; // chunks per tap
    auto issue = [&](int t) {
        const int chunk = chunk_of(t);
        uint8_t *st = wl + (t % R) * STAGE;
        if (CONVX) {
            const int tap = chunk / cpt, coff = (chunk - tap * cpt) * 128 + xoff;
            const int kr = tap / a.S, ks = tap - kr * a.S;
#pragma unroll
            for (int j = 0; j < XI; j++) {
                const int ih = wih[j] + kr, iw = wiw[j] + ks;
                const bool ok = (unsigned)ih < (unsigned)a.H && (unsigned)iw < (unsigned)a.W;
                const uint8_t *src = ok ? a.x + (uint32_t)((wpix[j] + ih * a.W + iw) * a.in_cs + coff) : a.padbuf + (xoff & 48);
                __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(st + j * 1024 + ((j + 1) >> 1) * 128), 16, 0, 0);
            }
        } else {
#pragma unroll
            for (int j = 0; j < XI; j++) {
                const int m = min(m0 + 8 * j + xrow, a.P - 1); // rows beyond the last pixel repeat it; their results are dropped
                const uint8_t *src = a.x + (uint32_t)(m * a.in_cs + chunk * 128 + xoff);
                __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(st + j * 1024 + ((j + 1) >> 1) * 128), 16, 0, 0);
            }
        }
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
                __builtin_amdgcn_global_load_lds((gptr_t)(wsrc + (size_t)(2 * chunk + h) * wslab + nb * 1024),
                                                 (lptr_t)(st + WOFF + (h * NB + nb) * 1024), 16, 0, 0);
    };

    v4i acc[MB][NB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
            acc[mb][nb] = v4i{0, 0, 0, 0};

    for (int u = 0; u < R - 1 && u < cnt; u++)
        issue(u);
    // fragment addresses inside a stage: weights in packed order; pixel row 16 mb + r lives in block 2 mb + (r >> 3)
    // (rows r and r + 8 fall into different halves of the banks), piece (4 h + q) of the row at piece ^ (r & 7)
    const int wfo = WOFF + r * 64 + ((q ^ ((r >> 2) & 3)) << 4);
    const int xfo = (r >> 3) * 1152 + (r & 7) * 128; // + 2176 per 16-row fragment
    for (int t = 0; t < cnt; t++) {
        // this wave's fragment reads of chunk t - 1 have returned (the load unit's LDS writes are not ordered against
        // pending reads), then its stage is refilled
        __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
        if (t + R - 1 < cnt)
            issue(t + R - 1);
        const int ahead = min(R - 1, cnt - 1 - t); // chunks younger than t in flight
        if (ahead >= 3)
            wait_vmcnt<3 * PER>();
        else if (ahead == 2)
            wait_vmcnt<(R > 2 ? 2 : 0) * PER>();
        else if (ahead == 1)
            wait_vmcnt<PER>();
        else
            wait_vmcnt<0>();
        const uint8_t *st = wl + (t % R) * STAGE;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            v4i wf[NB];
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
                wf[nb] = *reinterpret_cast<const v4i *>(st + wfo + (h * NB + nb) * 1024);
#pragma unroll
            for (int mb = 0; mb < MB; mb++) {
                const v4i xs = *reinterpret_cast<const v4i *>(st + mb * 2176 + xfo + (((4 * h + q) ^ (r & 7)) << 4)) ^ (int)a.xmask;
#pragma unroll
                for (int nb = 0; nb < NB; nb++)
                    acc[mb][nb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[nb], xs, acc[mb][nb], 0, 0, 0);
            }
        }
    }

    // ---- the waves' partial sums meet in LDS; wave w finishes the tiles w, w + NW, ...
    __syncthreads(); // every wave is done with its stages; no load is in flight any more
    int32_t *red = reinterpret_cast<int32_t *>(lds); // [wave][tile][register][lane]
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
            for (int v = 0; v < 4; v++)
                red[((wave * NT + mb * NB + nb) * 4 + v) * 64 + lane] = acc[mb][nb][v];
    __syncthreads();
#pragma unroll
    for (int tl = 0; tl < (NT + NW - 1) / NW; tl++) {
        const int tile = wave + tl * NW;
        if (tile >= NT)
            break;
        const int mb = tile / NB, nb = tile % NB;
        const int m = m0 + mb * 16 + r, ko = n0 + nb * 16 + 4 * q; // this lane: 4 consecutive channels of one pixel
        const v4i bias = *reinterpret_cast<const v4i *>(a.bias2 + ko);
        int32_t v[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            uint32_t s = (uint32_t)bias[e];
#pragma unroll
            for (int w = 0; w < NW; w++)
                s += (uint32_t)red[((w * NT + tile) * 4 + e) * 64 + lane];
            v[e] = (int32_t)s;
        }
        if (m >= a.P || ko >= a.out_cs)
            continue;
        if (a.acc_out != nullptr)
            *reinterpret_cast<v4i *>(a.acc_out + (size_t)m * a.out_cs + ko) = v4i{v[0], v[1], v[2], v[3]};
        int32_t rq[4];
#pragma unroll
        for (int e = 0; e < 4; e++)
            rq[e] = a.qmult ? conv_requant_ch(a, v[e], ko + e) : a.fastq ? conv_requant<true>(a, v[e]) : conv_requant<false>(a, v[e]);
        if (a.deq_out != nullptr) { // fused dequantize (op_dequantize_run_u8, art/modules/quant/src/op/dequantize.c:111-123)
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (ko + e < a.K)
                    a.deq_out[(size_t)m * a.K + ko + e] = __fmul_rn((float)(rq[e] - a.q.zp), a.deq_alpha);
            continue;
        }
        uint32_t packed = pack_low_bytes(rq[0], rq[1], rq[2], rq[3]);
        if (a.res) { // fused residual add: exactly what the add operator computes from the convolution's stored bytes
            const uint32_t rv = *reinterpret_cast<const uint32_t *>(a.res + (size_t)m * a.out_cs + ko);
            packed = a.res_first ? add_dword<false>(rv, packed, a.addq) : add_dword<false>(packed, rv, a.addq);
        }
        *reinterpret_cast<uint32_t *>(a.y + (size_t)m * a.out_cs + ko) = packed;
    }
}

// ------------------------------------------------------------------------------------------------
// Depthwise 3x3 (group == C == K, stride 1 or 2): HBM-bound on paper (16 bytes in, 16 bytes out per output pixel and
// 16 channels), in practice bounded by vector ALU work, so the kernel is written for instruction count.
// One thread owns 4 channels (one dword of the channels-last tensors) of a strip of 4 output pixels along W; a
// wave covers 256 contiguous bytes per tap.  Bytes are re-centred as in the MFMA kernel (x ^ 0x80, w - 128).
// Stride 1: per kernel row the six input columns of the strip are byte-transposed (8 v_perm_b32 per 4x4 block)
// into per-channel dwords T0 = [x0 x1 x2 x3], T1 = [x2 x3 x4 x5]; outputs 0 / 1 are v_dot4_i32_i8 of T0 with the
// packed weights [w0 w1 w2 0] / [0 w0 w1 w2], outputs 2 / 3 the same with T1.  Stride 2: each output gathers its
// three taps with two v_perm_b32 into [x0 x1 x2 0].  bias + a * sum(w - 128) + 9ab is folded per channel; the
// b * sum(x - 128) term (wzp != 128 only) is one more dot with ones.  Taps outside the image are loaded from a
// clamped address (no divergent branch) and replaced by the byte izp.
// A thread computes 2 output rows x 4 output columns x 4 channels, so that every loaded and transposed input row
// serves up to three kernel rows of two output rows.
// QMODE 0: 64-bit requantisation; 1: one-multiply form; 2: one-multiply form and clamp range exactly [0, 255]
// (saturating packs instead of clamps).  DUMP: also write the int32 accumulators.
template <int STRIDE, bool HAS_WZP, int QMODE, bool DUMP>
__device__ static inline void depthwise3x3_body(const ConvArgs &a, int idx, int per_row, int cq, int ohp_count)
{
    constexpr int ROWS = 2;                      // output rows per thread
    constexpr int NCOL = 3 * STRIDE + 3;         // input columns a strip of 4 outputs touches
    constexpr int NIR = (ROWS - 1) * STRIDE + 3; // input rows the two output rows touch
    const uint32_t *wtab = reinterpret_cast<const uint32_t *>(a.wpack); // [3 rows][2 alignments][cs] dwords
    const int rowp = fast_div(idx, per_row, a.inv_ohw); // inv_ohw holds 1 / per_row for this kernel
    const int rem = idx - rowp * per_row;
    const int strip = fast_div(rem, cq, a.inv_ow), quad = rem - strip * cq; // inv_ow holds 1 / cq
    const int n = fast_div(rowp, ohp_count, a.inv_oh), oh0 = (rowp - n * ohp_count) * ROWS; // inv_oh: 1 / row pairs per image
    const int ow0 = strip * 4, iw0 = ow0 * STRIDE - a.pad_w, ih0 = oh0 * STRIDE - a.pad_h;
    const int c0 = quad * 4;
    const v4i bias = *reinterpret_cast<const v4i *>(a.bias2 + c0);
    v4i wa[3], wb[3];
#pragma unroll
    for (int r = 0; r < 3; r++) {
        wa[r] = *reinterpret_cast<const v4i *>(wtab + (r * 2 + 0) * a.in_cs + c0); // [w0 w1 w2 0] per channel
        if (STRIDE == 1)
            wb[r] = *reinterpret_cast<const v4i *>(wtab + (r * 2 + 1) * a.in_cs + c0); // [0 w0 w1 w2]
    }
    int32_t acc[ROWS][4][4], xsum[ROWS][4][4];
#pragma unroll
    for (int q = 0; q < ROWS; q++)
#pragma unroll
        for (int o = 0; o < 4; o++)
#pragma unroll
            for (int c = 0; c < 4; c++)
                acc[q][o][c] = bias[c], xsum[q][o][c] = 0;
    // 32-bit byte offsets from the tensor base (the host guarantees the tensor is smaller than 2 GiB)
    const uint32_t nbase = (uint32_t)(n * a.H * a.W * a.in_cs + c0);
    // threads whose whole NIR x NCOL footprint is inside the image (nearly all of them) skip the border logic
    const bool interior = ih0 >= 0 && ih0 + NIR - 1 < a.H && iw0 >= 0 && iw0 + NCOL - 1 < a.W;
    const uint32_t padx = a.padword ^ 0x80808080u;
    // all loads first (NIR x NCOL dwords in flight per thread), arithmetic afterwards: the kernel lives on memory
    // latency, not on occupancy
    uint32_t colr[NIR][NCOL];
#pragma unroll
    for (int ir = 0; ir < NIR; ir++) {
        uint32_t (&col)[NCOL] = colr[ir];
        if (interior) {
            const uint32_t rbase = nbase + (uint32_t)(((ih0 + ir) * a.W + iw0) * a.in_cs);
#pragma unroll
            for (int j = 0; j < NCOL; j++)
                col[j] = *reinterpret_cast<const uint32_t *>(a.x + (rbase + (uint32_t)(j * a.in_cs))) ^ 0x80808080u;
        } else {
            // loaded from a clamped (always valid) address, then replaced by the pad byte where outside the image
            const int ih = ih0 + ir;
            const bool row_ok = (unsigned)ih < (unsigned)a.H;
            const uint32_t rbase = nbase + (uint32_t)((ih < 0 ? 0 : (ih >= a.H ? a.H - 1 : ih)) * a.W * a.in_cs);
#pragma unroll
            for (int j = 0; j < NCOL; j++) {
                const int iw = iw0 + j;
                const uint32_t off = (uint32_t)((iw < 0 ? 0 : (iw >= a.W ? a.W - 1 : iw)) * a.in_cs);
                const uint32_t v = *reinterpret_cast<const uint32_t *>(a.x + (rbase + off)) ^ 0x80808080u;
                col[j] = (row_ok && (unsigned)iw < (unsigned)a.W) ? v : padx;
            }
        }
    }
#pragma unroll
    for (int ir = 0; ir < NIR; ir++) {
        const uint32_t (&col)[NCOL] = colr[ir];
        if (STRIDE == 1) {
#pragma unroll
            for (int h = 0; h < 2; h++) { // columns 2h .. 2h+3 serve outputs 2h and 2h+1
                const uint32_t A = col[2 * h], B = col[2 * h + 1], C = col[2 * h + 2], D = col[2 * h + 3];
                // v_perm_b32(S0, S1, sel): selector bytes 0-3 pick from S1, 4-7 from S0
                const uint32_t t0 = __builtin_amdgcn_perm(B, A, 0x05010400u), t1 = __builtin_amdgcn_perm(B, A, 0x07030602u);
                const uint32_t t2 = __builtin_amdgcn_perm(D, C, 0x05010400u), t3 = __builtin_amdgcn_perm(D, C, 0x07030602u);
                const uint32_t T[4] = {__builtin_amdgcn_perm(t2, t0, 0x05040100u), __builtin_amdgcn_perm(t2, t0, 0x07060302u),
                                       __builtin_amdgcn_perm(t3, t1, 0x05040100u), __builtin_amdgcn_perm(t3, t1, 0x07060302u)};
#pragma unroll
                for (int q = 0; q < ROWS; q++) {
                    const int kr = ir - q * STRIDE; // kernel row this input row is for output row q
                    if (kr < 0 || kr > 2)
                        continue;
#pragma unroll
                    for (int c = 0; c < 4; c++) {
                        acc[q][2 * h][c] = __builtin_amdgcn_sdot4((int)T[c], wa[kr][c], acc[q][2 * h][c], false);
                        acc[q][2 * h + 1][c] = __builtin_amdgcn_sdot4((int)T[c], wb[kr][c], acc[q][2 * h + 1][c], false);
                        if (HAS_WZP) {
                            xsum[q][2 * h][c] = __builtin_amdgcn_sdot4((int)T[c], 0x00010101, xsum[q][2 * h][c], false);
                            xsum[q][2 * h + 1][c] = __builtin_amdgcn_sdot4((int)T[c], 0x01010100, xsum[q][2 * h + 1][c], false);
                        }
                    }
                }
            }
        } else {
#pragma unroll
            for (int o = 0; o < 4; o++) {
                const uint32_t A = col[o * STRIDE], B = col[o * STRIDE + 1], C = col[o * STRIDE + 2];
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    // selector 0x0c gives a zero byte
                    const uint32_t t = __builtin_amdgcn_perm(B, A, 0x0c0c0000u | ((4u + c) << 8) | (uint32_t)c);
                    const uint32_t T = __builtin_amdgcn_perm(C, t, 0x0c000100u | ((4u + c) << 16));
#pragma unroll
                    for (int q = 0; q < ROWS; q++) {
                        const int kr = ir - q * STRIDE;
                        if (kr < 0 || kr > 2)
                            continue;
                        acc[q][o][c] = __builtin_amdgcn_sdot4((int)T, wa[kr][c], acc[q][o][c], false);
                        if (HAS_WZP)
                            xsum[q][o][c] = __builtin_amdgcn_sdot4((int)T, 0x00010101, xsum[q][o][c], false);
                    }
                }
            }
        }
    }
#pragma unroll
    for (int q = 0; q < ROWS; q++) {
        if (oh0 + q >= a.OH)
            break;
        const uint32_t obase = (uint32_t)((((n * a.OH + oh0 + q) * a.OW) + ow0) * a.out_cs + c0);
#pragma unroll
        for (int o = 0; o < 4; o++) {
            if (ow0 + o >= a.OW)
                break;
            int32_t v[4];
#pragma unroll
            for (int c = 0; c < 4; c++) {
                v[c] = (int32_t)((uint32_t)acc[q][o][c] + (HAS_WZP ? (uint32_t)(a.bwz * xsum[q][o][c]) : 0u));
                if (DUMP)
                    a.acc_out[(size_t)(obase + o * a.out_cs) + c] = v[c];
            }
            uint32_t packed = 0;
            if (QMODE == 2) {
                packed = conv_requant4<true>(a, v[0], v[1], v[2], v[3]);
            } else {
#pragma unroll
                for (int c = 0; c < 4; c++)
                    packed |= (uint32_t)((QMODE == 0 && a.qmult) ? conv_requant_ch(a, v[c], c0 + c) : conv_requant<QMODE == 1>(a, v[c])) << (8 * c);
            }
            *reinterpret_cast<uint32_t *>(a.y + (obase + (uint32_t)(o * a.out_cs))) = packed;
        }
    }
}

template <int STRIDE, bool HAS_WZP>
__global__ __launch_bounds__(256) void conv_depthwise3x3_kernel(const ConvArgs a)
{
    const int cq = a.in_cs >> 2, nstrip = (a.OW + 3) >> 2, ohp = (a.OH + 1) >> 1;
    const int per_row = nstrip * cq;
    const int total = a.N * ohp * per_row; // the host guarantees it fits in 31 bits
    const int qmode = (a.fastq && a.qmult == nullptr) ? (a.lo == 0 && a.q.hi == 255 ? 2 : 1) : 0;
    // work-groups go to the 8 XCDs in turn: renumbered so that each XCD works on one contiguous eighth of the (image-major)
    // index space, the eighth whose pixels its convolution tiles read and write (the grid is a multiple of 8)
    const int L = (int)(blockIdx.x & 7) * (int)(gridDim.x >> 3) + (int)(blockIdx.x >> 3);
    for (int idx = L * 256 + threadIdx.x; idx < total; idx += gridDim.x * 256) {
        if (a.acc_out != nullptr)
            depthwise3x3_body<STRIDE, HAS_WZP, 0, true>(a, idx, per_row, cq, ohp); // test path: exactness only
        else if (qmode == 2)
            depthwise3x3_body<STRIDE, HAS_WZP, 2, false>(a, idx, per_row, cq, ohp);
        else if (qmode == 1)
            depthwise3x3_body<STRIDE, HAS_WZP, 1, false>(a, idx, per_row, cq, ohp);
        else
            depthwise3x3_body<STRIDE, HAS_WZP, 0, false>(a, idx, per_row, cq, ohp);
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
                    acc[e] += ((int)(((xv >> (8 * e)) & 255) ^ (uint32_t)a.sx) - a.izp) * (int)wp[e];
            }
        }
        uint32_t packed = 0;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            if (a.acc_out)
                a.acc_out[(size_t)m * a.out_cs + c0 + e] = acc[e];
            packed |= (uint32_t)((a.qmult ? conv_requant_ch(a, acc[e], c0 + e) : conv_requant<false>(a, acc[e])) & 255) << (8 * e);
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
                    acc += (uint32_t)(((int)(xp[c] ^ a.sx) - a.izp) * ((int)(wp[(size_t)c * a.R * a.S] ^ a.sx) - a.wzp));
            }
        }
        if (a.acc_out)
            a.acc_out[(size_t)m * a.out_cs + k] = (int32_t)acc;
        a.y[(size_t)m * a.out_cs + k] = (uint8_t)(a.qmult ? conv_requant_ch(a, (int32_t)acc, k) : conv_requant<false>(a, (int32_t)acc));
    }
}

} // namespace hipq

// =================================================================================================
// host side
using namespace hipq;

enum ConvVariant { kMfma, kMfmaSmallC, kDepthwise3x3, kDepthwise, kDirect };

// Tile shapes of the MFMA kernel: BM pixels x BN channels per work-group, waves arranged WM x WN.
struct TileShape {
    int bm, bn;
};
static const TileShape kTiles[] = {{128, 128}, {256, 64}, {128, 64}, {64, 128}, {64, 64}};
constexpr int kNumTiles = sizeof(kTiles) / sizeof(kTiles[0]);

// conv_mfma_stream_kernel: a work-group's share is 16 * mb pixel rows by 16 * nb output channels, nw waves
struct StreamShape {
    int mb, nb, nw;
};

struct hipq_conv2d_plan {
    hipq_conv2d_desc d;
    ConvArgs args;
    ConvVariant variant;
    int tile;       // index into kTiles
    int stages = 0; // load stages of the DMA kernel; 0 = the built-in rule
    int special = 1; // the halo-tile and pointwise kernels: 0 never, 1 built-in rule, 2 wherever they apply
    bool tile_selected = false;     // hipq_conv2d_plan_select named a tile: the tile kernels, not the streaming kernel
    StreamShape stream = {0, 0, 0}; // explicit shape of the streaming kernel (hipq_conv2d_plan_stream); mb = 0: built-in rule
    bool has_wzp;
    void *d_w = nullptr, *d_bias = nullptr, *d_q = nullptr;
    std::string name;
};

// conv_mfma_halo_kernel: 3x3, stride 1, pad 1, 64-byte channel slabs, weight zero point 128 (or int8), and a halo of
// BM + 2W + 2 pixel rows within the BM + 128 rows the kernel holds; not for the 256-pixel tile.
static bool halo_applies(const hipq_conv2d_plan *p)
{
    const hipq_conv2d_desc &d = p->d;
    if (!(p->special && p->variant == kMfma && !p->has_wzp && d.in_cs % 64 == 0 && d.R == 3 && d.S == 3 && d.stride_h == 1
          && d.stride_w == 1 && d.pad_h == 1 && d.pad_w == 1 && d.W <= 63 && kTiles[p->tile].bm <= 128))
        return false;
    const int nc = d.in_cs / 64, bm = kTiles[p->tile].bm;
    if (nc == 1)
        return true;
    // Several channel slabs (all halo tiles resident at once): measured slower than the streaming kernel on 14x14 and
    // 7x7 images and equal on 28x28, so only on request.
    return p->special == 2 && (nc == 2 || nc == 4 || nc == 8) && kTiles[p->tile].bn == 128 && bm + 2 * d.W + 2 <= bm + 64;
}

// conv_mfma_pointwise_kernel: 1x1, stride 1, no padding, at most 64 input and 256 output channels, weight zero point
// 128 (or int8), one-multiply requantisation.
static bool pointwise_applies(const hipq_conv2d_plan *p)
{
    const hipq_conv2d_desc &d = p->d;
    return p->special && p->variant == kMfma && !p->has_wzp && d.R == 1 && d.S == 1 && d.stride_h == 1 && d.stride_w == 1
        && d.pad_h == 0 && d.pad_w == 0 && d.in_cs % 16 == 0 && d.in_cs <= 64 && d.out_cs % 16 == 0 && p->args.kout_pad <= 256
        && p->args.fastq && p->args.qmult == nullptr;
}

constexpr int kCUs = 256;
static bool k2_applies(const hipq_conv2d_plan *p);

// conv_mfma_stream_kernel: layers over at most 256 pixels (fully-connected layers: the pixels are the batch; the last
// stages of a network at batch 1) whose pixels are whole 128-byte lines, weight zero point 128 (or int8).  Shape of a work-group's share: 16 * mb
// pixel rows by 16 * nb output channels.  A strip that holds every pixel row reads each weight byte once; two m-tiles
// per strip halve the pixel bytes a CU pulls through its L1 (what bounds the kernel once the weights stream at full
// rate) and read the weights twice, the second time from L2.
static bool stream_applies(const hipq_conv2d_plan *p, StreamShape *shape = nullptr)
{
    const hipq_conv2d_desc &d = p->d;
    const ConvArgs &a = p->args;
    // up to 256 pixels whatever the layer; up to 1024 where the reduction is at least 512 bytes long (measured against the
    // tile kernels: 3x3 on 784 pixels 4.8 against 7.0 us at 128 channels, 6.2 against 10.7 at 256, 12.3 against 18.4 at
    // 512; 1x1 1024 -> 256 on 784 pixels 3.9 against 6.3; behind from 1568 pixels on, and at 256 -> 1024 from 392)
    if (!(p->special && !p->tile_selected && p->variant == kMfma && !p->has_wzp && d.in_cs % 128 == 0
          && (a.P <= 256 || (a.P <= 1024 && d.R * d.S * d.in_cs >= 512)) && (long long)d.N * d.H * d.W * d.in_cs < (1ll << 31)))
        return false;
    if (shape) {
        if (p->stream.mb) {
            *shape = p->stream;
            return true;
        }
        // What a CU pulls through its L1 bounds the kernel once the weights stream at full rate: per work-group
        // (16 mb + 16 nb) rows of k bytes, times the rounds of work-groups the chip needs.  The smallest product wins,
        // more work-groups on a tie (measured: 128 x 4096 x 4096 takes 8.6 us as 64 x 32, 11.3 as 128 x 16, 10.1 as
        // 32 x 32; 64 x 2048 x 1000 takes 3.5 us as 16 x 16, 4.7 as 64 x 16).
        static const StreamShape cand[] = {{8, 1, 4}, {4, 2, 4}, {4, 1, 4}, {2, 2, 4}, {2, 1, 4}, {1, 2, 4}, {1, 1, 4}};
        const int rows = (a.P + 15) / 16;
        long long best = -1, best_wgs = 0;
        for (const StreamShape &c : cand) {
            if (c.mb > 1 && c.mb / 2 >= rows)
                continue; // half of the rows would be padding
            const long long wgs = (long long)((rows + c.mb - 1) / c.mb) * ((a.out_cs + 16 * c.nb - 1) / (16 * c.nb));
            const long long cost = ((wgs + kCUs - 1) / kCUs) * (c.mb + c.nb);
            if (best < 0 || cost < best || (cost == best && wgs > best_wgs))
                best = cost, best_wgs = wgs, *shape = c;
        }
    }
    return true;
}

// conv_mfma_expand_kernel (conv_expand.hip): a 1x1 layer that widens the channels, for this launch's arguments (with a
// residual to add or without)
static bool expand_applies(const hipq_conv2d_plan *p, const ConvArgs &a)
{
    return p->variant == kMfma && p->special && !p->tile_selected && !p->has_wzp && conv_expand_applies(a, p->special == 2);
}

// conv3x3_c64_rows_kernel (conv_rows.hip): 3x3 / stride 1 / pad 1 with 64 channels in and out, rows resident in LDS
static bool rows_applies(const hipq_conv2d_plan *p, const ConvArgs &a)
{
    return p->variant == kMfma && p->special == 1 && !p->tile_selected && !p->has_wzp && conv_rows_applies(a);
}

// conv_wreg_kernel (conv_wreg.hip): 1x1 / 3x3 layers whose weight operands go straight from memory to the waves' registers
static bool wreg_applies(const hipq_conv2d_plan *p, const ConvArgs &a)
{
    if (!(p->variant == kMfma && p->special && !p->tile_selected && !p->has_wzp && p->d.dtype == HIPQ_DTYPE_U8 && conv_wreg_applies(a)))
        return false;
    if (p->special == 3)
        return true;
    if (p->special == 2)
        return false; // mode 2 asks for the halo / two-group / widening kernels wherever they apply
    // built-in rule (measured at batch 64 against the tile kernels): the 3x3 layers of the 14x14 and 7x7 stages (256 -> 256 at
    // 14x14 16.5 -> 13.2 us, 512 -> 512 at 7x7 18.2 -> 13.7, the stride-2 layers into them 17.2 -> 15.3 and 18.1 -> 15.6) and the
    // 1x1 layers there that reduce the channels four times (1024 -> 256: 9.0 -> 7.9 us, 2048 -> 512: 10.1 -> 8.0); level or behind
    // on the other 1x1 layers and on larger images
    if (a.P > 16384 || a.P <= 1024)
        return false;
    if (a.R == 3)
        return true;
    return a.res == nullptr && a.stride_h == 1 && a.in_cs >= 4 * a.out_cs;
}

// conv_stem3x3_kernel (conv_stem.hip): 3x3 / stride 2 from an image with at most 4 channels to at most 32
static bool stem3_applies(const hipq_conv2d_plan *p, const ConvArgs &a)
{
    return p->variant == kMfmaSmallC && p->special >= 1 && !p->tile_selected && !p->has_wzp && conv_stem3x3_applies(a, a.rowb);
}

static void set_mfma_name(hipq_conv2d_plan *p, bool smallc)
{
    char nm[96];
    StreamShape ss;
    if (!smallc && wreg_applies(p, p->args))
        snprintf(nm, sizeof nm, "conv_mfma_i8_wreg");
    else if (!smallc && stream_applies(p, &ss))
        snprintf(nm, sizeof nm, "conv_mfma_i8_stream_%dx%d%s", 16 * ss.mb, 16 * ss.nb, p->d.dtype == HIPQ_DTYPE_I8 ? "_signed" : "");
    else if (!smallc && rows_applies(p, p->args))
        snprintf(nm, sizeof nm, "conv_mfma_i8_rows3x3%s", p->d.dtype == HIPQ_DTYPE_I8 ? "_signed" : "");
    else if (!smallc && expand_applies(p, p->args))
        snprintf(nm, sizeof nm, "conv_mfma_i8_expand%s", p->d.dtype == HIPQ_DTYPE_I8 ? "_signed" : "");
    else if (pointwise_applies(p))
        snprintf(nm, sizeof nm, "conv_mfma_i8_pointwise%s", p->d.dtype == HIPQ_DTYPE_I8 ? "_signed" : "");
    else if (smallc && stem3_applies(p, p->args))
        snprintf(nm, sizeof nm, "conv_mfma_i8_stem3x3");
    else
        snprintf(nm, sizeof nm, "conv_mfma_i8_%dx%d%s%s%s%s", kTiles[p->tile].bm, kTiles[p->tile].bn, smallc ? "_c4" : "",
                 p->has_wzp ? "_wzp" : "", p->d.dtype == HIPQ_DTYPE_I8 ? "_signed" : "",
                 halo_applies(p) ? "_halo" : (!smallc && k2_applies(p)) ? "_k2" : "");
    p->name = nm;
    if (p->d_q)
        p->name += "_perchannel";
}

static int conv_out_dim(int in, int pad, int k, int stride)
{
    // art/src/op.c:549-555 (unsigned arithmetic, hole == 1)
    return (int)(((uint32_t)in + 2u * (uint32_t)pad - (uint32_t)k) / (uint32_t)stride + 1u);
}

// Largest tile that still gives every CU a few work-groups to overlap (two waves per SIMD hide the
// global-load latency of one another).
static int choose_tile(long long P, int out_cs, bool expand, int in_cs)
{
    auto count = [&](int t) { return ((P + kTiles[t].bm - 1) / kTiles[t].bm) * ((out_cs + kTiles[t].bn - 1) / kTiles[t].bn); };
    // one tile of channels, or a width that would leave 15 % or more of the 128-channel tiles' columns empty (96, 160,
    // 320 channels): 64x64 tiles (MobileNetV2 at batch 64, inside the network: 0.463 -> 0.459 ms for the first, -> 0.460
    // for the second; alone, 128x64 tiles are 5 % faster on the 56x56 layers)
    if (out_cs <= 64 || ((out_cs + 127) / 128 * 128 - out_cs) * 100 >= 15 * ((out_cs + 127) / 128 * 128))
        return 4;
    if (expand && P >= 8000) // short reduction, wide output: store-bound, many small work-groups overlap best; from 512
        return in_cs >= 512 ? 3 : 4; // input channels on the reduction is long enough for the wider tile (17.4 -> 14.9 us)
    if (expand && count(0) >= 200 && count(0) < kCUs)
        return 4; // a widening layer whose 128x128 tiles would leave CUs idle: small tiles (MobileNetV2's 160 -> 960 and
                  // 320 -> 1280 at 7x7, batch 64: the pass 0.470 -> 0.463 ms; 64x128 tiles 0.465)
    if (count(3) <= 128)
        return 4; // tiles for at most half the CUs (fully-connected layers, 7x7 layers at batch 32): the smallest tile, to
                  // put more CUs on the weight stream (512 -> 512 3x3 on 1568 pixels: 16.1 -> 14.3 us)
    return count(0) >= 200 ? 0 : 3;      // 128x128, or 64x128 when that leaves most CUs idle
}

// walpha_pc: nullptr, or K weight scales (one per output channel), which replace desc.walpha
static int plan_create(const hipq_conv2d_desc *dp, const uint8_t *w, const int32_t *bias, const float *walpha_pc,
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
    HIPQ_REQUIRE(d.dtype == HIPQ_DTYPE_U8 || d.dtype == HIPQ_DTYPE_I8, "conv: dtype must be HIPQ_DTYPE_U8 or HIPQ_DTYPE_I8");
    // int8 symmetric tensors (op_conv_2d_i8xi8_run, conv_2d_int8_impl.c:34-174): no zero points, out-of-image taps
    // are 0, the result is clipped to +-(2^obits - 1) and stored as the low byte.  An int8 byte b is the uint8 byte
    // b ^ 0x80 with zero point 128, which is how the kernels that are not specialised read it.
    const bool sgn = d.dtype == HIPQ_DTYPE_I8;

    auto *p = new hipq_conv2d_plan();
    p->d = d;
    ConvArgs &a = p->args;
    memset(&a, 0, sizeof(a));
    a.N = d.N, a.C = d.C, a.H = d.H, a.W = d.W, a.K = d.K, a.R = d.R, a.S = d.S;
    a.pad_h = d.pad_h, a.pad_w = d.pad_w, a.stride_h = d.stride_h, a.stride_w = d.stride_w, a.group = d.group;
    a.in_cs = d.in_cs, a.out_cs = d.out_cs;
    a.OH = conv_out_dim(d.H, d.pad_h, d.R, d.stride_h);
    a.OW = conv_out_dim(d.W, d.pad_w, d.S, d.stride_w);
    a.izp = sgn ? 128 : d.izp, a.wzp = sgn ? 128 : d.wzp;
    a.sx = sgn ? 0x80 : 0;
    a.xmask = sgn ? 0u : 0x80808080u;
    const long long P = (long long)d.N * a.OH * a.OW;
    if (P <= 0 || P * (long long)d.out_cs >= (1ll << 31) || (long long)d.N * d.H * d.W * d.in_cs >= (1ll << 31)) {
        delete p;
        return fail("conv: tensor too large for 32-bit indexing (or empty output)");
    }
    a.P = (int)P;
    // per-channel weight scales: one (mult, shift) per output channel, derived exactly like the tensor's pair; the
    // tensor's own pair is that of channel 0 (what the reference CPU module, which reads walpha[0] only, would use)
    std::vector<uint32_t> qbuf;
    if (walpha_pc != nullptr) {
        const size_t npad = ((size_t)std::max(d.K, d.out_cs) + 127) / 128 * 128;
        qbuf.assign(2 * npad, 0);
        for (size_t k = 0; k < npad; k++) {
            uint32_t m;
            int sh;
            hipq_quant_scale(d.ialpha * walpha_pc[k < (size_t)d.K ? k : 0] / d.oalpha, 32, &m, &sh);
            if (!valid_shift(sh)) {
                delete p;
                return fail("conv: requantisation shift %d of channel %zu outside 1..62 (scale %g)", sh, k,
                            (double)(d.ialpha * walpha_pc[k < (size_t)d.K ? k : 0] / d.oalpha));
            }
            qbuf[k] = m, qbuf[npad + k] = (uint32_t)sh;
        }
    }
    hipq_quant_scale(d.ialpha * (walpha_pc ? walpha_pc[0] : d.walpha) / d.oalpha, 32, &a.q.mult, &a.q.shift);
    a.q.zp = sgn ? 0 : d.ozp;
    a.q.hi = (1 << d.obits) - 1;
    // fused ReLU: max(y, ozp); a zero point beyond the saturation value (obits < 8) leaves only that value, as the
    // reference's relu applied to the saturated convolution output would
    a.lo = sgn ? (d.relu ? 0 : -a.q.hi) : (d.relu ? std::min(d.ozp, a.q.hi) : 0);
    if (!valid_shift(a.q.shift)) {
        delete p;
        return fail("conv: requantisation shift %d outside 1..62 (scale %g)", a.q.shift,
                    (double)(d.ialpha * (walpha_pc ? walpha_pc[0] : d.walpha) / d.oalpha));
    }
    // the one-multiply form needs one shift for the whole tensor: never for per-channel scales, whatever channel 0's is
    a.fastq = walpha_pc == nullptr && a.q.shift >= 33 && a.q.shift <= 52;
    a.qt = a.fastq ? a.q.shift - 32 : 1;
    a.qadd = a.fastq ? (1 << (a.qt - 1)) + (a.q.zp << a.qt) : 0;
    a.inv_ohw = 1.0 / ((double)a.OH * a.OW);
    a.inv_ow = 1.0 / (double)a.OW;
    const int pad_byte = sgn ? 0 : d.izp; // the byte an out-of-image tap reads
    a.padword = 0x01010101u * (uint32_t)pad_byte;
    const int aoff = 128 - a.izp, boff = 128 - a.wzp; // both 0 for int8
    // weight byte -> signed value relative to 128 (uint8) or the int8 value itself
    auto wval = [&](uint8_t b) { return sgn ? (int)(int8_t)b : (int)b - 128; };
    a.bwz = boff;

    const int cg = d.C / d.group;
    std::vector<uint8_t> wbuf;
    std::vector<int32_t> bbuf;
    size_t pad_off = 0, frag_off = 0;
    if (d.group == 1 && (d.in_cs % 16 == 0 || d.in_cs == 4)) {
        const bool smallc = d.in_cs == 4;
        p->variant = smallc ? kMfmaSmallC : kMfma;
        p->tile = choose_tile(a.P, d.out_cs, d.R == 1 && d.S == 1 && d.out_cs >= 2 * d.in_cs, d.in_cs);
        const int BM = kTiles[p->tile].bm, BN = kTiles[p->tile].bn;
        a.nbm = (a.P + BM - 1) / BM;
        a.nbn = (d.out_cs + BN - 1) / BN;
        a.rowb = smallc ? 4 * ((d.S + 3) / 4 * 4) : d.in_cs;
        a.Ktot = smallc ? d.R * a.rowb : d.R * d.S * d.in_cs;
        a.nslab = (a.Ktot + 63) / 64;
        // every tile kernel indexes weight rows and folded constants by output-channel TILE, i.e. up to out_cs rounded up
        // to its tile width: the padding covers the output stride, not just K (a caller may write into a wider buffer)
        a.kout_pad = (std::max(d.K, d.out_cs) + 127) / 128 * 128;
        p->has_wzp = boff != 0;
        // weights: [slab][kout_pad][64 bytes]; chunk c of row ko is stored at chunk c ^ ((ko >> 2) & 3),
        // the order the kernel keeps in LDS.  Rows of pad output channels stay zero (their outputs are
        // don't-care bytes in the pad channels of y).
        wbuf.assign((size_t)a.nslab * a.kout_pad * 64, 0);
        bbuf.assign((size_t)a.kout_pad, 0);
        for (int ko = 0; ko < d.K; ko++) {
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
                        ws = wval(w[(((size_t)ko * d.C + c) * d.R + r) * d.S + s]);
                }
                wsum += ws;
                const int slab = kp >> 6, chunk = ((kp >> 4) & 3) ^ ((ko >> 2) & 3);
                wbuf[((size_t)slab * a.kout_pad + ko) * 64 + chunk * 16 + (kp & 15)] = (uint8_t)(int8_t)ws;
            }
            const long long c0 = (bias ? (long long)bias[ko] : 0) + (long long)aoff * wsum
                + (long long)a.nslab * 64 * aoff * boff;
            bbuf[ko] = (int32_t)(uint32_t)(unsigned long long)c0;
        }
        pad_off = wbuf.size();
        wbuf.resize(pad_off + 64, (uint8_t)pad_byte); // source of out-of-image taps
        // the same weights in fragment order (ConvArgs::wfrag) for the kernels whose waves load their MFMA weight
        // operands straight from memory: layers of a bottleneck block
        if (!smallc && boff == 0 && d.in_cs % 64 == 0 && d.in_cs <= 2048 && d.out_cs <= 2048 && d.C == d.in_cs
            && ((d.R == 1 && d.S == 1) || (d.R == 3 && d.S == 3))) {
            frag_off = (wbuf.size() + 255) / 256 * 256;
            wbuf.resize(frag_off + pad_off, 0);
            for (int sl = 0; sl < a.nslab; sl++)
                for (int T = 0; T < a.kout_pad / 32; T++)
                    for (int kk = 0; kk < 2; kk++)
                        for (int l = 0; l < 64; l++) {
                            const int pp = l & 31, hh = l >> 5;
                            const int ko = 32 * T + 16 * ((pp >> 2) & 1) + 4 * (pp >> 3) + (pp & 3);
                            const uint8_t *src = &wbuf[((size_t)sl * a.kout_pad + ko) * 64 + (((2 * kk + hh) ^ ((ko >> 2) & 3)) << 4)];
                            memcpy(&wbuf[frag_off + ((((size_t)sl * (a.kout_pad / 32) + T) * 2 + kk) * 64 + l) * 16], src, 16);
                        }
        }
        p->special = 1;
        set_mfma_name(p, smallc);
    } else if (!sgn && d.group == d.C && d.K == d.C && d.in_cs == d.out_cs && d.R == 3 && d.S == 3 && d.stride_h == d.stride_w
               && (d.stride_h == 1 || d.stride_h == 2)
               && (long long)d.N * a.OH * ((a.OW + 3) / 4) * (d.in_cs / 4) < (1ll << 31)) {
        p->variant = kDepthwise3x3;
        p->has_wzp = boff != 0;
        // weights: [kernel row][alignment][cs] dwords, {w0 - 128, w1 - 128, w2 - 128, 0} and {0, w0 - 128, w1 - 128, w2 - 128}
        wbuf.assign((size_t)3 * 2 * d.in_cs * 4, 0);
        bbuf.assign(d.in_cs, 0);
        for (int c = 0; c < d.C; c++) {
            long long wsum = 0;
            for (int r = 0; r < 3; r++)
                for (int t = 0; t < 3; t++) {
                    const int ws = (int)w[(size_t)c * 9 + r * 3 + t] - 128;
                    wsum += ws;
                    wbuf[((size_t)(r * 2 + 0) * d.in_cs + c) * 4 + t] = (uint8_t)(int8_t)ws;
                    wbuf[((size_t)(r * 2 + 1) * d.in_cs + c) * 4 + t + 1] = (uint8_t)(int8_t)ws;
                }
            const long long c0 = (bias ? (long long)bias[c] : 0) + (long long)aoff * wsum + 9ll * aoff * boff;
            bbuf[c] = (int32_t)(uint32_t)(unsigned long long)c0;
        }
        a.inv_ohw = 1.0 / ((double)((a.OW + 3) / 4) * (d.in_cs / 4));
        a.inv_ow = 1.0 / (double)(d.in_cs / 4);
        a.inv_oh = 1.0 / (double)((a.OH + 1) / 2);
        p->name = std::string("conv_depthwise3x3_u8_s") + (d.stride_h == 1 ? "1" : "2") + (p->has_wzp ? "_wzp" : "");
    } else if (d.group == d.C && d.K == d.C && d.in_cs == d.out_cs) {
        p->variant = kDepthwise;
        wbuf.assign((size_t)d.R * d.S * d.in_cs * 2, 0);
        int16_t *wq = reinterpret_cast<int16_t *>(wbuf.data());
        for (int c = 0; c < d.C; c++)
            for (int t = 0; t < d.R * d.S; t++)
                wq[(size_t)t * d.in_cs + c] = (int16_t)(wval(w[(size_t)c * d.R * d.S + t]) + boff);
        bbuf.assign(d.in_cs, 0);
        for (int c = 0; c < d.C; c++)
            bbuf[c] = bias ? bias[c] : 0;
        p->name = sgn ? "conv_depthwise_i8" : "conv_depthwise_u8";
    } else {
        p->variant = kDirect;
        wbuf.assign(w, w + (size_t)d.K * cg * d.R * d.S);
        bbuf.assign(d.K, 0);
        for (int k = 0; k < d.K; k++)
            bbuf[k] = bias ? bias[k] : 0;
        p->name = sgn ? "conv_direct_i8" : "conv_direct_u8";
    }

    hipError_t e = hipMalloc(&p->d_w, wbuf.size());
    if (e == hipSuccess)
        e = hipMalloc(&p->d_bias, bbuf.size() * sizeof(int32_t));
    if (e == hipSuccess && !qbuf.empty()) {
        e = hipMalloc(&p->d_q, qbuf.size() * sizeof(uint32_t));
        if (e == hipSuccess)
            e = hipMemcpy(p->d_q, qbuf.data(), qbuf.size() * sizeof(uint32_t), hipMemcpyHostToDevice);
    }
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
    a.padbuf = a.wpack + pad_off;
    a.wfrag = frag_off ? a.wpack + frag_off : nullptr;
    if (frag_off)
        set_mfma_name(p, false); // the register-fed kernel's rule looks at the fragment-order copy
    if (p->d_q) {
        a.qmult = static_cast<const uint32_t *>(p->d_q);
        a.qshift = reinterpret_cast<const int32_t *>(a.qmult + qbuf.size() / 2);
        if (p->variant == kMfma || p->variant == kMfmaSmallC)
            set_mfma_name(p, p->variant == kMfmaSmallC); // the pointwise kernel does not serve per-channel scales
        else
            p->name += "_perchannel";
    }
    *plan_out = p;
    return 0;
}

extern "C" int hipq_conv2d_plan_create(const hipq_conv2d_desc *dp, const uint8_t *w, const int32_t *bias,
                                       hipq_conv2d_plan **plan_out)
{
    return plan_create(dp, w, bias, nullptr, plan_out);
}

extern "C" int hipq_conv2d_plan_create_per_channel(const hipq_conv2d_desc *dp, const uint8_t *w, const int32_t *bias,
                                                   const float *walpha, hipq_conv2d_plan **plan_out)
{
    clear_error();
    HIPQ_REQUIRE(walpha, "hipq_conv2d_plan_create_per_channel: null walpha");
    return plan_create(dp, w, bias, walpha, plan_out);
}

extern "C" void hipq_conv2d_plan_destroy(hipq_conv2d_plan *p)
{
    if (!p)
        return;
    if (p->d_w)
        (void)hipFree(p->d_w);
    if (p->d_bias)
        (void)hipFree(p->d_bias);
    if (p->d_q)
        (void)hipFree(p->d_q);
    delete p;
}

extern "C" const char *hipq_conv2d_plan_kernel(const hipq_conv2d_plan *p) { return p ? p->name.c_str() : ""; }

extern "C" const char *hipq_conv2d_plan_kernel_add(const hipq_conv2d_plan *p)
{
    if (!p || (p->variant != kMfma && p->variant != kMfmaSmallC))
        return "";
    static thread_local std::string nm;
    ConvArgs a = p->args;
    a.res = a.padbuf; // any non-null pointer: the question is which kernel a launch with a residual goes to
    a.addq.fast = 1;  // the 32-bit form of the add, which ordinary scale ratios allow
    a.addq.hi = 255;  // to 8 bits
    char buf[96];
    StreamShape ss;
    if (wreg_applies(p, a))
        snprintf(buf, sizeof buf, "conv_mfma_i8_wreg+add");
    else if (stream_applies(p, &ss))
        snprintf(buf, sizeof buf, "conv_mfma_i8_stream_%dx%d%s+add", 16 * ss.mb, 16 * ss.nb, p->d.dtype == HIPQ_DTYPE_I8 ? "_signed" : "");
    else if (rows_applies(p, a))
        snprintf(buf, sizeof buf, "conv_mfma_i8_rows3x3+add");
    else if (expand_applies(p, a))
        snprintf(buf, sizeof buf, "conv_mfma_i8_expand%s+add", p->d.dtype == HIPQ_DTYPE_I8 ? "_signed" : "");
    else
        snprintf(buf, sizeof buf, "conv_mfma_i8_%dx%d%s%s%s%s+add", kTiles[p->tile].bm, kTiles[p->tile].bn,
                 p->variant == kMfmaSmallC ? "_c4" : "", p->has_wzp ? "_wzp" : "", p->d.dtype == HIPQ_DTYPE_I8 ? "_signed" : "",
                 p->variant == kMfma && k2_applies(p) ? "_k2" : "");
    nm = buf;
    if (p->d_q)
        nm += "_perchannel";
    return nm.c_str();
}

extern "C" int hipq_conv2d_plan_select(hipq_conv2d_plan *p, int tile, int stages)
{
    clear_error();
    HIPQ_REQUIRE(p, "hipq_conv2d_plan_select: null plan");
    HIPQ_REQUIRE(p->variant == kMfma, "hipq_conv2d_plan_select: only the DMA-fed MFMA kernel has variants (this plan runs %s)",
                 p->name.c_str());
    HIPQ_REQUIRE(tile >= -1 && tile < kNumTiles && (stages == 0 || (stages >= 2 && stages <= 4) || stages == 8),
                 "hipq_conv2d_plan_select: tile must be -1 (keep) or 0..%d, stages 0 (built-in rule), 2..4 or 8", kNumTiles - 1);
    if (tile >= 0) {
        p->tile_selected = true;
        p->tile = tile;
        p->args.nbm = (p->args.P + kTiles[tile].bm - 1) / kTiles[tile].bm;
        p->args.nbn = (p->d.out_cs + kTiles[tile].bn - 1) / kTiles[tile].bn;
    }
    p->stages = stages;
    set_mfma_name(p, false);
    return 0;
}

extern "C" int hipq_conv2d_plan_special(hipq_conv2d_plan *p, int mode)
{
    clear_error();
    HIPQ_REQUIRE(p, "hipq_conv2d_plan_special: null plan");
    HIPQ_REQUIRE(p->variant == kMfma || p->variant == kMfmaSmallC,
                 "hipq_conv2d_plan_special: only the MFMA kernels have variants (this plan runs %s)", p->name.c_str());
    HIPQ_REQUIRE(mode >= 0 && mode <= 3, "hipq_conv2d_plan_special: mode must be 0 (never), 1 (built-in rule), 2 (wherever they apply) or 3 (the register-fed kernel wherever it applies)");
    p->special = mode;
    set_mfma_name(p, p->variant == kMfmaSmallC);
    return 0;
}

extern "C" int hipq_conv2d_plan_stream(hipq_conv2d_plan *p, int rows, int cols, int waves)
{
    clear_error();
    HIPQ_REQUIRE(p, "hipq_conv2d_plan_stream: null plan");
    HIPQ_REQUIRE(stream_applies(p), "hipq_conv2d_plan_stream: this plan does not run the streaming kernel (it runs %s)", p->name.c_str());
    if (rows == 0 && cols == 0 && waves == 0) {
        p->stream = {0, 0, 0};
    } else {
        const int key = rows / 16 * 100 + cols / 16 * 10 + waves;
        static const int ok[] = {814, 424, 414, 224, 214, 124, 114};
        bool found = rows % 16 == 0 && cols % 16 == 0;
        if (found) {
            found = false;
            for (int k : ok)
                found = found || k == key;
        }
        HIPQ_REQUIRE(found, "hipq_conv2d_plan_stream: no instantiation for %d rows x %d columns with %d waves", rows, cols, waves);
        p->stream = {rows / 16, cols / 16, waves};
    }
    set_mfma_name(p, false);
    return 0;
}

// Load stages.  Short reductions (few slabs) run with two stages: the smaller LDS footprint lets four work-groups
// share a CU and overlap their load, multiply and store phases.  Long reductions (3x3 layers, wide 1x1 layers) run
// with four (three for the largest tile): measured inside the whole network, where a layer's input comes from HBM
// or the last-level cache rather than from a warm L2, the deeper stream is worth 10 % of the ResNet-50 step.
constexpr int kStages = 2;
constexpr int kDeepFrom = 8; // slabs

template <int BM, int BN, int WM, int WN, int NS, bool FUSED>
static void launch_dma_aligned(const dim3 grid, const ConvArgs &a, hipStream_t st)
{
    hipLaunchKernelGGL((conv_mfma_dma_kernel<BM, BN, WM, WN, NS, false, true, FUSED>), grid, dim3(256), 0, st, a);
}

// Weight stages of the halo kernel beside nab halo buffers of nph * 64 rows: as many as leave two work-groups to a CU
// (80 KB each), at most 8; where the halo buffers alone leave fewer than 4, one work-group per CU and 7 stages.
constexpr int halo_stages(int bn, int nph, int nab)
{
    const int n = (80 * 1024 - 64 - nab * nph * 4096) / (bn * 64);
    return n > 8 ? 8 : n < 4 ? 7 : n;
}

// The halo-tile kernel serves 3x3 / stride 1 / pad 1 layers whose halo (BM + 2W + 2 pixel rows) fits BM + 128 LDS rows
// (one channel slab) or BM + 64 rows (2, 4 or 8 channel slabs; 128x128 and 64x128 tiles).
template <int BM, int BN, int WM, int WN>
static bool launch_halo(const hipq_conv2d_plan *p, const ConvArgs &a, const dim3 grid, hipStream_t st)
{
    if constexpr (BM > 128) {
        return false;
    } else {
        if (!halo_applies(p) || a.res != nullptr) // the fused residual add stays with the streaming kernel
            return false;
        constexpr int N0 = BM / 64 + 1;
        const bool wide = BM + 2 * a.W + 2 > N0 * 64;
        const int nc = a.in_cs / 64;
        const dim3 block(256);
        if (nc == 1) {
            // a single channel slab has nine steps in all
            if (wide)
                hipLaunchKernelGGL((conv_mfma_halo_kernel<BM, BN, WM, WN, 4, N0 + 1, 1>), grid, block, 0, st, a);
            else
                hipLaunchKernelGGL((conv_mfma_halo_kernel<BM, BN, WM, WN, 4, N0, 1>), grid, block, 0, st, a);
            return true;
        }
        if constexpr (BN == 128) {
            // A step is 128-256 clocks of MFMA work against a load latency of well over a thousand, so the weight stream
            // runs as deep as LDS allows (a weight stage is only BN * 64 bytes here).
            if (wide)
                return false;
            if (nc == 2)
                hipLaunchKernelGGL((conv_mfma_halo_kernel<BM, BN, WM, WN, halo_stages(BN, N0, 2), N0, 2>), grid, block, 0, st, a);
            else if (nc == 4)
                hipLaunchKernelGGL((conv_mfma_halo_kernel<BM, BN, WM, WN, halo_stages(BN, N0, 4), N0, 4>), grid, block, 0, st, a);
            else if (nc == 8)
                hipLaunchKernelGGL((conv_mfma_halo_kernel<BM, BN, WM, WN, halo_stages(BN, N0, 8), N0, 8>), grid, block, 0, st, a);
            else
                return false;
            return true;
        }
        return false;
    }
}

// conv_mfma_dma_k2_kernel (the reduction shared by two groups of four waves): convolutions - with or without a fused
// residual add, which its epilogue applies to the staged tile like the generic kernels' - with aligned addressing, an even number of at least 8 slabs, a tile of at most 128 + 64 or 64 + 128 rows per stage
// pair, and - by the built-in rule - no more tiles than the chip has CUs, i.e. layers that would otherwise run one wave
// per SIMD.  Measured inside the ResNet-50 pass the 7x7 layers gain 20 %; layers with one to two tiles per CU gain
// nothing (two four-wave work-groups already share their CUs) and 128x128 tiles lose.  An explicit stage count
// (hipq_conv2d_plan_select) keeps the four-wave kernel.
static bool k2_applies(const hipq_conv2d_plan *p)
{
    const ConvArgs &a = p->args;
    const bool aligned = a.in_cs % 64 == 0 || (a.R == 1 && a.S == 1 && a.in_cs % 16 == 0);
    if (!(p->special && p->stages == 0 && p->variant == kMfma && !p->has_wzp && aligned && (a.nslab & 1) == 0 && a.nslab >= 8))
        return false;
    if (kTiles[p->tile].bm + kTiles[p->tile].bn > 256)
        return false;
    // up to a tile and a half per CU as well, for 64x128 tiles on a long reduction (ResNet-50's 3x3 layers at 14x14: 392
    // tiles, 36 slabs, 15.3 -> 14.9 us inside the network; shorter reductions lose there: 1x1 1024 -> 256 8.8 -> 9.4)
    if (a.nslab >= 32 && kTiles[p->tile].bm == 64 && kTiles[p->tile].bn == 128 && a.nbm * a.nbn <= 400)
        return true;
    return p->special == 2 || a.nbm * a.nbn <= kCUs;
}

template <int BM, int BN, int WM, int WN>
static bool launch_k2(const hipq_conv2d_plan *p, const ConvArgs &a, const dim3 grid, hipStream_t st)
{
    if constexpr (BM + BN > 256) {
        return false;
    } else {
        if (!k2_applies(p))
            return false;
        if (a.nbm * a.nbn <= kCUs || BM + BN > 192) {
            // one work-group per CU: LDS is no constraint, so the deepest stream the stages allow
            hipLaunchKernelGGL((conv_mfma_dma_k2_kernel<BM, BN, WM, WN, (BM + BN <= 192 ? 4 : 3)>), grid, dim3(512), 0, st, a);
        } else {
            // more tiles than CUs (on request only): three stages per group, so that two work-groups still share a CU
            hipLaunchKernelGGL((conv_mfma_dma_k2_kernel<BM, BN, WM, WN, 3>), grid, dim3(512), 0, st, a);
        }
        return true;
    }
}

template <int BM, int BN, int WM, int WN>
static void launch_mfma(const hipq_conv2d_plan *p, const ConvArgs &a, hipStream_t st)
{
    const int nblk = a.nbm * a.nbn;
    const dim3 grid((nblk + 7) / 8 * 8), block(256);
    StreamShape ss;
    const bool streams = stream_applies(p, &ss); // the kernel the plan is named after wins over the halo kernel
    if (p->variant == kMfma && !streams && launch_halo<BM, BN, WM, WN>(p, a, grid, st))
        return;
    if (streams) {
        const bool fc = a.R == 1 && a.S == 1 && a.stride_h == 1 && a.stride_w == 1 && a.pad_h == 0 && a.pad_w == 0;
        const int mtiles = (a.P + 16 * ss.mb - 1) / (16 * ss.mb), ntiles = (a.out_cs + 16 * ss.nb - 1) / (16 * ss.nb);
        const dim3 sgrid((ntiles + 7) / 8 * 8 * mtiles);
        const int key = ss.mb * 100 + ss.nb * 10 + ss.nw;
        switch (key) {
#define HIPQ_STREAM_CASE(MB_, NB_)                                                                                       \
    case MB_ * 100 + NB_ * 10 + 4:                                                                                      \
        if (fc)                                                                                                         \
            hipLaunchKernelGGL((conv_mfma_stream_kernel<MB_, NB_, false>), sgrid, dim3(256), 0, st, a, mtiles);         \
        else                                                                                                            \
            hipLaunchKernelGGL((conv_mfma_stream_kernel<MB_, NB_, true>), sgrid, dim3(256), 0, st, a, mtiles);          \
        return;
            HIPQ_STREAM_CASE(8, 1)
            HIPQ_STREAM_CASE(4, 2)
            HIPQ_STREAM_CASE(4, 1)
            HIPQ_STREAM_CASE(2, 2)
            HIPQ_STREAM_CASE(2, 1)
            HIPQ_STREAM_CASE(1, 2)
            HIPQ_STREAM_CASE(1, 1)
#undef HIPQ_STREAM_CASE
        default: break; // an unknown forced shape: the tile kernels below
        }
    }
    if (pointwise_applies(p) && a.acc_out == nullptr && a.res == nullptr) {
        // persistent work-groups (four waves, a strip of 32 pixels each per turn), five to a CU
        const int nstrips = (a.P + 31) / 32, want = (nstrips + 3) / 4;
        const dim3 pgrid(((want < 1280 ? want : 1280) + 7) / 8 * 8);
        if (a.in_cs <= 32)
            hipLaunchKernelGGL(conv_mfma_pointwise_kernel<1>, pgrid, block, 0, st, a);
        else
            hipLaunchKernelGGL(conv_mfma_pointwise_kernel<2>, pgrid, block, 0, st, a);
        return;
    }
    // "aligned" addressing: a 64-byte slab never straddles two taps.  True when a pixel's channels are whole slabs, and
    // for 1x1 kernels with any channel stride (a multiple of 16): there is one tap, and the pad chunks of the last
    // slab (beyond the pixel's own bytes) are read from the pad buffer.
    const bool aligned = a.in_cs % 64 == 0 || (a.R == 1 && a.S == 1 && a.in_cs % 16 == 0);
    if (p->variant == kMfmaSmallC) {
        if (p->has_wzp)
            hipLaunchKernelGGL((conv_mfma_kernel<BM, BN, WM, WN, true, true>), grid, block, 0, st, a);
        else
            hipLaunchKernelGGL((conv_mfma_kernel<BM, BN, WM, WN, false, true>), grid, block, 0, st, a);
    } else if (p->has_wzp) { // rare (asymmetric weights): generic addressing only
        hipLaunchKernelGGL((conv_mfma_dma_kernel<BM, BN, WM, WN, kStages, true, false>), grid, block, 0, st, a);
    } else if (aligned && a.res != nullptr && launch_k2<BM, BN, WM, WN>(p, a, grid, st)) {
        // few tiles and a long reduction: the two-group kernel, the add applied to its staged tile
    } else if (aligned && a.res != nullptr && a.fastq && a.addq.fast && !plain_epilogue(a)) {
        // residual add in the accumulator layout, residual tile prefetched into LDS
        const int ns = p->stages ? p->stages : (a.nslab >= kDeepFrom ? 3 : kStages);
        if (ns >= 4)
            launch_dma_aligned<BM, BN, WM, WN, 4, true>(grid, a, st);
        else if (ns == 3)
            launch_dma_aligned<BM, BN, WM, WN, 3, true>(grid, a, st);
        else
            launch_dma_aligned<BM, BN, WM, WN, 2, true>(grid, a, st);
    } else if (aligned && launch_k2<BM, BN, WM, WN>(p, a, grid, st)) {
        // the reduction shared by two groups of waves
    } else if (aligned) {
        // Few tiles, long reduction (fully-connected layers at small batch): the weights stream from HBM through a
        // handful of CUs, and only the bytes each of them keeps in flight cover the memory latency: eight stages.
        const bool stream = nblk <= 128 && a.nslab >= 16 && BM + BN <= 192;
        const int ns = p->stages ? p->stages : stream ? 8 : (a.nslab >= kDeepFrom ? (BM + BN >= 320 ? 3 : 4) : kStages);
        if (ns >= 8 && BM + BN <= 192)
            launch_dma_aligned<BM, BN, WM, WN, (BM + BN <= 192 ? 8 : 4), false>(grid, a, st);
        else if (ns >= 4)
            launch_dma_aligned<BM, BN, WM, WN, 4, false>(grid, a, st);
        else if (ns == 3)
            launch_dma_aligned<BM, BN, WM, WN, 3, false>(grid, a, st);
        else
            launch_dma_aligned<BM, BN, WM, WN, 2, false>(grid, a, st);
    } else {
        hipLaunchKernelGGL((conv_mfma_dma_kernel<BM, BN, WM, WN, kStages, false, false>), grid, block, 0, st, a);
    }
}

static int run_conv(const hipq_conv2d_plan *p, ConvArgs &a, hipStream_t st);

extern "C" int hipq_conv2d_run(const hipq_conv2d_plan *p, const void *x, void *y, int32_t *acc_out, void *stream)
{
    clear_error();
    HIPQ_REQUIRE(p && x && y, "hipq_conv2d_run: null argument");
    ConvArgs a = p->args;
    a.x = static_cast<const uint8_t *>(x);
    a.y = static_cast<uint8_t *>(y);
    a.acc_out = acc_out;
    return run_conv(p, a, static_cast<hipStream_t>(stream));
}

extern "C" int hipq_conv2d_run_relu(const hipq_conv2d_plan *p, const void *x, void *y, void *stream)
{
    clear_error();
    HIPQ_REQUIRE(p && x && y, "hipq_conv2d_run_relu: null argument");
    HIPQ_REQUIRE(p->d.dtype == HIPQ_DTYPE_U8, "hipq_conv2d_run_relu: uint8 plans only (op_quant_relu_run is a uint8 operator)");
    ConvArgs a = p->args;
    a.x = static_cast<const uint8_t *>(x);
    a.y = static_cast<uint8_t *>(y);
    a.acc_out = nullptr;
    a.lo = std::min(p->d.ozp, a.q.hi); // what plan creation sets for relu = 1
    return run_conv(p, a, static_cast<hipStream_t>(stream));
}

extern "C" int hipq_conv2d_dequant_fusable(const hipq_conv2d_plan *p, float alpha, int zp)
{
    if (!p || p->variant != kMfma || p->d.dtype != HIPQ_DTYPE_U8 || p->args.OH * p->args.OW != 1 || p->args.qmult != nullptr)
        return 0;
    // the dequantize must read the bytes with the scale and zero point they are written with
    return stream_applies(p) && alpha == p->d.oalpha && zp == p->d.ozp ? 1 : 0;
}

extern "C" int hipq_conv2d_run_dequant(const hipq_conv2d_plan *p, const void *x, float *y, void *stream)
{
    clear_error();
    HIPQ_REQUIRE(p && x && y, "hipq_conv2d_run_dequant: null argument");
    HIPQ_REQUIRE(hipq_conv2d_dequant_fusable(p, p->d.oalpha, p->d.ozp),
                 "hipq_conv2d_run_dequant: only fully-connected uint8 plans on the streaming kernel (this plan runs %s)", p->name.c_str());
    ConvArgs a = p->args;
    a.x = static_cast<const uint8_t *>(x);
    a.y = nullptr; // never written
    a.acc_out = nullptr;
    a.deq_out = y;
    a.deq_alpha = p->d.oalpha;
    return run_conv(p, a, static_cast<hipStream_t>(stream));
}

extern "C" int hipq_conv2d_run_add(const hipq_conv2d_plan *p, const void *x, const void *residual, int residual_is_input0,
                                   float res_alpha, int res_zp, float oalpha, int ozp, int obits, void *y, void *stream)
{
    clear_error();
    HIPQ_REQUIRE(p && x && y && residual, "hipq_conv2d_run_add: null argument");
    HIPQ_REQUIRE(p->variant == kMfma || p->variant == kMfmaSmallC,
                 "hipq_conv2d_run_add: only the MFMA convolution kernels fuse the add (this plan runs %s)", p->name.c_str());
    HIPQ_REQUIRE(p->d.dtype == HIPQ_DTYPE_U8, "hipq_conv2d_run_add: the fused add exists for uint8 tensors only (op_quant_add_run)");
    HIPQ_REQUIRE(res_zp >= 0 && res_zp <= 255 && ozp >= 0 && ozp <= 255 && obits >= 1 && obits <= 8,
                 "hipq_conv2d_run_add: zero points must be in 0..255, obits in 1..8");
    ConvArgs a = p->args;
    a.x = static_cast<const uint8_t *>(x);
    a.y = static_cast<uint8_t *>(y);
    a.res = static_cast<const uint8_t *>(residual);
    a.res_first = residual_is_input0 ? 1 : 0;
    const bool ok = residual_is_input0
        ? make_add_params(res_alpha, res_zp, p->d.oalpha, p->d.ozp, oalpha, ozp, obits, &a.addq)
        : make_add_params(p->d.oalpha, p->d.ozp, res_alpha, res_zp, oalpha, ozp, obits, &a.addq);
    HIPQ_REQUIRE(ok, "hipq_conv2d_run_add: scales out of the fixed-point range");
    return run_conv(p, a, static_cast<hipStream_t>(stream));
}

// the launch arguments of hipq_conv2d_run_add for plan p (everything but the tensors)
static bool add_args(const hipq_conv2d_plan *p, int residual_is_input0, float res_alpha, int res_zp, float oalpha, int ozp,
                     int obits, ConvArgs *a)
{
    *a = p->args;
    a->res = a->padbuf; // any non-null pointer; the caller sets the real one
    a->res_first = residual_is_input0 ? 1 : 0;
    return residual_is_input0 ? make_add_params(res_alpha, res_zp, p->d.oalpha, p->d.ozp, oalpha, ozp, obits, &a->addq)
                              : make_add_params(p->d.oalpha, p->d.ozp, res_alpha, res_zp, oalpha, ozp, obits, &a->addq);
}

extern "C" int hipq_conv2d_add_conv_fusable(const hipq_conv2d_plan *p, int residual_is_input0, float res_alpha, int res_zp,
                                            float oalpha, int ozp, int obits, const hipq_conv2d_plan *next)
{
    if (!p || !next || p->variant != kMfma || next->variant != kMfma || !p->special || p->tile_selected || p->has_wzp
        || next->has_wzp || p->d.dtype != HIPQ_DTYPE_U8 || next->d.dtype != HIPQ_DTYPE_U8 || obits != 8)
        return 0;
    if (res_zp < 0 || res_zp > 255 || ozp < 0 || ozp > 255)
        return 0;
    // the next layer must read the sum with the scale and zero point it is written with
    if (next->d.ialpha != oalpha || next->d.izp != ozp)
        return 0;
    ConvArgs a;
    if (!add_args(p, residual_is_input0, res_alpha, res_zp, oalpha, ozp, obits, &a))
        return 0;
    return conv_expand_chain_applies(a, next->args) ? 1 : 0;
}

extern "C" int hipq_conv2d_run_add_conv(const hipq_conv2d_plan *p, const void *x, const void *residual, int residual_is_input0,
                                        float res_alpha, int res_zp, float oalpha, int ozp, int obits, void *y,
                                        const hipq_conv2d_plan *next, int next_relu, void *y_next, void *stream)
{
    clear_error();
    HIPQ_REQUIRE(p && next && x && y && residual && y_next, "hipq_conv2d_run_add_conv: null argument");
    HIPQ_REQUIRE(hipq_conv2d_add_conv_fusable(p, residual_is_input0, res_alpha, res_zp, oalpha, ozp, obits, next),
                 "hipq_conv2d_run_add_conv: these two plans (%s, then %s) do not run as one kernel: run hipq_conv2d_run_add and "
                 "hipq_conv2d_run", p->name.c_str(), next->name.c_str());
    ConvArgs a, a2 = next->args;
    add_args(p, residual_is_input0, res_alpha, res_zp, oalpha, ozp, obits, &a);
    a.x = static_cast<const uint8_t *>(x);
    a.y = static_cast<uint8_t *>(y);
    a.res = static_cast<const uint8_t *>(residual);
    a.acc_out = nullptr;
    a2.x = nullptr;
    a2.y = static_cast<uint8_t *>(y_next);
    a2.acc_out = nullptr;
    if (next_relu)
        a2.lo = std::min(next->d.ozp, a2.q.hi); // the ReLU clamp, as in hipq_conv2d_run_relu
    launch_conv_expand_chain(a, a2, static_cast<hipStream_t>(stream));
    return launch_status("conv_mfma_expand_kernel (chained)");
}

// the launch arguments of the three layers of an identity bottleneck block (hipq_bottleneck_run); false if the add's
// scales are outside the fixed-point range
static bool block_args(const hipq_conv2d_plan *p1, const hipq_conv2d_plan *p2, const hipq_conv2d_plan *p3, int residual_is_input0,
                       float oalpha, int ozp, int obits, ConvArgs *a1, ConvArgs *a2, ConvArgs *a3)
{
    *a1 = p1->args, *a2 = p2->args;
    // the residual is the block's input: the tensor the first layer reads, with that layer's input scale and zero point
    return add_args(p3, residual_is_input0, p1->d.ialpha, p1->d.izp, oalpha, ozp, obits, a3);
}

extern "C" int hipq_bottleneck_fusable(const hipq_conv2d_plan *p1, const hipq_conv2d_plan *p2, const hipq_conv2d_plan *p3,
                                       int residual_is_input0, float oalpha, int ozp, int obits)
{
    for (const hipq_conv2d_plan *p : {p1, p2, p3})
        if (!p || p->variant != kMfma || !p->special || p->tile_selected || p->has_wzp || p->d.dtype != HIPQ_DTYPE_U8 || p->d.obits != 8)
            return 0;
    if (obits != 8 || ozp < 0 || ozp > 255)
        return 0;
    // each layer must read its input with the zero point the previous one writes it with
    if (p2->d.izp != p1->d.ozp || p3->d.izp != p2->d.ozp || p2->d.ialpha != p1->d.oalpha || p3->d.ialpha != p2->d.oalpha)
        return 0;
    ConvArgs a1, a2, a3;
    if (!block_args(p1, p2, p3, residual_is_input0, oalpha, ozp, obits, &a1, &a2, &a3))
        return 0;
    if (!conv_block_applies(a1, a2, a3, nullptr))
        return 0;
    // built-in rule: where it measured faster than the three launches it replaces - blocks of 256 middle channels (14x14
    // images at batch 64: 31 against 41 us and two launch gaps); hipq_conv2d_plan_special(reduce, 2): wherever it applies
    return p1->special == 2 || conv_block_preferred(a1) ? 1 : 0;
}

extern "C" int hipq_bottleneck_run(const hipq_conv2d_plan *p1, const hipq_conv2d_plan *p2, const hipq_conv2d_plan *p3, const void *x,
                                   int residual_is_input0, float oalpha, int ozp, int obits, void *y, void *stream)
{
    clear_error();
    HIPQ_REQUIRE(p1 && p2 && p3 && x && y, "hipq_bottleneck_run: null argument");
    HIPQ_REQUIRE(x != y, "hipq_bottleneck_run: the sum cannot overwrite the block's input (neighbouring patches read it)");
    HIPQ_REQUIRE(hipq_bottleneck_fusable(p1, p2, p3, residual_is_input0, oalpha, ozp, obits),
                 "hipq_bottleneck_run: these three plans (%s, %s, %s) and this add do not run as one kernel: run hipq_conv2d_run "
                 "twice and hipq_conv2d_run_add", p1->name.c_str(), p2->name.c_str(), p3->name.c_str());
    ConvArgs a1, a2, a3;
    block_args(p1, p2, p3, residual_is_input0, oalpha, ozp, obits, &a1, &a2, &a3);
    a1.x = static_cast<const uint8_t *>(x);
    a1.y = a2.y = nullptr;
    a1.acc_out = a2.acc_out = a3.acc_out = nullptr;
    a3.res = a1.x;
    a3.y = static_cast<uint8_t *>(y);
    launch_conv_block(a1, a2, a3, nullptr, static_cast<hipStream_t>(stream));
    return launch_status("conv_bottleneck_kernel");
}

extern "C" int hipq_bottleneck_conv_fusable(const hipq_conv2d_plan *p1, const hipq_conv2d_plan *p2, const hipq_conv2d_plan *p3,
                                            int residual_is_input0, float oalpha, int ozp, int obits, const hipq_conv2d_plan *next)
{
    if (!next || !hipq_bottleneck_fusable(p1, p2, p3, residual_is_input0, oalpha, ozp, obits))
        return 0;
    if (next->variant != kMfma || !next->special || next->tile_selected || next->has_wzp || next->d.dtype != HIPQ_DTYPE_U8
        || next->d.obits != 8 || next->d.izp != ozp || next->d.ialpha != oalpha)
        return 0;
    ConvArgs a1, a2, a3;
    block_args(p1, p2, p3, residual_is_input0, oalpha, ozp, obits, &a1, &a2, &a3);
    return conv_block_applies(a1, a2, a3, &next->args) ? 1 : 0;
}

extern "C" int hipq_bottleneck_run_conv(const hipq_conv2d_plan *p1, const hipq_conv2d_plan *p2, const hipq_conv2d_plan *p3, const void *x,
                                        int residual_is_input0, float oalpha, int ozp, int obits, void *y,
                                        const hipq_conv2d_plan *next, int next_relu, void *y_next, void *stream)
{
    clear_error();
    HIPQ_REQUIRE(p1 && p2 && p3 && x && y && next && y_next, "hipq_bottleneck_run_conv: null argument");
    HIPQ_REQUIRE(x != y && x != y_next && y != y_next,
                 "hipq_bottleneck_run_conv: the sum and the next layer's output cannot overwrite the block's input or each other");
    HIPQ_REQUIRE(hipq_bottleneck_conv_fusable(p1, p2, p3, residual_is_input0, oalpha, ozp, obits, next),
                 "hipq_bottleneck_run_conv: these plans (%s, %s, %s, next layer %s) and this add do not run as one kernel: run "
                 "hipq_bottleneck_run and hipq_conv2d_run", p1->name.c_str(), p2->name.c_str(), p3->name.c_str(), next->name.c_str());
    ConvArgs a1, a2, a3, an = next->args;
    block_args(p1, p2, p3, residual_is_input0, oalpha, ozp, obits, &a1, &a2, &a3);
    a1.x = static_cast<const uint8_t *>(x);
    a1.y = a2.y = nullptr;
    a1.acc_out = a2.acc_out = a3.acc_out = an.acc_out = nullptr;
    a3.res = a1.x;
    a3.y = static_cast<uint8_t *>(y);
    an.x = nullptr;
    an.y = static_cast<uint8_t *>(y_next);
    if (next_relu)
        an.lo = std::min(next->d.ozp, an.q.hi); // the ReLU clamp, as in hipq_conv2d_run_relu
    launch_conv_block(a1, a2, a3, &an, static_cast<hipStream_t>(stream));
    return launch_status("conv_bottleneck_kernel");
}

extern "C" int hipq_conv2d_add2_fusable(const hipq_conv2d_plan *p, const hipq_conv2d_plan *sc, int shortcut_is_input0, float oalpha,
                                        int ozp, int obits)
{
    for (const hipq_conv2d_plan *q : {p, sc})
        if (!q || q->variant != kMfma || !q->special || q->tile_selected || q->has_wzp || q->d.dtype != HIPQ_DTYPE_U8 || q->d.obits != 8)
            return 0;
    if (obits != 8 || ozp < 0 || ozp > 255)
        return 0;
    ConvArgs a;
    if (!add_args(p, shortcut_is_input0, sc->d.oalpha, sc->d.ozp, oalpha, ozp, obits, &a) || !conv_wreg_dual_applies(a, sc->args))
        return 0;
    // built-in rule: where it measured at least as fast as the two launches at batch 64 - 256 -> 1024 with a 512-channel
    // shortcut on 14x14 images, and 512 -> 2048 with a 1024-channel shortcut on 7x7 images (one work-group of four waves
    // per CU: level with the two launches inside a ResNet-50 pass, 0.6543 against 0.6555 ms, one launch fewer);
    // hipq_conv2d_plan_special(plan, 2): wherever it applies
    return p->special == 2 || (a.P <= 16384 && (a.in_cs == 256 || a.in_cs == 512)) ? 1 : 0;
}

extern "C" int hipq_conv2d_run_add2(const hipq_conv2d_plan *p, const void *x, const hipq_conv2d_plan *sc, const void *x_shortcut,
                                    int shortcut_is_input0, float oalpha, int ozp, int obits, void *y, void *stream)
{
    clear_error();
    HIPQ_REQUIRE(p && sc && x && x_shortcut && y, "hipq_conv2d_run_add2: null argument");
    HIPQ_REQUIRE(hipq_conv2d_add2_fusable(p, sc, shortcut_is_input0, oalpha, ozp, obits),
                 "hipq_conv2d_run_add2: these two plans (%s, %s) and this add do not run as one kernel: run hipq_conv2d_run and "
                 "hipq_conv2d_run_add", p->name.c_str(), sc->name.c_str());
    ConvArgs a, b = sc->args;
    add_args(p, shortcut_is_input0, sc->d.oalpha, sc->d.ozp, oalpha, ozp, obits, &a);
    a.x = static_cast<const uint8_t *>(x);
    a.y = static_cast<uint8_t *>(y);
    a.acc_out = b.acc_out = nullptr;
    b.x = static_cast<const uint8_t *>(x_shortcut);
    b.y = nullptr;
    launch_conv_wreg_dual(a, b, static_cast<hipStream_t>(stream));
    return launch_status("conv_wreg_dual_kernel");
}

// hipq_bottleneck_tail_*: the launch arguments of the three layers; false if the chain does not run as one kernel
static bool tail_args(const hipq_conv2d_plan *p2, const hipq_conv2d_plan *p3, int residual_is_input0, float res_alpha, int res_zp,
                      float oalpha, int ozp, int obits, const hipq_conv2d_plan *next, ConvArgs *a2, ConvArgs *a3, ConvArgs *an)
{
    for (const hipq_conv2d_plan *p : {p2, p3, next})
        if (p && (p->variant != kMfma || !p->special || p->tile_selected || p->has_wzp || p->d.dtype != HIPQ_DTYPE_U8 || p->d.obits != 8))
            return false;
    if (!p2 || !p3 || obits != 8 || ozp < 0 || ozp > 255 || res_zp < 0 || res_zp > 255)
        return false;
    // each layer must read its input with the scale and zero point the previous one writes it with
    if (p3->d.izp != p2->d.ozp || p3->d.ialpha != p2->d.oalpha || (next && (next->d.izp != ozp || next->d.ialpha != oalpha)))
        return false;
    *a2 = p2->args;
    if (!add_args(p3, residual_is_input0, res_alpha, res_zp, oalpha, ozp, obits, a3))
        return false;
    if (next)
        *an = next->args;
    return conv_block_tail_applies(*a2, *a3, next ? an : nullptr);
}

extern "C" int hipq_bottleneck_tail_fusable(const hipq_conv2d_plan *p2, const hipq_conv2d_plan *p3, int residual_is_input0,
                                            float res_alpha, int res_zp, float oalpha, int ozp, int obits,
                                            const hipq_conv2d_plan *next)
{
    ConvArgs a2, a3, an;
    if (!tail_args(p2, p3, residual_is_input0, res_alpha, res_zp, oalpha, ozp, obits, next, &a2, &a3, &an))
        return 0;
    // hipq_conv2d_plan_special(mid, 2): wherever it applies; else the built-in rule
    return p2->special == 2 || conv_block_tail_preferred(a2, next != nullptr) ? 1 : 0;
}

extern "C" int hipq_bottleneck_tail_run(const hipq_conv2d_plan *p2, const hipq_conv2d_plan *p3, const void *x, const void *residual,
                                        int residual_is_input0, float res_alpha, int res_zp, float oalpha, int ozp, int obits,
                                        void *y, const hipq_conv2d_plan *next, int next_relu, void *y_next, void *stream)
{
    clear_error();
    HIPQ_REQUIRE(p2 && p3 && x && residual && y && (!next || y_next), "hipq_bottleneck_tail_run: null argument");
    ConvArgs a2, a3, an;
    HIPQ_REQUIRE(tail_args(p2, p3, residual_is_input0, res_alpha, res_zp, oalpha, ozp, obits, next, &a2, &a3, &an),
                 "hipq_bottleneck_tail_run: these plans (%s, %s%s%s) and this add do not run as one kernel: run hipq_conv2d_run, "
                 "hipq_conv2d_run_add and hipq_conv2d_run", p2->name.c_str(), p3->name.c_str(), next ? ", " : "",
                 next ? next->name.c_str() : "");
    a2.x = static_cast<const uint8_t *>(x);
    a2.y = nullptr;
    a2.acc_out = a3.acc_out = nullptr;
    a3.res = static_cast<const uint8_t *>(residual);
    a3.y = static_cast<uint8_t *>(y);
    if (next) {
        an.x = nullptr;
        an.y = static_cast<uint8_t *>(y_next);
        an.acc_out = nullptr;
        if (next_relu)
            an.lo = std::min(next->d.ozp, an.q.hi); // the ReLU clamp, as in hipq_conv2d_run_relu
    }
    launch_conv_block_tail(a2, a3, next ? &an : nullptr, static_cast<hipStream_t>(stream));
    return launch_status("conv_bottleneck_tail_kernel");
}

extern "C" int hipq_conv2d_maxpool_fusable(const hipq_conv2d_plan *p, int OH, int OW, int kernel, int stride, int pad,
                                           float ialpha, int izp, float oalpha, int ozp, int obits)
{
    if (!p || p->variant != kMfmaSmallC || p->has_wzp || p->d.dtype != HIPQ_DTYPE_U8 || p->d.obits != 8 || obits != 8)
        return 0;
    const ConvArgs &a = p->args;
    // the pooling's rescale must be the identity (equal scale and zero point on both sides, which are the convolution's
    // output parameters), and its geometry the one the kernel implements
    if (kernel != 3 || stride != 2 || pad != 1 || ialpha != oalpha || izp != ozp || ialpha != p->d.oalpha || izp != p->d.ozp)
        return 0;
    if (OH != (a.OH - 1) / 2 + 1 || OW != (a.OW - 1) / 2 + 1)
        return 0;
    return conv_stem_maxpool_applies(a, a.rowb) ? 1 : 0;
}

extern "C" int hipq_conv2d_run_maxpool(const hipq_conv2d_plan *p, const void *x, void *y, int OH, int OW, int relu, void *stream)
{
    clear_error();
    HIPQ_REQUIRE(p && x && y, "hipq_conv2d_run_maxpool: null argument");
    HIPQ_REQUIRE(hipq_conv2d_maxpool_fusable(p, OH, OW, 3, 2, 1, p->d.oalpha, p->d.ozp, p->d.oalpha, p->d.ozp, 8),
                 "hipq_conv2d_run_maxpool: this plan (%s) does not fuse with a 3x3 / stride 2 / pad 1 max pooling to %d x %d: run "
                 "the two operators separately", p->name.c_str(), OH, OW);
    ConvArgs a = p->args;
    a.x = static_cast<const uint8_t *>(x);
    a.y = nullptr;
    a.acc_out = nullptr;
    if (relu)
        a.lo = std::min(p->d.ozp, a.q.hi); // the ReLU clamp, as in hipq_conv2d_run_relu
    launch_conv_stem_maxpool(a, static_cast<uint8_t *>(y), OH, OW, nullptr, nullptr, static_cast<hipStream_t>(stream));
    return launch_status("conv_stem_maxpool_kernel");
}

extern "C" int hipq_conv2d_maxpool_conv_fusable(const hipq_conv2d_plan *p, int OH, int OW, const hipq_conv2d_plan *next,
                                                const hipq_conv2d_plan *next2)
{
    if (!p || !next || !hipq_conv2d_maxpool_fusable(p, OH, OW, 3, 2, 1, p->d.oalpha, p->d.ozp, p->d.oalpha, p->d.ozp, 8))
        return 0;
    for (const hipq_conv2d_plan *q : {next, next2})
        if (q && (q->variant != kMfma || !q->special || q->tile_selected || q->has_wzp || q->d.dtype != HIPQ_DTYPE_U8 || q->d.obits != 8
                  || q->d.izp != p->d.ozp || q->d.ialpha != p->d.oalpha))
            return 0;
    return conv_stem_next_applies(p->args, OH, OW, next->args, next2 ? &next2->args : nullptr) ? 1 : 0;
}

extern "C" int hipq_conv2d_run_maxpool_conv(const hipq_conv2d_plan *p, const void *x, void *y, int OH, int OW, int relu,
                                            const hipq_conv2d_plan *next, int next_relu, void *y_next,
                                            const hipq_conv2d_plan *next2, int next2_relu, void *y_next2, void *stream)
{
    clear_error();
    HIPQ_REQUIRE(p && x && y && next && y_next && (!next2 || y_next2), "hipq_conv2d_run_maxpool_conv: null argument");
    HIPQ_REQUIRE(hipq_conv2d_maxpool_conv_fusable(p, OH, OW, next, next2),
                 "hipq_conv2d_run_maxpool_conv: these plans (%s, %s%s%s) do not run as one kernel with a 3x3 / stride 2 / pad 1 max "
                 "pooling to %d x %d between them: run hipq_conv2d_run_maxpool and hipq_conv2d_run", p->name.c_str(),
                 next->name.c_str(), next2 ? ", " : "", next2 ? next2->name.c_str() : "", OH, OW);
    HIPQ_REQUIRE(y_next != y && y_next != x && (!next2 || (y_next2 != y && y_next2 != x && y_next2 != y_next)),
                 "hipq_conv2d_run_maxpool_conv: a chained layer cannot overwrite a tensor the kernel reads or writes");
    ConvArgs a = p->args, an = next->args, an2 = next2 ? next2->args : next->args;
    a.x = static_cast<const uint8_t *>(x);
    a.y = nullptr;
    a.acc_out = nullptr;
    if (relu)
        a.lo = std::min(p->d.ozp, a.q.hi); // the ReLU clamp, as in hipq_conv2d_run_relu
    an.x = an2.x = nullptr;
    an.y = static_cast<uint8_t *>(y_next);
    an2.y = static_cast<uint8_t *>(y_next2);
    an.acc_out = an2.acc_out = nullptr;
    if (next_relu)
        an.lo = std::min(next->d.ozp, an.q.hi);
    if (next2 && next2_relu)
        an2.lo = std::min(next2->d.ozp, an2.q.hi);
    launch_conv_stem_maxpool(a, static_cast<uint8_t *>(y), OH, OW, &an, next2 ? &an2 : nullptr, static_cast<hipStream_t>(stream));
    return launch_status("conv_stem_maxpool_kernel");
}

static int run_conv(const hipq_conv2d_plan *p, ConvArgs &a, hipStream_t st)
{
    switch (p->variant) {
    case kMfma:
    case kMfmaSmallC:
        if (wreg_applies(p, a)) {
            launch_conv_wreg(a, st); // few pixels: the pixel operand in LDS once, weight operands straight into registers
            break;
        }
        if (rows_applies(p, a)) {
            launch_conv_rows(a, st); // 3x3 with 64 channels: the input rows stay in LDS, the weights in registers
            break;
        }
        if (expand_applies(p, a)) {
            launch_conv_expand(a, st); // a channel-widening 1x1 layer: pixel operands in registers, channel tiles in a loop
            break;
        }
        if (stem3_applies(p, a)) {
            launch_conv_stem3x3(a, st); // 3x3 / stride 2 on an RGB image: the input rows stay in LDS
            break;
        }
        switch (p->tile) {
        case 0: launch_mfma<128, 128, 2, 2>(p, a, st); break;
        case 1: launch_mfma<256, 64, 4, 1>(p, a, st); break;
        case 2: launch_mfma<128, 64, 2, 2>(p, a, st); break;
        case 3: launch_mfma<64, 128, 1, 4>(p, a, st); break;
        default: launch_mfma<64, 64, 2, 2>(p, a, st); break;
        }
        break;
    case kDepthwise3x3: {
        if (!p->has_wzp && conv_dw_slide_applies(a)) {
            launch_conv_dw_slide(a, st); // a thread walks down the image: every input row loaded and transposed once
            break;
        }
        const size_t total = (size_t)a.N * ((a.OH + 1) / 2) * ((a.OW + 3) / 4) * (a.in_cs / 4);
        const dim3 grid((unsigned)((std::min<size_t>((total + 255) / 256, 256 * 64) + 7) / 8 * 8)), block(256); // a multiple of 8
        if (p->d.stride_h == 1) {
            if (p->has_wzp)
                hipLaunchKernelGGL((conv_depthwise3x3_kernel<1, true>), grid, block, 0, st, a);
            else
                hipLaunchKernelGGL((conv_depthwise3x3_kernel<1, false>), grid, block, 0, st, a);
        } else {
            if (p->has_wzp)
                hipLaunchKernelGGL((conv_depthwise3x3_kernel<2, true>), grid, block, 0, st, a);
            else
                hipLaunchKernelGGL((conv_depthwise3x3_kernel<2, false>), grid, block, 0, st, a);
        }
        break;
    }
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
