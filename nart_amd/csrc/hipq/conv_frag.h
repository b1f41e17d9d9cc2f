// Building blocks of the kernels whose waves load their MFMA weight operands straight from memory in fragment order
// (ConvArgs::wfrag) while the pixel operands wait in LDS: the LDS row swizzle, the requantising epilogues on a lane's 16
// consecutive channels, the ring of weight operands a wave keeps ahead of its multiplies and a wave's reduction of one
// 32-channel tile.  gfx950 only.
#pragma once

#include "conv_shared.h"

namespace hipq {
namespace frag {

// chunk (16 bytes) c of pixel row `row` is kept at chunk c ^ swz(row) of its LDS row, so that 16 lanes that read the same
// chunk of 16 consecutive rows fall on 16 different bank groups whatever the row length
template <int ROWBYTES>
__device__ static inline int swz(int row)
{
    return ROWBYTES >= 256 ? (row & 15) : ROWBYTES == 128 ? ((row >> 1) & 7) : ((row >> 2) & 3);
}

// 16 accumulators (16 consecutive channels of one pixel) -> 16 requantised bytes, each XORed with the low byte of flip.
// For clamp ranges within [0, 255] (a.lo >= 0: the callers' hosts check it).
__device__ static inline v4i requant16(const ConvArgs &a, const v16i &acc, uint32_t flip)
{
    v4i o;
    if (a.lo == 0 && a.q.hi == 255) {
#pragma unroll
        for (int g = 0; g < 4; g++)
            o[g] = (int)(conv_requant4<true>(a, acc[g * 4], acc[g * 4 + 1], acc[g * 4 + 2], acc[g * 4 + 3]) ^ flip);
    } else {
#pragma unroll
        for (int g = 0; g < 4; g++)
            o[g] = (int)(conv_requant4<false>(a, acc[g * 4], acc[g * 4 + 1], acc[g * 4 + 2], acc[g * 4 + 3]) ^ flip);
    }
    return o;
}

// The same followed by the residual add (op_quant_add_run on the requantised bytes and the residual's 16 bytes `res`),
// in the 32-bit form: per element the convolution's clamped result minus its zero point is clamp(q, lo - zp, hi - zp)
// with q = (mulhi(acc, mult) + 2^(t-1)) >> t; the add's terms are (d * m + c) >> s; the sum's last shift and its
// saturation to [0, 255] are the shifting, saturating pack.
__device__ static inline v4i requant_add16(const ConvArgs &a, const v16i &acc, const v4i res)
{
    const AddParams &q = a.addq;
    const int mc = (int)(a.res_first ? q.m1 : q.m0), sc = a.res_first ? q.s1 : q.s0;
    const int mr = (int)(a.res_first ? q.m0 : q.m1), sr = a.res_first ? q.s0 : q.s1, cr = a.res_first ? q.c0 : q.c1;
    const int rc = 1 << (sc - 1); // rounding of the convolution's term (its zero point cancels)
    const int qround = 1 << (a.qt - 1);
    const int dlo = a.lo - a.q.zp, dhi = a.q.hi - a.q.zp;
    v4i o;
#pragma unroll
    for (int g = 0; g < 4; g++) {
        const uint32_t rv = (uint32_t)res[g];
        int32_t y[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            int32_t d = (__mulhi(acc[g * 4 + e], (int)a.q.mult) + qround) >> a.qt;
            asm("v_med3_i32 %0, %1, %2, %3" : "=v"(d) : "v"(d), "s"(dlo), "v"(dhi));
            const int32_t t0 = (__mul24(d, mc) + rc) >> sc;
            const int32_t t1 = (__mul24((int)((rv >> (8 * e)) & 255), mr) + cr) >> sr;
            y[e] = t0 + t1 + q.cadd;
        }
        o[g] = (int)ashr_sat_u8x4(y[0], y[1], y[2], y[3], q.sh);
    }
    return o;
}

// accumulators of a lane <- the folded bias of its 16 consecutive channels (or zero for the wave that does not carry it)
__device__ static inline void init_acc(v16i &acc, const int32_t *bias16, bool zero)
{
#pragma unroll
    for (int g = 0; g < 4; g++) {
        const v4i bv = *reinterpret_cast<const v4i *>(bias16 + g * 4);
#pragma unroll
        for (int e = 0; e < 4; e++)
            acc[g * 4 + e] = zero ? 0 : bv[e];
    }
}

// A wave owns ONE 32-channel tile for MT pixel tiles of 32 and all STOT 64-byte slabs of the reduction, so the waves of a
// work-group exchange nothing and the loop has no barrier.  (Splitting a reduction between two waves read every pixel
// operand once instead of twice, but the exchange of partial sums through LDS and its barriers cost more in every kernel
// that tried both.)  The weight operands wait in a ring of D slabs, two k-steps each: ldw(s, kk) loads the operand of slab
// s, k-step kk from global memory, D slabs ahead of its multiplies (ring_fill1 issues the first D, as early as the caller
// likes); ldb(s, kk, t): the pixel operand of pixel tile t from LDS, one slab ahead; flip is XORed onto the pixel operands
// (0x80808080 re-centres raw uint8 bytes, 0 leaves re-centred ones alone).  The code has no branch, so the compiler's
// wait counts stay exact.
template <int D>
struct WeightRing1 {
    v4i w[D][2];
};

template <int STOT, int D, class FW>
__device__ static inline void ring_fill1(WeightRing1<D> &r, FW ldw)
{
#pragma unroll
    for (int i = 0; i < D && i < STOT; i++)
#pragma unroll
        for (int kk = 0; kk < 2; kk++)
            r.w[i][kk] = ldw(i, kk);
}

template <int STOT, int MT, int D, class FW, class FB>
__device__ static inline void reduce_all(v16i (&acc)[MT], WeightRing1<D> &r, const int flip, FW ldw, FB ldb)
{
    v4i br[2][MT][2];
    auto loadb = [&](int i, v4i(&b)[MT][2]) {
#pragma unroll
        for (int t = 0; t < MT; t++)
#pragma unroll
            for (int kk = 0; kk < 2; kk++)
                b[t][kk] = ldb(i, kk, t);
    };
    loadb(0, br[0]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < STOT; i++) {
        if (i + 1 < STOT)
            loadb(i + 1, br[(i + 1) & 1]);
#pragma unroll
        for (int kk = 0; kk < 2; kk++)
#pragma unroll
            for (int t = 0; t < MT; t++)
                acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(r.w[i % D][kk], br[i & 1][t][kk] ^ flip, acc[t], 0, 0, 0);
        if (i + D < STOT) {
#pragma unroll
            for (int kk = 0; kk < 2; kk++)
                r.w[i % D][kk] = ldw(i + D, kk);
        }
        __builtin_amdgcn_sched_barrier(0); // keep every slab's loads, reads and multiplies where they are written
    }
}

} // namespace frag
} // namespace hipq
