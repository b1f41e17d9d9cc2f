// Building blocks of the kernels whose waves load their MFMA weight operands straight from memory in fragment order
// (ConvArgs::wfrag) while the pixel operands wait in LDS: the LDS row swizzle, the requantising epilogues on a lane's 16
// consecutive channels, the ring of weight operands a wave keeps ahead of its multiplies, a wave's half of a reduction
// and the exchange that adds the two halves of a pair of waves.  gfx950 only.
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

// The weight operands a wave holds ahead of its multiplies: D slabs of four (channel tile nt, k-step kk at [2 nt + kk]),
// and the two of an odd slab count's last half slab.
template <int D>
struct WeightRing {
    v4i w[D][4], wt[2];
};

// One wave's half of a layer's reduction, accumulated into acc[pixel tile][channel tile] (MT pixel tiles of 32, 2
// channel tiles of 32): the slabs kh, kh + 2, ... of the first STOT - (STOT & 1), and, when STOT is odd, k-step kh of
// the last slab - both waves of a pair do the same amount of work and the code has no branch, so the compiler's wait
// counts stay exact.  ldw(s, kk, nt): the weight operand of slab s, k-step kk, channel tile nt, from global memory, D
// slabs ahead of its multiplies (ring_fill issues the first D, as early as the caller likes); ldb(s, kk, t): the pixel
// operand of pixel tile t from LDS, one slab ahead; flip is XORed onto the pixel operands (0x80808080 re-centres raw
// uint8 bytes, 0 leaves re-centred ones alone).
template <int STOT, int D, class FW>
__device__ static inline void ring_fill(WeightRing<D> &r, const int kh, FW ldw)
{
    constexpr int NS = STOT / 2;
#pragma unroll
    for (int i = 0; i < D && i < NS; i++)
#pragma unroll
        for (int nt = 0; nt < 2; nt++)
#pragma unroll
            for (int kk = 0; kk < 2; kk++)
                r.w[i][2 * nt + kk] = ldw(2 * i + kh, kk, nt);
    if ((STOT & 1) && NS <= D)
        r.wt[0] = ldw(STOT - 1, kh, 0), r.wt[1] = ldw(STOT - 1, kh, 1);
}

template <int STOT, int MT, int D, class FW, class FB>
__device__ static inline void reduce_half(v16i (&acc)[MT][2], WeightRing<D> &r, const int kh, const int flip, FW ldw, FB ldb)
{
    constexpr int NS = STOT / 2;
    constexpr bool TAIL = (STOT & 1) != 0;
    v4i br[2][MT][2], bt[MT];
    auto loadb = [&](int i, v4i(&b)[MT][2]) {
#pragma unroll
        for (int t = 0; t < MT; t++)
#pragma unroll
            for (int kk = 0; kk < 2; kk++)
                b[t][kk] = ldb(2 * i + kh, kk, t);
    };
    loadb(0, br[0]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < NS; i++) {
        if (i + 1 < NS) {
            loadb(i + 1, br[(i + 1) & 1]);
        } else if (TAIL) {
#pragma unroll
            for (int t = 0; t < MT; t++)
                bt[t] = ldb(STOT - 1, kh, t);
        }
#pragma unroll
        for (int kk = 0; kk < 2; kk++)
#pragma unroll
            for (int t = 0; t < MT; t++)
#pragma unroll
                for (int nt = 0; nt < 2; nt++)
                    acc[t][nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(r.w[i % D][2 * nt + kk], br[i & 1][t][kk] ^ flip, acc[t][nt], 0, 0, 0);
        if (i + D < NS) {
#pragma unroll
            for (int nt = 0; nt < 2; nt++)
#pragma unroll
                for (int kk = 0; kk < 2; kk++)
                    r.w[i % D][2 * nt + kk] = ldw(2 * (i + D) + kh, kk, nt);
        } else if (TAIL && i + D == NS) {
            r.wt[0] = ldw(STOT - 1, kh, 0), r.wt[1] = ldw(STOT - 1, kh, 1);
        }
        __builtin_amdgcn_sched_barrier(0); // keep every slab's loads, reads and multiplies where they are written
    }
    if (TAIL) {
#pragma unroll
        for (int t = 0; t < MT; t++)
#pragma unroll
            for (int nt = 0; nt < 2; nt++)
                acc[t][nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(r.wt[nt], bt[t] ^ flip, acc[t][nt], 0, 0, 0);
    }
}

// The same without sharing the reduction: a wave owns ONE 32-channel tile and all STOT slabs, so nothing is exchanged.
// Every wave then reads every pixel operand (twice the LDS traffic of the split), which the kernels that are bound by
// the weight stream or by vector arithmetic can afford.  ldw(s, kk): the weight operand of slab s, k-step kk; ldb as above.
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

// The two waves of a pair add their partial sums: each sends its channel tile 1 and keeps tile 0 (the pair's waves order
// their channel tiles oppositely, so one wave's tile 1 is the other's tile 0) through 4 KB slots in LDS - all pixel
// tiles at once where the slots hold them (ONE_ROUND: MT slots per wave), else one pixel tile per round with a barrier
// before a slot is written again.  No barrier at the end: the caller has one before it reuses the slots.
template <int MT, bool ONE_ROUND>
__device__ static inline void pair_reduce(v16i (&acc)[MT][2], uint8_t *scr, const int wave, const int partner, const int lane)
{
    constexpr int SLOT = ONE_ROUND ? MT * 4096 : 4096;
    auto send = [&](int t) {
#pragma unroll
        for (int g = 0; g < 4; g++) {
            v4i v;
#pragma unroll
            for (int e = 0; e < 4; e++)
                v[e] = acc[t][1][g * 4 + e];
            *reinterpret_cast<v4i *>(scr + wave * SLOT + (ONE_ROUND ? t * 4096 : 0) + g * 1024 + lane * 16) = v;
        }
    };
    auto receive = [&](int t) {
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const v4i v = *reinterpret_cast<const v4i *>(scr + partner * SLOT + (ONE_ROUND ? t * 4096 : 0) + g * 1024 + lane * 16);
#pragma unroll
            for (int e = 0; e < 4; e++)
                acc[t][0][g * 4 + e] += v[e];
        }
    };
    if (ONE_ROUND) {
#pragma unroll
        for (int t = 0; t < MT; t++)
            send(t);
        __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
#pragma unroll
        for (int t = 0; t < MT; t++)
            receive(t);
        return;
    }
#pragma unroll
    for (int t = 0; t < MT; t++) {
        if (t > 0) { // every wave has read the previous round's slots
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_s_barrier();
        }
        send(t);
        __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
        receive(t);
    }
}

} // namespace frag
} // namespace hipq
