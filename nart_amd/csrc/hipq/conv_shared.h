// Device code shared by the convolution kernels' translation units: kernel arguments, the requantising epilogues of
// the MFMA kernels, wait-count and address-space helpers.  gfx950 only.
#pragma once

#include <type_traits>

#include "common.h"

namespace hipq {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
struct __attribute__((packed, aligned(4))) v4i_a4 { v4i v; }; // a 16-byte load that is only 4-byte aligned

struct ConvArgs {
    const uint8_t *x;
    uint8_t *y;
    int32_t *acc_out;
    const uint8_t *wpack; // MFMA: [slab][kout_pad][64] swizzled int8; depthwise: [tap][cs] int16
    // MFMA plans over whole 64-byte channel slabs with at most 1024 input and output channels: the same weights in
    // fragment order - the 1 KB that a wave loads as one MFMA operand (32-channel tile T, k-step kk of slab s: lane
    // 32 h + p holds bytes [32 kk + 16 h, + 16) of channel 32 T + 16 ((p >> 2) & 1) + 4 (p >> 3) + (p & 3), so that a lane's 16
    // accumulators are 16 consecutive channels) contiguous at ((s * kout_pad / 32 + T) * 2 + kk) * 1024; else nullptr
    const uint8_t *wfrag;
    const int32_t *bias2; // per output channel, padded to kout_pad
    const uint8_t *padbuf; // 64 bytes of the byte izp (source of out-of-image taps)
    int N, C, H, W, K, OH, OW;
    int in_cs, out_cs;
    int R, S, pad_h, pad_w, stride_h, stride_w, group;
    int P;        // N*OH*OW output pixels
    int rowb;     // bytes of one k "row": in_cs (generic) or 4*round_up(S,4) (small-C mode)
    int Ktot;     // generic: R*S*in_cs; small-C: R*rowb
    int nslab;    // ceil(Ktot / 64)
    int kout_pad; // K rounded up to a multiple of 128
    int nbm, nbn;
    int bwz;          // b = 128 - wzp
    int izp, wzp;     // for the non-MFMA kernels
    uint32_t padword; // byte izp in all four lanes
    uint32_t xmask;   // MFMA kernels: 0x80808080 re-centres uint8 activations, 0 leaves int8 activations alone
    int sx;           // other kernels: bytes are read as (byte ^ sx) - zero point; 0x80 with zero points 128 == int8
    Requant q;
    int lo;    // lower clamp: ozp when ReLU is fused, else 0
    int fastq; // 1: the one-multiply requantisation is valid for q.shift
    int qt;    // shift - 32
    int qadd;  // 2^(qt-1) + zp * 2^qt
    double inv_ohw, inv_ow; // 1 / (OH*OW), 1 / OW (depthwise 3x3: 1 / work items per row, 1 / channel quads)
    double inv_oh;          // 1 / OH
    // per-output-channel requantisation (a weight scale per channel): multipliers and shifts, padded like bias2;
    // nullptr = the per-tensor pair in q.  Such plans requantise with the 64-bit form, channel by channel.
    const uint32_t *qmult;
    const int32_t *qshift;
    const uint8_t *res; // fused residual add: the other operand (same layout as y), or nullptr
    int res_first;      // 1: the residual is input 0 of the add, the convolution's output input 1
    AddParams addq;
    // fused dequantize (streaming kernel only): the float value of every output byte, (byte - zero point) * deq_alpha, goes
    // to deq_out[pixel][K] and the bytes themselves are not written; nullptr = off
    float *deq_out;
    float deq_alpha;
};

// x / d for 0 <= x < 2^31, d >= 1, inv = 1.0 / d: the double product is within one of the quotient, one
// compare settles it (a handful of full-rate instructions instead of the generic 32-bit division sequence)
__device__ static inline int fast_div(int x, int d, double inv)
{
    int q = (int)((double)x * inv);
    q -= q * d > x;
    q += (q + 1) * d <= x;
    return q;
}

__device__ static inline v4i ldg128(const uint8_t *p) { return *reinterpret_cast<const v4i *>(p); }

// ------------------------------------------------------------------------------------------------
// Epilogue shared by the MFMA kernels: requantise the wave's accumulators and write the tile.
// FAST selects the one-multiply requantisation (valid for 33 <= shift <= 52, see the file header).
// The caller guarantees that no wave still reads the LDS stages and that no load into them is in flight.
template <bool FAST>
__device__ static inline int32_t conv_requant(const ConvArgs &a, int32_t v)
{
    int32_t r;
    if (FAST)
        r = (__mulhi(v, (int)a.q.mult) + a.qadd) >> a.qt;
    else
        r = (int32_t)(rshift_rn((int64_t)v * (int64_t)a.q.mult, a.q.shift) + a.q.zp);
    int32_t out;
    asm("v_med3_i32 %0, %1, %2, %3" : "=v"(out) : "v"(r), "s"(a.lo), "v"(a.q.hi)); // lo <= hi: the median is the clamp
    return out;
}

// Per-channel form: channel ch has its own (mult, shift); zero point and clamps are the tensor's.
__device__ static inline int32_t conv_requant_ch(const ConvArgs &a, int32_t v, int ch)
{
    const int32_t r = (int32_t)(rshift_rn((int64_t)v * (int64_t)a.qmult[ch], a.qshift[ch]) + a.q.zp);
    return r < a.lo ? a.lo : (r > a.q.hi ? a.q.hi : r);
}

// The element-wise epilogue (no LDS transpose): accumulator dumps, outputs too narrow for 128-bit rows, per-channel scales.
__host__ __device__ static inline bool plain_epilogue(const ConvArgs &a) { return a.acc_out != nullptr || (a.out_cs & 15) || a.qmult != nullptr; }

// Pack the low bytes of four values into a dword (three v_perm_b32 / v_or_b32; works for negative values, whose
// low byte is their two's complement int8).
__device__ static inline uint32_t pack_low_bytes(int32_t r0, int32_t r1, int32_t r2, int32_t r3)
{
    return __builtin_amdgcn_perm((uint32_t)r1, (uint32_t)r0, 0x0c0c0400u) | __builtin_amdgcn_perm((uint32_t)r3, (uint32_t)r2, 0x04000c0cu);
}

// One-multiply requantisation of four accumulators to the four bytes of a dword, for outputs whose clamp range lies in
// [0, 255] (a.lo >= 0): mulhi and the rounding / zero-point constant as in conv_requant<true>, then the clamp IN FRONT of
// the shift - lo << t and ((hi + 1) << t) - 1 are the smallest and largest values that shift to lo and hi - and the
// shifting, saturating pack.  SAT: the range is exactly [0, 255], the pack's saturation is the clamp.
template <bool SAT>
__device__ static __forceinline__ uint32_t conv_requant4(const ConvArgs &a, int32_t v0, int32_t v1, int32_t v2, int32_t v3)
{
    int32_t r[4] = {v0, v1, v2, v3};
    const int32_t plo = a.lo << a.qt, phi = ((a.q.hi + 1) << a.qt) - 1;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        r[e] = __mulhi(r[e], (int)a.q.mult) + a.qadd;
        if (!SAT)
            asm("v_med3_i32 %0, %1, %2, %3" : "=v"(r[e]) : "v"(r[e]), "s"(plo), "v"(phi));
    }
    return ashr_sat_u8x4(r[0], r[1], r[2], r[3], a.qt);
}

template <int BM, int BN, int WM, int WN, bool HAS_WZP, bool FAST, bool PLAIN_SAT, int TM, int TN>
__device__ static __forceinline__ void conv_epilogue(const ConvArgs &a, v16i (&acc)[TN][TM], int (&colsum)[TM], uint8_t *lds,
                                            int bm, int bn, int wm, int wn)
{
    constexpr int OSTR = BN + 16; // row stride of the output staging tile
    const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5;
    const int ch0 = bn * BN + wn * (TN * 32);
    const int m0 = bm * BM; // first pixel of the tile
    if (plain_epilogue(a)) {
        // plain path: accumulator dump requested, an output too narrow for 128-bit rows, or per-channel scales
#pragma unroll
        for (int tm = 0; tm < TM; tm++) {
            const int m = m0 + wm * (TM * 32) + tm * 32 + (lane & 31);
            if (m >= a.P)
                continue;
#pragma unroll
            for (int tn = 0; tn < TN; tn++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int ko = ch0 + tn * 32 + g * 8 + half * 4;
                    if (ko >= a.out_cs)
                        continue;
                    // one requantisation form for this path (it is never the fast one): the 64-bit product with the
                    // channel's own multiplier and shift where the plan has them, the tensor's otherwise
                    int32_t rq[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int32_t v = (int32_t)((uint32_t)acc[tn][tm][g * 4 + e] + (HAS_WZP ? (uint32_t)colsum[tm] : 0u));
                        if (a.acc_out)
                            a.acc_out[(size_t)m * a.out_cs + ko + e] = v;
                        const uint32_t qm = a.qmult ? a.qmult[ko + e] : a.q.mult;
                        const int qs = a.qmult ? a.qshift[ko + e] : a.q.shift;
                        const int32_t r = (int32_t)(rshift_rn((int64_t)v * (int64_t)qm, qs) + a.q.zp);
                        rq[e] = r < a.lo ? a.lo : (r > a.q.hi ? a.q.hi : r);
                    }
                    uint32_t packed = pack_low_bytes(rq[0], rq[1], rq[2], rq[3]);
                    if (a.res) {
                        const uint32_t rv = *reinterpret_cast<const uint32_t *>(a.res + (size_t)m * a.out_cs + ko);
                        packed = a.res_first ? add_dword<false>(rv, packed, a.addq) : add_dword<false>(packed, rv, a.addq);
                    }
                    *reinterpret_cast<uint32_t *>(a.y + (size_t)m * a.out_cs + ko) = packed;
                }
        }
        return;
    }
    // each lane holds 4 consecutive channels of one pixel per accumulator quad: transpose the packed dwords
    // through LDS so that every pixel's channels leave as 128-bit stores
#pragma unroll
    for (int tm = 0; tm < TM; tm++) {
        const int pl = wm * (TM * 32) + tm * 32 + (lane & 31);
#pragma unroll
        for (int tn = 0; tn < TN; tn++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                uint32_t packed = 0;
                if (FAST && PLAIN_SAT) {
                    // clamp range is exactly [0, 255]: the shifting, saturating pack replaces four clamps and the shifts
                    int32_t v[4];
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        v[e] = (int32_t)((uint32_t)acc[tn][tm][g * 4 + e] + (HAS_WZP ? (uint32_t)colsum[tm] : 0u));
                    packed = conv_requant4<true>(a, v[0], v[1], v[2], v[3]);
                } else {
                    int32_t rq[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int32_t v = (int32_t)((uint32_t)acc[tn][tm][g * 4 + e] + (HAS_WZP ? (uint32_t)colsum[tm] : 0u));
                        rq[e] = conv_requant<FAST>(a, v);
                    }
                    packed = pack_low_bytes(rq[0], rq[1], rq[2], rq[3]);
                }
                *reinterpret_cast<uint32_t *>(lds + pl * OSTR + wn * (TN * 32) + tn * 32 + g * 8 + half * 4) = packed;
            }
    }
    // own LDS writes complete, then the barrier: deliberately NOT __syncthreads(), whose fence would also wait for
    // every vector-memory operation in flight
    __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0), vmcnt / expcnt untouched
    __builtin_amdgcn_s_barrier();
    constexpr int LPR = BN / 16;   // lanes per pixel row
    constexpr int RPP = 256 / LPR; // rows per pass
    const int c16 = (tid % LPR) * 16;
    if (bn * BN + c16 >= a.out_cs)
        return;
    if (a.res == nullptr) {
#pragma unroll
        for (int r = tid / LPR; r < BM; r += RPP) {
            const int m = m0 + r;
            if (m < a.P)
                *reinterpret_cast<v4i *>(a.y + (size_t)m * a.out_cs + bn * BN + c16)
                    = *reinterpret_cast<const v4i *>(lds + r * OSTR + c16);
        }
        return;
    }
    // fused residual add (the convolution's own uint8 result exists only in LDS): y = add(conv, residual),
    // exactly what a separate add kernel would compute from the stored bytes
    auto fused = [&](auto fast) {
        constexpr bool AF = decltype(fast)::value;
#pragma unroll
        for (int r = tid / LPR; r < BM; r += RPP) {
            const int m = m0 + r;
            if (m >= a.P)
                continue;
            const size_t off = (size_t)m * a.out_cs + bn * BN + c16;
            const u32x4 cv = *reinterpret_cast<const u32x4 *>(lds + r * OSTR + c16);
            const u32x4 rv = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(a.res + off));
            *reinterpret_cast<u32x4 *>(a.y + off) = a.res_first ? add_16<AF>(rv, cv, a.addq) : add_16<AF>(cv, rv, a.addq);
        }
    };
    if (a.addq.fast)
        fused(std::true_type{});
    else
        fused(std::false_type{});
}

// Epilogue with the residual add applied in the accumulator layout.  The residual tile [BM][BN] was fetched into
// LDS by the load unit at kernel start (chunk c of row r at chunk c ^ ((r >> 1) & (BN/16 - 1))), so its latency is
// long gone; each lane reads the dword holding its 4 channels.  Requires the one-multiply requantisation and the
// 32-bit form of the add (the host checks).  Per element: the convolution's clamped result minus its zero point is
// clamp(q, lo - zp, hi - zp) with q = (mulhi(acc, mult) + 2^(t-1)) >> t; the add's terms are (d * m + c) >> s; the sum
// is clamped and packed.  Bit-identical to storing the convolution's bytes and running the add on them.
template <int BM, int BN, int WM, int WN, int TM, int TN>
__device__ static __forceinline__ void conv_epilogue_fused_add(const ConvArgs &a, v16i (&acc)[TN][TM], uint8_t *lds_out,
                                                      const uint8_t *lds_res, int bm, int bn, int wm, int wn)
{
    constexpr int OSTR = BN + 16, CMASK = BN / 16 - 1;
    const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5;
    const AddParams &q = a.addq;
    // operand order of the add: the convolution is input 1 when the residual comes first
    const int mc = (int)(a.res_first ? q.m1 : q.m0), sc = a.res_first ? q.s1 : q.s0;
    const int mr = (int)(a.res_first ? q.m0 : q.m1), sr = a.res_first ? q.s0 : q.s1, cr = a.res_first ? q.c0 : q.c1;
    const int rc = 1 << (sc - 1);                    // rounding of the convolution's term (its zero point cancels)
    const int qround = 1 << (a.qt - 1);
    const int dlo = a.lo - a.q.zp, dhi = a.q.hi - a.q.zp; // clamp range of (conv byte - conv zero point)
    const int yhi = ((q.hi + 1) << q.sh) - 1;             // the largest value that the last shift takes to q.hi
#pragma unroll
    for (int tm = 0; tm < TM; tm++) {
        const int pl = wm * (TM * 32) + tm * 32 + (lane & 31);
        const int rsw = (pl >> 1) & CMASK;
#pragma unroll
        for (int tn = 0; tn < TN; tn++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int chl = wn * (TN * 32) + tn * 32 + g * 8 + half * 4;
                const uint32_t rv = *reinterpret_cast<const uint32_t *>(lds_res + pl * BN + (((chl >> 4) ^ rsw) << 4) + (chl & 15));
                int32_t y[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    int32_t d = (__mulhi(acc[tn][tm][g * 4 + e], (int)a.q.mult) + qround) >> a.qt;
                    asm("v_med3_i32 %0, %1, %2, %3" : "=v"(d) : "v"(d), "s"(dlo), "v"(dhi));
                    const int32_t t0 = (__mul24(d, mc) + rc) >> sc;
                    const int32_t t1 = (__mul24((int)((rv >> (8 * e)) & 255), mr) + cr) >> sr;
                    y[e] = min(t0 + t1 + q.cadd, yhi); // the upper clamp in front of the last shift, the lower one is the pack's
                }
                *reinterpret_cast<uint32_t *>(lds_out + pl * OSTR + chl) = ashr_sat_u8x4(y[0], y[1], y[2], y[3], q.sh);
            }
    }
    __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    constexpr int LPR = BN / 16, RPP = 256 / LPR;
    const int c16 = (tid % LPR) * 16;
    if (bn * BN + c16 >= a.out_cs)
        return;
#pragma unroll
    for (int r = tid / LPR; r < BM; r += RPP) {
        const int m = bm * BM + r;
        if (m < a.P)
            *reinterpret_cast<v4i *>(a.y + (size_t)m * a.out_cs + bn * BN + c16) = *reinterpret_cast<const v4i *>(lds_out + r * OSTR + c16);
    }
}

// vmcnt counts a wave's vector-memory loads in issue order: wait until at most N are outstanding.
template <int N>
__device__ static inline void wait_vmcnt()
{
    // gfx9 encoding: vmcnt = {imm[15:14], imm[3:0]}, expcnt = imm[6:4], lgkmcnt = imm[11:8] (left at their maxima)
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

typedef const __attribute__((address_space(1))) void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;

} // namespace hipq
