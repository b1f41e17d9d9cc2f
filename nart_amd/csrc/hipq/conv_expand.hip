// 1x1 convolutions that widen the channels (the last layer of a bottleneck block: 64 -> 256, 128 -> 512, 256 -> 1024),
// with or without the residual add of the block fused in.  gfx950 only.
//
// Reproduces op_conv_2d_u8xu8_run (art/modules/quant/src/op/conv_2d_uint8_impl.c:39-165) and, fused, op_quant_add_run
// (art/modules/quant/src/op/add.c:83-148) bit for bit, like the tile kernels of conv.hip.
//
// Such a layer writes (and, with the add, also reads) 4 bytes per byte of activations it consumes and does very little
// arithmetic per output byte on the matrix cores; what it does a lot of is VECTOR arithmetic - requantising an
// accumulator and adding the residual costs about sixteen vector instructions per output byte (three rounded shifts
// that do not merge) - and what it needs is many bytes in flight to and from HBM.  The tile kernels pay, on top of
// that, a prologue of about as many instructions again per output tile (pixel addresses, bounds, the pipeline fill),
// re-read the activations once per 64 output channels, and come in grids that leave CUs with one work-group or none at
// the end.  Here:
//   * the output is cut into tiles of 128 pixels x 64 channels, ordered channel tile fastest; the grid is as many
//     work-groups as the chip holds at once, and each takes a CONTIGUOUS range of that list, equal to within one tile;
//   * a wave owns 32 of the 128 pixels; its pixel operands for the whole reduction (at most 256 input channels: 32
//     registers) come straight from global memory - lane (p, h) loads bytes [32 s + 16 h, +16) of pixel p for k-step s,
//     which IS the MFMA operand - and stay in registers until the range moves on to the next 128 pixels;
//   * the weights of a tile (64 rows x in_cs bytes, in the packed order of the tile kernels) and its residual tile are
//     fetched by the load unit (global_load_lds_dwordx4) into one of two LDS buffers while the previous tile is being
//     requantised: the vector arithmetic of one tile hides the memory latency of the next;
//   * the result bytes overwrite the residual tile in place (every lane writes the dword it read), in a layout whose
//     16-byte pieces then leave as 128-bit stores; without a residual they go to a staging tile.  Those stores are issued
//     one tile late, after the next tile's multiplies, so that the wait for the next tile's operands - vmcnt counts loads
//     and stores alike - never waits for a store that was issued a moment ago.
//   * chained form: the 1x1 convolution that READS the sum (the first layer of the next bottleneck block: 256 -> 64,
//     512 -> 128) runs in the same kernel.  A wave owns all 64 channels of its 32 pixels in every tile, so the bytes it has
//     just written to LDS are, for those pixels, one 64-byte slab of the next convolution's reduction: after each tile
//     it multiplies them with that slab of the next layer's weights (fetched beside the tile's own) into a second set of
//     accumulators, and after the last tile it requantises those and stores the next layer's output.  The sum is still
//     written (the next block's add reads it), but never read back: a launch, and one pass over the largest tensors
//     of the network, disappear.  A work-group then takes whole rows of tiles (all channels of 128 pixels).
// Requirements (checked by the host): 1x1 kernel, no padding, one group, input channel stride 64, 128 or 256, at most
// 1024 output channels (their folded biases sit in LDS), weight zero point 128 (or int8), one-multiply requantisation,
// 32-bit form of the add, output rows of whole 16-byte pieces.
#include "conv_expand.h"

namespace hipq {

namespace {

constexpr int kBM = 128, kBN = 64, kOSTR = kBN + 16; // pixels and channels of a tile; row stride of the staging tile
constexpr int kMaxTiles = 16;                        // channel tiles, at most (their folded biases sit in LDS)

// The wave's 32 x 64 accumulators -> bytes in the staging tile (row = pixel of the work-group, 80-byte rows).
template <bool PLAIN_SAT, int TN = 2>
__device__ inline void plain_to_staging(const ConvArgs &a, const v16i (&acc)[TN], uint8_t *stg, int pl, int half)
{
    constexpr int kOSTR = TN * 32 + 16; // shadows the tile's: rows of TN * 32 channels
#pragma unroll
    for (int tn = 0; tn < TN; tn++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            uint32_t packed;
            if (PLAIN_SAT) {
                // clamp range exactly [0, 255]: two saturating packs replace four clamps and the shifts
                packed = conv_requant4<true>(a, acc[tn][g * 4], acc[tn][g * 4 + 1], acc[tn][g * 4 + 2], acc[tn][g * 4 + 3]);
            } else {
                int32_t rq[4];
#pragma unroll
                for (int e = 0; e < 4; e++)
                    rq[e] = conv_requant<true>(a, acc[tn][g * 4 + e]);
                packed = pack_low_bytes(rq[0], rq[1], rq[2], rq[3]);
            }
            *reinterpret_cast<uint32_t *>(stg + pl * kOSTR + tn * 32 + g * 8 + half * 4) = packed;
        }
}

// The same with the residual add applied in the accumulator layout, on a residual tile in LDS (16-byte piece c of
// pixel row r at piece c ^ ((r >> 1) & 3) of its 64-byte row), which the result bytes overwrite: per element the
// convolution's clamped result minus its zero point is clamp(q, lo - zp, hi - zp) with q = (mulhi(acc, mult) + 2^(t-1)) >> t;
// the add's terms are (d * m + c) >> s; the sum is clamped and packed.  ADD_SAT: the add's clamp range is exactly [0, 255].
template <bool ADD_SAT>
__device__ inline void fused_in_place(const ConvArgs &a, const v16i (&acc)[2], uint8_t *rtile, int pl, int half)
{
    const AddParams &q = a.addq;
    const int mc = (int)(a.res_first ? q.m1 : q.m0), sc = a.res_first ? q.s1 : q.s0;
    const int mr = (int)(a.res_first ? q.m0 : q.m1), sr = a.res_first ? q.s0 : q.s1, cr = a.res_first ? q.c0 : q.c1;
    const int rc = 1 << (sc - 1);                    // rounding of the convolution's term (its zero point cancels)
    const int qround = 1 << (a.qt - 1);
    const int dlo = a.lo - a.q.zp, dhi = a.q.hi - a.q.zp; // clamp range of (conv byte - conv zero point)
    const int rsw = (pl >> 1) & 3;
#pragma unroll
    for (int tn = 0; tn < 2; tn++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const int chl = tn * 32 + g * 8 + half * 4;
            uint32_t *slot = reinterpret_cast<uint32_t *>(rtile + pl * kBN + (((chl >> 4) ^ rsw) << 4) + (chl & 15));
            const uint32_t rv = *slot;
            int32_t y[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                int32_t d = (__mulhi(acc[tn][g * 4 + e], (int)a.q.mult) + qround) >> a.qt;
                asm("v_med3_i32 %0, %1, %2, %3" : "=v"(d) : "v"(d), "s"(dlo), "v"(dhi));
                const int32_t t0 = (__mul24(d, mc) + rc) >> sc;
                const int32_t t1 = (__mul24((int)((rv >> (8 * e)) & 255), mr) + cr) >> sr;
                y[e] = t0 + t1 + q.cadd;
            }
            uint32_t packed;
            if (ADD_SAT) {
                packed = ashr_sat_u8x4(y[0], y[1], y[2], y[3], q.sh); // the last shift, the clamp to [0, 255], the pack
            } else {
                packed = 0;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    int32_t v = y[e] >> q.sh;
                    asm("v_med3_i32 %0, %1, %2, %3" : "=v"(v) : "v"(v), "s"(0), "v"(q.hi));
                    packed |= (uint32_t)v << (8 * e);
                }
            }
            *slot = packed; // the lane that read the residual dword replaces it with the result: no other lane touches it
        }
}

} // namespace

// MID: 0, or the output channels (64 / 128) of the chained 1x1 convolution a2, whose output goes to a2.y
template <int NSLAB, bool FUSED, bool SAT, int MID>
__global__ __launch_bounds__(256) void conv_mfma_expand_kernel(const ConvArgs a, const ConvArgs a2, const int ntiles, const int total)
{
    constexpr int WBYTES = NSLAB * 4096;         // one channel tile of weights: NSLAB slabs of 64 rows x 64 bytes
    constexpr int RBYTES = kBM * kBN;            // one residual tile
    constexpr int R_OFF = 2 * WBYTES;            // fused: two residual tiles; plain: one staging tile
    constexpr int B_OFF = R_OFF + (FUSED ? 2 * RBYTES : kBM * kOSTR);
    constexpr int W2BYTES = MID * 64;            // chained: one slab of the next layer's weights (MID rows x 64 bytes)
    constexpr int W2_OFF = B_OFF + kMaxTiles * kBN * 4, S2_OFF = W2_OFF + 2 * W2BYTES; // then its output staging tile
    constexpr int TN2 = MID / 32;
    static_assert(MID == 0 || (FUSED && SAT && (MID == 64 || MID == 128)), "the chained form follows a fused add to uint8");
    __shared__ __attribute__((aligned(1024))) uint8_t lds[S2_OFF + (MID ? kBM * (MID + 16) : 0)];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5, p = lane & 31, swz = (lane >> 2) & 3;
    // work-groups go to the 8 XCDs in turn: XCD x takes the x-th contiguous eighth of the tile list (the grid is a
    // multiple of 8), so neighbours in the list - which share pixels or weights - share an L2
    const int g = (int)(blockIdx.x % 8) * (int)(gridDim.x / 8) + (int)(blockIdx.x / 8);
    int t0, t1;
    if (MID) { // whole rows of tiles: work-group g takes the 128 pixels of row g
        t0 = g * ntiles, t1 = t0 + ntiles;
        if (t0 >= total)
            return;
    } else {
        t0 = (int)((long long)total * g / (int)gridDim.x), t1 = (int)((long long)total * (g + 1) / (int)gridDim.x);
        if (t0 >= t1)
            return;
    }

    // ---- tile t -> LDS buffer (t - t0) & 1: its weights, and its residual tile when fused ----
    const size_t wslab = (size_t)a.kout_pad * 64;
    const int wave_off = wave * 1024;
    auto issue = [&](int mt, int nt, int buf) {
        uint8_t *wb = lds + buf * WBYTES + wave_off;
        const uint8_t *ws = a.wpack + (size_t)nt * 4096 + tid * 16;
#pragma unroll
        for (int s = 0; s < NSLAB; s++)
            __builtin_amdgcn_global_load_lds((gptr_t)(ws + s * wslab), (lptr_t)(wb + s * 4096), 16, 0, 0);
        if (FUSED) {
            // slot sl of the tile = 16-byte piece (sl & 3) ^ ((r >> 1) & 3) of pixel row r = sl >> 2
            uint8_t *rb = lds + R_OFF + buf * RBYTES + wave_off;
#pragma unroll
            for (int jj = 0; jj < 2; jj++) {
                const int sl = tid + 256 * jj, r = sl >> 2, c = (sl & 3) ^ ((r >> 1) & 3);
                const int m = mt * kBM + r, ch = nt * kBN + c * 16;
                const uint8_t *src = m < a.P && ch < a.out_cs ? a.res + (size_t)m * a.out_cs + ch : a.padbuf;
                __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(rb + jj * 4096), 16, 0, 0);
            }
        }
        if (MID) { // slab nt of the next layer's weights: its input channels 64 nt .. 64 nt + 63 are this tile's outputs
            const uint8_t *w2 = a2.wpack + (size_t)nt * a2.kout_pad * 64 + tid * 16;
#pragma unroll
            for (int jj = 0; jj < W2BYTES / 4096; jj++)
                __builtin_amdgcn_global_load_lds((gptr_t)(w2 + jj * 4096), (lptr_t)(lds + W2_OFF + buf * W2BYTES + wave_off + jj * 4096), 16, 0, 0);
        }
    };
    int mt = t0 / ntiles, nt = t0 - mt * ntiles; // the current tile; the list is walked without further divisions
    issue(mt, nt, 0);

    // ---- the folded biases -> LDS; the wave's pixel operands -> registers.  Every global load of the prologue is issued
    // before the first result is used (bias values wait in registers, the pixel operands are re-centred after the
    // loop's first wait): one round trip to memory instead of three in a row ----
    int32_t *lbias = reinterpret_cast<int32_t *>(lds + B_OFF);
    int32_t bv[kMaxTiles * kBN / 256];
#pragma unroll
    for (int j = 0; j < kMaxTiles * kBN / 256; j++)
        bv[j] = tid + 256 * j < ntiles * kBN ? a.bias2[tid + 256 * j] : 0;
    const int pl = wave * 32 + p;                 // this lane's pixel within the tile's 128
    v4i bf[NSLAB][2];
    auto load_pixels = [&](int mt) {
        const int m = min(mt * kBM + pl, a.P - 1); // rows beyond the tensor compute a copy that is never stored
        const uint8_t *xrow;
        if (a.stride_h == 1 && a.stride_w == 1) {
            xrow = a.x + (size_t)m * a.in_cs;
        } else {
            const int ohw = a.OH * a.OW;
            const int n = fast_div(m, ohw, a.inv_ohw), rem = m - n * ohw;
            const int oh = fast_div(rem, a.OW, a.inv_ow), ow = rem - oh * a.OW;
            xrow = a.x + ((size_t)(n * a.H + oh * a.stride_h) * a.W + ow * a.stride_w) * a.in_cs;
        }
#pragma unroll
        for (int s = 0; s < NSLAB; s++)
#pragma unroll
            for (int k = 0; k < 2; k++)
                bf[s][k] = ldg128(xrow + s * 64 + k * 32 + half * 16); // raw bytes: re-centred at the top of the next tile
    };
    load_pixels(mt);
    bool fresh = true; // bf holds raw bytes
#pragma unroll
    for (int j = 0; j < kMaxTiles * kBN / 256; j++)
        if (tid + 256 * j < ntiles * kBN)
            lbias[tid + 256 * j] = bv[j];
    v16i acc2[MID ? TN2 : 1]; // chained: 32 pixels x MID channels of the next layer, from its folded bias
    if (MID) {
#pragma unroll
        for (int tn = 0; tn < TN2; tn++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const v4i bv = *reinterpret_cast<const v4i *>(a2.bias2 + tn * 32 + q * 8 + half * 4);
#pragma unroll
                for (int e = 0; e < 4; e++)
                    acc2[tn][q * 4 + e] = bv[e];
            }
    }
    const int foff[2] = {p * 64 + (((0 + half) ^ swz) << 4), p * 64 + (((2 + half) ^ swz) << 4)};

    // the finished tile's 16-byte pieces: four lanes per pixel row, two passes of 64 rows
    const int srow = tid >> 2, spiece = tid & 3;
    auto read_staged = [&](int buf, v4i(&v)[2]) {
#pragma unroll
        for (int k = 0; k < 2; k++) {
            const int r = srow + 64 * k;
            v[k] = FUSED ? *reinterpret_cast<const v4i *>(lds + R_OFF + buf * RBYTES + r * kBN + ((spiece ^ ((r >> 1) & 3)) << 4))
                         : *reinterpret_cast<const v4i *>(lds + R_OFF + r * kOSTR + spiece * 16);
        }
    };
    auto store_tile = [&](int smt, int snt, const v4i(&v)[2]) {
        const int ch = snt * kBN + spiece * 16;
#pragma unroll
        for (int k = 0; k < 2; k++) {
            const int m = smt * kBM + srow + 64 * k;
            if (m < a.P && ch < a.out_cs)
                *reinterpret_cast<v4i *>(a.y + (size_t)m * a.out_cs + ch) = v[k];
        }
    };

    int pmt = mt, pnt = nt; // the previous tile
    for (int t = t0; t < t1; t++) {
        const int buf = (t - t0) & 1;
        const bool wrap = nt + 1 == ntiles;
        const int nmt = wrap ? mt + 1 : mt, nnt = wrap ? 0 : nt + 1; // the next tile
        // tile t's operands have landed (issued a whole requantisation ago, like the stores of tile t - 2); this wave's
        // LDS writes of the previous tile's bytes (and of the biases) are done; the barrier makes all of it visible
        wait_vmcnt<0>();
        __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
        if (fresh) { // the pixel operands loaded during the previous tile (or the prologue) have landed with that wait
#pragma unroll
            for (int s = 0; s < NSLAB; s++)
#pragma unroll
                for (int k = 0; k < 2; k++)
                    bf[s][k] ^= (int)a.xmask;
            fresh = false;
        }
        const uint8_t *wb = lds + buf * WBYTES;
        v16i acc[2];
#pragma unroll
        for (int tn = 0; tn < 2; tn++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const v4i bv = *reinterpret_cast<const v4i *>(lbias + nt * kBN + tn * 32 + q * 8 + half * 4);
#pragma unroll
                for (int e = 0; e < 4; e++)
                    acc[tn][q * 4 + e] = bv[e];
            }
#pragma unroll
        for (int s = 0; s < NSLAB; s++)
#pragma unroll
            for (int k = 0; k < 2; k++) {
                const v4i af0 = *reinterpret_cast<const v4i *>(wb + s * 4096 + foff[k]);
                const v4i af1 = *reinterpret_cast<const v4i *>(wb + s * 4096 + 2048 + foff[k]);
                acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af0, bf[s][k], acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af1, bf[s][k], acc[1], 0, 0, 0);
            }
        if (t + 1 < t1 && wrap) {
            load_pixels(nmt); // the range moves on to the next 128 pixels: their operands arrive during this tile's arithmetic
            fresh = true;
        }
        v4i staged[2];
        if (t > t0)
            read_staged(buf ^ 1, staged);
        // every thread's reads of the previous tile's bytes have returned, every wave is done with the other weight buffer
        __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
        if (t + 1 < t1)
            issue(nmt, nnt, buf ^ 1);
        if (t > t0)
            store_tile(pmt, pnt, staged);
        if (FUSED)
            fused_in_place<SAT>(a, acc, lds + R_OFF + buf * RBYTES, pl, half);
        else
            plain_to_staging<SAT>(a, acc, lds + R_OFF, pl, half);
        if (MID) {
            // the 64 bytes this wave has just written for each of its pixels are slab nt of the next layer's reduction
            __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): own writes
            const uint8_t *row = lds + R_OFF + buf * RBYTES + pl * kBN, *w2b = lds + W2_OFF + buf * W2BYTES;
            const int rsw = (pl >> 1) & 3;
#pragma unroll
            for (int k = 0; k < 2; k++) {
                const v4i b2 = *reinterpret_cast<const v4i *>(row + (((2 * k + half) ^ rsw) << 4)) ^ (int)a2.xmask;
#pragma unroll
                for (int tn = 0; tn < TN2; tn++) {
                    const v4i af = *reinterpret_cast<const v4i *>(w2b + tn * 2048 + foff[k]);
                    acc2[tn] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, b2, acc2[tn], 0, 0, 0);
                }
            }
        }
        pmt = mt, pnt = nt;
        mt = nmt, nt = nnt;
    }
    __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    v4i staged[2];
    read_staged((t1 - 1 - t0) & 1, staged);
    store_tile(pmt, pnt, staged);
    if (MID) {
        // the next layer's 128 pixels x MID channels: requantise, transpose through LDS, 128-bit stores
        uint8_t *stg2 = lds + S2_OFF;
        if (a2.lo == 0 && a2.q.hi == 255)
            plain_to_staging<true, MID ? TN2 : 1>(a2, acc2, stg2, pl, half);
        else
            plain_to_staging<false, MID ? TN2 : 1>(a2, acc2, stg2, pl, half);
        __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
        constexpr int LPR = (MID ? MID : 64) / 16, RPP = 256 / LPR; // lanes per pixel row, rows per pass
        const int c16 = (tid % LPR) * 16;
#pragma unroll
        for (int r = tid / LPR; r < kBM; r += RPP) {
            const int m = pmt * kBM + r;
            if (m < a2.P && c16 < a2.out_cs)
                *reinterpret_cast<v4i *>(a2.y + (size_t)m * a2.out_cs + c16) = *reinterpret_cast<const v4i *>(stg2 + r * (MID + 16) + c16);
        }
    }
}

bool conv_expand_applies(const ConvArgs &a, bool wherever)
{
    const int ntiles = (a.out_cs + kBN - 1) / kBN;
    return a.R == 1 && a.S == 1 && a.pad_h == 0 && a.pad_w == 0 && a.group == 1 && a.bwz == 0
        && (a.in_cs == 64 || a.in_cs == 128 || a.in_cs == 256) && a.nslab == a.in_cs / 64 && a.fastq && !plain_epilogue(a)
        && ntiles >= 4 && ntiles <= kMaxTiles && a.out_cs >= 2 * a.in_cs && a.P >= 1024 && (a.res == nullptr || a.addq.fast)
        // where it beats the kernels it replaces: with the add at 64 input channels (31.7 against 35.7 us at 64 -> 256
        // on 200 704 pixels; level at 128 -> 512, behind at 256 -> 1024), without at 256 (16.7 against 19.7 us at
        // 256 -> 512 on 50 176 pixels) and at 64 on very many pixels (64 -> 256 on 200 704: 16.3 against the pointwise
        // kernel's 17.8 us alone, and the ResNet-50 pass it sits in 0.880 -> 0.869 ms); inside that pass the add at 128 input
        // channels on 50 176 pixels gains 0.25 %, the one at 256 on 12 544 loses 0.5 % - and only on many pixels: its grid is
        // three work-groups per CU whatever the size, a launch of it takes 6.6 us or more, and the tile kernels need
        // 4 to 7 us up to some 12 000 pixels (256 -> 512: level at 25 000; 64 -> 256 with the add: 19.6 against 18.7 us
        // at 100 352)
        && (wherever || (a.res != nullptr ? (a.in_cs == 64 && a.P >= 150000) || (a.in_cs == 128 && a.P >= 50000) : (a.in_cs == 256 && a.P >= 20000) || (a.in_cs == 64 && a.P >= 150000)));
}

template <int NSLAB, int MID>
static void launch_expand_n(const ConvArgs &a, const ConvArgs &a2, hipStream_t st)
{
    const bool fused = a.res != nullptr;
    const int mtiles = (a.P + kBM - 1) / kBM, ntiles = (a.out_cs + kBN - 1) / kBN, total = mtiles * ntiles;
    if (MID) {
        const dim3 grid((unsigned)((mtiles + 7) / 8 * 8)), block(256);
        hipLaunchKernelGGL((conv_mfma_expand_kernel<NSLAB, true, true, MID>), grid, block, 0, st, a, a2, ntiles, total);
        return;
    }
    // three work-groups per CU (measured: two leave the vector units idle while a work-group waits for its tile, four slow
    // every work-group's arithmetic down by more than they hide), fewer where their LDS does not fit; at least two tiles each
    const int lds = 2 * NSLAB * 4096 + (fused ? 2 * kBM * kBN : kBM * kOSTR) + kMaxTiles * kBN * 4;
    const int per_cu = std::max(1, std::min(3, 160 * 1024 / lds));
    const int wgs = std::max(8, std::min(256 * per_cu, total / 2) / 8 * 8);
    const dim3 grid((unsigned)wgs), block(256);
    if (fused) {
        if (a.addq.hi == 255)
            hipLaunchKernelGGL((conv_mfma_expand_kernel<NSLAB, true, true, 0>), grid, block, 0, st, a, a2, ntiles, total);
        else
            hipLaunchKernelGGL((conv_mfma_expand_kernel<NSLAB, true, false, 0>), grid, block, 0, st, a, a2, ntiles, total);
    } else if (a.lo == 0 && a.q.hi == 255) {
        hipLaunchKernelGGL((conv_mfma_expand_kernel<NSLAB, false, true, 0>), grid, block, 0, st, a, a2, ntiles, total);
    } else {
        hipLaunchKernelGGL((conv_mfma_expand_kernel<NSLAB, false, false, 0>), grid, block, 0, st, a, a2, ntiles, total);
    }
}

void launch_conv_expand(const ConvArgs &a, hipStream_t st)
{
    switch (a.nslab) {
    case 1: launch_expand_n<1, 0>(a, a, st); break;
    case 2: launch_expand_n<2, 0>(a, a, st); break;
    default: launch_expand_n<4, 0>(a, a, st); break; // conv_expand_applies: in_cs is 64, 128 or 256
    }
}

bool conv_expand_chain_applies(const ConvArgs &a, const ConvArgs &a2)
{
    return a.res != nullptr && conv_expand_applies(a, true) && a.in_cs <= 128 && a.out_cs % kBN == 0 && a.addq.hi == 255
        && a2.R == 1 && a2.S == 1 && a2.pad_h == 0 && a2.pad_w == 0 && a2.stride_h == 1 && a2.stride_w == 1 && a2.group == 1
        && a2.bwz == 0 && a2.xmask != 0 && a2.N == a.N && a2.H == a.OH && a2.W == a.OW && a2.in_cs == a.out_cs && a2.P == a.P
        && a2.nslab == a.out_cs / kBN && (a2.out_cs == 64 || a2.out_cs == 128) && a2.kout_pad >= a2.out_cs && a2.fastq
        && !plain_epilogue(a2) && a2.res == nullptr;
}

void launch_conv_expand_chain(const ConvArgs &a, const ConvArgs &a2, hipStream_t st)
{
    if (a2.out_cs == 64) {
        if (a.nslab == 1)
            launch_expand_n<1, 64>(a, a2, st);
        else
            launch_expand_n<2, 64>(a, a2, st);
    } else {
        if (a.nslab == 1)
            launch_expand_n<1, 128>(a, a2, st);
        else
            launch_expand_n<2, 128>(a, a2, st);
    }
}

} // namespace hipq
