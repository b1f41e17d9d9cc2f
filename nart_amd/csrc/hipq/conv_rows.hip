// 3x3 / stride 1 / pad 1 convolutions with 64 input and at most 64 output channels on images up to 64 pixels wide (the
// middle layer of ResNet-50's first bottleneck stage, every layer of ResNet-18's first stage, the single-layer case of
// the benchmark configurations).  gfx950 only.
//
// Reproduces op_conv_2d_u8xu8_run (art/modules/quant/src/op/conv_2d_uint8_impl.c:39-165) bit for bit, like the tile
// kernels of conv.hip; int8 tensors (conv_2d_int8_impl.c:34-174) through the same code with xmask = 0.
//
// The tile kernels stream, for every output tile, nine weight slabs and nine shifted copies of the input through LDS,
// with a barrier per slab; such a layer then takes 18 us for 3 us of matrix work.  With 64 channels the whole weight
// tensor is 36 KB - 144 registers per lane as MFMA operands - and an image row is a few KB, so:
//   * a work-group owns `rb` output rows of one image (the host picks rb so that the grid fills the chip in whole
//     rounds); the rb + 2 input rows go into LDS ONCE with the load unit, 1 KB per instruction, beside a pad pixel left
//     and right of every row and pad rows above / below the image that hold the byte izp;
//   * the weights of all nine taps (both k-steps, both halves of the 64 output channels) go into LDS once per work-group
//     with the load unit - into the space of the input rows that are not needed yet - and from there into every wave's
//     registers, where they stay (eight waves of a CU fetching 36 KB each straight from memory kept the CU's load path
//     busy for 2 us before the first multiply);
//   * a wave computes 32 pixels of an output row x 64 channels at a time: per tap and k-step its pixel operand - lane
//     (p, h): bytes [32 s + 16 h, +16) of pixel (row + dr, col + ds) - is one 128-bit LDS read, closed-form addressing,
//     no border tests, no barrier anywhere in the loop; the reads run three steps ahead of the multiplies;
//   * the 32 x 64 result bytes are transposed through a 2 KB LDS patch private to the wave (no barrier either) and leave
//     as two 128-bit stores per lane, 2 KB contiguous in memory - after the residual add of hipq_conv2d_run_add
//     (op_quant_add_run, art/modules/quant/src/op/add.c:116-152) where one is fused: the other operand's bytes are
//     requested before the requantisation and added to the transposed bytes.
// Where the time goes (cycle stamps in a throw-away build, 64 x 56 x 56, 7 output rows per work-group, two work-groups
// per CU, 12 us inside the kernel): 1.9 us until the weights and the first four rows are in LDS, 1.1 us for the eight
// waves of a CU to read their 36 KB of weights out of it (LDS bandwidth), then 1.7 - 2.1 us per unit and wave against
// 0.5 us of multiplies: a unit's multiplies and its requantisation (a quarter-rate 32-bit multiply per output) follow
// one another, and the two waves of a SIMD run in step.  Interleaving the previous unit's epilogue with the multiplies
// needs a second set of accumulators, i.e. more than the 256 registers a wave has at two waves per SIMD; at one wave
// per SIMD (512 registers) the interleaved form measured 16 us against 13.4: nothing fills a single wave's stalls.
// Requirements (checked by the host): 3x3, stride 1, pad 1, one group, input and output channel stride 64, image rows
// of at most 64 pixels, weight zero point 128 (or int8), one-multiply requantisation, per-tensor weight scale.
#include "conv_rows.h"

namespace hipq {

namespace {
constexpr int kMaxRB = 9;                   // output rows per work-group, at most (rows 4 .. 10 of the patch first hold the weights)
constexpr int kRowPitch = 64 + 5 * 1024;    // bytes of an input row in LDS: the left pad pixel, then up to 5 loads of 1 KB
                                            // (64 pixels and the pad pixel to their right)
constexpr int kPatch = 32 * 64;             // a wave's output staging: 32 pixels x 64 channels
constexpr int kWBytes = 9 * 64 * 64;        // the weights: 9 taps x 64 channels x 64 bytes
static_assert(4 * kRowPitch + kWBytes <= (kMaxRB + 2) * kRowPitch + 4 * kPatch,
              "the weights pass through the space of the rows behind the first four (and of the patches, unused until then)");
}

template <bool PLAIN_SAT, bool ADD>
__global__ __launch_bounds__(256, 2) void conv3x3_c64_rows_kernel(const ConvArgs a, const int nrb, const int rb)
{
    constexpr int P_OFF = (kMaxRB + 2) * kRowPitch;
    __shared__ __attribute__((aligned(1024))) uint8_t lds[P_OFF + 4 * kPatch + 256]; // rows, the waves' patches, the bias

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5, p = lane & 31, swz = (lane >> 2) & 3;
    const int n = (int)blockIdx.x / nrb, r0 = ((int)blockIdx.x % nrb) * rb;
    const int nrows = min(rb, a.H - r0);      // output rows of this work-group
    const int nin = nrows + 2;                // input rows r0 - 1 .. r0 + nrows

    // ---- the first four input rows (all that the first two output rows need) and, behind them, the weights: row j of the
    // patch = image row r0 - 1 + j; beyond the image: the byte izp.  Item i = (row j, 1 KB block) goes to wave i % 4 ----
    const int nblk = (a.W * 64 + 64 + 1023) >> 10; // 1 KB loads per row: its pixels and the pad pixel to their right
    auto load_rows = [&](int j0, int j1) {
        for (int i = j0 * nblk + wave; i < j1 * nblk; i += 4) {
            const int j = i / nblk, blk = i - j * nblk, ir = r0 - 1 + j;
            const int off = blk * 1024 + lane * 16;
            const bool ok = (unsigned)ir < (unsigned)a.H && off < a.W * 64;
            // the lanes of a row's loads that lie beyond its pixels read the pad source: that is the pad pixel to the right
            const uint8_t *src = ok ? a.x + ((size_t)(n * a.H + ir) * a.W) * 64 + off : a.padbuf;
            __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(lds + j * kRowPitch + 64 + blk * 1024), 16, 0, 0);
        }
    };
    const int nfirst = min(nin, 4);
    load_rows(0, nfirst);
    uint8_t *wl = lds + 4 * kRowPitch; // tap t: 64 channel rows of 64 bytes, in the packed (swizzled) order
#pragma unroll
    for (int i = 0; i < 9; i++) {
        const int blk = wave + 4 * i, t = blk >> 2, q = blk & 3; // 1 KB block q of tap t
        __builtin_amdgcn_global_load_lds((gptr_t)(a.wpack + (size_t)t * a.kout_pad * 64 + q * 1024 + lane * 16),
                                         (lptr_t)(wl + blk * 1024), 16, 0, 0);
    }
    int32_t *lbias = reinterpret_cast<int32_t *>(lds + P_OFF + 4 * kPatch);
    if (tid < 64)
        lbias[tid] = a.bias2[tid];
    // the pad pixel left of every row (those of rows 4 and up once the weights have left that space)
    auto left_pads = [&](int j0, int j1) {
        if (tid < (j1 - j0) * 4) {
            const uint32_t pw = a.padword;
            *reinterpret_cast<u32x4 *>(lds + (j0 + (tid >> 2)) * kRowPitch + (tid & 3) * 16) = u32x4{pw, pw, pw, pw};
        }
    };
    left_pads(0, nfirst);
    wait_vmcnt<0>();
    __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    // ---- this lane's weight operands for the whole kernel: [tap][k-step][channel half] ----
    v4i wreg[9][2][2];
#pragma unroll
    for (int t = 0; t < 9; t++)
#pragma unroll
        for (int s = 0; s < 2; s++)
#pragma unroll
            for (int tn = 0; tn < 2; tn++)
                wreg[t][s][tn] = *reinterpret_cast<const v4i *>(wl + t * 4096 + (tn * 32 + p) * 64 + (((2 * s + half) ^ swz) << 4));
    __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): every wave holds its weights, then the rows may overwrite them
    __builtin_amdgcn_s_barrier();
    load_rows(nfirst, nin); // in flight while the first two output rows are computed
    left_pads(nfirst, nin);

    const int nseg = (a.W + 31) >> 5;         // 32-pixel segments of a row
    uint8_t *patch = lds + P_OFF + wave * kPatch;
    // one unit: 32 pixels of an output row x 64 channels
    auto compute = [&](int u) {
        const int row = u / nseg, seg = u - row * nseg;
        const int col = min(seg * 32 + p, a.W - 1); // lanes beyond the row compute a copy that is never stored
        // pixel (row + dr, col + ds) of the patch, ds = -1 .. 1: patch row row + dr, pixel slot col + ds + 1
        const uint8_t *base = lds + row * kRowPitch + col * 64 + half * 16;
        v16i acc[2];
#pragma unroll
        for (int tn = 0; tn < 2; tn++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const v4i b = *reinterpret_cast<const v4i *>(lbias + tn * 32 + g * 8 + half * 4);
#pragma unroll
                for (int e = 0; e < 4; e++)
                    acc[tn][g * 4 + e] = b[e];
            }
        // step k = (tap, k-step): the pixel operand is read three steps before its two multiplies
        auto rd = [&](int k) {
            const int t = k >> 1;
            return *reinterpret_cast<const v4i *>(base + (t / 3) * kRowPitch + (t % 3) * 64 + (k & 1) * 32);
        };
        v4i bfr[4];
        bfr[0] = rd(0), bfr[1] = rd(1), bfr[2] = rd(2);
#pragma unroll
        for (int k = 0; k < 18; k++) {
            if (k + 3 < 18)
                bfr[(k + 3) & 3] = rd(k + 3);
            __builtin_amdgcn_sched_barrier(0); // keep the read ahead of the multiplies (the scheduler would sink it to its use)
            const v4i bf = bfr[k & 3] ^ (int)a.xmask;
            acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wreg[k >> 1][k & 1][0], bf, acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wreg[k >> 1][k & 1][1], bf, acc[1], 0, 0, 0);
        }
        uint8_t *yrow = a.y + ((size_t)(n * a.H + r0 + row) * a.W + seg * 32) * 64;
        // fused residual add: the other operand's bytes for the two 16-byte pieces this lane will store, requested now
        // and used after the requantisation
        u32x4 rv[2] = {};
        if (ADD) {
            const uint8_t *rrow = a.res + (yrow - a.y);
#pragma unroll
            for (int k = 0; k < 2; k++) {
                const int q = (lane >> 2) + 16 * k, c = lane & 3;
                if (seg * 32 + q < a.W)
                    rv[k] = *reinterpret_cast<const u32x4 *>(rrow + q * 64 + c * 16);
            }
        }
        // requantise, transpose through the wave's own patch (16-byte piece c of pixel q at piece c ^ (q & 3)), store
#pragma unroll
        for (int tn = 0; tn < 2; tn++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                uint32_t packed;
                if (PLAIN_SAT) {
                    packed = conv_requant4<true>(a, acc[tn][g * 4], acc[tn][g * 4 + 1], acc[tn][g * 4 + 2], acc[tn][g * 4 + 3]);
                } else {
                    int32_t rq[4];
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        rq[e] = conv_requant<true>(a, acc[tn][g * 4 + e]);
                    packed = pack_low_bytes(rq[0], rq[1], rq[2], rq[3]);
                }
                const int ch = tn * 32 + g * 8 + half * 4;
                *reinterpret_cast<uint32_t *>(patch + p * 64 + (((ch >> 4) ^ (p & 3)) << 4) + (ch & 15)) = packed;
            }
        __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): the wave's own writes
#pragma unroll
        for (int k = 0; k < 2; k++) {
            const int q = (lane >> 2) + 16 * k, c = lane & 3; // pixel of the segment, 16-byte piece
            u32x4 v = *reinterpret_cast<const u32x4 *>(patch + q * 64 + ((c ^ (q & 3)) << 4));
            if (ADD) { // exactly what the add operator computes from the convolution's stored bytes
                if (a.addq.fast)
                    v = a.res_first ? add_16<true>(rv[k], v, a.addq) : add_16<true>(v, rv[k], a.addq);
                else
                    v = a.res_first ? add_16<false>(rv[k], v, a.addq) : add_16<false>(v, rv[k], a.addq);
            }
            if (seg * 32 + q < a.W)
                *reinterpret_cast<u32x4 *>(yrow + q * 64 + c * 16) = v;
        }
        __builtin_amdgcn_s_waitcnt(0xC07F); // the patch is read before the next unit overwrites it
    };
    const int units = nrows * nseg, early = min(2 * nseg, units); // (row, segment) pairs; those of the first two rows
    int u = wave;
    for (; u < early; u += 4)
        compute(u);
    wait_vmcnt<0>(); // this wave's loads of the remaining rows have landed (its stores so far as well), then everybody's
    __builtin_amdgcn_s_barrier();
    for (; u < units; u += 4)
        compute(u);
}

bool conv_rows_applies(const ConvArgs &a)
{
    return a.R == 3 && a.S == 3 && a.stride_h == 1 && a.stride_w == 1 && a.pad_h == 1 && a.pad_w == 1 && a.group == 1
        && a.in_cs == 64 && a.out_cs == 64 && a.K <= 64 && a.nslab == 9 && a.W <= 64 && a.W >= 1 && a.OH == a.H && a.OW == a.W
        && a.bwz == 0 && a.fastq && !plain_epilogue(a);
}

// Output rows per work-group: two work-groups fit a CU (their registers), so the grid runs in rounds of 512; the cost of
// a choice is its number of rounds times the rows a work-group loads and computes.
static int rows_per_wg(int N, int H)
{
    int best = 1;
    long best_cost = 0;
    for (int rb = 1; rb <= kMaxRB; rb++) {
        const long wgs = (long)N * ((H + rb - 1) / rb);
        const long cost = ((wgs + 511) / 512) * (rb + 2 + 2); // + 2 input rows, + 2: the fixed part (weights, first loads)
        if (rb == 1 || cost < best_cost) {
            best = rb;
            best_cost = cost;
        }
    }
    return best;
}

void launch_conv_rows(const ConvArgs &a, hipStream_t st)
{
    const int rb = rows_per_wg(a.N, a.H), nrb = (a.H + rb - 1) / rb;
    const dim3 grid(a.N * nrb), block(256);
    const bool sat = a.lo == 0 && a.q.hi == 255;
    if (a.res != nullptr) { // the residual add of hipq_conv2d_run_add applied to the bytes on their way out
        if (sat)
            hipLaunchKernelGGL((conv3x3_c64_rows_kernel<true, true>), grid, block, 0, st, a, nrb, rb);
        else
            hipLaunchKernelGGL((conv3x3_c64_rows_kernel<false, true>), grid, block, 0, st, a, nrb, rb);
    } else if (sat) {
        hipLaunchKernelGGL((conv3x3_c64_rows_kernel<true, false>), grid, block, 0, st, a, nrb, rb);
    } else {
        hipLaunchKernelGGL((conv3x3_c64_rows_kernel<false, false>), grid, block, 0, st, a, nrb, rb);
    }
}

} // namespace hipq
