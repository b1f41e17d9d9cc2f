// Depthwise 3x3 convolution (group == C == K, stride 1 or 2, weight zero point 128) for gfx950, written for
// instruction count: the layer is bound by vector arithmetic, not by its 2 bytes of traffic per output byte.
//
// A thread owns 4 channels (one dword of the channels-last tensors) of a strip of 4 output columns and walks down RB
// output rows of it.  Per INPUT row it loads the 6 (stride 1) or 9 (stride 2) dwords of the strip's columns once,
// transposes them once into per-channel dwords of four consecutive pixels (8 v_perm_b32 per 4x4 block), and feeds
// them to the partial sums of every output row that input row belongs to: three rows in flight for stride 1 (kernel
// rows 0, 1, 2 of output rows i, i-1, i-2), two for stride 2.  An output row is requantised and stored when its last
// kernel row is in: every loaded and transposed input row serves all the output rows it belongs to, and none of the
// work is for rows that the thread does not produce (RB = 2 measured fastest: see kRowsPerThread).
//   stride 1: T0 = [x0 x1 x2 x3], T1 = [x2 x3 x4 x5] per channel; outputs 0 / 1 are v_dot4_i32_i8 of T0 with the packed
//             weights [w0 w1 w2 0] / [0 w0 w1 w2], outputs 2 / 3 the same with T1;
//   stride 2: T0 = [x0..x3], T1 = [x4..x7]; outputs 0 and 2 use T0 and T1, output 1 v_alignbyte(T1, T0) = [x2 x3 x4 x5],
//             output 3 a v_perm of T1 and the ninth column = [x6 x7 x8 0]; all with [w0 w1 w2 0].
// Bytes are re-centred (x ^ 0x80, w - 128); bias + 128 * sum(w - 128) is folded per channel by the host.  Columns and
// rows outside the image are loaded from a clamped address and replaced by the zero-point byte (a select per dword,
// no divergent branch).  Rows three ahead are requested before the current row is used.
#include "conv_dw.h"
#include "hipq.h"

#include <algorithm>
#include <cstdlib>
#include <type_traits>

namespace hipq {

namespace {

template <int V>
using ic = std::integral_constant<int, V>;

// f(ic<B>{}), f(ic<B + 1>{}), ..., f(ic<E - 1>{}): a loop whose index is a constant expression inside the body
template <int B, int E, class F>
__device__ static inline void static_for(F &&f)
{
    if constexpr (B < E) {
        f(ic<B>{});
        static_for<B + 1, E>(f);
    }
}

// dwords A..D: 4 channels of four consecutive pixels; T[c]: channel c of the four pixels
// (v_perm_b32(S0, S1, sel): selector bytes 0-3 pick from S1, 4-7 from S0)
__device__ static inline void transpose4(uint32_t A, uint32_t B, uint32_t C, uint32_t D, uint32_t (&T)[4])
{
    const uint32_t t0 = __builtin_amdgcn_perm(B, A, 0x05010400u), t1 = __builtin_amdgcn_perm(B, A, 0x07030602u);
    const uint32_t t2 = __builtin_amdgcn_perm(D, C, 0x05010400u), t3 = __builtin_amdgcn_perm(D, C, 0x07030602u);
    T[0] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
    T[1] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
    T[2] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
    T[3] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
}

// dot(a, b) + c into a new register: the compiler's own choice for this is a copy of c followed by the accumulating form
__device__ static inline int32_t dot4_from(uint32_t a, int32_t b, int32_t c)
{
    int32_t d;
    asm("v_dot4_i32_i8 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
}

// QMODE 0: 64-bit requantisation (any shift, per-channel scales); 1: one-multiply form; 2: one-multiply form and a
// clamp range of exactly [0, 255] (saturating packs instead of clamps).  DUMP: also write the int32 sums.
template <int QMODE, bool DUMP>
__device__ static inline void emit_row(const ConvArgs &a, const int32_t (&acc)[4][4], uint32_t obase, int ncols, int c0)
{
#pragma unroll
    for (int o = 0; o < 4; o++) {
        if (o >= ncols)
            break;
        const uint32_t off = obase + (uint32_t)(o * a.out_cs);
        if (DUMP)
            *reinterpret_cast<v4i *>(a.acc_out + off) = v4i{acc[o][0], acc[o][1], acc[o][2], acc[o][3]};
        uint32_t packed = 0;
        if (QMODE == 2) {
            packed = conv_requant4<true>(a, acc[o][0], acc[o][1], acc[o][2], acc[o][3]);
        } else {
            int32_t r[4];
#pragma unroll
            for (int c = 0; c < 4; c++)
                r[c] = (QMODE == 0 && a.qmult) ? conv_requant_ch(a, acc[o][c], c0 + c) : conv_requant<QMODE == 1>(a, acc[o][c]);
            packed = pack_low_bytes(r[0], r[1], r[2], r[3]);
        }
        *reinterpret_cast<uint32_t *>(a.y + off) = packed;
    }
}

// How the grid maps to work: a work-group is ONE wave and takes 64 consecutive (strip, channel quad) items of one row block
// of one image, so image and row block are the same for all its lanes and everything derived from them - row addresses,
// row validity, the output row's base - is scalar-unit arithmetic, off the vector ALU that bounds this kernel.  The two
// divisions that take a block number apart, and the one that splits an item, are multiplications by reciprocals the
// host has computed (and verified for every dividend that can occur).
struct DwMap {
    int nrb, chunks, per_img, items; // row blocks per image, waves per row block, their product, items per row block
    uint32_t m_img, m_chunk, m_cq;   // floor(x / d) = (x * m) >> (32 + s)
    int s_img, s_chunk, s_cq;
    int cq;
};

// m == 0: the divisor is 1 (no 32-bit reciprocal multiplies to the identity)
__device__ static inline uint32_t div_magic(uint32_t x, uint32_t m, int s) { return m ? (uint32_t)(((uint64_t)x * m) >> 32) >> s : x; }

template <int STRIDE, int QMODE, bool DUMP, int RB>
__global__ __launch_bounds__(64) void conv_depthwise3x3_slide_kernel(const ConvArgs a, const DwMap mp)
{
    constexpr int NCOL = 3 * STRIDE + 3; // input columns under a strip of 4 outputs
    // work-groups go to the 8 XCDs in turn: renumbered so that each XCD works on one contiguous eighth of the
    // (image-major) block list (the grid is a multiple of 8; blocks beyond the list end at once)
    const uint32_t L = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    const uint32_t n = div_magic(L, mp.m_img, mp.s_img), r1 = L - n * mp.per_img;
    const uint32_t rb = div_magic(r1, mp.m_chunk, mp.s_chunk), chunk = r1 - rb * mp.chunks;
    if ((int)n >= a.N)
        return;
    const uint32_t item = chunk * 64 + threadIdx.x;
    if ((int)item >= mp.items)
        return;
    const int strip = (int)div_magic(item, mp.m_cq, mp.s_cq), quad = (int)item - strip * mp.cq;
    const int oh0 = (int)rb * RB, ow0 = strip * 4, c0 = quad * 4;
    const int ih0 = oh0 * STRIDE - a.pad_h, iw0 = ow0 * STRIDE - a.pad_w;
    const int ncols = min(4, a.OW - ow0);

    const uint32_t *wtab = reinterpret_cast<const uint32_t *>(a.wpack); // [3 rows][2 alignments][cs] dwords
    const v4i bias = *reinterpret_cast<const v4i *>(a.bias2 + c0);
    v4i wa[3], wb[3];
#pragma unroll
    for (int r = 0; r < 3; r++) {
        wa[r] = *reinterpret_cast<const v4i *>(wtab + (r * 2 + 0) * a.in_cs + c0); // [w0 w1 w2 0] per channel
        if (STRIDE == 1)
            wb[r] = *reinterpret_cast<const v4i *>(wtab + (r * 2 + 1) * a.in_cs + c0); // [0 w0 w1 w2]
    }

    // 32-bit byte offsets from the tensor base (the host guarantees the tensors are smaller than 2 GiB)
    const uint32_t nbase = (uint32_t)(n * a.H * a.W * a.in_cs + c0);
    const uint32_t rowbytes = (uint32_t)(a.W * a.in_cs);
    const uint32_t padx = a.padword ^ 0x80808080u;
    uint32_t coff[NCOL];
    bool cok[NCOL];
    const int off0 = iw0 * a.in_cs, offmax = (a.W - 1) * a.in_cs; // one multiply per thread: the clamp commutes with the scaling
#pragma unroll
    for (int j = 0; j < NCOL; j++) {
        cok[j] = (unsigned)(iw0 + j) < (unsigned)a.W;
        coff[j] = (uint32_t)min(max(off0 + j * a.in_cs, 0), offmax);
    }
    auto issue = [&](int i, uint32_t (&dst)[NCOL]) {
        const uint32_t rbase = nbase + (uint32_t)min(max(ih0 + i, 0), a.H - 1) * rowbytes;
#pragma unroll
        for (int j = 0; j < NCOL; j++)
            dst[j] = *reinterpret_cast<const uint32_t *>(a.x + (rbase + coff[j]));
    };
    auto fix = [&](int i, const uint32_t (&src)[NCOL], uint32_t (&col)[NCOL]) {
        const bool rok = (unsigned)(ih0 + i) < (unsigned)a.H;
#pragma unroll
        for (int j = 0; j < NCOL; j++)
            col[j] = (rok && cok[j]) ? (src[j] ^ 0x80808080u) : padx;
    };
    auto emit = [&](const int32_t (&r)[4][4], int oh) {
        if (oh < a.OH)
            emit_row<QMODE, DUMP>(a, r, (uint32_t)(((n * a.OH + oh) * a.OW + ow0) * a.out_cs + c0), ncols, c0);
    };

    constexpr int PD = 3, NSET = PD + 1; // rows requested ahead of the row in use; register sets for rows in flight
    if constexpr (STRIDE == 1) {
        // input row i (relative to the block's first) is kernel row 0 of output row i, 1 of i - 1, 2 of i - 2; the sums of
        // output row r live in acc[r % 3], input row i in raw[i % NSET].  Everything below is straight-line code (RB is a
        // template argument), so the compiler's wait counts are exact: a loop would make it wait for every load in
        // flight at each trip.
        constexpr int NIN = RB + 2;
        int32_t acc[3][4][4];
        uint32_t raw[NSET][NCOL];
        static_for<0, (PD < NIN ? PD : NIN)>([&](auto ii) { issue(decltype(ii)::value, raw[decltype(ii)::value % NSET]); });
        static_for<0, NIN>([&](auto ii) {
            constexpr int i = decltype(ii)::value;
            if constexpr (i + PD < NIN)
                issue(i + PD, raw[(i + PD) % NSET]);
            uint32_t col[NCOL];
            fix(i, raw[i % NSET], col);
#pragma unroll
            for (int h = 0; h < 2; h++) {
                uint32_t T[4];
                transpose4(col[2 * h], col[2 * h + 1], col[2 * h + 2], col[2 * h + 3], T);
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    if constexpr (i < RB) {
                        acc[i % 3][2 * h][c] = dot4_from(T[c], wa[0][c], bias[c]);
                        acc[i % 3][2 * h + 1][c] = dot4_from(T[c], wb[0][c], bias[c]);
                    }
                    if constexpr (i >= 1 && i - 1 < RB) {
                        constexpr int s = (i + 2) % 3;
                        acc[s][2 * h][c] = __builtin_amdgcn_sdot4((int)T[c], wa[1][c], acc[s][2 * h][c], false);
                        acc[s][2 * h + 1][c] = __builtin_amdgcn_sdot4((int)T[c], wb[1][c], acc[s][2 * h + 1][c], false);
                    }
                    if constexpr (i >= 2) {
                        constexpr int s = (i + 1) % 3;
                        acc[s][2 * h][c] = __builtin_amdgcn_sdot4((int)T[c], wa[2][c], acc[s][2 * h][c], false);
                        acc[s][2 * h + 1][c] = __builtin_amdgcn_sdot4((int)T[c], wb[2][c], acc[s][2 * h + 1][c], false);
                    }
                }
            }
            if constexpr (i >= 2)
                emit(acc[(i + 1) % 3], oh0 + i - 2);
        });
    } else {
        // input rows 2 o and 2 o + 1 are kernel rows 0 and 1 of output row o, row 2 o is also kernel row 2 of output row
        // o - 1; the sums of output row r live in acc[r % 2], input row i in raw[i % NSET]
        constexpr int NIN = 2 * RB + 1;
        int32_t acc[2][4][4];
        uint32_t raw[NSET][NCOL];
        auto operands = [&](const uint32_t (&col)[NCOL], uint32_t (&op)[4][4]) {
            uint32_t T0[4], T1[4];
            transpose4(col[0], col[1], col[2], col[3], T0);
            transpose4(col[4], col[5], col[6], col[7], T1);
#pragma unroll
            for (int c = 0; c < 4; c++) {
                op[0][c] = T0[c];
                op[1][c] = __builtin_amdgcn_alignbyte(T1[c], T0[c], 2);
                op[2][c] = T1[c];
                op[3][c] = __builtin_amdgcn_perm(col[NCOL - 1], T1[c], 0x0c000302u | ((4u + c) << 16)); // 0x0c: a zero byte
            }
        };
        static_for<0, (PD < NIN ? PD : NIN)>([&](auto ii) { issue(decltype(ii)::value, raw[decltype(ii)::value % NSET]); });
        static_for<0, NIN>([&](auto ii) {
            constexpr int i = decltype(ii)::value, o = i >> 1;
            if constexpr (i + PD < NIN)
                issue(i + PD, raw[(i + PD) % NSET]);
            uint32_t col[NCOL], op[4][4];
            fix(i, raw[i % NSET], col);
            operands(col, op);
#pragma unroll
            for (int q = 0; q < 4; q++)
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    if constexpr ((i & 1) == 0) {
                        if constexpr (o < RB)
                            acc[o % 2][q][c] = dot4_from(op[q][c], wa[0][c], bias[c]);
                        if constexpr (o >= 1)
                            acc[(o + 1) % 2][q][c] = __builtin_amdgcn_sdot4((int)op[q][c], wa[2][c], acc[(o + 1) % 2][q][c], false);
                    } else {
                        acc[o % 2][q][c] = __builtin_amdgcn_sdot4((int)op[q][c], wa[1][c], acc[o % 2][q][c], false);
                    }
                }
            if constexpr ((i & 1) == 0 && o >= 1)
                emit(acc[(o + 1) % 2], oh0 + o - 1);
        });
    }
}

} // namespace

bool conv_dw_slide_applies(const ConvArgs &a)
{
    return a.R == 3 && a.S == 3 && a.stride_h == a.stride_w && (a.stride_h == 1 || a.stride_h == 2) && a.bwz == 0
        && a.in_cs == a.out_cs && (a.in_cs & 3) == 0;
}

template <int STRIDE, int RB>
static void launch_rb(const ConvArgs &a, hipStream_t st)
{
    DwMap mp;
    mp.nrb = (a.OH + RB - 1) / RB;
    mp.cq = a.in_cs / 4;
    mp.items = ((a.OW + 3) / 4) * mp.cq;
    mp.chunks = (mp.items + 63) / 64;
    mp.per_img = mp.nrb * mp.chunks;
    const long long grid_l = ((long long)a.N * mp.per_img + 7) / 8 * 8; // the plan bounds N * OH * strips * quads by 2^31
    // reciprocals for the three divisions (include/hipq.h: hipq_div_magic)
    hipq_div_magic((uint32_t)mp.per_img, &mp.m_img, &mp.s_img);
    hipq_div_magic((uint32_t)mp.chunks, &mp.m_chunk, &mp.s_chunk);
    hipq_div_magic((uint32_t)mp.cq, &mp.m_cq, &mp.s_cq);
    const dim3 grid((unsigned)grid_l), block(64);
    const int qmode = (a.fastq && a.qmult == nullptr) ? (a.lo == 0 && a.q.hi == 255 ? 2 : 1) : 0;
    if (a.acc_out)
        hipLaunchKernelGGL((conv_depthwise3x3_slide_kernel<STRIDE, 0, true, RB>), grid, block, 0, st, a, mp);
    else if (qmode == 2)
        hipLaunchKernelGGL((conv_depthwise3x3_slide_kernel<STRIDE, 2, false, RB>), grid, block, 0, st, a, mp);
    else if (qmode == 1)
        hipLaunchKernelGGL((conv_depthwise3x3_slide_kernel<STRIDE, 1, false, RB>), grid, block, 0, st, a, mp);
    else
        hipLaunchKernelGGL((conv_depthwise3x3_slide_kernel<STRIDE, 0, false, RB>), grid, block, 0, st, a, mp);
}

// Output rows per thread.  Longer walks share loaded and transposed rows among more output rows (4 rows: 25 % fewer
// vector instructions per row than 2), but leave the chip fewer, longer threads: measured on the depthwise layers of a
// MobileNetV2 at batch 64, 2 rows are fastest from 7x7 to 112x112 (3, 4, 6 and 8 rows: equal on the largest layers,
// up to 40 % slower on the small ones).
constexpr int kRowsPerThread = 2;

void launch_conv_dw_slide(const ConvArgs &a, hipStream_t st)
{
    if (a.stride_h == 1)
        launch_rb<1, kRowsPerThread>(a, st);
    else
        launch_rb<2, kRowsPerThread>(a, st);
}

} // namespace hipq
