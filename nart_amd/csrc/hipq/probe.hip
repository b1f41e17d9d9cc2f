// Machine probes for gfx950 behind hipq_probe_launch: a few lines of HIP around one loop each, so that the rates the
// kernels of this library are judged against - what the matrix pipes sustain on random bytes, what a CU's load path
// delivers per clock and per instruction width, what a launch costs inside a graph - are measured on the box the
// benchmark runs on instead of quoted.  No counterpart in the reference.  bench.py times them (HIP events around graph
// replays) and reports them as `machine_probes`.
//
// Every probe reads or writes only inside the caller's buffer (at least 64 MiB, 1 KB aligned) and ends by itself: the
// loops have fixed trip counts.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "common.h"
#include "conv_shared.h"
#include "hipq.h"

namespace hipq {

namespace {

constexpr size_t kProbeBytes = 64ull << 20;
constexpr int kWgs = 512; // two work-groups of four waves per CU

// 0 / 1: v_mfma_i32_32x32x32_i8 on four independent accumulators, operands in registers: all-ones bytes / whatever the
// buffer holds (the caller fills it with random bytes: the matrix pipes' sustained rate depends on the data)
template <bool FROM_BUFFER>
__global__ __launch_bounds__(256) void probe_mfma_kernel(const uint8_t *buf, int iters, int *sink)
{
    const int lane = threadIdx.x & 63;
    v4i a[2], b[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        if (FROM_BUFFER) {
            a[i] = *reinterpret_cast<const v4i *>(buf + ((size_t)(blockIdx.x * 4 + i) * 64 + lane) * 16);
            b[i] = *reinterpret_cast<const v4i *>(buf + ((size_t)(blockIdx.x * 4 + 2 + i) * 64 + lane) * 16);
        } else {
            a[i] = v4i{0x01010101, 0x01010101, 0x01010101, 0x01010101};
            b[i] = a[i];
        }
    }
    v16i acc[4] = {};
    for (int it = 0; it < iters; it++) {
        acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[0], b[0], acc[0], 0, 0, 0);
        acc[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[1], b[0], acc[1], 0, 0, 0);
        acc[2] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[0], b[1], acc[2], 0, 0, 0);
        acc[3] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[1], b[1], acc[3], 0, 0, 0);
    }
    int s = 0;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int e = 0; e < 16; e++)
            s ^= acc[i][e];
    if (s == 0x5a5a5a5b)
        sink[0] = s;
}

// 2: nothing (the cost of a launch in a chain of dependent launches)
__global__ void probe_empty_kernel() {}

// 3: the load unit streaming into LDS (global_load_lds_dwordx4), every wave its own 40 KB-strided walk through the first
// `region` bytes of the buffer, three stages of two 1 KB instructions deep
__global__ __launch_bounds__(256) void probe_lds_dma_kernel(const uint8_t *buf, size_t mask, int steps, int *sink)
{
    constexpr int IPS = 2, DEPTH = 3;
    __shared__ __attribute__((aligned(1024))) uint8_t lds[4 * DEPTH * IPS * 1024];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    size_t off = ((size_t)(blockIdx.x * 4 + wave) * 40960) & mask;
    uint8_t *wl = lds + wave * DEPTH * IPS * 1024;
    v4i acc = {0, 0, 0, 0};
    auto issue = [&](int s) {
#pragma unroll
        for (int j = 0; j < IPS; j++)
            __builtin_amdgcn_global_load_lds((gptr_t)(buf + ((off + j * 1024) & mask) + lane * 16),
                                             (lptr_t)(wl + ((s % DEPTH) * IPS + j) * 1024), 16, 0, 0);
        off += IPS * 1024;
    };
    for (int d = 0; d < DEPTH - 1; d++)
        issue(d);
    for (int s = 0; s < steps; s++) {
        issue(s + DEPTH - 1);
        wait_vmcnt<(DEPTH - 1) * IPS>();
        acc ^= *reinterpret_cast<const v4i *>(wl + (s % DEPTH) * IPS * 1024 + lane * 16);
    }
    wait_vmcnt<0>();
    if (acc[0] == 0x12345678 && acc[1] == 0x09abcdef)
        sink[0] = acc[2] ^ acc[3];
}

// 4 .. 9: one vector-memory instruction shape in a loop, each wave on 4 KB of its own (resident in the CU's L1):
// MODE 0 32-bit loads, 64 lanes on 256 contiguous bytes; 1 32-bit loads, eight pieces of 32 bytes in eight lines;
// 2 128-bit loads, 1 KB contiguous; 3 32-bit stores contiguous; 4 32-bit stores in eight pieces; 5 128-bit stores
template <int MODE>
__global__ __launch_bounds__(256) void probe_vmem_kernel(uint8_t *buf, int iters, size_t span_mask, int *sink)
{
    constexpr size_t SPAN = 4096; // span_mask = SPAN - 1, passed at run time: with a constant the compiler sees that the
                                  // addresses repeat and hoists the loads out of the loop
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint8_t *base = buf + ((size_t)blockIdx.x * 4 + wave) * SPAN;
    constexpr bool PIECES = MODE == 1 || MODE == 4, WIDE = MODE == 2 || MODE == 5;
    const size_t lo = PIECES ? (size_t)(lane >> 3) * 128 + (lane & 7) * 4 : WIDE ? (size_t)lane * 16 : (size_t)lane * 4;
    constexpr int STEP = PIECES ? 32 : WIDE ? 1024 : 256;
    int acc = 0;
    size_t off = 0;
    for (int i = 0; i < iters; i++) {
#pragma unroll
        for (int u = 0; u < 8; u++) {
            uint8_t *p = base + ((off + lo) & span_mask);
            if (MODE == 0 || MODE == 1) {
                acc ^= *reinterpret_cast<const int *>(p);
            } else if (MODE == 2) {
                const v4i v = *reinterpret_cast<const v4i *>(p);
                acc ^= v[0] ^ v[1] ^ v[2] ^ v[3];
            } else if (MODE == 3 || MODE == 4) {
                *reinterpret_cast<int *>(p) = i + u;
            } else {
                *reinterpret_cast<v4i *>(p) = v4i{i, u, i, u};
            }
            off += STEP;
            if (PIECES && (u & 3) == 3)
                off += 1024 - 128;
        }
    }
    if (acc == 0x12345679)
        sink[0] = acc;
}

} // namespace

} // namespace hipq

using namespace hipq;

// which: 0 MFMA on constant operands, 1 MFMA on the buffer's bytes (units: integer operations);
// 2 an empty kernel (units: 0); 3 load-unit streaming of the first `param` bytes (a power of two; units: bytes);
// 4 .. 9 the vector-memory instruction shapes of probe_vmem_kernel (units: wave instructions per CU).
extern "C" int hipq_probe_launch(int which, void *buf, size_t bytes, int iters, size_t param, double *units, void *stream)
{
    clear_error();
    HIPQ_REQUIRE(which >= 0 && which <= 9, "hipq_probe_launch: probes are numbered 0 to 9");
    HIPQ_REQUIRE(buf && bytes >= kProbeBytes && (reinterpret_cast<uintptr_t>(buf) & 1023) == 0 && iters > 0 && iters <= (1 << 20),
                 "hipq_probe_launch: needs a 1 KB aligned buffer of at least 64 MiB and 1 to 2^20 iterations");
    hipStream_t st = static_cast<hipStream_t>(stream);
    uint8_t *b = static_cast<uint8_t *>(buf);
    int *sink = reinterpret_cast<int *>(b + kProbeBytes - 64);
    double u = 0;
    switch (which) {
    case 0:
        hipLaunchKernelGGL(probe_mfma_kernel<false>, dim3(kWgs), dim3(256), 0, st, b, iters, sink);
        u = (double)kWgs * 4 * iters * 4 * 65536.0;
        break;
    case 1:
        hipLaunchKernelGGL(probe_mfma_kernel<true>, dim3(kWgs), dim3(256), 0, st, b, iters, sink);
        u = (double)kWgs * 4 * iters * 4 * 65536.0;
        break;
    case 2:
        hipLaunchKernelGGL(probe_empty_kernel, dim3(1), dim3(64), 0, st);
        break;
    case 3:
        HIPQ_REQUIRE(param >= (1u << 16) && param <= kProbeBytes / 2 && (param & (param - 1)) == 0,
                     "hipq_probe_launch: the streamed region must be a power of two between 64 KiB and 32 MiB");
        hipLaunchKernelGGL(probe_lds_dma_kernel, dim3(kWgs), dim3(256), 0, st, b, param - 1, iters, sink);
        u = (double)kWgs * 4 * iters * 2 * 1024.0;
        break;
    default: {
        const int mode = which - 4;
        uint8_t *area = b + (kProbeBytes / 2); // stores stay clear of the bytes probe 1 multiplies
#define HIPQ_VMEM(M) hipLaunchKernelGGL(probe_vmem_kernel<M>, dim3(kWgs), dim3(256), 0, st, area, iters, (size_t)4095, sink)
        if (mode == 0)
            HIPQ_VMEM(0);
        else if (mode == 1)
            HIPQ_VMEM(1);
        else if (mode == 2)
            HIPQ_VMEM(2);
        else if (mode == 3)
            HIPQ_VMEM(3);
        else if (mode == 4)
            HIPQ_VMEM(4);
        else
            HIPQ_VMEM(5);
#undef HIPQ_VMEM
        u = 2.0 * 4 * iters * 8; // per CU: two work-groups of four waves, eight instructions per iteration
        break;
    }
    }
    if (units)
        *units = u;
    return launch_status("hipq_probe_launch");
}
