// Measurement aids of bench.py (built into bench_mfma_probe.so, not part of libbittorch_hip.so or its ABI):
// the int8 MFMA rate the chip sustains when nothing else is in the way, and (at the end of the file) the rate at which
// the memory system feeds a pure reader.
// Every wave issues back-to-back v_mfma_i32_16x16x64_i8 on eight independent accumulators
// held in registers; no memory traffic inside the loop.  The prefill GEMM's TOPS are
// reported against this figure as well as against the nominal peak.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef int v4i __attribute__((ext_vector_type(4)));

namespace {

__global__ __launch_bounds__(512) void mfma_i8_probe_kernel(int iters, int random_operands, int* __restrict__ out) {
    const int lane = threadIdx.x & 63;
    v4i a = {lane, lane + 1, lane + 2, lane + 3};
    v4i b = {lane ^ 5, lane ^ 9, lane ^ 17, lane ^ 33};
    if (random_operands) {
        // full-range pseudo-random bytes (switching activity of real operands): A like
        // quantized activations, B ternary {-1, 0, +1}
        uint32_t h = (uint32_t)(blockIdx.x * 512 + threadIdx.x) * 2654435761u + 12345u;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            h = h * 1664525u + 1013904223u;
            a[i] = (int)h;
            h = h * 1664525u + 1013904223u;
            uint32_t w = 0;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const uint32_t c = (h >> (8 * e + 3)) % 3u;  // 0, 1, 2 -> 0, +1, -1
                w |= (c == 0 ? 0x00u : c == 1 ? 0x01u : 0xFFu) << (8 * e);
            }
            b[i] = (int)w;
        }
    }
    v4i acc[8];
#pragma unroll
    for (int t = 0; t < 8; t++) acc[t] = v4i{t, 0, 0, 0};
    for (int i = 0; i < iters; i++) {
#pragma unroll
        for (int t = 0; t < 8; t++) acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc[t], 0, 0, 0);
    }
    int s = 0;
#pragma unroll
    for (int t = 0; t < 8; t++) s += acc[t][0] + acc[t][1] + acc[t][2] + acc[t][3];
    if (s == 0x7fffffff) out[0] = s;  // keeps the loop alive; practically never true
}

// Same measurement with the register footprint of the prefill GEMM's inner product: a
// 128 x 64 accumulator tile per wave (32 accumulators = 128 VGPRs), four A and four B operand
// fragments per 32 MFMAs.
// out[2], out[3]: shader-clock cycles and 100 MHz real-time ticks workgroup 0 spent in the loop (the ratio is the clock
// the chip sustains under this load).
__global__ __launch_bounds__(512) void mfma_i8_probe_tile_kernel(int iters, int* __restrict__ out) {
    const int lane = threadIdx.x & 63;
    v4i a[8], b[4], acc[8][4];
    uint32_t h = (uint32_t)(blockIdx.x * 512 + threadIdx.x) * 2654435761u + 12345u;
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int e = 0; e < 4; e++) { h = h * 1664525u + 1013904223u; a[i][e] = (int)h; }
#pragma unroll
    for (int t = 0; t < 4; t++)
#pragma unroll
        for (int e = 0; e < 4; e++) { h = h * 1664525u + 1013904223u; b[t][e] = (int)(h & 0x01010101u); }
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int t = 0; t < 4; t++) acc[i][t] = v4i{lane, i, t, 0};
    const unsigned long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
    for (int it = 0; it < iters; it += 4) {
#pragma unroll
        for (int i = 0; i < 8; i++)
#pragma unroll
            for (int t = 0; t < 4; t++) acc[i][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[i], b[t], acc[i][t], 0, 0, 0);
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        out[2] = (int)(__builtin_readcyclecounter() - c0);
        out[3] = (int)(__builtin_amdgcn_s_memrealtime() - r0);
    }
    int s = 0;
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int t = 0; t < 4; t++) s += acc[i][t][0] + acc[i][t][1] + acc[i][t][2] + acc[i][t][3];
    if (s == 0x7fffffff) out[0] = s;
}

}  // namespace

// Launches `blocks` workgroups of 8 waves that each issue `iters` x 8 back-to-back v_mfma_i32_16x16x64_i8 on register
// operands and writes the operation count of the launch (2*16*16*64 per instruction) to *ops_per_launch.
// random_operands = 0: small constant operands; 1: pseudo-random int8 activations and ternary weights; 2: the prefill
// GEMM's register footprint (32 accumulators per wave).  `out` is a device int the kernel may write.  Returns 0 / -1.
extern "C" int bench_probe_mfma_i8(int blocks, int iters, int random_operands, int* out, double* ops_per_launch,
                                void* stream) {
    if (blocks <= 0 || iters <= 0 || !out) return -1;
    if (random_operands == 2)  // 32 accumulators per wave; iters is rounded up to a multiple of 4
        hipLaunchKernelGGL(mfma_i8_probe_tile_kernel, dim3((unsigned)blocks), dim3(512), 0, (hipStream_t)stream,
                           iters, out);
    else
        hipLaunchKernelGGL(mfma_i8_probe_kernel, dim3((unsigned)blocks), dim3(512), 0, (hipStream_t)stream, iters,
                           random_operands, out);
    // 8 waves per block, 8 MFMAs per iteration, 2*16*16*64 operations each
    if (ops_per_launch) *ops_per_launch = (double)blocks * 8.0 * (double)iters * 8.0 * 32768.0;
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

// ---- what the memory system delivers to a pure reader ----------------------------------------------------------------
// A read-only kernel over `bytes` of device memory, xor-reduced so that the loads stay alive; three address patterns:
//   0  grid-stride 16-byte loads over the whole buffer (the textbook streaming loop);
//   1  every workgroup reads its own contiguous share front to back, a wave 2 KiB (8 loads of 4 bytes per lane) at a time;
//   2  the same with the non-temporal hint on the loads.
// The grouped GEMV walks its weights in pattern 2; its GB/s are reported against this figure as well as against the
// nominal 8 TB/s.
namespace {
__global__ __launch_bounds__(256) void read_probe_grid(const uint4* __restrict__ p, size_t n, int* out) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 256;
    uint32_t a = 0;
    for (; i + 7 * stride < n; i += 8 * stride) {
        uint4 v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = p[i + u * stride];
#pragma unroll
        for (int u = 0; u < 8; u++) a ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    if (a == 0x12345678u) out[1] = (int)a;
}
template <bool NT>
__global__ __launch_bounds__(512) void read_probe_chunk(const uint32_t* __restrict__ p, size_t ndw, int* out) {
    const size_t per_wg = ndw / gridDim.x;  // dwords
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t* base = p + (size_t)blockIdx.x * per_wg;
    uint32_t a = 0;
    constexpr int U = 8, BLK = U * 64;  // dwords per wave block
    for (size_t blk = wave; (blk + 1) * BLK <= per_wg; blk += 8) {
        uint32_t v[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const uint32_t* q = base + blk * BLK + (size_t)u * 64 + lane;
            v[u] = NT ? __builtin_nontemporal_load(q) : *q;
        }
#pragma unroll
        for (int u = 0; u < U; u++) a ^= v[u];
    }
    if (a == 0x12345678u) out[1] = (int)a;
}
}  // namespace

// One launch of the read probe over `bytes` (a multiple of 1 MiB) at `buf`; pattern as above.  Returns 0 / -1.
extern "C" int bench_probe_hbm_read(const void* buf, size_t bytes, int pattern, int* out, void* stream) {
    if (!buf || !out || bytes < (1u << 20) || bytes % (1u << 20) != 0) return -1;
    hipStream_t st = (hipStream_t)stream;
    if (pattern == 0) hipLaunchKernelGGL(read_probe_grid, dim3(4096), dim3(256), 0, st, (const uint4*)buf, bytes / 16, out);
    else if (pattern == 1) hipLaunchKernelGGL(read_probe_chunk<false>, dim3(512), dim3(512), 0, st, (const uint32_t*)buf, bytes / 4, out);
    else hipLaunchKernelGGL(read_probe_chunk<true>, dim3(512), dim3(512), 0, st, (const uint32_t*)buf, bytes / 4, out);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}
