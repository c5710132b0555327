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

// ---- what a grid-wide hand-over costs ---------------------------------------------------------------------------------
// A chain of dependent GEMVs in ONE launch would have persistent workgroups produce a stage's output vector, make it
// visible to the whole chip and consume it in the next stage.  This probe measures that hand-over by itself: every
// workgroup writes its slice of an n-entry vector (agent-scope stores that go through to memory), then either
//   mode 0  arrives at a barrier -- a counter per XCD in the XCD's own L2, the last arriver of an XCD adds to one
//           agent-scope counter, everybody polls that one -- and reads the whole vector with plain 16-byte loads from
//           addresses nobody has read before (a fresh buffer every round), or
//   mode 1  has no barrier: every 32-bit entry carries the round number in its upper half and the consumers poll the
//           data itself with agent-scope 8-byte loads until every entry is of this round, or
//   mode 2  the barrier of mode 0 alone (nothing written or read).
// Every wait is bounded by `spin_limit` polls: a workgroup that gives up writes the round to *status and all of its
// threads leave; the others then give up in turn.  `check` counts entries that arrived with a wrong value.
namespace {
template <int MODE>
__global__ __launch_bounds__(512) void handover_probe_kernel(int rounds, uint32_t* ctr, uint32_t* xcd_ctr, uint32_t* data,
                                                            int n_data, int* status, int spin_limit, uint32_t* check) {
    const int nwg = gridDim.x, wg = blockIdx.x, tid = threadIdx.x;
    uint32_t bad = 0;
    __shared__ int ok_s;
    const int per = (n_data + nwg - 1) / nwg;
    for (int r = 1; r <= rounds; r++) {
        uint32_t* buf = data + (size_t)r * n_data;  // a fresh buffer every round
        if (MODE != 2) {
            for (int i = tid; i < per; i += 512) {
                const int idx = wg * per + i;
                if (idx < n_data) {
                    const uint32_t val = (MODE == 1) ? (((uint32_t)r << 16) | (uint32_t)((idx * 7 + r) & 0xffff)) : (uint32_t)(r * 1000003 + idx);
                    __hip_atomic_store(&buf[idx], val, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
        }
        if (MODE == 0 || MODE == 2) {
            __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0): this wave's stores have been acknowledged
            __syncthreads();
            if (tid == 0) {
                const int xcd = wg & 7, per_xcd = nwg >> 3;
                const uint32_t old = __hip_atomic_fetch_add(&xcd_ctr[xcd * 32], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                if (old == (uint32_t)(r * per_xcd - 1)) __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                int spins = 0;
                while (__hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < (uint32_t)(r * 8) && ++spins < spin_limit) {}
                ok_s = spins < spin_limit;
            }
            __syncthreads();
            if (!ok_s) {
                if (tid == 0) atomicExch(status, r);
                return;
            }
            if (MODE == 0) {
                const uint4* b4 = (const uint4*)buf;
                for (int i = tid; i < n_data / 4; i += 512) {
                    const uint4 v = b4[i];
                    bad += v.x != (uint32_t)(r * 1000003 + 4 * i) || v.w != (uint32_t)(r * 1000003 + 4 * i + 3);
                }
            }
        } else {
            int spins = 0;
            const unsigned long long* b8 = (const unsigned long long*)buf;
            for (int i = tid; i < n_data / 2; i += 512) {
                unsigned long long v;
                do {
                    v = __hip_atomic_load(&b8[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                } while (((uint32_t)(v >> 48) != (uint32_t)r || (((uint32_t)v) >> 16) != (uint32_t)r) && ++spins < spin_limit);
                bad += ((uint32_t)v & 0xffff) != (uint32_t)((2 * i * 7 + r) & 0xffff);
            }
            if (spins >= spin_limit) atomicExch(status, r);
            if (__syncthreads_or(spins >= spin_limit)) return;
        }
    }
    if (bad) atomicAdd(check, bad);
}
}  // namespace

// One launch of `rounds` hand-overs by `workgroups` (a multiple of 8, at most two per compute unit: all of them must be
// resident) persistent workgroups of 512 threads.  ctr: 1 dword, xcd_ctr: 256 dwords, status / check: 1 dword each, all
// zeroed by the caller before every launch; data: (rounds + 1) * n_data dwords, zeroed likewise (n_data a multiple of
// 4).  Returns 0 / -1.
extern "C" int bench_probe_grid_handover(int mode, int workgroups, int rounds, int n_data, void* ctr, void* xcd_ctr, void* data,
                                         void* status, void* check, int spin_limit, void* stream) {
    if (mode < 0 || mode > 2 || workgroups <= 0 || workgroups % 8 != 0 || workgroups > 512 || rounds <= 0 || n_data <= 0 ||
        n_data % 4 != 0 || spin_limit <= 0 || !ctr || !xcd_ctr || !data || !status || !check)
        return -1;
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid((unsigned)workgroups), block(512);
    if (mode == 0)
        hipLaunchKernelGGL(handover_probe_kernel<0>, grid, block, 0, st, rounds, (uint32_t*)ctr, (uint32_t*)xcd_ctr, (uint32_t*)data,
                           n_data, (int*)status, spin_limit, (uint32_t*)check);
    else if (mode == 1)
        hipLaunchKernelGGL(handover_probe_kernel<1>, grid, block, 0, st, rounds, (uint32_t*)ctr, (uint32_t*)xcd_ctr, (uint32_t*)data,
                           n_data, (int*)status, spin_limit, (uint32_t*)check);
    else
        hipLaunchKernelGGL(handover_probe_kernel<2>, grid, block, 0, st, rounds, (uint32_t*)ctr, (uint32_t*)xcd_ctr, (uint32_t*)data,
                           n_data, (int*)status, spin_limit, (uint32_t*)check);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}
