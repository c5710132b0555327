// Fused ternary quantize + 2-bit pack for gfx950 (HBM-bound, one pass over W).
//
// Arithmetic restated from the reference quantizer and codec
// (bittorch/quant/ternary.py:122-142, bittorch/quant/ternary_packed.py:50-73,
// :202-206): scale = row (or tensor) absmax floored at 1e-8, threshold =
// fl(tf * scale) in the weight dtype, code = |w| > thr ? (w > 0 ? 1 : 2) : 0,
// byte[kb, n] = c0 | c1<<2 | c2<<4 | c3<<6 for k = 4kb..4kb+3.
//
// Two kernels share that arithmetic:
//   * quantize_pack_fast_kernel: K a multiple of 256, N a multiple of the row tile,
//     aligned pointers.  A wave keeps one whole row in registers (K/64 values per
//     lane), reduces its absmax across the 64 lanes, encodes, and hands the row's
//     bytes to LDS; a workgroup owns R = WAVES*RPW consecutive rows, so the
//     transposed store writes R contiguous bytes per packed_T row.  One read of W.
//   * quantize_pack_generic_kernel: any shape, alignment and dtype, optional dense
//     ternary output; reads every row twice (absmax pass, encode pass) and walks K
//     in segments so that the LDS tile is bounded.
#include <cstdlib>

#include "bt_common.h"

namespace bt {

// Workgroup b of a grid of 8*per_xcd workgroups -> tile index such that
// consecutive tiles run on the same XCD (workgroups are dealt round-robin over
// the 8 XCDs), so the pieces of one packed_T cache line that neighbouring tiles
// write meet in one L2.
__device__ __forceinline__ int64_t xcd_tile(int64_t b, int64_t per_xcd) {
    return (b & 7) * per_xcd + (b >> 3);
}

__device__ __forceinline__ uint32_t encode4(const float (&v)[4], float thr, uint32_t& tern4) {
    uint32_t byte = 0;
    tern4 = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const bool keep = fabsf(v[i]) > thr;
        const bool neg = v[i] < 0.0f;
        const uint32_t code = keep ? (neg ? 2u : 1u) : 0u;
        byte |= code << (2 * i);
        tern4 |= (keep ? (neg ? 0xFFu : 0x01u) : 0u) << (8 * i);
    }
    return byte;
}

// ---- fast kernel ---------------------------------------------------------------------
// ITERS float4 groups per lane, WAVES waves, RPW rows per wave one after another; SPLIT waves share a row (wave w
// holds 256-element chunks ITERS * (w % SPLIT) .. + ITERS - 1 of row slot w / SPLIT, ITERS * SPLIT >= K / 256): a long
// row in one wave's registers leaves room for four waves per compute unit, whose encode then runs one wave per SIMD
// with nothing to overlap it (4096 x 11008 fp32: 45.4 us, of which 9.4 us encode; split over four waves: see below).
// LDS tile: byte (kb, row) at kb*PITCHB + row, PITCHB = R + 4: the odd dword pitch keeps the
// column writes (lanes = consecutive kb) and the row reads free of bank conflicts.
template <int DT, int ITERS, int WAVES, int RPW, int SPLIT = 1>
__global__ __launch_bounds__(WAVES * 64) void quantize_pack_fast_kernel(
    const void* __restrict__ W, int N, int K, float tf, float clamp_min, int per_channel,
    uint8_t* __restrict__ packed_T, float* __restrict__ scale, int tiles, int per_xcd) {
    constexpr int SLOTS = WAVES / SPLIT;  // rows in flight
    constexpr int R = SLOTS * RPW;
    constexpr int PITCHB = R + 4;
    static_assert(WAVES % SPLIT == 0, "whole row slots");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_b[];
    __shared__ float part_max[RPW][WAVES];
    const int tile = (int)xcd_tile(blockIdx.x, per_xcd);
    if (tile >= tiles) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int slot = wave / SPLIT, part = wave % SPLIT;
    const int n0 = tile * R;
    const int nfull = (K >> 8) - part * ITERS;  // complete 256-element chunks of this wave's share (uniform)
    const int Kb = K >> 2;
    const float tensor_scale = per_channel ? 0.0f : fmaxf(scale[0], clamp_min);
    // The tensor scale arrives unfloored; one thread stores the floored value.  Workgroups that read it afterwards
    // floor it again, which changes nothing.
    if (!per_channel && tile == 0 && threadIdx.x == 0) scale[0] = tensor_scale;
    uint32_t pk[ITERS];
#pragma unroll
    for (int j = 0; j < ITERS; j++) pk[j] = 0;
    // the row's scale from its absolute maximum (this lane's share of it), stored once, and the threshold that goes with it
    auto row_threshold = [&](int r, int n, float amax) __attribute__((always_inline)) -> float {
        float s;
        if (per_channel) {
            amax = wave_max(amax);
            if constexpr (SPLIT > 1) {  // the row's other waves (per_channel is uniform: every wave meets the barrier)
                if (lane == 0) part_max[r][wave] = amax;
                __syncthreads();
#pragma unroll
                for (int q = 0; q < SPLIT; q++) amax = fmaxf(amax, part_max[r][slot * SPLIT + q]);
            }
            s = fmaxf(amax, clamp_min);
            if (lane == 0 && part == 0) scale[n] = s;
        } else {
            s = tensor_scale;
        }
        return round_to_dtype(__fmul_rn(tf, s), DT);
    };
#pragma unroll 1  // one row in registers at a time
    for (int r = 0; r < RPW; r++) {
        const int n = n0 + RPW * slot + r;
        float4 v[ITERS];
        if constexpr (DT == BT_F32) {
            const float4* rowp = (const float4*)((const float*)W + (int64_t)n * K) + part * ITERS * 64 + lane;
#pragma unroll
            for (int j = 0; j < ITERS; j++) {
                if (j < nfull) {
                    const uint4 t = ldw4_nt(rowp + j * 64);
                    v[j] = make_float4(__builtin_bit_cast(float, t.x), __builtin_bit_cast(float, t.y),
                                       __builtin_bit_cast(float, t.z), __builtin_bit_cast(float, t.w));
                } else {
                    v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
                }
            }
        } else {
            const uint2* rowp = (const uint2*)((const uint16_t*)W + (int64_t)n * K) + part * ITERS * 64 + lane;
#pragma unroll
            for (int j = 0; j < ITERS; j++) {
                const uint2 t = (j < nfull) ? ldw2_nt(rowp + j * 64) : make_uint2(0u, 0u);
                if constexpr (DT == BT_F16)
                    v[j] = make_float4(f16_bits_to_f32((uint16_t)t.x), f16_bits_to_f32((uint16_t)(t.x >> 16)),
                                       f16_bits_to_f32((uint16_t)t.y), f16_bits_to_f32((uint16_t)(t.y >> 16)));
                else
                    v[j] = make_float4(bf16_bits_to_f32((uint16_t)t.x), bf16_bits_to_f32((uint16_t)(t.x >> 16)),
                                       bf16_bits_to_f32((uint16_t)t.y), bf16_bits_to_f32((uint16_t)(t.y >> 16)));
            }
        }
        float amax = 0.0f;
#pragma unroll
        for (int j = 0; j < ITERS; j++)
            amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v[j].x), fabsf(v[j].y)), fmaxf(fabsf(v[j].z), fabsf(v[j].w))));
        const float thr = row_threshold(r, n, amax);
#pragma unroll
        for (int j = 0; j < ITERS; j++) {
            const float a[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
            uint32_t t4;
            pk[j] |= encode4(a, thr, t4) << (8 * r);
        }
    }
#pragma unroll
    for (int j = 0; j < ITERS; j++) {
        if (j < nfull) {
            uint8_t* dst = lds_b + ((part * ITERS + j) * 64 + lane) * PITCHB + slot * RPW;
            if constexpr (RPW == 4) *(uint32_t*)dst = pk[j];
            else if constexpr (RPW == 2) *(uint16_t*)dst = (uint16_t)pk[j];
            else *dst = (uint8_t)pk[j];
        }
    }
    __syncthreads();
    constexpr int Q = R / 16;  // 16-byte pieces per packed_T row segment
    for (int idx = threadIdx.x; idx < Kb * Q; idx += WAVES * 64) {
        const int kb = idx / Q, q = idx % Q;
        const uint32_t* src = (const uint32_t*)(lds_b + kb * PITCHB + 16 * q);
        *(uint4*)(packed_T + (int64_t)kb * N + n0 + 16 * q) = make_uint4(src[0], src[1], src[2], src[3]);
    }
}

template <int DT, int ITERS, int WAVES, int RPW, int SPLIT = 1>
static int launch_fast_cfg(const void* W, int64_t N, int64_t K, float tf, float clamp_min, int per_channel,
                           uint8_t* packed_T, float* scale, hipStream_t st) {
    constexpr int R = (WAVES / SPLIT) * RPW;
    const int tiles = (int)(N / R);
    const int per_xcd = (int)ceil_div(tiles, 8);
    const size_t lds = (size_t)(K / 4) * (R + 4);
    auto kern = quantize_pack_fast_kernel<DT, ITERS, WAVES, RPW, SPLIT>;
    if (lds > 64 * 1024 &&
        hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
        set_error("bt_quantize_pack: cannot reserve %zu bytes of LDS", lds);
        return BT_ERR_LAUNCH;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)(per_xcd * 8)), dim3(WAVES * 64), lds, st, W, (int)N, (int)K, tf,
                       clamp_min, per_channel, packed_T, scale, tiles, per_xcd);
    return check_launch("bt_quantize_pack");
}

// Row tile for the fast kernel: as many rows per wave (bytes per packed_T segment) as still
// leave more than one tile per CU; at least 16 rows per workgroup (one 16-byte piece).
template <int DT, int ITERS, int WAVES>
static int launch_fast_rows(const void* W, int64_t N, int64_t K, float tf, float clamp_min, int per_channel,
                            uint8_t* packed_T, float* scale, hipStream_t st, int* rc) {
    constexpr int MIN_RPW = (WAVES >= 16) ? 1 : (WAVES >= 8) ? 2 : 4;
    int rpw = 0;
    if (const char* env = tuning_env("BITTORCH_QP_RPW")) rpw = atoi(env);
    if (rpw != 1 && rpw != 2 && rpw != 4) {
        // (workgroups of 8 waves run two to a compute unit: at least 640 of them, so that both places stay filled)
        const int64_t min_tiles = (WAVES == 8 && ITERS <= 16) ? 640 : 320;
        rpw = 4;
        while (rpw > MIN_RPW && (N % (WAVES * rpw) != 0 || N / (WAVES * rpw) < min_tiles)) rpw >>= 1;
    }
    if (rpw < MIN_RPW) rpw = MIN_RPW;
    if (N % (WAVES * rpw) != 0 || (size_t)(K / 4) * (WAVES * rpw + 4) > 150 * 1024) return 0;
    if (rpw == 4) {
        *rc = launch_fast_cfg<DT, ITERS, WAVES, 4>(W, N, K, tf, clamp_min, per_channel, packed_T, scale, st);
    } else if (rpw == 2) {
        if constexpr (MIN_RPW <= 2)
            *rc = launch_fast_cfg<DT, ITERS, WAVES, 2>(W, N, K, tf, clamp_min, per_channel, packed_T, scale, st);
    } else {
        if constexpr (MIN_RPW <= 1)
            *rc = launch_fast_cfg<DT, ITERS, WAVES, 1>(W, N, K, tf, clamp_min, per_channel, packed_T, scale, st);
    }
    return 1;
}

// returns 1 if the fast kernel took the call (rc holds its status), 0 if the shape does not
// qualify.  Register budget: a row of K elements costs K/64 data registers per lane, so 16 waves
// per workgroup fit K <= 4096 with a row per wave, K <= 8192 with a row over two waves and K <= 16384 over four.
template <int DT>
static int try_launch_fast(const void* W, int64_t N, int64_t K, float tf, float clamp_min, int per_channel,
                           uint8_t* packed_T, float* scale, int8_t* w_tern, hipStream_t st, int* rc) {
    if (!packed_T || w_tern || K % 256 != 0 || ((uintptr_t)W) % 16 != 0 || ((uintptr_t)packed_T) % 16 != 0 ||
        N * K >= (1ll << 31) || tuning_env("BITTORCH_QP_GENERIC"))
        return 0;
    const int chunks = (int)(K / 256);
#define BT_QF(IT, WV) \
    if (chunks <= IT) return launch_fast_rows<DT, IT, WV>(W, N, K, tf, clamp_min, per_channel, packed_T, scale, st, rc)
    BT_QF(4, 16);
    BT_QF(8, 16);
    // 2048 < K <= 4096 and many rows: workgroups of 8 waves (16 rows), two per compute unit, so that one loads while the
    // other encodes and stores, and the last round is cut finer (11008 x 4096: 34.9 against 40.0 us; 4096 x 4096, one
    // workgroup per compute unit either way, stays on 16 waves: 15.4 against 16.4 us)
    if (chunks > 8 && chunks <= 16 && N >= 6144 && N % 16 == 0)
        return launch_fast_rows<DT, 16, 8>(W, N, K, tf, clamp_min, per_channel, packed_T, scale, st, rc);
    BT_QF(16, 16);
#undef BT_QF
    // Longer rows are split over two or four waves of a 16-wave workgroup (16 rows per tile either way)
    if (N % 16 != 0 || (size_t)(K / 4) * 20 > 150 * 1024) return 0;
    const bool two = chunks <= 32 && !tuning_env("BITTORCH_QP_SPLIT4");
    const int per_wave = (int)ceil_div(chunks, two ? 2 : 4);
#define BT_QS(IT, SP, RP) \
    if (per_wave <= IT) { \
        *rc = launch_fast_cfg<DT, IT, 16, RP, SP>(W, N, K, tf, clamp_min, per_channel, packed_T, scale, st); \
        return 1; \
    }
    if (two) {
        BT_QS(10, 2, 2) BT_QS(12, 2, 2) BT_QS(14, 2, 2) BT_QS(16, 2, 2)
    } else {
        BT_QS(6, 4, 4) BT_QS(8, 4, 4) BT_QS(10, 4, 4) BT_QS(11, 4, 4) BT_QS(12, 4, 4) BT_QS(14, 4, 4) BT_QS(16, 4, 4)
    }
#undef BT_QS
    return 0;
}

// ---- generic kernel --------------------------------------------------------------------
template <int DT>
__device__ __forceinline__ void load4(const void* W, int64_t elem, int64_t row_end, bool vec_ok, float (&v)[4]) {
    // four consecutive elements starting at `elem`; zero past row_end
    if (vec_ok && elem + 4 <= row_end) {
        if constexpr (DT == BT_F32) {
            const float4 t = *(const float4*)((const float*)W + elem);
            v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
        } else if constexpr (DT == BT_I8) {
            const uint32_t t = *(const uint32_t*)((const int8_t*)W + elem);
#pragma unroll
            for (int i = 0; i < 4; i++) v[i] = (float)(int8_t)(t >> (8 * i));
        } else {
            const uint2 t = *(const uint2*)((const uint16_t*)W + elem);
            const uint16_t h[4] = {(uint16_t)(t.x & 0xffff), (uint16_t)(t.x >> 16),
                                   (uint16_t)(t.y & 0xffff), (uint16_t)(t.y >> 16)};
#pragma unroll
            for (int i = 0; i < 4; i++) v[i] = (DT == BT_F16) ? f16_bits_to_f32(h[i]) : bf16_bits_to_f32(h[i]);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++) v[i] = (elem + i < row_end) ? load_elem<DT>(W, elem + i) : 0.0f;
    }
}

// 256 threads own 16 rows (wave w rows n0+4w .. +3).  Pass 1: the four row scales.
// Pass 2, per segment of up to G_SEG packed rows: encode, put the four rows' bytes into one
// dword per kb in LDS (pitch 5 dwords), then 16-byte transposed stores.
constexpr int G_SEG = 2048;
template <int DT>
__global__ __launch_bounds__(256) void quantize_pack_generic_kernel(
    const void* __restrict__ W, int64_t N, int64_t K, int64_t Kb, float tf, float clamp_min, int per_channel,
    uint8_t* __restrict__ packed_T, float* __restrict__ scale, int8_t* __restrict__ w_tern, int64_t tiles,
    int64_t per_xcd, float fixed_thr) {
    // fixed_thr >= 0: no scale at all, the threshold is given (packing of already ternary weights)
    constexpr int PITCH = 5;
    __shared__ uint32_t lds[G_SEG * PITCH];
    const int64_t tile = xcd_tile(blockIdx.x, per_xcd);
    if (tile >= tiles) return;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t n0 = tile * 16;
    const bool vec_ok = (K % 4 == 0) && (((uintptr_t)W) % 16 == 0);
    const bool tern_vec = vec_ok && (((uintptr_t)w_tern) % 4 == 0);
    const float tensor_scale = (per_channel || fixed_thr >= 0.0f) ? 0.0f : fmaxf(scale[0], clamp_min);
    // (the floored value goes back; readers that come later floor it again, which changes nothing)
    if (!per_channel && fixed_thr < 0.0f && tile == 0 && threadIdx.x == 0) scale[0] = tensor_scale;

    float thr[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int64_t n = n0 + 4 * wave + r;
        float s = tensor_scale;
        if (per_channel && n < N) {  // uniform per wave
            const int64_t row0 = n * K;
            float amax = 0.0f;
            for (int64_t kb = lane; kb < Kb; kb += 64) {
                float v[4];
                load4<DT>(W, row0 + 4 * kb, row0 + K, vec_ok, v);
                amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))));
            }
            s = fmaxf(wave_max(amax), clamp_min);
            if (lane == 0) scale[n] = s;
        }
        thr[r] = (fixed_thr >= 0.0f) ? fixed_thr : round_to_dtype(__fmul_rn(tf, s), DT);
    }

    const bool full = (n0 + 16 <= N) && (N % 16 == 0) && (((uintptr_t)packed_T) % 16 == 0);
    for (int64_t seg0 = 0; seg0 < Kb; seg0 += G_SEG) {
        const int seg_len = (int)((Kb - seg0 < G_SEG) ? (Kb - seg0) : G_SEG);
        for (int kl = lane; kl < seg_len; kl += 64) {
            const int64_t kb = seg0 + kl;
            uint32_t word = 0;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int64_t n = n0 + 4 * wave + r;
                if (n < N) {
                    const int64_t row0 = n * K, row_end = row0 + K;
                    float v[4];
                    load4<DT>(W, row0 + 4 * kb, row_end, vec_ok, v);
                    uint32_t tern4;
                    word |= encode4(v, thr[r], tern4) << (8 * r);
                    if (w_tern) {
                        const int64_t e = row0 + 4 * kb;
                        if (tern_vec && e + 4 <= row_end) {
                            *(uint32_t*)(w_tern + e) = tern4;
                        } else {
                            for (int i = 0; i < 4; i++)
                                if (e + i < row_end) w_tern[e + i] = (int8_t)((tern4 >> (8 * i)) & 0xff);
                        }
                    }
                }
            }
            if (packed_T) lds[kl * PITCH + wave] = word;
        }
        if (!packed_T) continue;  // uniform
        __syncthreads();
        for (int kl = threadIdx.x; kl < seg_len; kl += 256) {
            const uint32_t d[4] = {lds[kl * PITCH], lds[kl * PITCH + 1], lds[kl * PITCH + 2], lds[kl * PITCH + 3]};
            uint8_t* dst = packed_T + (seg0 + kl) * N + n0;
            if (full) {
                *(uint4*)dst = make_uint4(d[0], d[1], d[2], d[3]);
            } else {
                for (int i = 0; i < 16; i++)
                    if (n0 + i < N) dst[i] = (uint8_t)((d[i >> 2] >> (8 * (i & 3))) & 0xff);
            }
        }
        __syncthreads();
    }
}

// tensor absmax into scale[0] (the bit pattern of a non-negative float orders like a uint)
template <int DT>
__global__ __launch_bounds__(256) void absmax_kernel(const void* __restrict__ W, int64_t total, int vec_ok,
                                                     float* __restrict__ scale) {
    float amax = 0.0f;
    const int64_t stride = (int64_t)gridDim.x * 256;
    const int64_t tid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    int64_t done = 0;
    if (vec_ok) {
        // 16-byte loads, four per thread in flight; every workgroup reads its own contiguous run front to back,
        // 4 KiB at a time.  Plain loads: the quantizing kernel reads the same bytes next and finds part of them
        // in the memory-side cache (with the non-temporal hint here the pair of kernels takes 3 us longer).
        constexpr int EPV = (DT == BT_F32) ? 4 : 8;  // elements per 16 bytes
        const int64_t nvec = total / EPV;
        const uint4* p = (const uint4*)W;
        const int64_t run = (nvec + gridDim.x - 1) / gridDim.x;
        const int64_t first = (int64_t)blockIdx.x * run;
        const int64_t last = (first + run < nvec) ? first + run : nvec;
        for (int64_t i = first + threadIdx.x; i < last; i += 4 * 256) {
            uint4 q[4];
#pragma unroll
            for (int u = 0; u < 4; u++)
                q[u] = (i + u * 256 < last) ? p[i + u * 256] : make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const uint32_t d[4] = {q[u].x, q[u].y, q[u].z, q[u].w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    if constexpr (DT == BT_F32) {
                        amax = fmaxf(amax, fabsf(__builtin_bit_cast(float, d[e])));
                    } else if constexpr (DT == BT_F16) {
                        amax = fmaxf(amax, fabsf(f16_bits_to_f32((uint16_t)d[e])));
                        amax = fmaxf(amax, fabsf(f16_bits_to_f32((uint16_t)(d[e] >> 16))));
                    } else {
                        amax = fmaxf(amax, fabsf(bf16_bits_to_f32((uint16_t)d[e])));
                        amax = fmaxf(amax, fabsf(bf16_bits_to_f32((uint16_t)(d[e] >> 16))));
                    }
                }
            }
        }
        done = nvec * EPV;
    }
    for (int64_t i = done + tid; i < total; i += stride) amax = fmaxf(amax, fabsf(load_elem<DT>(W, i)));
    // one atomic per workgroup, and only if it can still raise the maximum: atomics of all
    // XCDs on one address serialise at roughly ten nanoseconds each
    __shared__ float part[4];
    amax = wave_max(amax);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = amax;
    __syncthreads();
    if (threadIdx.x == 0) {
        amax = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
        if (amax > __hip_atomic_load(scale, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
            atomicMax((unsigned int*)scale, __builtin_bit_cast(unsigned int, amax));
    }
}

__global__ void set_scalar_kernel(float* p, float v) { *p = v; }

template <int DT>
static int launch_quantize(const void* W, int64_t N, int64_t K, float tf, float clamp_min, int per_channel,
                           uint8_t* packed_T, float* scale, int8_t* w_tern, hipStream_t st) {
    int rc = BT_OK;
    if (try_launch_fast<DT>(W, N, K, tf, clamp_min, per_channel, packed_T, scale, w_tern, st, &rc)) return rc;
    const int64_t Kb = ceil_div(K, 4);
    const int64_t tiles = ceil_div(N, 16);
    const int64_t per_xcd = ceil_div(tiles, 8);
    hipLaunchKernelGGL(quantize_pack_generic_kernel<DT>, dim3((unsigned)(per_xcd * 8)), dim3(256), 0, st, W, N, K,
                       Kb, tf, clamp_min, per_channel, packed_T, scale, w_tern, tiles, per_xcd, -1.0f);
    return check_launch("bt_quantize_pack");
}

template <int DT>
static void launch_absmax(const void* W, int64_t total, float* scale, hipStream_t st) {
    const int vec_ok = (((uintptr_t)W) % 16 == 0) ? 1 : 0;
    const unsigned blocks = (unsigned)std::min<int64_t>(std::max<int64_t>(ceil_div(total, 256 * 16), 1), 1024);
    hipLaunchKernelGGL(absmax_kernel<DT>, dim3(blocks), dim3(256), 0, st, W, total, vec_ok, scale);
}

}  // namespace bt

extern "C" int bt_quantize_pack(const void* W, int w_dtype, int64_t N, int64_t K, double threshold_factor,
                                int per_channel, uint8_t* packed_T, float* scale, int8_t* w_tern, void* stream) {
    using namespace bt;
    if (!W || !scale || N <= 0 || K <= 0) {
        set_error("bt_quantize_pack: null pointer or empty shape (N=%lld K=%lld)", (long long)N, (long long)K);
        return BT_ERR_INVALID;
    }
    if (w_dtype != BT_F32 && w_dtype != BT_F16 && w_dtype != BT_BF16) {
        set_error("bt_quantize_pack: unsupported weight dtype %d", w_dtype);
        return BT_ERR_INVALID;
    }
    hipStream_t st = (hipStream_t)stream;
    const float tf = (float)threshold_factor;
    // 1e-8 rounded to the weight dtype (fp16: 0, bf16: nearest bf16)
    float clamp_min = 1e-8f;
    if (w_dtype == BT_F16) clamp_min = 0.0f;
    if (w_dtype == BT_BF16) {
        uint32_t u = __builtin_bit_cast(uint32_t, clamp_min);
        u += 0x7fffu + ((u >> 16) & 1u);
        u &= 0xffff0000u;
        clamp_min = __builtin_bit_cast(float, u);
    }
    if (!per_channel) {
        // tensor scale: zero, absmax over everything; the quantizing kernel floors it, for itself and in place
        hipLaunchKernelGGL(set_scalar_kernel, dim3(1), dim3(1), 0, st, scale, 0.0f);
        const int64_t total = N * K;
        if (w_dtype == BT_F32) launch_absmax<BT_F32>(W, total, scale, st);
        else if (w_dtype == BT_F16) launch_absmax<BT_F16>(W, total, scale, st);
        else launch_absmax<BT_BF16>(W, total, scale, st);
    }
    int rc;
    if (w_dtype == BT_F32)
        rc = launch_quantize<BT_F32>(W, N, K, tf, clamp_min, per_channel, packed_T, scale, w_tern, st);
    else if (w_dtype == BT_F16)
        rc = launch_quantize<BT_F16>(W, N, K, tf, clamp_min, per_channel, packed_T, scale, w_tern, st);
    else
        rc = launch_quantize<BT_BF16>(W, N, K, tf, clamp_min, per_channel, packed_T, scale, w_tern, st);
    return rc;
}

extern "C" int bt_pack_ternary_i8(const int8_t* W_tern, int64_t N, int64_t K, uint8_t* packed_T, void* stream) {
    using namespace bt;
    if (!W_tern || !packed_T || N <= 0 || K <= 0) {
        set_error("bt_pack_ternary_i8: null pointer or empty shape (N=%lld K=%lld)", (long long)N, (long long)K);
        return BT_ERR_INVALID;
    }
    const int64_t Kb = ceil_div(K, 4);
    const int64_t tiles = ceil_div(N, 16);
    const int64_t per_xcd = ceil_div(tiles, 8);
    // codes: +1 -> 1, -1 -> 2, anything of magnitude <= 0.5 (i.e. 0) -> 0
    hipLaunchKernelGGL(quantize_pack_generic_kernel<BT_I8>, dim3((unsigned)(per_xcd * 8)), dim3(256), 0,
                       (hipStream_t)stream, (const void*)W_tern, N, K, Kb, 0.0f, 0.0f, 0, packed_T, (float*)nullptr,
                       (int8_t*)nullptr, tiles, per_xcd, 0.5f);
    return check_launch("bt_pack_ternary_i8");
}
