// Fused ternary quantize + 2-bit pack for gfx950 (HBM-bound, one pass over W).
//
// Arithmetic restated from the reference quantizer and codec
// (bittorch/quant/ternary.py:122-142, bittorch/quant/ternary_packed.py:50-73,
// :202-206): scale = row (or tensor) absmax floored at 1e-8, threshold =
// fl(tf * scale) in the weight dtype, code = |w| > thr ? (w > 0 ? 1 : 2) : 0,
// byte[kb, n] = c0 | c1<<2 | c2<<4 | c3<<6 for k = 4kb..4kb+3.
//
// Layout of the work: a 256-thread workgroup owns 16 consecutive output rows
// n0..n0+15, wave w the four rows n0+4w..n0+4w+3.  A wave keeps one whole row in
// registers (ITERS float4 groups per lane), reduces its absmax across the 64
// lanes, encodes, and ORs the row's bytes into a dword per kb that ends up
// holding the four rows of the wave.  The dwords go through LDS so that the
// transposed store writes 16 contiguous bytes per kb row.
#include "bt_common.h"

namespace bt {

// Workgroup b of a grid of 8*per_xcd workgroups -> tile index such that
// consecutive tiles run on the same XCD (workgroups are dealt round-robin over
// the 8 XCDs), so the 16-byte pieces of one packed_T cache line that
// neighbouring tiles write meet in one L2.
__device__ __forceinline__ int64_t xcd_tile(int64_t b, int64_t per_xcd) {
    return (b & 7) * per_xcd + (b >> 3);
}

template <int DT>
__device__ __forceinline__ void load4(const void* W, int64_t elem, int64_t row_end, bool vec_ok,
                                      float (&v)[4]) {
    // four consecutive elements starting at `elem`; zero past row_end
    if (vec_ok && elem + 4 <= row_end) {
        if constexpr (DT == BT_F32) {
            const float4 t = *(const float4*)((const float*)W + elem);
            v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
        } else {
            const uint2 t = *(const uint2*)((const uint16_t*)W + elem);
            const uint16_t h[4] = {(uint16_t)(t.x & 0xffff), (uint16_t)(t.x >> 16),
                                   (uint16_t)(t.y & 0xffff), (uint16_t)(t.y >> 16)};
#pragma unroll
            for (int i = 0; i < 4; i++)
                v[i] = (DT == BT_F16) ? f16_bits_to_f32(h[i]) : bf16_bits_to_f32(h[i]);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++) v[i] = (elem + i < row_end) ? load_elem<DT>(W, elem + i) : 0.0f;
    }
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

// ITERS > 0: rows of up to ITERS*256 elements held in registers (single pass).
// ITERS == 0: any K; the row is read twice (absmax pass, encode pass).
template <int DT, int ITERS>
__global__ __launch_bounds__(256) void quantize_pack_kernel(
    const void* __restrict__ W, int64_t N, int64_t K, int64_t Kb, float tf, float clamp_min,
    int per_channel, uint8_t* __restrict__ packed_T, float* __restrict__ scale,
    int8_t* __restrict__ w_tern, int64_t tiles, int64_t per_xcd) {
    extern __shared__ uint32_t lds[];  // [Kb][4]: dword (kb, wave) = 4 row bytes

    const int64_t tile = xcd_tile(blockIdx.x, per_xcd);
    if (tile >= tiles) return;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t n0 = tile * 16;
    // 16-byte (fp32) / 8-byte (16-bit) vector loads need aligned rows
    const bool vec_ok = (K % 4 == 0) && (((uintptr_t)W) % 16 == 0);
    const float tensor_scale = per_channel ? 0.0f : fmaxf(scale[0], clamp_min);

    if constexpr (ITERS > 0) {
        uint32_t pk[ITERS];
#pragma unroll
        for (int j = 0; j < ITERS; j++) pk[j] = 0;

        for (int r = 0; r < 4; r++) {
            const int64_t n = n0 + 4 * wave + r;
            if (n >= N) break;  // uniform per wave
            const int64_t row0 = n * K, row_end = row0 + K;
            float v[ITERS][4];
            float amax = 0.0f;
#pragma unroll
            for (int j = 0; j < ITERS; j++) {
                const int64_t kb = (int64_t)j * 64 + lane;
                if (kb < Kb) {
                    load4<DT>(W, row0 + 4 * kb, row_end, vec_ok, v[j]);
                } else {
                    v[j][0] = v[j][1] = v[j][2] = v[j][3] = 0.0f;
                }
                amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v[j][0]), fabsf(v[j][1])),
                                         fmaxf(fabsf(v[j][2]), fabsf(v[j][3]))));
            }
            float s;
            if (per_channel) {
                s = fmaxf(wave_max(amax), clamp_min);
                if (lane == 0) scale[n] = s;
            } else {
                s = tensor_scale;
            }
            const float thr = round_to_dtype(__fmul_rn(tf, s), DT);
#pragma unroll
            for (int j = 0; j < ITERS; j++) {
                const int64_t kb = (int64_t)j * 64 + lane;
                uint32_t tern4;
                const uint32_t byte = encode4(v[j], thr, tern4);
                pk[j] |= byte << (8 * r);
                if (w_tern && kb < Kb) {
                    const int64_t e = row0 + 4 * kb;
                    if (vec_ok && e + 4 <= row_end) {
                        *(uint32_t*)(w_tern + e) = tern4;
                    } else {
                        for (int i = 0; i < 4; i++)
                            if (e + i < row_end) w_tern[e + i] = (int8_t)((tern4 >> (8 * i)) & 0xff);
                    }
                }
            }
        }
        if (packed_T) {
#pragma unroll
            for (int j = 0; j < ITERS; j++) {
                const int64_t kb = (int64_t)j * 64 + lane;
                if (kb < Kb) lds[kb * 4 + wave] = pk[j];
            }
        }
    } else {
        for (int r = 0; r < 4; r++) {
            const int64_t n = n0 + 4 * wave + r;
            if (n >= N) break;
            const int64_t row0 = n * K, row_end = row0 + K;
            float s;
            if (per_channel) {
                float amax = 0.0f;
                for (int64_t kb = lane; kb < Kb; kb += 64) {
                    float v[4];
                    load4<DT>(W, row0 + 4 * kb, row_end, vec_ok, v);
                    amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])),
                                             fmaxf(fabsf(v[2]), fabsf(v[3]))));
                }
                s = fmaxf(wave_max(amax), clamp_min);
                if (lane == 0) scale[n] = s;
            } else {
                s = tensor_scale;
            }
            const float thr = round_to_dtype(__fmul_rn(tf, s), DT);
            for (int64_t kb = lane; kb < Kb; kb += 64) {
                float v[4];
                load4<DT>(W, row0 + 4 * kb, row_end, vec_ok, v);
                uint32_t tern4;
                const uint32_t byte = encode4(v, thr, tern4);
                if (packed_T) {
                    // bytes of the wave's four rows share a dword; rows run one after
                    // another in this wave, so a plain read-modify-write is race free
                    uint32_t cur = (r == 0) ? 0u : lds[kb * 4 + wave];
                    lds[kb * 4 + wave] = cur | (byte << (8 * r));
                }
                if (w_tern) {
                    const int64_t e = row0 + 4 * kb;
                    for (int i = 0; i < 4; i++)
                        if (e + i < row_end) w_tern[e + i] = (int8_t)((tern4 >> (8 * i)) & 0xff);
                }
            }
        }
    }
    if (!packed_T) return;
    // rows past N in a ragged last tile leave their byte lanes untouched: zero them
    // by construction (pk starts at 0; for ITERS == 0 a wave with no valid row
    // never wrote its dword), so make such dwords explicit zeros
    if (n0 + 4 * wave >= N) {
        for (int64_t kb = lane; kb < Kb; kb += 64) lds[kb * 4 + wave] = 0u;
    }
    __syncthreads();

    const bool full = (n0 + 16 <= N) && (N % 16 == 0) && (((uintptr_t)packed_T) % 16 == 0);
    for (int64_t kb = threadIdx.x; kb < Kb; kb += 256) {
        const uint4 q = *(const uint4*)(lds + kb * 4);
        uint8_t* dst = packed_T + kb * N + n0;
        if (full) {
            *(uint4*)dst = q;
        } else {
            const uint32_t d[4] = {q.x, q.y, q.z, q.w};
            for (int i = 0; i < 16; i++)
                if (n0 + i < N) dst[i] = (uint8_t)((d[i >> 2] >> (8 * (i & 3))) & 0xff);
        }
    }
}

// tensor absmax into scale[0] (bit pattern of a non-negative float orders like a uint)
template <int DT>
__global__ __launch_bounds__(256) void absmax_kernel(const void* __restrict__ W, int64_t total,
                                                     float* __restrict__ scale) {
    float amax = 0.0f;
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride)
        amax = fmaxf(amax, fabsf(load_elem<DT>(W, i)));
    amax = wave_max(amax);
    if ((threadIdx.x & 63) == 0) atomicMax((unsigned int*)scale, __builtin_bit_cast(unsigned int, amax));
}

__global__ void set_scalar_kernel(float* p, float v) { *p = v; }
__global__ void floor_scalar_kernel(float* p, float floor_v) { *p = fmaxf(*p, floor_v); }

template <int DT>
static int launch_quantize(const void* W, int64_t N, int64_t K, float tf, float clamp_min,
                           int per_channel, uint8_t* packed_T, float* scale, int8_t* w_tern,
                           hipStream_t st) {
    const int64_t Kb = ceil_div(K, 4);
    const int64_t tiles = ceil_div(N, 16);
    const int64_t per_xcd = ceil_div(tiles, 8);
    const dim3 grid((unsigned)(per_xcd * 8)), block(256);
    const size_t lds = packed_T ? (size_t)Kb * 16 : 0;
    if (lds > 160 * 1024 - 1024) {
        set_error("bt_quantize_pack: K=%lld too large for the LDS transpose tile", (long long)K);
        return BT_ERR_INVALID;
    }
#define BT_QP(IT)                                                                              \
    hipLaunchKernelGGL((quantize_pack_kernel<DT, IT>), grid, block, lds, st, W, N, K, Kb, tf,  \
                       clamp_min, per_channel, packed_T, scale, w_tern, tiles, per_xcd)
    if (lds > 64 * 1024) {
        // beyond the default dynamic LDS limit: raise it for the generic variant
        if (hipFuncSetAttribute((const void*)quantize_pack_kernel<DT, 0>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
            set_error("bt_quantize_pack: cannot reserve %zu bytes of LDS", lds);
            return BT_ERR_LAUNCH;
        }
    }
    if (K <= 1024) BT_QP(4);
    else if (K <= 2048) BT_QP(8);
    else if (K <= 4096) BT_QP(16);
    else if (K <= 8192) BT_QP(32);
    else if (K <= 12288) BT_QP(48);
    else BT_QP(0);
#undef BT_QP
    return check_launch("bt_quantize_pack");
}

}  // namespace bt

extern "C" int bt_quantize_pack(const void* W, int w_dtype, int64_t N, int64_t K,
                                double threshold_factor, int per_channel, uint8_t* packed_T,
                                float* scale, int8_t* w_tern, void* stream) {
    using namespace bt;
    if (!W || !scale || N <= 0 || K <= 0) {
        set_error("bt_quantize_pack: null pointer or empty shape (N=%lld K=%lld)", (long long)N,
                  (long long)K);
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
        hipLaunchKernelGGL(set_scalar_kernel, dim3(1), dim3(1), 0, st, scale, 0.0f);
        const int64_t total = N * K;
        const unsigned blocks = (unsigned)std::min<int64_t>(ceil_div(total, 256 * 16), 2048);
        if (w_dtype == BT_F32)
            hipLaunchKernelGGL(absmax_kernel<BT_F32>, dim3(blocks), dim3(256), 0, st, W, total, scale);
        else if (w_dtype == BT_F16)
            hipLaunchKernelGGL(absmax_kernel<BT_F16>, dim3(blocks), dim3(256), 0, st, W, total, scale);
        else
            hipLaunchKernelGGL(absmax_kernel<BT_BF16>, dim3(blocks), dim3(256), 0, st, W, total, scale);
    }
    int rc;
    if (w_dtype == BT_F32)
        rc = launch_quantize<BT_F32>(W, N, K, tf, clamp_min, per_channel, packed_T, scale, w_tern, st);
    else if (w_dtype == BT_F16)
        rc = launch_quantize<BT_F16>(W, N, K, tf, clamp_min, per_channel, packed_T, scale, w_tern, st);
    else
        rc = launch_quantize<BT_BF16>(W, N, K, tf, clamp_min, per_channel, packed_T, scale, w_tern, st);
    if (rc != BT_OK) return rc;
    if (!per_channel) {
        hipLaunchKernelGGL(floor_scalar_kernel, dim3(1), dim3(1), 0, st, scale, clamp_min);
        return check_launch("bt_quantize_pack(floor)");
    }
    return BT_OK;
}
