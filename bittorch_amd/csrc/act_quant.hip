// Per-row int8 activation quantization for gfx950 (HBM-bound).
//
// Arithmetic restated from the reference (csrc/kernels/ternary_gemm_tensor_core.cu:343-347,
// :439, :456-457) with the row scale taken over the whole row:
//   amax = max_k |x[b,k]|;  s_x[b] = amax > 1e-6 ? amax / 127 : 1
//   q[b,k] = (int8) clamp(roundf(x[b,k] * (1 / s_x[b])), -127, 127)
// Optionally the rows' sums of q (int32), which the field-layout prefill GEMM starts its accumulators from.
#include <cstdlib>

#include "bt_common.h"

namespace bt {

// Per-row int8 activation quantizer: one wave per row, two passes over the row
// (the second pass hits in cache; a row is at most a few tens of KiB).
template <int DT>
__global__ __launch_bounds__(256) void act_quant_kernel(const void* __restrict__ X, int64_t B, int64_t K,
                                                        int8_t* __restrict__ Q, float* __restrict__ s_x,
                                                        int q_layout, int32_t* __restrict__ rowsum) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= B) return;
    const int64_t base = row * K;
    constexpr int ES = (DT == BT_F32) ? 4 : 2;
    const bool vec_ok = (K % 8 == 0) && (((uintptr_t)X) % 16 == 0) && (((uintptr_t)Q) % 8 == 0);

    auto load8 = [&](int64_t k, float (&v)[8]) {
        if (vec_ok) {
            if constexpr (DT == BT_F32) {
                const float4 a = *(const float4*)((const float*)X + base + k);
                const float4 b = *(const float4*)((const float*)X + base + k + 4);
                v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
                v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
            } else {
                const uint4 u = *(const uint4*)((const uint16_t*)X + base + k);
                const uint32_t d[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const uint16_t h = (uint16_t)(d[e >> 1] >> (16 * (e & 1)));
                    v[e] = (DT == BT_F16) ? f16_bits_to_f32(h) : bf16_bits_to_f32(h);
                }
            }
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++) v[e] = (k + e < K) ? load_elem<DT>(X, base + k + e) : 0.0f;
        }
    };
    (void)ES;

    float amax = 0.0f;
    for (int64_t k = (int64_t)lane * 8; k < K; k += 512) {
        float v[8];
        load8(k, v);
#pragma unroll
        for (int e = 0; e < 8; e++) amax = fmaxf(amax, fabsf(v[e]));
    }
    amax = wave_max(amax);
    const float s = (amax > 1e-6f) ? __fdiv_rn(amax, 127.0f) : 1.0f;
    const float inv = __fdiv_rn(1.0f, s);
    if (lane == 0) s_x[row] = s;

    int qsum = 0;
    for (int64_t k = (int64_t)lane * 8; k < K; k += 512) {
        float v[8];
        load8(k, v);
        uint32_t lo = 0, hi = 0;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            float r = round_half_away(__fmul_rn(v[e], inv));
            r = fmaxf(-127.0f, fminf(127.0f, r));
            qsum += (int)r;  // (elements past K were loaded as zero)
            const uint32_t byte = (uint32_t)(uint8_t)(int8_t)(int)r;
            if (e < 4) lo |= byte << (8 * e);
            else hi |= byte << (8 * (e - 4));
        }
        if (vec_ok) {  // (operand order is only requested with K % 16 == 0 and aligned rows: this path)
            *(uint2*)(Q + base + k) = q_layout == Q_OPERAND_ORDER ? q_to_operand_order(lo, hi, lane & 1) : make_uint2(lo, hi);
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++)
                if (k + e < K) Q[base + k + e] = (int8_t)(((e < 4 ? lo : hi) >> (8 * (e & 3))) & 0xff);
        }
    }
    if (rowsum) {  // (uniform)
        qsum = wave_sum_i32(qsum);
        if (lane == 0) rowsum[row] = qsum;
    }
}

// One workgroup per row, the row held in registers between the absmax pass and the
// quantization: X is read once and the row's latency chain is load -> reduce -> store.
// Needs K % 8 == 0, K <= 2048*ITERS and aligned pointers (16 bytes X, 8 bytes Q).
template <int DT, int ITERS>
__global__ __launch_bounds__(256) void act_quant_row_kernel(const void* __restrict__ X, int K,
                                                            int8_t* __restrict__ Q, float* __restrict__ s_x,
                                                            int q_layout, int32_t* __restrict__ rowsum) {
    __shared__ float part[4];
    __shared__ int part_sum[4];
    const int tid = threadIdx.x;
    const int64_t base = (int64_t)blockIdx.x * K;
    float v[ITERS][8];
#pragma unroll
    for (int i = 0; i < ITERS; i++) {
        const int k = (i * 256 + tid) * 8;
        const int kc = min(k, K - 8);  // clamped, unconditional loads; zeroed below
        if constexpr (DT == BT_F32) {
            const uint4 a = *(const uint4*)((const float*)X + base + kc);
            const uint4 b = *(const uint4*)((const float*)X + base + kc + 4);
            const uint32_t da[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int e = 0; e < 8; e++) v[i][e] = __builtin_bit_cast(float, da[e]);
        } else {
            const uint4 u = *(const uint4*)((const uint16_t*)X + base + kc);
            const uint32_t d[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const uint16_t h = (uint16_t)(d[e >> 1] >> (16 * (e & 1)));
                v[i][e] = (DT == BT_F16) ? f16_bits_to_f32(h) : bf16_bits_to_f32(h);
            }
        }
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < ITERS; i++) {
        const bool ok = (i * 256 + tid) * 8 < K;
#pragma unroll
        for (int e = 0; e < 8; e++) amax = fmaxf(amax, ok ? fabsf(v[i][e]) : 0.0f);
    }
    amax = wave_max(amax);
    if ((tid & 63) == 0) part[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
    const float s = (amax > 1e-6f) ? __fdiv_rn(amax, 127.0f) : 1.0f;
    const float inv = __fdiv_rn(1.0f, s);
    if (tid == 0) s_x[blockIdx.x] = s;
    int qsum = 0;
#pragma unroll
    for (int i = 0; i < ITERS; i++) {
        const int k = (i * 256 + tid) * 8;
        uint32_t lo = 0, hi = 0;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            float r = round_half_away(__fmul_rn(v[i][e], inv));
            r = fmaxf(-127.0f, fminf(127.0f, r));
            if (k < K) qsum += (int)r;  // (a clamped group past the end repeats the row's last one)
            const uint32_t byte = (uint32_t)(uint8_t)(int8_t)(int)r;
            if (e < 4) lo |= byte << (8 * e);
            else hi |= byte << (8 * (e - 4));
        }
        const uint2 o = q_layout == Q_OPERAND_ORDER ? q_to_operand_order(lo, hi, tid & 1) : make_uint2(lo, hi);
        if (k < K) st2_nt(Q + base + k, o.x, o.y);  // K % 16 == 0 in operand order: both lanes of a pair store
    }
    if (rowsum) {  // (uniform)
        qsum = wave_sum_i32(qsum);
        if ((tid & 63) == 0) part_sum[tid >> 6] = qsum;
        __syncthreads();
        if (tid == 0) rowsum[blockIdx.x] = part_sum[0] + part_sum[1] + part_sum[2] + part_sum[3];
    }
}

// Many short rows: one wave per row (four rows per workgroup), lane l holding the 8-element chunks i * 64 + l -- all
// 64 lanes busy where the workgroup kernel above leaves lanes idle, the absmax a shuffle tree, no LDS and no barrier.
// The same bits.
template <int DT, int ITERS>
__global__ __launch_bounds__(256) void act_quant_wave_kernel(const void* __restrict__ X, int64_t B, int K,
                                                             int8_t* __restrict__ Q, float* __restrict__ s_x,
                                                             int q_layout, int32_t* __restrict__ rowsum) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= B) return;  // (whole waves; the kernel has no barrier)
    const int64_t base = row * K;
    float v[ITERS][8];
#pragma unroll
    for (int i = 0; i < ITERS; i++) {
        const int kc = min((i * 64 + lane) * 8, K - 8);  // clamped, unconditional loads; masked below
        if constexpr (DT == BT_F32) {
            const uint4 a = *(const uint4*)((const float*)X + base + kc);
            const uint4 b = *(const uint4*)((const float*)X + base + kc + 4);
            const uint32_t da[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int e = 0; e < 8; e++) v[i][e] = __builtin_bit_cast(float, da[e]);
        } else {
            const uint4 u = *(const uint4*)((const uint16_t*)X + base + kc);
            const uint32_t d[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const uint16_t h = (uint16_t)(d[e >> 1] >> (16 * (e & 1)));
                v[i][e] = (DT == BT_F16) ? f16_bits_to_f32(h) : bf16_bits_to_f32(h);
            }
        }
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < ITERS; i++) {
        const bool ok = (i * 64 + lane) * 8 < K;
#pragma unroll
        for (int e = 0; e < 8; e++) amax = fmaxf(amax, ok ? fabsf(v[i][e]) : 0.0f);
    }
    amax = wave_max(amax);
    const float s = (amax > 1e-6f) ? __fdiv_rn(amax, 127.0f) : 1.0f;
    const float inv = __fdiv_rn(1.0f, s);
    if (lane == 0) s_x[row] = s;
    int qsum = 0;
#pragma unroll
    for (int i = 0; i < ITERS; i++) {
        const int k = (i * 64 + lane) * 8;
        uint32_t lo = 0, hi = 0;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            float r = round_half_away(__fmul_rn(v[i][e], inv));
            r = fmaxf(-127.0f, fminf(127.0f, r));
            if (k < K) qsum += (int)r;
            const uint32_t byte = (uint32_t)(uint8_t)(int8_t)(int)r;
            if (e < 4) lo |= byte << (8 * e);
            else hi |= byte << (8 * (e - 4));
        }
        const uint2 o = q_layout == Q_OPERAND_ORDER ? q_to_operand_order(lo, hi, lane & 1) : make_uint2(lo, hi);
        if (k < K) st2_nt(Q + base + k, o.x, o.y);
    }
    if (rowsum) {  // (uniform)
        qsum = wave_sum_i32(qsum);
        if (lane == 0) rowsum[row] = qsum;
    }
}

template <int DT>
static bool launch_act_quant_rows(const void* X, int64_t B, int64_t K, int8_t* Q, float* s_x, int ql, int32_t* rs,
                                  hipStream_t st) {
    if (K % 8 != 0 || K > 16384 || ((uintptr_t)X) % 16 != 0 || ((uintptr_t)Q) % 8 != 0 || B > 0x7fffffff ||
        tuning_env("BITTORCH_ACTQ_GENERIC"))
        return false;
    const dim3 grid((unsigned)B), block(256);
    const int k = (int)K;
    if (B >= 2048 && K <= 3072) {  // many short rows: a wave per row (4096 x 2560 bf16 9.4 -> 7.6 us, 4096 x 1024 6.9 -> 4.5,
                                   // 4096 x 2048 7.3 -> 6.6; from K = 3584 on the workgroup kernel is as fast or faster)
        const dim3 wgrid((unsigned)((B + 3) / 4));
        switch ((k + 511) / 512) {
            case 1: hipLaunchKernelGGL((act_quant_wave_kernel<DT, 1>), wgrid, block, 0, st, X, B, k, Q, s_x, ql, rs); break;
            case 2: hipLaunchKernelGGL((act_quant_wave_kernel<DT, 2>), wgrid, block, 0, st, X, B, k, Q, s_x, ql, rs); break;
            case 3: hipLaunchKernelGGL((act_quant_wave_kernel<DT, 3>), wgrid, block, 0, st, X, B, k, Q, s_x, ql, rs); break;
            case 4: hipLaunchKernelGGL((act_quant_wave_kernel<DT, 4>), wgrid, block, 0, st, X, B, k, Q, s_x, ql, rs); break;
            case 5: hipLaunchKernelGGL((act_quant_wave_kernel<DT, 5>), wgrid, block, 0, st, X, B, k, Q, s_x, ql, rs); break;
            default: hipLaunchKernelGGL((act_quant_wave_kernel<DT, 6>), wgrid, block, 0, st, X, B, k, Q, s_x, ql, rs); break;
        }
        return true;
    }
    if (K <= 2048) hipLaunchKernelGGL((act_quant_row_kernel<DT, 1>), grid, block, 0, st, X, k, Q, s_x, ql, rs);
    else if (K <= 4096) hipLaunchKernelGGL((act_quant_row_kernel<DT, 2>), grid, block, 0, st, X, k, Q, s_x, ql, rs);
    else if (K <= 8192) hipLaunchKernelGGL((act_quant_row_kernel<DT, 4>), grid, block, 0, st, X, k, Q, s_x, ql, rs);
    else if (K <= 12288) hipLaunchKernelGGL((act_quant_row_kernel<DT, 6>), grid, block, 0, st, X, k, Q, s_x, ql, rs);
    else hipLaunchKernelGGL((act_quant_row_kernel<DT, 8>), grid, block, 0, st, X, k, Q, s_x, ql, rs);
    return true;
}

// q_layout = Q_OPERAND_ORDER needs K % 16 == 0, X 16-byte and Q 8-byte aligned (the callers check)
int launch_act_quant(const void* X, int x_dtype, int64_t B, int64_t K, int8_t* Q, float* s_x, int q_layout,
                     int32_t* rowsum, hipStream_t st) {
    const int ql = q_layout;
    // the operand order is written 16 bytes at a time: callers check this too, but a buffer that cannot take it
    // must never be written row-major under that name
    if (ql == Q_OPERAND_ORDER && (K % 16 != 0 || ((uintptr_t)X) % 16 != 0 || ((uintptr_t)Q) % 16 != 0)) {
        set_error("bt_act_quant_i8: the operand-order layout needs K %% 16 == 0 and 16-byte aligned X and Q");
        return BT_ERR_INVALID;
    }
    int32_t* rs = rowsum;
    const bool done = (x_dtype == BT_F32)   ? launch_act_quant_rows<BT_F32>(X, B, K, Q, s_x, ql, rs, st)
                      : (x_dtype == BT_F16) ? launch_act_quant_rows<BT_F16>(X, B, K, Q, s_x, ql, rs, st)
                                            : launch_act_quant_rows<BT_BF16>(X, B, K, Q, s_x, ql, rs, st);
    if (done) return check_launch("bt_act_quant_i8");
    const dim3 grid((unsigned)ceil_div(B, 4)), block(256);
    if (x_dtype == BT_F32) hipLaunchKernelGGL(act_quant_kernel<BT_F32>, grid, block, 0, st, X, B, K, Q, s_x, ql, rs);
    else if (x_dtype == BT_F16) hipLaunchKernelGGL(act_quant_kernel<BT_F16>, grid, block, 0, st, X, B, K, Q, s_x, ql, rs);
    else hipLaunchKernelGGL(act_quant_kernel<BT_BF16>, grid, block, 0, st, X, B, K, Q, s_x, ql, rs);
    return check_launch("bt_act_quant_i8");
}

// fp32 activations as three bf16 planes: x = hi + mid + lo exactly, each term the truncation to
// bf16 (upper 16 bits) of what the terms before it leave (24 significand bits = 3 x 8).  Ternary
// weights are exact in bf16, so the three products per weight are exact and the 16-bit matrix
// cores accumulate them in fp32: fp32 inputs run on the bf16 kernels without losing a bit of
// the activations.  X [B,K] fp32 -> P [B,3*Kp] bf16 bits, row b = [hi(Kp) | mid(Kp) | lo(Kp)] / 2,
// Kp = K rounded up to the kernels' 64-wide step, the padding zero (it meets padding codes or clamped
// weight rows: 0 * w = 0 exactly).
__device__ __forceinline__ void split3(float x, uint16_t& hi, uint16_t& mid, uint16_t& lo) {
    const uint32_t u0 = __builtin_bit_cast(uint32_t, x) & 0xFFFF0000u;
    const float r1 = x - __builtin_bit_cast(float, u0);
    const uint32_t u1 = __builtin_bit_cast(uint32_t, r1) & 0xFFFF0000u;
    const float r2 = r1 - __builtin_bit_cast(float, u1);
    // stored halved (exact): the bf16 kernels decode the weights as +-2.0, and x * 2 would
    // overflow for |x| above half the fp32 range
    hi = (uint16_t)(__builtin_bit_cast(uint32_t, __builtin_bit_cast(float, u0) * 0.5f) >> 16);
    mid = (uint16_t)(__builtin_bit_cast(uint32_t, __builtin_bit_cast(float, u1) * 0.5f) >> 16);
    lo = (uint16_t)(__builtin_bit_cast(uint32_t, r2 * 0.5f) >> 16);
}
// VEC: K % 4 == 0 and X 16-byte aligned (one float4 per thread and trip); otherwise element by element
template <bool VEC>
__global__ __launch_bounds__(256) void split_f32_planes_kernel(const float* __restrict__ X, int64_t B, int64_t K, int64_t Kp,
                                                               uint16_t* __restrict__ P) {
    const int64_t kq = Kp >> 2;  // groups of four per padded row
    const int64_t total = B * kq;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t b = i / kq, c = i - b * kq;
        float x[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        if constexpr (VEC) {
            if (4 * c < K) {
                const float4 v = *(const float4*)(X + b * K + 4 * c);
                x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
            }
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (4 * c + e < K) x[e] = X[b * K + 4 * c + e];
        }
        uint16_t hi[4], mid[4], lo[4];
#pragma unroll
        for (int e = 0; e < 4; e++) split3(x[e], hi[e], mid[e], lo[e]);
        uint16_t* row = P + b * 3 * Kp + 4 * c;
        *(uint2*)(row) = make_uint2((uint32_t)hi[0] | ((uint32_t)hi[1] << 16), (uint32_t)hi[2] | ((uint32_t)hi[3] << 16));
        *(uint2*)(row + Kp) = make_uint2((uint32_t)mid[0] | ((uint32_t)mid[1] << 16), (uint32_t)mid[2] | ((uint32_t)mid[3] << 16));
        *(uint2*)(row + 2 * Kp) = make_uint2((uint32_t)lo[0] | ((uint32_t)lo[1] << 16), (uint32_t)lo[2] | ((uint32_t)lo[3] << 16));
    }
}

// Kp: plane length, a multiple of 64 and >= K; P is 8-byte aligned
int launch_split_f32_planes(const void* X, int64_t B, int64_t K, int64_t Kp, void* P, hipStream_t st) {
    const int64_t total = B * (Kp >> 2);
    const unsigned blocks = (unsigned)std::min<int64_t>(std::max<int64_t>(ceil_div(total, 256), 1), 8192);
    if (K % 4 == 0 && ((uintptr_t)X) % 16 == 0)
        hipLaunchKernelGGL(split_f32_planes_kernel<true>, dim3(blocks), dim3(256), 0, st, (const float*)X, B, K, Kp, (uint16_t*)P);
    else
        hipLaunchKernelGGL(split_f32_planes_kernel<false>, dim3(blocks), dim3(256), 0, st, (const float*)X, B, K, Kp, (uint16_t*)P);
    return check_launch("bt_ternary_linear_packed_forward(split)");
}

}  // namespace bt
