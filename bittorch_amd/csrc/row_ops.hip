// Row-wise producers of the ternary GEMMs' activations for gfx950 (HBM-bound), fusing what a
// transformer block does between two ternary layers (block structure of the reference's JS
// runtime, js/src/models/TernaryTransformer.ts:366-423 (SwiGLU MLP), :489-521 (pre-norm block)):
//
//   SwiGLU   h[b,k] = rd( rd(silu(g[b,k])) * u[b,k] ),   silu(x) = x / (1 + exp(-x))
//   RMSNorm  y[b,k] = rd( (x[b,k] * r_b) * w[k] ),        r_b = 1 / sqrt(ss_b / K + eps),
//                                                         ss_b = float(sum_k double(x[b,k])^2)
// (rd = round to the tensor dtype; every fp32 operation rounded on its own, no contraction; exp is
// the fixed polynomial below, so a host restatement reproduces every bit), each optionally
// followed in the same kernel by the per-row int8 activation quantizer of the int8 GEMM
// (csrc/kernels/ternary_gemm_tensor_core.cu:343-347, :439, :456-457, whole-row scale):
//   amax = max_k |v|;  s_x = amax > 1e-6 ? amax / 127 : 1;  q = clamp(roundf(v * (1 / s_x)), -127, 127)
// so that the activation makes one trip through HBM instead of three or four.
#include <cstdlib>

#include "row_math.h"

namespace bt {

enum { ROW_SWIGLU = 0, ROW_RMSNORM = 1 };

struct RowOpParams {
    const void* A;      // SwiGLU: gate [B, K] (row stride lda);  RMSNorm: x [B, K] (row stride lda)
    const void* Bv;     // SwiGLU: up [B, K] (row stride ldb);    RMSNorm: weight [K] or null
    int64_t lda, ldb;   // row strides in elements
    void* H;            // optional [B, K] output in the input dtype
    int8_t* Q;          // optional [B, K] int8 output (with s_x)
    float* s_x;         // [B]
    int32_t* rowsum;    // optional [B]: the rows' sums of Q (for the field-layout prefill GEMM)
    float eps;
    int K;
    int q_layout;       // Q_ROW_MAJOR / Q_OPERAND_ORDER (K % 16 == 0)
};

// NT = true reads with the non-temporal hint.  Not used for activations: they were written by the kernel before and come
// out of the memory-side cache, where the hint costs 5-10 % (RMSNorm of 4096 x 2560 bf16: 10.0 us plain, 11.5 us with it);
// the stores below carry it (written through instead of at the end of the kernel: 10.7 -> 10.0 us, 2048 x 4096 8.7 -> 6.9 us).
template <int DT, bool NT = false>
__device__ __forceinline__ void load8(const void* base, int64_t idx, float (&v)[8]) {
    if constexpr (DT == BT_F32) {
        const uint4 a = NT ? ldw4_nt((const float*)base + idx) : *(const uint4*)((const float*)base + idx);
        const uint4 b = NT ? ldw4_nt((const float*)base + idx + 4) : *(const uint4*)((const float*)base + idx + 4);
        const uint32_t d[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = __builtin_bit_cast(float, d[e]);
    } else {
        const uint4 u = NT ? ldw4_nt((const uint16_t*)base + idx) : *(const uint4*)((const uint16_t*)base + idx);
        const uint32_t d[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const uint16_t h = (uint16_t)(d[e >> 1] >> (16 * (e & 1)));
            v[e] = (DT == BT_F16) ? f16_bits_to_f32(h) : bf16_bits_to_f32(h);
        }
    }
}
template <int DT>
__device__ __forceinline__ void store8(void* base, int64_t idx, const float (&v)[8]) {
    if constexpr (DT == BT_F32) {
        st4_nt((float*)base + idx, __builtin_bit_cast(uint32_t, v[0]), __builtin_bit_cast(uint32_t, v[1]),
               __builtin_bit_cast(uint32_t, v[2]), __builtin_bit_cast(uint32_t, v[3]));
        st4_nt((float*)base + idx + 4, __builtin_bit_cast(uint32_t, v[4]), __builtin_bit_cast(uint32_t, v[5]),
               __builtin_bit_cast(uint32_t, v[6]), __builtin_bit_cast(uint32_t, v[7]));
    } else {
        uint32_t d[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const uint32_t lo = (DT == BT_F16) ? f32_to_f16_bits(v[2 * e]) : f32_to_bf16_bits(v[2 * e]);
            const uint32_t hi = (DT == BT_F16) ? f32_to_f16_bits(v[2 * e + 1]) : f32_to_bf16_bits(v[2 * e + 1]);
            d[e] = lo | (hi << 16);
        }
        st4_nt((uint16_t*)base + idx, d[0], d[1], d[2], d[3]);
    }
}

// One workgroup per row, the row held in registers: the operands are read once, the outputs
// written once.  Needs K % 8 == 0, K <= 2048*ITERS, 16-byte aligned rows.
// QUANT = false: nothing outlives the store of an element, so SwiGLU streams through few registers.
template <int OP, int DT, int ITERS, bool QUANT>
__global__ __launch_bounds__(256) void row_op_kernel(RowOpParams p) {
    __shared__ double part_d[4];
    __shared__ float part_f[4];
    const int tid = threadIdx.x;
    const int K = p.K;
    const int64_t row = blockIdx.x;
    float v[ITERS][8];
    // clamped, unconditional loads; lanes past the row are masked where it matters
#pragma unroll
    for (int i = 0; i < ITERS; i++) {
        const int k = (i * 256 + tid) * 8;
        const int kc = min(k, K - 8);
        load8<DT>(p.A, row * p.lda + kc, v[i]);
    }
    if constexpr (OP == ROW_SWIGLU) {
#pragma unroll
        for (int i = 0; i < ITERS; i++) {
            const int k = (i * 256 + tid) * 8;
            const int kc = min(k, K - 8);
            float u[8];
            load8<DT>(p.Bv, row * p.ldb + kc, u);
#pragma unroll
            for (int e = 0; e < 8; e++) v[i][e] = swiglu_value(v[i][e], u[e], DT);
        }
    } else {
        double ss = 0.0;
#pragma unroll
        for (int i = 0; i < ITERS; i++) {
            const bool ok = (i * 256 + tid) * 8 < K;
#pragma unroll
            for (int e = 0; e < 8; e++) ss += ok ? (double)v[i][e] * (double)v[i][e] : 0.0;
        }
        ss = wave_sum_f64(ss);
        if ((tid & 63) == 0) part_d[tid >> 6] = ss;
        __syncthreads();
        ss = (part_d[0] + part_d[1]) + (part_d[2] + part_d[3]);
        const float r = rms_rstd(ss, K, p.eps);
#pragma unroll
        for (int i = 0; i < ITERS; i++) {
            const int k = (i * 256 + tid) * 8;
            const int kc = min(k, K - 8);
            float w[8];
            if (p.Bv) load8<DT>(p.Bv, kc, w);
#pragma unroll
            for (int e = 0; e < 8; e++) v[i][e] = rmsnorm_value(v[i][e], r, p.Bv ? w[e] : 1.0f, DT);
        }
    }
    if (p.H) {
#pragma unroll
        for (int i = 0; i < ITERS; i++) {
            const int k = (i * 256 + tid) * 8;
            if (k < K) store8<DT>(p.H, row * (int64_t)K + k, v[i]);
        }
    }
    if constexpr (!QUANT) return;
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < ITERS; i++) {
        const bool ok = (i * 256 + tid) * 8 < K;
#pragma unroll
        for (int e = 0; e < 8; e++) amax = fmaxf(amax, ok ? fabsf(v[i][e]) : 0.0f);
    }
    amax = wave_max(amax);
    if ((tid & 63) == 0) part_f[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(part_f[0], part_f[1]), fmaxf(part_f[2], part_f[3]));
    const float s = (amax > 1e-6f) ? __fdiv_rn(amax, 127.0f) : 1.0f;
    const float inv = __fdiv_rn(1.0f, s);
    if (tid == 0) p.s_x[row] = s;
    int qsum = 0;
#pragma unroll
    for (int i = 0; i < ITERS; i++) {
        const int k = (i * 256 + tid) * 8;
        uint32_t lo = 0, hi = 0;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const int8_t qv = quant_i8(v[i][e], inv);
            if (k < K) qsum += (int)qv;
            const uint32_t byte = (uint32_t)(uint8_t)qv;
            if (e < 4) lo |= byte << (8 * e);
            else hi |= byte << (8 * (e - 4));
        }
        const uint2 o = p.q_layout == Q_OPERAND_ORDER ? q_to_operand_order(lo, hi, tid & 1) : make_uint2(lo, hi);
        if (k < K) st2_nt(p.Q + row * (int64_t)K + k, o.x, o.y);
    }
    if (p.rowsum) {  // (uniform)
        __shared__ int part_i[4];
        qsum = wave_sum_i32(qsum);
        if ((tid & 63) == 0) part_i[tid >> 6] = qsum;
        __syncthreads();
        if (tid == 0) p.rowsum[row] = (part_i[0] + part_i[1]) + (part_i[2] + part_i[3]);
    }
}

// Short rows: one WAVE per row (four rows per workgroup), the row in the wave's registers.  Lane l holds the 8-element
// chunks i * 64 + l, i < ITERS (K <= 512 * ITERS; the launcher says when): a row of 2560 elements fills five iterations of all 64 lanes, where
// the 256-thread kernel above leaves three of its eight wave-iterations idle, and every reduction is a shuffle tree
// inside the wave -- no LDS, no barrier between a row's passes.  Same element arithmetic, same results.
template <int OP, int DT, int ITERS, bool QUANT>
__global__ __launch_bounds__(256) void row_op_wave_kernel(RowOpParams p, int64_t B) {
    const int lane = threadIdx.x & 63;
    const int K = p.K;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= B) return;  // (whole waves; the kernel has no barrier)
    float v[ITERS][8];
#pragma unroll
    for (int i = 0; i < ITERS; i++) {
        const int k = (i * 64 + lane) * 8;
        load8<DT>(p.A, row * p.lda + min(k, K - 8), v[i]);
    }
    if constexpr (OP == ROW_SWIGLU) {
#pragma unroll
        for (int i = 0; i < ITERS; i++) {
            const int k = (i * 64 + lane) * 8;
            float u[8];
            load8<DT>(p.Bv, row * p.ldb + min(k, K - 8), u);
#pragma unroll
            for (int e = 0; e < 8; e++) v[i][e] = swiglu_value(v[i][e], u[e], DT);
        }
    } else {
        double ss = 0.0;
#pragma unroll
        for (int i = 0; i < ITERS; i++) {
            const bool ok = (i * 64 + lane) * 8 < K;
#pragma unroll
            for (int e = 0; e < 8; e++) ss += ok ? (double)v[i][e] * (double)v[i][e] : 0.0;
        }
        const float r = rms_rstd(wave_sum_f64(ss), K, p.eps);
#pragma unroll
        for (int i = 0; i < ITERS; i++) {
            const int k = (i * 64 + lane) * 8;
            float w[8];
            if (p.Bv) load8<DT>(p.Bv, min(k, K - 8), w);
#pragma unroll
            for (int e = 0; e < 8; e++) v[i][e] = rmsnorm_value(v[i][e], r, p.Bv ? w[e] : 1.0f, DT);
        }
    }
    if (p.H) {
#pragma unroll
        for (int i = 0; i < ITERS; i++) {
            const int k = (i * 64 + lane) * 8;
            if (k < K) store8<DT>(p.H, row * (int64_t)K + k, v[i]);
        }
    }
    if constexpr (!QUANT) return;
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
    if (lane == 0) p.s_x[row] = s;
    int qsum = 0;
#pragma unroll
    for (int i = 0; i < ITERS; i++) {
        const int k = (i * 64 + lane) * 8;
        uint32_t lo = 0, hi = 0;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const int8_t qv = quant_i8(v[i][e], inv);
            if (k < K) qsum += (int)qv;
            const uint32_t byte = (uint32_t)(uint8_t)qv;
            if (e < 4) lo |= byte << (8 * e);
            else hi |= byte << (8 * (e - 4));
        }
        const uint2 o = p.q_layout == Q_OPERAND_ORDER ? q_to_operand_order(lo, hi, lane & 1) : make_uint2(lo, hi);
        if (k < K) st2_nt(p.Q + row * (int64_t)K + k, o.x, o.y);
    }
    if (p.rowsum) {  // (uniform)
        qsum = wave_sum_i32(qsum);
        if (lane == 0) p.rowsum[row] = qsum;
    }
}

// Any K and alignment: one workgroup per row, element-wise passes that recompute the value
// (reduction passes hit in cache).
template <int OP, int DT>
__global__ __launch_bounds__(256) void row_op_generic_kernel(RowOpParams p) {
    __shared__ double part_d[4];
    __shared__ float part_f[4];
    const int tid = threadIdx.x;
    const int K = p.K;
    const int64_t row = blockIdx.x;
    float r = 0.0f;
    if constexpr (OP == ROW_RMSNORM) {
        double ss = 0.0;
        for (int k = tid; k < K; k += 256) {
            const double x = (double)load_elem<DT>(p.A, row * p.lda + k);
            ss += x * x;
        }
        ss = wave_sum_f64(ss);
        if ((tid & 63) == 0) part_d[tid >> 6] = ss;
        __syncthreads();
        ss = (part_d[0] + part_d[1]) + (part_d[2] + part_d[3]);
        r = rms_rstd(ss, K, p.eps);
    }
    auto value = [&](int k) {
        const float a = load_elem<DT>(p.A, row * p.lda + k);
        if constexpr (OP == ROW_SWIGLU) return swiglu_value(a, load_elem<DT>(p.Bv, row * p.ldb + k), DT);
        else return rmsnorm_value(a, r, p.Bv ? load_elem<DT>(p.Bv, k) : 1.0f, DT);
    };
    if (p.H)
        for (int k = tid; k < K; k += 256) store_elem<DT>(p.H, row * (int64_t)K + k, value(k));
    if (!p.Q) return;
    float amax = 0.0f;
    for (int k = tid; k < K; k += 256) amax = fmaxf(amax, fabsf(value(k)));
    amax = wave_max(amax);
    if ((tid & 63) == 0) part_f[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(part_f[0], part_f[1]), fmaxf(part_f[2], part_f[3]));
    const float s = (amax > 1e-6f) ? __fdiv_rn(amax, 127.0f) : 1.0f;
    const float inv = __fdiv_rn(1.0f, s);
    if (tid == 0) p.s_x[row] = s;
    int qsum = 0;
    for (int k = tid; k < K; k += 256) {
        const int64_t pos = p.q_layout == Q_OPERAND_ORDER ? q_operand_order_pos(k) : k;
        const int8_t qv = quant_i8(value(k), inv);
        qsum += (int)qv;
        p.Q[row * (int64_t)K + pos] = qv;
    }
    if (p.rowsum) {  // (uniform)
        __shared__ int part_i[4];
        qsum = wave_sum_i32(qsum);
        if ((tid & 63) == 0) part_i[tid >> 6] = qsum;
        __syncthreads();
        if (tid == 0) p.rowsum[row] = (part_i[0] + part_i[1]) + (part_i[2] + part_i[3]);
    }
}

template <int OP, int DT, bool QUANT>
static void launch_row_op_iters(const RowOpParams& p, dim3 grid, dim3 block, hipStream_t st) {
    if (p.K <= 2048) hipLaunchKernelGGL((row_op_kernel<OP, DT, 1, QUANT>), grid, block, 0, st, p);
    else if (p.K <= 4096) hipLaunchKernelGGL((row_op_kernel<OP, DT, 2, QUANT>), grid, block, 0, st, p);
    else if (p.K <= 6144) hipLaunchKernelGGL((row_op_kernel<OP, DT, 3, QUANT>), grid, block, 0, st, p);
    else if (p.K <= 8192) hipLaunchKernelGGL((row_op_kernel<OP, DT, 4, QUANT>), grid, block, 0, st, p);
    else if (p.K <= 12288) hipLaunchKernelGGL((row_op_kernel<OP, DT, 6, QUANT>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((row_op_kernel<OP, DT, 8, QUANT>), grid, block, 0, st, p);
}

// One wave per row where it measures faster than a workgroup per row: rows that leave a quarter or more of the
// workgroup kernel's lanes idle (K <= 1536, 2048 < K <= 3072) in launches with enough rows to keep every SIMD supplied
// with waves -- 4096 x 2560 bf16: RMSNorm 9.9 -> 8.6 us, RMSNorm + quantization 14.5 -> 11.5, SwiGLU + quantization
// 21.2 -> 16.7; 8192 x 1024: 16.6 -> 10.0, 21.4 -> 13.8.  With few rows a lone wave's chain of passes is the slower one
// (512 x 2560: 5.5 -> 8.0 us), and rows that fill the workgroup's lanes gain nothing (K = 2048, 3584, 4096).
static bool wave_per_row(int64_t B, int K, bool quant) {
    const bool idle_lanes = K <= 1536 || (K > 2048 && K <= 3072);
    return idle_lanes && B >= (quant ? 2048 : 4096) && (quant || K <= 2560);
}
template <int OP, int DT, bool QUANT>
static void launch_row_op_wave(const RowOpParams& p, int64_t B, hipStream_t st) {
    const dim3 grid((unsigned)((B + 3) / 4)), block(256);
    switch ((p.K + 511) / 512) {  // (1..3, 5, 6: what wave_per_row lets through)
        case 1: hipLaunchKernelGGL((row_op_wave_kernel<OP, DT, 1, QUANT>), grid, block, 0, st, p, B); break;
        case 2: hipLaunchKernelGGL((row_op_wave_kernel<OP, DT, 2, QUANT>), grid, block, 0, st, p, B); break;
        case 3: hipLaunchKernelGGL((row_op_wave_kernel<OP, DT, 3, QUANT>), grid, block, 0, st, p, B); break;
        case 5: hipLaunchKernelGGL((row_op_wave_kernel<OP, DT, 5, QUANT>), grid, block, 0, st, p, B); break;
        default: hipLaunchKernelGGL((row_op_wave_kernel<OP, DT, 6, QUANT>), grid, block, 0, st, p, B); break;
    }
}

template <int OP, int DT>
static void launch_row_op_dt(const RowOpParams& p, int64_t B, bool fast, hipStream_t st) {
    const dim3 grid((unsigned)B), block(256);
    if (!fast) {
        hipLaunchKernelGGL((row_op_generic_kernel<OP, DT>), grid, block, 0, st, p);
        return;
    }
    if (wave_per_row(B, p.K, p.Q != nullptr)) {
        if (p.Q) launch_row_op_wave<OP, DT, true>(p, B, st);
        else launch_row_op_wave<OP, DT, false>(p, B, st);
        return;
    }
    if (p.Q) launch_row_op_iters<OP, DT, true>(p, grid, block, st);
    else launch_row_op_iters<OP, DT, false>(p, grid, block, st);
}

// op: ROW_SWIGLU / ROW_RMSNORM.  The callers have checked pointers, shapes and dtypes.
int launch_row_op(int op, int dtype, const void* A, int64_t lda, const void* Bv, int64_t ldb, float eps, int64_t B,
                  int64_t K, void* H, int8_t* Q, float* s_x, int q_layout, int32_t* rowsum, hipStream_t st,
                  const char* who) {
    RowOpParams p;
    p.A = A; p.Bv = Bv; p.lda = lda; p.ldb = ldb; p.H = H; p.Q = Q; p.s_x = s_x; p.rowsum = Q ? rowsum : nullptr; p.eps = eps; p.K = (int)K;
    p.q_layout = q_layout;
    const int es = dtype_size(dtype);
    auto aligned = [&](const void* ptr, int64_t ld) { return !ptr || (((uintptr_t)ptr) % 16 == 0 && (ld * es) % 16 == 0); };
    const bool fast = K % 8 == 0 && K <= 16384 && aligned(A, lda) && aligned(Bv, op == ROW_SWIGLU ? ldb : 8) &&
                      aligned(H, K) && (!Q || ((uintptr_t)Q) % 8 == 0) && !option(OPT_ROWOP_GENERIC);
    if (op == ROW_SWIGLU) {
        if (dtype == BT_F32) launch_row_op_dt<ROW_SWIGLU, BT_F32>(p, B, fast, st);
        else if (dtype == BT_F16) launch_row_op_dt<ROW_SWIGLU, BT_F16>(p, B, fast, st);
        else launch_row_op_dt<ROW_SWIGLU, BT_BF16>(p, B, fast, st);
    } else {
        if (dtype == BT_F32) launch_row_op_dt<ROW_RMSNORM, BT_F32>(p, B, fast, st);
        else if (dtype == BT_F16) launch_row_op_dt<ROW_RMSNORM, BT_F16>(p, B, fast, st);
        else launch_row_op_dt<ROW_RMSNORM, BT_BF16>(p, B, fast, st);
    }
    return check_launch(who);
}

}  // namespace bt
