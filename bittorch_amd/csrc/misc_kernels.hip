// Shape-generic kernels: any N, K, B and fp32/fp16/bf16 activations.  They back
// the matrix-core kernels for shapes or alignments those do not take, the
// dense-int8-weight entry point, and the packed -> dense conversion.
// fp32 accumulation runs over k in ascending order, exactly the order of the
// reference kernels (csrc/kernels/ternary_gemm.cu:59-63,
// csrc/kernels/ternary_gemm_production.cu:126-133).
#include "bt_common.h"

namespace bt {

// Y[b,n] = (sum_k x[b,k] * decode(W_T[k/4,n], k%4)) * scale[n] + bias[n]
// One thread per output column, 256 columns per workgroup; grid.y walks the batch rows (any number of them: a
// workgroup takes rows blockIdx.y, blockIdx.y + gridDim.y, ...).
template <int XDT>
__global__ __launch_bounds__(256) void packed_generic_kernel(const void* __restrict__ X,
                                                             const uint8_t* __restrict__ W_T, Epilogue epi,
                                                             void* __restrict__ Y, int64_t B, int64_t N, int64_t K,
                                                             int64_t Kb) {
    const int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (n >= N) return;
    const float s = epi_scale(epi, n), bv = epi_bias(epi, n);
    for (int64_t b = blockIdx.y; b < B; b += gridDim.y) {
        const int64_t xrow = b * K;
        float acc = 0.0f;
        for (int64_t kb = 0; kb < Kb; kb++) {
            const uint32_t byte = W_T[kb * N + n];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int64_t k = 4 * kb + i;
                if (k < K) {
                    const float w = (float)decode2((byte >> (2 * i)) & 3u);
                    acc = __fadd_rn(acc, __fmul_rn(load_elem<XDT>(X, xrow + k), w));
                }
            }
        }
        float y = epi_float(acc, s, bv);
        if (epi.residual) y = add_residual(y, epi.residual, XDT, b * N + n);
        store_elem<XDT>(Y, b * N + n, y);
    }
}

int launch_packed_generic(const void* X, int x_dtype, const uint8_t* W_T, const Epilogue& epi, void* Y,
                          int64_t B, int64_t N, int64_t K, hipStream_t st) {
    const int64_t Kb = ceil_div(K, 4);
    const dim3 grid((unsigned)ceil_div(N, 256), (unsigned)(B < 65535 ? B : 65535)), block(256);
    if (x_dtype == BT_F32)
        hipLaunchKernelGGL(packed_generic_kernel<BT_F32>, grid, block, 0, st, X, W_T, epi, Y, B, N, K, Kb);
    else if (x_dtype == BT_F16)
        hipLaunchKernelGGL(packed_generic_kernel<BT_F16>, grid, block, 0, st, X, W_T, epi, Y, B, N, K, Kb);
    else
        hipLaunchKernelGGL(packed_generic_kernel<BT_BF16>, grid, block, 0, st, X, W_T, epi, Y, B, N, K, Kb);
    return check_launch("packed_generic");
}

// Dense int8 weights W [N,K]: 64 columns x 16 batch rows per workgroup, K in
// tiles of 64 staged through LDS (weights transposed there so that the k loop
// reads conflict-free).
template <int XDT>
__global__ __launch_bounds__(256) void unpacked_kernel(const void* __restrict__ X, const int8_t* __restrict__ W,
                                                       Epilogue epi, void* __restrict__ Y, int64_t B, int64_t N,
                                                       int64_t K) {
    __shared__ float xs[16][64];
    __shared__ int8_t ws[64][68];  // [k][n], padded
    const int nl = threadIdx.x & 63;
    const int bs = threadIdx.x >> 6;  // rows bs*4 .. bs*4+3
    const int64_t n0 = (int64_t)blockIdx.x * 64;
    const int64_t b0 = (int64_t)blockIdx.y * 16;
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int64_t k0 = 0; k0 < K; k0 += 64) {
        for (int idx = threadIdx.x; idx < 16 * 64; idx += 256) {
            const int r = idx >> 6, kk = idx & 63;
            const int64_t b = b0 + r, k = k0 + kk;
            xs[r][kk] = (b < B && k < K) ? load_elem<XDT>(X, b * K + k) : 0.0f;
        }
        for (int idx = threadIdx.x; idx < 64 * 64; idx += 256) {
            const int r = idx >> 6, kk = idx & 63;  // r: column n, kk: k (contiguous in memory)
            const int64_t n = n0 + r, k = k0 + kk;
            ws[kk][r] = (n < N && k < K) ? W[n * K + k] : (int8_t)0;
        }
        __syncthreads();
        const int klim = (K - k0 < 64) ? (int)(K - k0) : 64;
        for (int kk = 0; kk < klim; kk++) {
            const float w = (float)ws[kk][nl];
#pragma unroll
            for (int r = 0; r < 4; r++) acc[r] = __fadd_rn(acc[r], __fmul_rn(xs[bs * 4 + r][kk], w));
        }
        __syncthreads();
    }
    const int64_t n = n0 + nl;
    if (n >= N) return;
    const float s = epi_scale(epi, n);
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int64_t b = b0 + bs * 4 + r;
        if (b >= B) continue;
        // acc *= scale; acc += bias (only when a bias is given)
        float v = __fmul_rn(acc[r], s);
        if (epi.bias) v = __fadd_rn(v, epi_bias(epi, n));
        if (epi.residual) v = add_residual(v, epi.residual, XDT, b * N + n);
        store_elem<XDT>(Y, b * N + n, v);
    }
}

int launch_unpacked(const void* X, int x_dtype, const int8_t* W, const Epilogue& epi, void* Y, int64_t B,
                    int64_t N, int64_t K, hipStream_t st) {
    // one launch covers 65535 blocks of 16 rows; a taller batch is served in slices of that many rows
    const int64_t max_rows = 65535ll * 16;
    if (B > max_rows) {
        const int64_t esz = dtype_size(x_dtype);
        for (int64_t r0 = 0; r0 < B; r0 += max_rows) {
            Epilogue e = epi;
            if (e.residual) e.residual = (const uint8_t*)epi.residual + r0 * N * esz;
            const int rc = launch_unpacked((const uint8_t*)X + r0 * K * esz, x_dtype, W, e, (uint8_t*)Y + r0 * N * esz,
                                           (B - r0 < max_rows) ? B - r0 : max_rows, N, K, st);
            if (rc) return rc;
        }
        return BT_OK;
    }
    const dim3 grid((unsigned)ceil_div(N, 64), (unsigned)ceil_div(B, 16)), block(256);
    if (x_dtype == BT_F32) hipLaunchKernelGGL(unpacked_kernel<BT_F32>, grid, block, 0, st, X, W, epi, Y, B, N, K);
    else if (x_dtype == BT_F16) hipLaunchKernelGGL(unpacked_kernel<BT_F16>, grid, block, 0, st, X, W, epi, Y, B, N, K);
    else hipLaunchKernelGGL(unpacked_kernel<BT_BF16>, grid, block, 0, st, X, W, epi, Y, B, N, K);
    return check_launch("bt_ternary_linear_forward");
}

// out[n, k] = decode(W_T[k/4, n]) * scale[n]   (scale == nullptr: plain decode)
// Tile: 64 columns x 16 kb rows (64 k) through LDS for the transpose.
template <int ODT>
__global__ __launch_bounds__(256) void unpack_dequant_kernel(const uint8_t* __restrict__ W_T,
                                                             const float* __restrict__ scale, int scale_bcast,
                                                             void* __restrict__ out, int64_t N, int64_t K,
                                                             int64_t Kb) {
    __shared__ uint8_t tile[16][65];
    const int64_t n0 = (int64_t)blockIdx.x * 64;
    const int64_t kb0 = (int64_t)blockIdx.y * 16;
    for (int idx = threadIdx.x; idx < 16 * 64; idx += 256) {
        const int r = idx >> 6, c = idx & 63;
        const int64_t kb = kb0 + r, n = n0 + c;
        tile[r][c] = (kb < Kb && n < N) ? W_T[kb * N + n] : (uint8_t)0;
    }
    __syncthreads();
    const int c = threadIdx.x >> 2;     // column within the tile
    const int part = threadIdx.x & 3;   // kb rows part*4 .. part*4+3
    const int64_t n = n0 + c;
    if (n >= N) return;
    const float s = scale ? scale[scale_bcast ? 0 : n] : 1.0f;
    // 16 consecutive k of one output row per thread; the four threads of a column cover 64 k
    float w[16];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const uint32_t byte = tile[part * 4 + r][c];
#pragma unroll
        for (int i = 0; i < 4; i++) w[4 * r + i] = (float)decode2((byte >> (2 * i)) & 3u);
    }
    const int64_t k0 = 4 * (kb0 + part * 4);
    constexpr int OES = (ODT == 3) ? 1 : (ODT == BT_F32) ? 4 : 2;
    uint8_t* dst = (uint8_t*)out + (n * K + k0) * OES;
    if (k0 + 16 <= K && (((uintptr_t)dst) % 16 == 0)) {
        if constexpr (ODT == 3) {
            uint32_t d[4];
#pragma unroll
            for (int q = 0; q < 4; q++)
                d[q] = (uint32_t)(uint8_t)(int8_t)w[4 * q] | ((uint32_t)(uint8_t)(int8_t)w[4 * q + 1] << 8) |
                       ((uint32_t)(uint8_t)(int8_t)w[4 * q + 2] << 16) | ((uint32_t)(uint8_t)(int8_t)w[4 * q + 3] << 24);
            *(uint4*)dst = make_uint4(d[0], d[1], d[2], d[3]);
        } else if constexpr (ODT == BT_F32) {
#pragma unroll
            for (int q = 0; q < 4; q++)
                ((float4*)dst)[q] = make_float4(__fmul_rn(w[4 * q], s), __fmul_rn(w[4 * q + 1], s),
                                                __fmul_rn(w[4 * q + 2], s), __fmul_rn(w[4 * q + 3], s));
        } else {
#pragma unroll
            for (int q = 0; q < 2; q++) {
                uint32_t d[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float a = __fmul_rn(w[8 * q + 2 * e], s), b = __fmul_rn(w[8 * q + 2 * e + 1], s);
                    const uint32_t lo = (ODT == BT_F16) ? f32_to_f16_bits(a) : f32_to_bf16_bits(a);
                    const uint32_t hi = (ODT == BT_F16) ? f32_to_f16_bits(b) : f32_to_bf16_bits(b);
                    d[e] = lo | (hi << 16);
                }
                ((uint4*)dst)[q] = make_uint4(d[0], d[1], d[2], d[3]);
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < 16; i++) {
            if (k0 + i < K) {
                if constexpr (ODT == 3) ((int8_t*)out)[n * K + k0 + i] = (int8_t)w[i];
                else store_elem<ODT>(out, n * K + k0 + i, __fmul_rn(w[i], s));
            }
        }
    }
}

// ---- decode-tiled copy of the packed weights (W_LAYOUT_TILED) -----------------------------------
// One thread per dword of the tiled copy: lane = 16 g + j of step s of tile t collects the bytes of
// rows 16 s + 4 g .. + 3 of column 16 t + j.  The sixteen threads of a g read 16 contiguous bytes per row.
// pairs (N % 32 == 0): tile 2P of the copy is tile P of the matrix, tile 2P + 1 is tile N/32 + P, so that
// column h of the first half (gate) and column h of the second half (up) land in one workgroup.
__device__ __forceinline__ int64_t source_tile(int64_t t, int64_t tiles, int pairs) {
    return pairs ? ((t & 1) ? (tiles >> 1) + (t >> 1) : (t >> 1)) : t;
}

__global__ __launch_bounds__(256) void retile_kernel(const uint8_t* __restrict__ W_T, uint32_t* __restrict__ T,
                                                     int64_t N, int64_t Kb, int64_t S, int64_t total, int pairs) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int lane = (int)(i & 63);
    const int64_t s = (i >> 6) % S, t = source_tile((i >> 6) / S, total / (64 * S), pairs);
    const int64_t n = 16 * t + (lane & 15), kb0 = 16 * s + 4 * (lane >> 4);
    uint32_t d = 0;
    if (n < N) {
#pragma unroll
        for (int r = 0; r < 4; r++)
            if (kb0 + r < Kb) d |= (uint32_t)W_T[(kb0 + r) * N + n] << (8 * r);
    }
    T[i] = d;
}

// the inverse: one thread per byte of W_T
__global__ __launch_bounds__(256) void untile_kernel(const uint32_t* __restrict__ T, uint8_t* __restrict__ W_T,
                                                     int64_t N, int64_t Kb, int64_t S, int pairs) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= N * Kb) return;
    const int64_t kb = i / N, n = i % N;
    int64_t t = n >> 4;  // tile of the matrix -> tile of the copy
    if (pairs) {
        const int64_t half = N >> 5;
        t = (t < half) ? 2 * t : 2 * (t - half) + 1;
    }
    const int64_t idx = (t * S + (kb >> 4)) * 64 + 16 * ((kb & 15) >> 2) + (n & 15);
    W_T[i] = (uint8_t)(T[idx] >> (8 * (kb & 3)));
}

// ---- the field layout of the tiled copy (W_LAYOUT_TILED_FIELDS) ----------------------------------------------------
// One thread per aligned group of four dwords of the tiled copy (columns 4 q .. 4 q + 3 of a tile at one step and row
// group): a transpose of the 2-bit fields inside the group.  In the tiled copy dword t holds column t with the code of
// k = 4 b + c at bits 8 b + 2 c; in the field layout dword c holds, at bits 8 b + 2 t, column t at k = 4 b + c --
// as w + 1 (codes 0 / +1 / -1 -> 1 / 2 / 0) for t < 3 and as w in two's complement (0 / 1 / 3) for t = 3.
__global__ __launch_bounds__(256) void retile_fields_kernel(const uint4* __restrict__ T, uint4* __restrict__ F, int64_t groups) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= groups) return;
    const uint4 in = T[i];
    const uint32_t old[4] = {in.x, in.y, in.z, in.w};
    uint32_t out[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int t = 0; t < 4; t++) {
#pragma unroll
        for (int c = 0; c < 4; c++) {
#pragma unroll
            for (int b = 0; b < 4; b++) {
                const uint32_t code = (old[t] >> (8 * b + 2 * c)) & 3u;  // 0: 0, 1: +1, 2: -1
                const uint32_t f = (t < 3) ? ((code == 1u) ? 2u : (code == 2u) ? 0u : 1u) : ((code == 2u) ? 3u : code);
                out[c] |= f << (8 * b + 2 * t);
            }
        }
    }
    F[i] = make_uint4(out[0], out[1], out[2], out[3]);
}

int launch_retile_fields(const uint8_t* W_tiled, int64_t N, int64_t K, uint8_t* W_fields, hipStream_t st) {
    const int64_t Kb = ceil_div(K, 4), S = ceil_div(Kb, 16);
    const int64_t groups = ceil_div(N, 16) * S * 16;  // 64 dwords per step
    hipLaunchKernelGGL(retile_fields_kernel, dim3((unsigned)ceil_div(groups, 256)), dim3(256), 0, st, (const uint4*)W_tiled,
                       (uint4*)W_fields, groups);
    return check_launch("bt_retile_fields");
}

// forward: W_T [Kb, N] -> T;  inverse: T -> W_out [Kb, N]
int launch_retile(const uint8_t* W_T, int64_t N, int64_t K, int pairs, void* T, bool inverse, uint8_t* W_out, hipStream_t st) {
    const int64_t Kb = ceil_div(K, 4), S = ceil_div(Kb, 16);
    if (!inverse) {
        const int64_t total = ceil_div(N, 16) * S * 64;
        hipLaunchKernelGGL(retile_kernel, dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, st, W_T, (uint32_t*)T, N, Kb, S,
                           total, pairs);
    } else {
        hipLaunchKernelGGL(untile_kernel, dim3((unsigned)ceil_div(N * Kb, 256)), dim3(256), 0, st, (const uint32_t*)T, W_out,
                           N, Kb, S, pairs);
    }
    return check_launch(inverse ? "untile" : "retile");
}

}  // namespace bt

extern "C" int bt_unpack_dequant(const uint8_t* W_T, const float* scale, int64_t scale_len, void* out,
                                 int out_dtype, int64_t N, int64_t K, void* stream) {
    using namespace bt;
    if (!W_T || !out || N <= 0 || K <= 0) {
        set_error("bt_unpack_dequant: null pointer or empty shape");
        return BT_ERR_INVALID;
    }
    if (scale && scale_len != N && scale_len != 1) {
        set_error("bt_unpack_dequant: scale has %lld entries, expected %lld or 1", (long long)scale_len, (long long)N);
        return BT_ERR_INVALID;
    }
    const int64_t Kb = ceil_div(K, 4);
    const dim3 grid((unsigned)ceil_div(N, 64), (unsigned)ceil_div(Kb, 16)), block(256);
    hipStream_t st = (hipStream_t)stream;
    const int bc = (scale_len == 1) ? 1 : 0;
    switch (out_dtype) {
        case BT_F32: hipLaunchKernelGGL(unpack_dequant_kernel<BT_F32>, grid, block, 0, st, W_T, scale, bc, out, N, K, Kb); break;
        case BT_F16: hipLaunchKernelGGL(unpack_dequant_kernel<BT_F16>, grid, block, 0, st, W_T, scale, bc, out, N, K, Kb); break;
        case BT_BF16: hipLaunchKernelGGL(unpack_dequant_kernel<BT_BF16>, grid, block, 0, st, W_T, scale, bc, out, N, K, Kb); break;
        case 3: hipLaunchKernelGGL(unpack_dequant_kernel<3>, grid, block, 0, st, W_T, scale, bc, out, N, K, Kb); break;
        default:
            set_error("bt_unpack_dequant: unsupported output dtype %d", out_dtype);
            return BT_ERR_INVALID;
    }
    return check_launch("bt_unpack_dequant");
}
