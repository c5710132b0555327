// G independent small-batch int8 units in one launch (HBM-bound): unit u multiplies its int8-quantized activation
// rows Q_u [M <= 16, K] (row scales s_x_u [M]) with the decode-tiled ternary weights W_u into Y_u [M, N].
//
// Arithmetic of the reference's tensor-core kernel with the whole-row activation scale
// (csrc/kernels/ternary_gemm_tensor_core.cu:343-347, :439, :583-589, :652), exactly as bt_ternary_gemm_i8_tiled
// computes it for the same unit: acc_i32[m,n] = sum_k q[m,k] * 127 w[k,n] (summed on +-1 weights and multiplied by
// 127 exactly), y = ((float(acc) * s_x[m]) / 127) * scale[n] + bias[n].  Integer sums: the result does not depend
// on how K is split, so every unit equals the single call bit for bit.
//
// The reference serves one matrix per launch (ternary_gemm_production.cu:286-362); a decode-shape matrix streams in
// less time than a kernel takes to start, and at M = 16 a one-matrix kernel re-reads the activations in every
// workgroup (176 KB per workgroup for K = 11008, four times the weight bytes it streams).  Here persistent
// workgroups walk the flat sequence of (unit, 16-column tile) pairs: a workgroup owns a contiguous run of it, its
// waves split K -- wave w reads steps w * SPW .. + SPW - 1 of every tile, SPW * 256 consecutive bytes -- so the
// workgroup reads its share of the weights front to back, the pattern that streams fastest on this chip.  A wave's
// slice of the unit's 16 activation rows is the same for every tile of the unit: it is loaded once per unit into
// SPW * 4 registers, already in matrix-core operand order, and the loop has no activation traffic at all.  The waves'
// partial sums (16 rows x 16 columns of int32 per tile) meet in LDS atomics in one of two accumulator arrays; every
// 16 or 24 tiles a barrier ends the chunk and the threads finish its outputs (epilogue, stores, clearing) while the
// waves already add the next chunk into the other array.  TB tiles of weight loads are in flight per wave at all
// times, across chunk and unit boundaries.
#include <cstddef>

#include "bt_common.h"

namespace bt {

// Tiles per chunk (I8_EB tiles x 16 rows x 16 columns of int32 per accumulator array): 24 with 8 waves, 16 with 16,
// as measured (G = 32 units of 16 x 4096 -> 11008: 16 tiles 80.3 us, 24 tiles 73.6, 30 tiles 77.0; 16 x 11008 -> 4096
// on 16 waves: 77.7, 81.0, 83.4).
template <int WAVES> constexpr int i8_eb() { return WAVES == 8 ? 24 : 16; }

struct I8GroupParams {
    // tables of G device pointers
    const int8_t* const* Q_tab;
    const uint8_t* const* W_tab;
    const float* const* sx_tab;
    const void* const* scale_tab;
    const void* const* bias_tab;  // may be null
    void* const* Y_tab;
    int32_t* const* acc_tab;      // may be null: raw accumulators [M, N] per unit
    int64_t K, N;
    int wsteps;        // 16-row steps of the weights (64 k each)
    int tiles16;       // 16-column tiles
    int G, M;
    int tiles_per_wg;  // a multiple of TB
    int q_operand_order;
    int y_dtype, scale_dtype, bias_dtype, scale_bcast;
};

// A pointer read from one of the tables, pinned to scalar registers (the compiler cannot always prove a table index
// uniform, and a pointer fetched with a vector load costs a wait for all of the wave's outstanding memory operations
// wherever it is first used).  Rebuilt as a pointer into global memory: a bare integer cast would leave the compiler
// with generic-address loads and stores, which wait on two counters and complete out of order.
template <typename T>
__device__ __forceinline__ T* uniform_ptr(T* ptr) {
    const uint64_t v = (uint64_t)(uintptr_t)ptr;
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
    typedef __attribute__((address_space(1))) T* global_ptr;
    return (T*)(global_ptr)(uintptr_t)(((uint64_t)hi << 32) | lo);
}

template <int YDT> struct I8YTag { static constexpr int value = YDT; };

template <int SPW, int TB, int WAVES>
__global__ __launch_bounds__(WAVES * 64, 4) void gemv_i8_walk_kernel(I8GroupParams p) {
    constexpr int I8_EB = i8_eb<WAVES>();
    // Row stride of an accumulator array in ints: 4 past a multiple of 8 puts the four row groups a matrix-core result
    // spreads over the lanes (rows 4g .. 4g+3) on two sets of banks instead of one (G = 32 units as above, 16 tiles
    // per chunk: 87.1 -> 80.3 us).
    constexpr int I8_ROW = I8_EB * 16 + 4;
    static_assert(I8_EB % TB == 0, "chunks hold whole batches");
    constexpr int THREADS = WAVES * 64;
    __shared__ __attribute__((aligned(16))) int32_t accbuf[2][16][I8_ROW];    // [array][row][16 * tile + column]
    // the epilogue's operands of a chunk, staged while the chunk is computed: column scales and biases widened to
    // fp32 (zeros where there is no bias), the unit's row scales
    __shared__ __attribute__((aligned(16))) float ops_s[2][I8_EB * 16], ops_b[2][I8_EB * 16];
    __shared__ float ops_sx[2][16];
    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 15, g = lane >> 4;
    const int S = p.wsteps;
    const int T16 = p.tiles16;
    const int M = p.M;
    const int64_t total = (int64_t)p.G * T16;
    const int64_t t_begin = (int64_t)blockIdx.x * p.tiles_per_wg;
    const int64_t t_end = (t_begin + p.tiles_per_wg < total) ? t_begin + p.tiles_per_wg : total;
    if (t_begin >= t_end) return;

    for (int i = tid; i < 2 * 16 * I8_ROW; i += THREADS) (&accbuf[0][0][0])[i] = 0;

    // byte offset of this wave's SPW steps inside a tile (a step past the end repeats the last one and meets zeroed
    // activations)
    // (wave-uniform step offsets and one per-lane offset: the loads take a scalar base and a 32-bit lane offset)
    uint32_t soff[SPW];
#pragma unroll
    for (int f = 0; f < SPW; f++) soff[f] = (uint32_t)__builtin_amdgcn_readfirstlane(min(wave * SPW + f, S - 1) * 256);
    const uint32_t lane_off = (uint32_t)lane * 4u;
    const size_t tile_bytes = (size_t)S * 256;

    // prefetch cursor: (unit, tile) of the next tile to request
    int pf_u = (int)(t_begin / T16);
    int pf_t = (int)(t_begin - (int64_t)pf_u * T16);
    int64_t pf_left = t_end - t_begin;
    const uint8_t* pf_ptr = uniform_ptr(p.W_tab[pf_u]) + (size_t)pf_t * tile_bytes;
    uint32_t raw[TB][SPW];
    auto request = [&](uint32_t (&dst)[SPW]) {
        // (past the end of the run: the last tile again, never used)
#pragma unroll
        for (int f = 0; f < SPW; f++) dst[f] = ldw_nt((pf_ptr + soff[f]) + lane_off);
        if (pf_left > 1) {
            pf_left--;
            pf_t++;
            pf_ptr += tile_bytes;
            if (pf_t == T16) {
                pf_t = 0;
                pf_u++;
                pf_ptr = uniform_ptr(p.W_tab[pf_u]);
            }
        }
    };
    // A fragment of step f: lane (i = j, g) feeds row i, k = 64 step + 16 g .. + 15 (rows past M repeat the last row
    // and only reach outputs that are never stored; K is a multiple of 16, so a group below K lies inside its row)
    const uint32_t a_row = (uint32_t)min(j, M - 1) * (uint32_t)p.K;
    uint4 areg[SPW];
    auto load_a = [&](const int8_t* q) {
#pragma unroll
        for (int f = 0; f < SPW; f++) {
            const int k = (wave * SPW + f) * 64 + 16 * g;
            areg[f] = *(const uint4*)(q + a_row + (uint32_t)min(k, (int)p.K - 16));
        }
    };
    auto finish_a = [&]() {
#pragma unroll
        for (int f = 0; f < SPW; f++) {
            const int k = (wave * SPW + f) * 64 + 16 * g;
            uint4 v = areg[f];
            if (!p.q_operand_order) {  // (uniform) row-major bytes -> the matrix cores' order
                uint32_t t[4];
                transpose4x4_bytes(v.x, v.y, v.z, v.w, t);
                v = make_uint4(t[0], t[1], t[2], t[3]);
            }
            const bool ok = k < (int)p.K;
            areg[f] = make_uint4(ok ? v.x : 0u, ok ? v.y : 0u, ok ? v.z : 0u, ok ? v.w : 0u);
        }
    };
    // the first unit's activations are requested ahead of the weights (loads return in order; they are needed first)
    load_a(uniform_ptr(p.Q_tab[pf_u]));
#pragma unroll
    for (int i = 0; i < TB; i++) request(raw[i]);

    int cur = 0;
    __syncthreads();  // accumulators cleared

    int64_t t0 = t_begin;
    while (t0 < t_end) {
        const int u = __builtin_amdgcn_readfirstlane((int)(t0 / T16));
        const int tile0 = __builtin_amdgcn_readfirstlane((int)(t0 - (int64_t)u * T16));
        if (t0 != t_begin) load_a(uniform_ptr(p.Q_tab[u]));  // (uniform)
        finish_a();
        // the unit's pointers, once per unit and in scalar registers
        const float* sx_u = uniform_ptr(p.sx_tab[u]);
        const void* scale_u = uniform_ptr(p.scale_tab[u]);
        const void* bias_u = p.bias_tab ? uniform_ptr(p.bias_tab[u]) : nullptr;
        void* const y_u = uniform_ptr(p.Y_tab[u]);
        int32_t* const acc_u = p.acc_tab ? uniform_ptr(p.acc_tab[u]) : nullptr;
        // whole four-column pieces leave as vector stores: rows of N % 8 == 0 columns from 16-byte aligned bases
        const bool vec_u = (p.N & 7) == 0 && (((uintptr_t)y_u) & 15) == 0 && (((uintptr_t)acc_u) & 15) == 0;
        const int64_t unit_end = (int64_t)(u + 1) * T16;
        const int64_t u_stop = (unit_end < t_end) ? unit_end : t_end;
        for (int64_t c0 = t0; c0 < u_stop; c0 += I8_EB) {
            const int ntiles = (int)((u_stop - c0 < I8_EB) ? u_stop - c0 : I8_EB);  // a multiple of TB
            const int ctile = tile0 + (int)(c0 - t0);
            // The epilogue's operands are requested now, one column per thread, and parked in LDS at the end of the chunk:
            // the epilogue itself then waits for nothing but LDS.  (Requested by the epilogue's own threads after the
            // barrier they left every wave waiting on memory once per chunk; held in registers per output piece across
            // the chunk's matrix instructions they spilled.)
            uint32_t st_s = 0u, st_b = 0u;
            float st_sx = 0.0f;
            {
                const int64_t n = (int64_t)ctile * 16 + tid;
                if (tid < ntiles * 16 && n < p.N) {
                    st_s = load_bits_rt(scale_u, p.scale_dtype, p.scale_bcast ? 0 : n);
                    if (bias_u) st_b = load_bits_rt(bias_u, p.bias_dtype, n);
                }
                if (tid < 16) st_sx = sx_u[min(tid, M - 1)];
            }
            for (int tb = 0; tb < ntiles; tb += TB) {
                v4i acc[TB];
#pragma unroll
                for (int i = 0; i < TB; i++) acc[i] = v4i{0, 0, 0, 0};
#pragma unroll
                for (int f = 0; f < SPW; f++) {
                    const v4i a = {(int)areg[f].x, (int)areg[f].y, (int)areg[f].z, (int)areg[f].w};
#pragma unroll
                    for (int i = 0; i < TB; i++)
                        acc[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, decode16_i8(raw[i][f]), acc[i], 0, 0, 0);
                }
#pragma unroll
                for (int i = 0; i < TB; i++) request(raw[i]);
                // lane (j, g) holds rows 4g .. 4g+3 of column j
#pragma unroll
                for (int i = 0; i < TB; i++) {
#pragma unroll
                    for (int r = 0; r < 4; r++) atomicAdd(&accbuf[cur][4 * g + r][16 * (tb + i) + j], acc[i][r]);
                }
            }
            if (tid < I8_EB * 16) {
                ops_s[cur][tid] = bits_to_f32_rt(st_s, p.scale_dtype);
                ops_b[cur][tid] = bias_u ? bits_to_f32_rt(st_b, p.bias_dtype) : 0.0f;
            }
            if (tid < 16) ops_sx[cur][tid] = st_sx;
            __syncthreads();  // every wave has added its share of this chunk
            // The chunk's epilogue: 16 rows x (16 * tiles) columns in pieces of four columns (an 8-byte piece of a 16-bit
            // output row; consecutive threads cover a row's columns with full-line stores), in passes over the threads.
            // The operands arrive widened to fp32 and the output's type is decided once per chunk, so the loop is the
            // arithmetic and one store (about 60 instructions per piece).
            auto pieces = [&](auto ytag) {
                constexpr int YDT = decltype(ytag)::value;
#pragma unroll 1
                for (int item = tid; item < I8_EB * 64; item += THREADS) {
                    const int e_row = item / (4 * I8_EB);
                    const int col0 = (item - e_row * (4 * I8_EB)) * 4;  // first column of the piece inside the chunk
                    if (col0 >= ntiles * 16) continue;
                    int32_t* src = &accbuf[cur][e_row][col0];
                    const int4 v = *(const int4*)src;
                    *(int4*)src = make_int4(0, 0, 0, 0);
                    const int64_t n0 = (int64_t)ctile * 16 + col0;
                    if (n0 >= p.N || e_row >= M) continue;
                    const float4 s4 = *(const float4*)&ops_s[cur][col0], b4 = *(const float4*)&ops_b[cur][col0];
                    const float pre_sx = ops_sx[cur][e_row];
                    const int32_t a127[4] = {times127(v.x), times127(v.y), times127(v.z), times127(v.w)};  // +-1 weights
                    const float y[4] = {epi_int8(a127[0], pre_sx, s4.x, b4.x), epi_int8(a127[1], pre_sx, s4.y, b4.y),
                                        epi_int8(a127[2], pre_sx, s4.z, b4.z), epi_int8(a127[3], pre_sx, s4.w, b4.w)};
                    const int64_t idx = (int64_t)e_row * p.N + n0;
                    if (vec_u) {
                        if constexpr (YDT == BT_F32) {
                            st4_nt((float*)y_u + idx, __builtin_bit_cast(uint32_t, y[0]), __builtin_bit_cast(uint32_t, y[1]),
                                   __builtin_bit_cast(uint32_t, y[2]), __builtin_bit_cast(uint32_t, y[3]));
                        } else if constexpr (YDT == BT_F16) {
                            st2_nt((uint16_t*)y_u + idx, f32_to_f16_bits(y[0]) | ((uint32_t)f32_to_f16_bits(y[1]) << 16),
                                   f32_to_f16_bits(y[2]) | ((uint32_t)f32_to_f16_bits(y[3]) << 16));
                        } else {
                            st2_nt((uint16_t*)y_u + idx, f32_to_bf16_bits(y[0]) | ((uint32_t)f32_to_bf16_bits(y[1]) << 16),
                                   f32_to_bf16_bits(y[2]) | ((uint32_t)f32_to_bf16_bits(y[3]) << 16));
                        }
                        if (acc_u) st4_nt(acc_u + idx, (uint32_t)a127[0], (uint32_t)a127[1], (uint32_t)a127[2], (uint32_t)a127[3]);
                    } else {
#pragma unroll
                        for (int c = 0; c < 4; c++) {
                            if (n0 + c < p.N) {
                                store_elem<YDT>(y_u, idx + c, y[c]);
                                if (acc_u) acc_u[idx + c] = a127[c];
                            }
                        }
                    }
                }
            };
            if (p.y_dtype == BT_F32) pieces(I8YTag<BT_F32>{});
            else if (p.y_dtype == BT_F16) pieces(I8YTag<BT_F16>{});
            else pieces(I8YTag<BT_BF16>{});
            cur ^= 1;
        }
        t0 = u_stop;
    }
}

// ---- host side ------------------------------------------------------------------------------------------------------
static int64_t i8g_compute_units() {
    static int cus = 0;
    if (!cus) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
        cus = n;
    }
    return cus;
}

template <int SPW, int WAVES>
static void launch_i8_walk_tb(const I8GroupParams& p, int tb, unsigned grid, hipStream_t st) {
    if (tb == 2) hipLaunchKernelGGL((gemv_i8_walk_kernel<SPW, 2, WAVES>), dim3(grid), dim3(WAVES * 64), 0, st, p);
    else hipLaunchKernelGGL((gemv_i8_walk_kernel<SPW, 1, WAVES>), dim3(grid), dim3(WAVES * 64), 0, st, p);
}

// K up to 4096 (64 steps): 8 waves, two workgroups per compute unit; up to 11264 (176 steps): 16 waves, one.
bool i8_group_supported(int64_t K) { return K % 16 == 0 && K >= 16 && K <= 11264; }

int launch_i8_group(const int8_t* const* Q_tab, int q_layout, const float* const* sx_tab, const uint8_t* const* W_tab,
                    const void* const* scale_tab, int scale_dtype, int scale_bcast, const void* const* bias_tab,
                    int bias_dtype, void* const* Y_tab, int y_dtype, int32_t* const* acc_tab, int64_t G, int64_t M,
                    int64_t N, int64_t K, hipStream_t st) {
    I8GroupParams p = {};
    p.Q_tab = Q_tab; p.W_tab = W_tab; p.sx_tab = sx_tab; p.scale_tab = scale_tab; p.bias_tab = bias_tab;
    p.Y_tab = Y_tab; p.acc_tab = acc_tab;
    p.K = K; p.N = N;
    p.wsteps = (int)ceil_div(ceil_div(K, 4), 16);
    p.tiles16 = (int)ceil_div(N, 16);
    p.G = (int)G; p.M = (int)M;
    p.q_operand_order = q_layout == Q_OPERAND_ORDER;
    p.y_dtype = y_dtype; p.scale_dtype = scale_dtype; p.bias_dtype = bias_dtype; p.scale_bcast = scale_bcast;
    const bool wide = p.wsteps > 64;
    const int waves = wide ? 16 : 8;
    const int spw = (int)ceil_div(p.wsteps, waves);
    const int tb = (p.tiles16 % 2 == 0) ? 2 : 1;  // chunks inside a unit hold whole batches of tiles
    const int64_t wgs = (wide ? 1 : 2) * i8g_compute_units();
    const int64_t total = G * p.tiles16;
    const int64_t tpw = ceil_div(ceil_div(total, wgs), tb) * tb;
    p.tiles_per_wg = (int)tpw;
    const unsigned grid = (unsigned)ceil_div(total, tpw);
#define BT_I8G_CASE(SPW, WAVES) case SPW: launch_i8_walk_tb<SPW, WAVES>(p, tb, grid, st); break;
    if (!wide) {
        switch (spw) {
            BT_I8G_CASE(1, 8) BT_I8G_CASE(2, 8) BT_I8G_CASE(3, 8) BT_I8G_CASE(4, 8)
            BT_I8G_CASE(5, 8) BT_I8G_CASE(6, 8) BT_I8G_CASE(7, 8)
            default: launch_i8_walk_tb<8, 8>(p, tb, grid, st); break;
        }
    } else {
        switch (spw) {
            BT_I8G_CASE(5, 16) BT_I8G_CASE(6, 16) BT_I8G_CASE(7, 16) BT_I8G_CASE(8, 16)
            BT_I8G_CASE(9, 16) BT_I8G_CASE(10, 16)
            default: launch_i8_walk_tb<11, 16>(p, tb, grid, st); break;
        }
    }
#undef BT_I8G_CASE
    return check_launch("bt_ternary_gemm_i8_grouped");
}

}  // namespace bt
