// Decode-shape / small-batch packed-ternary GEMM for gfx950: streams the 2-bit
// weights W_T [Kb, N] from HBM once, decodes them in registers and feeds the
// matrix cores.  Rows of activations per launch: M <= 16 (one MFMA row block).
//
// Arithmetic restated from the reference kernels:
//   float path (csrc/kernels/ternary_gemm_production.cu:126-141):
//       acc_f32 = sum_k x[b,k] * w[k,n];  y = acc * scale[n] + bias[n]
//   int8 path (csrc/kernels/ternary_gemm_tensor_core.cu:583-589, :652):
//       acc_i32 = sum_k q[b,k] * (127 w[k,n]);  y = (acc * s_x[b] / 127) * scale[n] + bias[n]
//
// Work decomposition.  A wave "step" covers RS consecutive kb rows (16 for int8,
// 8 for 16-bit floats) and 16*NW output columns: lane (j = lane%16, g = lane/16)
// loads NW consecutive bytes (one dword, two, or four: a 128-bit load) from each
// of the KBG = RS/4 rows kb0 + g*KBG + r.  Those bytes are the B operands of NW
// MFMA instructions: MFMA t multiplies the 16 activation rows with output columns
// n = nb + NW*j + t.  The k order inside an MFMA is free as long as both operands
// agree, so the activation fragments are laid out once per workgroup (in LDS) in
// the order the cheapest weight decode produces.
// A workgroup covers one column tile and one slice of K (grid.y = split-K); its
// waves take steps round-robin and their accumulators are summed through LDS in
// a fixed order.  With split-K > 1 the per-slice sums go to a workspace and a
// second kernel adds them, again in a fixed order, and applies the epilogue.
#include "bt_common.h"

namespace bt {

struct StreamParams {
    const void* X;        // MODE_I8: int8 [M,K]; else 16-bit activations [M,K]
    const uint8_t* W_T;   // [Kb, N]
    const float* s_x;     // MODE_I8: per-row activation scales [M]
    void* Y;              // [M, N] of y_dtype
    int32_t* acc_out;     // MODE_I8, optional raw accumulators [M, N]
    void* partial;        // [S][M][N] 32-bit words when S > 1
    Epilogue epi;
    int64_t N, K, Kb;
    int64_t kb_per_split; // multiple of RS
    int M;                // 1..16
    int y_dtype;
    int x_vec_ok;         // activations may be read with 16-byte loads
};

template <int NW> struct RawVec;
template <> struct RawVec<16> { typedef uint4 type; };
template <> struct RawVec<8> { typedef uint2 type; };
template <> struct RawVec<4> { typedef uint32_t type; };

template <int NW>
__device__ __forceinline__ void load_raw(const uint8_t* p, bool ok, uint32_t (&d)[NW / 4]) {
    if (ok) {
        typename RawVec<NW>::type v = *(const typename RawVec<NW>::type*)p;
        __builtin_memcpy(d, &v, NW);
    } else {
#pragma unroll
        for (int i = 0; i < NW / 4; i++) d[i] = 0u;
    }
}

__device__ __forceinline__ void store_out(void* Y, int dt, int64_t idx, float v) {
    if (dt == BT_F32) ((float*)Y)[idx] = v;
    else if (dt == BT_F16) ((uint16_t*)Y)[idx] = f32_to_f16_bits(v);
    else ((uint16_t*)Y)[idx] = f32_to_bf16_bits(v);
}

template <int MODE>
__device__ __forceinline__ void finish_output(const StreamParams& p, int row, int64_t n, uint32_t bits) {
    const float s = epi_scale(p.epi, n);
    const float b = epi_bias(p.epi, n);
    float y;
    if constexpr (MODE == MODE_I8) {
        const int32_t acc127 = (int32_t)bits * 127;  // MFMA ran on +-1 weights
        if (p.acc_out) p.acc_out[(int64_t)row * p.N + n] = acc127;
        y = epi_int8(acc127, p.s_x[row], s, b);
    } else if constexpr (MODE == MODE_F16) {
        y = epi_float(__builtin_bit_cast(float, bits), s, b);
    } else {
        // bf16 weights were decoded as +-2.0 (low byte zero): undo exactly
        y = epi_float(__builtin_bit_cast(float, bits) * 0.5f, s, b);
    }
    store_out(p.Y, p.y_dtype, (int64_t)row * p.N + n, y);
}

template <int MODE, int NW, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void stream_kernel(StreamParams p) {
    constexpr int KBG = (MODE == MODE_I8) ? 4 : 2;  // kb rows per lane group
    constexpr int RS = 4 * KBG;                     // kb rows per wave step
    constexpr int GE = (MODE == MODE_I8) ? 16 : 8;  // activation elements per group
    constexpr int TILE_N = 16 * NW;
    constexpr int ND = NW / 4;
    typedef typename std::conditional<MODE == MODE_I8, v4i, v4f>::type acc_t;

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int j = lane & 15;
    const int g = lane >> 4;
    const int64_t nb = (int64_t)blockIdx.x * TILE_N;
    const int64_t kb0 = (int64_t)blockIdx.y * p.kb_per_split;
    const int64_t kb1 = (kb0 + p.kb_per_split < p.Kb) ? kb0 + p.kb_per_split : p.Kb;
    const int nsteps = (int)((kb1 - kb0 + RS - 1) / RS);
    const int64_t ncol = nb + (int64_t)NW * j;
    const bool col_ok = ncol < p.N;

    uint32_t raw[KBG][ND];
    auto load_step = [&](int step) {
#pragma unroll
        for (int r = 0; r < KBG; r++) {
            const int64_t kb = kb0 + (int64_t)step * RS + g * KBG + r;
            load_raw<NW>(p.W_T + kb * p.N + ncol, col_ok && kb < kb1, raw[r]);
        }
    };

    // weights first: their HBM latency overlaps the activation staging below
    int step = wave;
    if (step < nsteps) load_step(step);

    // ---- stage the activation fragments of this K slice into LDS --------------
    // slot (step s, lane l = gl*16 + i) holds the 16 bytes lane l feeds to the MFMA
    // in step s: row i, group gl, elements in decode order.
    {
        const int ngroups = nsteps * 4;
        const int64_t k_base = 4 * kb0;
        for (int idx = threadIdx.x; idx < ngroups * 16; idx += WAVES * 64) {
            const int i = idx & 15;
            const int gidx = idx >> 4;
            const int64_t k = k_base + (int64_t)gidx * GE;
            uint32_t d[4] = {0u, 0u, 0u, 0u};
            if (i < p.M && k < p.K) {
                if constexpr (MODE == MODE_I8) {
                    const int8_t* src = (const int8_t*)p.X + (int64_t)i * p.K + k;
                    if (p.x_vec_ok && k + 16 <= p.K) {
                        const uint4 v = *(const uint4*)src;
                        d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
                    } else {
                        for (int e = 0; e < 16; e++)
                            if (k + e < p.K) d[e >> 2] |= (uint32_t)(uint8_t)src[e] << (8 * (e & 3));
                    }
                    uint32_t t[4];
                    transpose4x4_bytes(d[0], d[1], d[2], d[3], t);
                    d[0] = t[0]; d[1] = t[1]; d[2] = t[2]; d[3] = t[3];
                } else {
                    const uint16_t* src = (const uint16_t*)p.X + (int64_t)i * p.K + k;
                    if (p.x_vec_ok && k + 8 <= p.K) {
                        const uint4 v = *(const uint4*)src;
                        d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
                    } else {
                        for (int e = 0; e < 8; e++)
                            if (k + e < p.K) d[e >> 1] |= (uint32_t)src[e] << (16 * (e & 1));
                    }
                    // natural halves h0..h7 -> dword c = { h[c], h[4+c] }
                    const uint32_t o0 = perm(d[2], d[0], 0x05040100u);
                    const uint32_t o1 = perm(d[2], d[0], 0x07060302u);
                    const uint32_t o2 = perm(d[3], d[1], 0x05040100u);
                    const uint32_t o3 = perm(d[3], d[1], 0x07060302u);
                    d[0] = o0; d[1] = o1; d[2] = o2; d[3] = o3;
                }
            }
            const int s = gidx >> 2, gl = gidx & 3;
            *(uint4*)(smem + ((size_t)(s * 64 + gl * 16 + i) << 4)) = make_uint4(d[0], d[1], d[2], d[3]);
        }
    }
    __syncthreads();

    acc_t acc[NW];
#pragma unroll
    for (int t = 0; t < NW; t++) acc[t] = acc_t{0, 0, 0, 0};

    while (step < nsteps) {
        uint32_t cur[KBG][ND];
#pragma unroll
        for (int r = 0; r < KBG; r++)
#pragma unroll
            for (int d = 0; d < ND; d++) cur[r][d] = raw[r][d];
        const int next = step + WAVES;
        if (next < nsteps) load_step(next);

        const uint4 av = *(const uint4*)(smem + ((size_t)(step * 64 + lane) << 4));
#pragma unroll
        for (int d = 0; d < ND; d++) {
            if constexpr (MODE == MODE_I8) {
                const v4i a = {(int)av.x, (int)av.y, (int)av.z, (int)av.w};
                uint32_t G[4];
                transpose4x4_bytes(cur[0][d], cur[1][d], cur[2][d], cur[3][d], G);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const v4i b = decode16_i8(G[i]);
                    acc[4 * d + i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc[4 * d + i], 0, 0, 0);
                }
            } else {
                const u32x4 au = {av.x, av.y, av.z, av.w};
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    // bytes: [zero, row0.byte i, zero, row1.byte i]
                    const uint32_t sel = ((uint32_t)(4 + i) << 24) | (0x0Cu << 16) | ((uint32_t)i << 8) | 0x0Cu;
                    const uint32_t M2 = perm(cur[1][d], cur[0][d], sel);
                    if constexpr (MODE == MODE_F16) {
                        const u32x4 bu = decode8_16bit<LUT_F16_ONE>(M2);
                        acc[4 * d + i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                            __builtin_bit_cast(v8h, au), __builtin_bit_cast(v8h, bu), acc[4 * d + i], 0, 0, 0);
                    } else {
                        const u32x4 bu = decode8_16bit<LUT_BF16_TWO>(M2);
                        acc[4 * d + i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            __builtin_bit_cast(v8bf, au), __builtin_bit_cast(v8bf, bu), acc[4 * d + i], 0, 0, 0);
                    }
                }
            }
        }
        step = next;
    }

    // ---- sum the waves' accumulators through LDS (fixed order) -------------------
    // red[row][t*16 + j] (32-bit words); lane (j, g) holds rows 4g..4g+3 of column t*16+j
    __syncthreads();  // every wave is done reading the activation stage
    uint32_t* red = (uint32_t*)smem;
    for (int w = 0; w < WAVES; w++) {
        if (wave == w) {
#pragma unroll
            for (int t = 0; t < NW; t++) {
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int row = 4 * g + r;
                    if (row < p.M) {
                        uint32_t* slot = red + row * TILE_N + t * 16 + j;
                        if constexpr (MODE == MODE_I8) {
                            const int32_t v = acc[t][r] + (w == 0 ? 0 : (int32_t)*slot);
                            *slot = (uint32_t)v;
                        } else {
                            const float v = (w == 0) ? acc[t][r] : __fadd_rn(__builtin_bit_cast(float, *slot), acc[t][r]);
                            *slot = __builtin_bit_cast(uint32_t, v);
                        }
                    }
                }
            }
        }
        __syncthreads();
    }

    // ---- write out: final values (no split-K) or this slice's partial sums ---------
    for (int idx = threadIdx.x; idx < p.M * TILE_N; idx += WAVES * 64) {
        const int row = idx / TILE_N;
        const int nl = idx % TILE_N;
        const int64_t n = nb + nl;
        if (n >= p.N) continue;
        const uint32_t bits = red[row * TILE_N + (nl % NW) * 16 + nl / NW];
        if (gridDim.y == 1) {
            finish_output<MODE>(p, row, n, bits);
        } else {
            ((uint32_t*)p.partial)[((int64_t)blockIdx.y * p.M + row) * p.N + n] = bits;
        }
    }
}

// Adds the S slices of split-K in slice order and applies the epilogue.
template <int MODE>
__global__ __launch_bounds__(256) void stream_reduce_kernel(StreamParams p, int S) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (int64_t)p.M * p.N) return;
    const int row = (int)(idx / p.N);
    const int64_t n = idx % p.N;
    const uint32_t* part = (const uint32_t*)p.partial;
    uint32_t bits;
    if constexpr (MODE == MODE_I8) {
        int32_t v = 0;
        for (int s = 0; s < S; s++) v += (int32_t)part[((int64_t)s * p.M + row) * p.N + n];
        bits = (uint32_t)v;
    } else {
        float v = __builtin_bit_cast(float, part[(int64_t)row * p.N + n]);
        for (int s = 1; s < S; s++)
            v = __fadd_rn(v, __builtin_bit_cast(float, part[((int64_t)s * p.M + row) * p.N + n]));
        bits = __builtin_bit_cast(uint32_t, v);
    }
    finish_output<MODE>(p, row, n, bits);
}

// ---- host side --------------------------------------------------------------------

struct StreamPlan {
    int nw;       // bytes per lane per row: 16, 8 or 4
    int waves;    // waves per workgroup
    int splits;   // split-K factor S
    int64_t kb_per_split;
};

static int rs_of(int mode) { return mode == MODE_I8 ? 16 : 8; }

// Largest K slice whose activation stage fits a 64 KiB LDS allocation: 64 steps.
static const int kMaxStepsPerWG = 64;

bool stream_supported(int64_t N, const void* W_T) {
    return N % 4 == 0 && ((uintptr_t)W_T) % 16 == 0;
}

StreamPlan stream_plan(int mode, int64_t N, int64_t Kb) {
    StreamPlan pl;
    const int rs = rs_of(mode);
    // optional override for tuning runs: BITTORCH_STREAM_CFG="nw,waves,splits"
    int o_nw = 0, o_waves = 0, o_splits = 0;
    if (const char* env = getenv("BITTORCH_STREAM_CFG")) sscanf(env, "%d,%d,%d", &o_nw, &o_waves, &o_splits);

    int nw = (N % 16 == 0) ? 16 : (N % 8 == 0) ? 8 : 4;
    if (o_nw == 16 || o_nw == 8 || o_nw == 4) {
        if (N % o_nw == 0) nw = o_nw;
    } else {
        // narrow the column tile until there are enough workgroups to cover the chip
        // without an excessive split-K (whose partial sums cost extra traffic)
        while (nw > 4 && ceil_div(N, 16 * nw) * ceil_div(Kb, (int64_t)rs * 8) < 512) nw >>= 1;
    }
    pl.nw = nw;
    pl.waves = (o_waves == 2 || o_waves == 4 || o_waves == 8 || o_waves == 16) ? o_waves : 4;
    const int64_t tiles = ceil_div(N, 16 * (int64_t)nw);
    const int64_t steps = ceil_div(Kb, rs);
    int64_t splits;
    if (o_splits > 0) {
        splits = o_splits;
    } else {
        // aim for ~2 workgroups per CU, but keep at least `waves` steps per workgroup
        splits = ceil_div(512, tiles);
        const int64_t max_splits = std::max<int64_t>(1, steps / pl.waves);
        if (splits > max_splits) splits = max_splits;
    }
    const int64_t min_splits = ceil_div(steps, kMaxStepsPerWG);
    if (splits < min_splits) splits = min_splits;
    if (splits > steps) splits = steps;
    if (splits < 1) splits = 1;
    int64_t steps_per = ceil_div(steps, splits);
    pl.kb_per_split = steps_per * rs;
    pl.splits = (int)ceil_div(Kb, pl.kb_per_split);
    return pl;
}

size_t stream_workspace_bytes(int mode, int64_t M, int64_t N, int64_t Kb) {
    // sized for the default plan and for any override (splits <= steps)
    const StreamPlan pl = stream_plan(mode, N, Kb);
    const int64_t rows = M < 16 ? M : 16;
    return pl.splits > 1 ? (size_t)pl.splits * rows * N * 4 : 0;
}

template <int MODE, int NW>
static void launch_stream_w(const StreamParams& p, const StreamPlan& pl, dim3 grid, size_t lds, hipStream_t st) {
    switch (pl.waves) {
        case 2: hipLaunchKernelGGL((stream_kernel<MODE, NW, 2>), grid, dim3(128), lds, st, p); break;
        case 8: hipLaunchKernelGGL((stream_kernel<MODE, NW, 8>), grid, dim3(512), lds, st, p); break;
        case 16: hipLaunchKernelGGL((stream_kernel<MODE, NW, 16>), grid, dim3(1024), lds, st, p); break;
        default: hipLaunchKernelGGL((stream_kernel<MODE, NW, 4>), grid, dim3(256), lds, st, p); break;
    }
}

template <int MODE>
static int launch_stream_mode(StreamParams p, const StreamPlan& pl, void* workspace, size_t ws_bytes,
                              hipStream_t st) {
    const int rs = rs_of(MODE);
    const int64_t tile_n = 16 * (int64_t)pl.nw;
    const dim3 grid((unsigned)ceil_div(p.N, tile_n), (unsigned)pl.splits);
    const int nsteps = (int)ceil_div(pl.kb_per_split, rs);
    size_t lds = (size_t)nsteps * 1024;
    const size_t red = (size_t)16 * tile_n * 4;
    if (lds < red) lds = red;
    p.kb_per_split = pl.kb_per_split;
    if (pl.splits > 1) {
        const size_t need = (size_t)pl.splits * p.M * p.N * 4;
        if (!workspace || ws_bytes < need) {
            set_error("packed forward: workspace of %zu bytes needed, %zu given", need, ws_bytes);
            return BT_ERR_WORKSPACE;
        }
        p.partial = workspace;
    }
    switch (pl.nw) {
        case 16: launch_stream_w<MODE, 16>(p, pl, grid, lds, st); break;
        case 8: launch_stream_w<MODE, 8>(p, pl, grid, lds, st); break;
        default: launch_stream_w<MODE, 4>(p, pl, grid, lds, st); break;
    }
    if (pl.splits > 1) {
        const int64_t total = (int64_t)p.M * p.N;
        hipLaunchKernelGGL((stream_reduce_kernel<MODE>), dim3((unsigned)ceil_div(total, 256)), dim3(256), 0,
                           st, p, pl.splits);
    }
    return check_launch("stream_gemm");
}

// One launch group per block of up to 16 activation rows.
int launch_stream(int mode, const void* X, int x_elem_size, const float* s_x, const uint8_t* W_T,
                  const Epilogue& epi, void* Y, int y_dtype, int32_t* acc_out, int64_t B, int64_t N,
                  int64_t K, void* workspace, size_t ws_bytes, hipStream_t st) {
    const int64_t Kb = ceil_div(K, 4);
    const StreamPlan pl = stream_plan(mode, N, Kb);
    const int y_size = dtype_size(y_dtype);
    for (int64_t m0 = 0; m0 < B; m0 += 16) {
        StreamParams p;
        p.X = (const uint8_t*)X + m0 * K * x_elem_size;
        p.W_T = W_T;
        p.s_x = s_x ? s_x + m0 : nullptr;
        p.Y = (uint8_t*)Y + m0 * N * y_size;
        p.acc_out = acc_out ? acc_out + m0 * N : nullptr;
        p.partial = nullptr;
        p.epi = epi;
        p.N = N; p.K = K; p.Kb = Kb;
        p.kb_per_split = pl.kb_per_split;
        p.M = (int)((B - m0 < 16) ? (B - m0) : 16);
        p.y_dtype = y_dtype;
        p.x_vec_ok = (((uintptr_t)p.X) % 16 == 0) && ((K * x_elem_size) % 16 == 0);
        int rc;
        if (mode == MODE_I8) rc = launch_stream_mode<MODE_I8>(p, pl, workspace, ws_bytes, st);
        else if (mode == MODE_F16) rc = launch_stream_mode<MODE_F16>(p, pl, workspace, ws_bytes, st);
        else rc = launch_stream_mode<MODE_BF16>(p, pl, workspace, ws_bytes, st);
        if (rc != BT_OK) return rc;
    }
    return BT_OK;
}

}  // namespace bt
