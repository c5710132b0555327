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
// loads NW consecutive bytes (a byte, a short, a dword, two or four dwords) from
// each of the KBG = RS/4 rows kb0 + g*KBG + r.  Those bytes are the B operands of
// NW MFMA instructions: MFMA t multiplies the 16 activation rows with output
// columns n = nb + NW*j + t.  The k order inside an MFMA is free as long as both
// operands agree, so each lane loads its 16 bytes of activations (row i = lane%16,
// the same k range as its weights) straight from global memory and permutes them
// into the order the cheapest weight decode produces.
// A wave issues the loads of PF steps before it computes any of them, which is
// what keeps enough bytes in flight to cover the HBM latency.
// A workgroup owns one column tile over the WHOLE of K: there is no split-K
// across workgroups, hence no partial sums in memory, no second pass and no
// inter-workgroup synchronisation.  The tile width is chosen so that there are
// enough tiles for every CU (down to 16 columns, one byte per lane and row);
// tiles that share 128-byte lines of W_T are placed on the same XCD so the
// line is fetched from HBM once.  The waves of a workgroup take steps
// round-robin and their accumulators are summed through LDS in wave order.
#include "bt_common.h"

namespace bt {

struct StreamParams {
    const void* X;        // MODE_I8: int8 [M,K]; else 16-bit activations [M,K]
    const uint8_t* W_T;   // [Kb, N]
    const float* s_x;     // MODE_I8: per-row activation scales [M]
    void* Y;              // [M, N] of y_dtype
    int32_t* acc_out;     // MODE_I8, optional raw accumulators [M, N]
    Epilogue epi;
    int64_t N, K, Kb;
    int tiles;            // column tiles
    int per_xcd;          // tiles per XCD (grid = 8 * per_xcd)
    int M;                // 1..16
    int y_dtype;
    int x_vec_ok;         // activation rows may be read with 16-byte loads
};

template <int NW> struct RawVec;
template <> struct RawVec<16> { typedef uint4 type; };
template <> struct RawVec<8> { typedef uint2 type; };
template <> struct RawVec<4> { typedef uint32_t type; };
template <> struct RawVec<2> { typedef uint16_t type; };
template <> struct RawVec<1> { typedef uint8_t type; };

// NW bytes at W_T + off into ceil(NW/4) dwords (zero extended).  The load is unconditional
// (the caller clamps `off` to a valid location): a load under a per-lane predicate becomes a
// branch with a wait behind it, which serialises the stream.
template <int NW>
__device__ __forceinline__ void load_raw(const uint8_t* base, uint32_t off, uint32_t (&d)[(NW + 3) / 4]) {
    const typename RawVec<NW>::type v = *(const typename RawVec<NW>::type*)(base + off);
    if constexpr (NW >= 4) __builtin_memcpy(d, &v, NW);
    else d[0] = (uint32_t)v;
}

__device__ __forceinline__ void store_out(void* Y, int dt, int64_t idx, float v) {
    if (dt == BT_F32) ((float*)Y)[idx] = v;
    else if (dt == BT_F16) ((uint16_t*)Y)[idx] = f32_to_f16_bits(v);
    else ((uint16_t*)Y)[idx] = f32_to_bf16_bits(v);
}

template <int MODE>
__device__ __forceinline__ void finish_output(const StreamParams& p, int row, int64_t n, uint32_t bits, float s,
                                              float b) {
    float y;
    if constexpr (MODE == MODE_I8) {
        const int32_t acc127 = times127((int32_t)bits);  // MFMA ran on +-1 weights
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

template <int MODE>
__device__ __forceinline__ uint32_t add_bits(uint32_t a, uint32_t b) {
    if constexpr (MODE == MODE_I8) return (uint32_t)((int32_t)a + (int32_t)b);
    else return __builtin_bit_cast(uint32_t, __builtin_bit_cast(float, a) + __builtin_bit_cast(float, b));
}

// 16 bytes of activations for lane (row i, group g) of one step, in natural k order.
// XV: rows are 16-byte aligned and K is a multiple of the 16-byte group, so a group that
// starts below K lies wholly inside its row; the load is unconditional on a clamped address
// (xrow = element offset of row min(i, M-1)) and the caller zeroes groups at k >= K when it
// consumes them.  !XV: element-wise gather (unaligned or ragged rows), zero filled.
template <int MODE, bool XV>
__device__ __forceinline__ uint4 load_x_frag(const StreamParams& p, uint32_t xrow, int i, int k) {
    constexpr int GE = (MODE == MODE_I8) ? 16 : 8;
    constexpr int ES = (MODE == MODE_I8) ? 1 : 2;
    if constexpr (XV) {
        const uint32_t kc = (uint32_t)min(k, (int)p.K - GE);
        return *(const uint4*)((const uint8_t*)p.X + (xrow + kc) * ES);
    } else {
        uint32_t d[4] = {0u, 0u, 0u, 0u};
        if (i < p.M && k < p.K) {
            if constexpr (MODE == MODE_I8) {
                const uint8_t* src = (const uint8_t*)p.X + (int64_t)i * p.K + k;
                for (int e = 0; e < GE; e++)
                    if (k + e < p.K) d[e >> 2] |= (uint32_t)src[e] << (8 * (e & 3));
            } else {
                const uint16_t* src = (const uint16_t*)p.X + (int64_t)i * p.K + k;
                for (int e = 0; e < GE; e++)
                    if (k + e < p.K) d[e >> 1] |= (uint32_t)src[e] << (16 * (e & 1));
            }
        }
        return make_uint4(d[0], d[1], d[2], d[3]);
    }
}

template <int MODE, int NW, int WAVES, int PF>
__global__ __launch_bounds__(WAVES * 64) void stream_kernel(StreamParams p) {
    constexpr int KBG = (MODE == MODE_I8) ? 4 : 2;  // kb rows per lane group
    constexpr int RS = 4 * KBG;                     // kb rows per wave step
    constexpr int TILE_N = 16 * NW;
    constexpr int ND = (NW + 3) / 4;                // dwords per lane and row
    typedef typename std::conditional<MODE == MODE_I8, v4i, v4f>::type acc_t;

    extern __shared__ __attribute__((aligned(16))) uint32_t red[];  // [WAVES][M][TILE_N]

    // consecutive tiles on one XCD (workgroups are dealt round-robin over 8 XCDs)
    const int tile = (int)(blockIdx.x & 7) * p.per_xcd + (int)(blockIdx.x >> 3);
    if (tile >= p.tiles) return;

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int j = lane & 15;
    const int g = lane >> 4;
    const int64_t nb = (int64_t)tile * TILE_N;
    const int nsteps = (int)((p.Kb + RS - 1) / RS);
    const int64_t ncol = nb + (int64_t)NW * j;
    const bool col_ok = ncol < p.N;
    // 32-bit offsets from the uniform base pointers (the host checks that they fit), advanced
    // by uniform strides: row kb of step s, group g, r is kb = s*RS + g*KBG + r.  Rows past the
    // end are clamped to the last row; their products vanish because the activations at
    // k >= K are zero, and columns past N are computed on column 0's bytes and never stored.
    const uint32_t col_off = col_ok ? (uint32_t)ncol : 0u;
    const uint32_t N32 = (uint32_t)p.N;
    const uint32_t last_off = (uint32_t)(p.Kb - 1) * N32 + col_off;
    const uint32_t step_stride = (uint32_t)(WAVES * RS) * N32;
    uint32_t woff = (uint32_t)(wave * RS + g * KBG) * N32 + col_off;
    int k0 = 4 * (wave * RS + g * KBG);
    const uint32_t xrow = (uint32_t)min(j, p.M - 1) * (uint32_t)p.K;

    // epilogue operands of this thread's output column, requested before the weight stream
    // so that their latency hides behind it (raw bits now, conversion after the reduction)
    constexpr bool PRE = (WAVES * 64) % TILE_N == 0;  // a thread finishes one column only
    uint32_t pre_s = 0u, pre_b = 0u;
    if constexpr (PRE) {
        const int64_t n = nb + (int)(threadIdx.x % TILE_N);
        if ((int)threadIdx.x < p.M * TILE_N && n < p.N) {
            pre_s = load_bits_rt(p.epi.scale, p.epi.scale_dtype, p.epi.scale_bcast ? 0 : n);
            if (p.epi.bias) pre_b = load_bits_rt(p.epi.bias, p.epi.bias_dtype, n);
        }
    }

    acc_t acc[NW];
#pragma unroll
    for (int t = 0; t < NW; t++) acc[t] = acc_t{0, 0, 0, 0};

    for (int base = wave; base < nsteps; base += WAVES * PF, woff += PF * step_stride, k0 += 4 * WAVES * RS * PF) {
        uint32_t raw[PF][KBG][ND];
        uint4 xa[PF];
#pragma unroll
        for (int f = 0; f < PF; f++) {
#pragma unroll
            for (int r = 0; r < KBG; r++)
                load_raw<NW>(p.W_T, min(woff + (uint32_t)f * step_stride + (uint32_t)r * N32, last_off), raw[f][r]);
        }
        if (p.x_vec_ok) {
#pragma unroll
            for (int f = 0; f < PF; f++) xa[f] = load_x_frag<MODE, true>(p, xrow, j, k0 + f * 4 * WAVES * RS);
        } else {
#pragma unroll
            for (int f = 0; f < PF; f++) xa[f] = load_x_frag<MODE, false>(p, xrow, j, k0 + f * 4 * WAVES * RS);
        }
#pragma unroll
        for (int f = 0; f < PF; f++) {
            if (base + f * WAVES >= nsteps) break;  // uniform per wave
            {
                const bool k_ok = k0 + f * 4 * WAVES * RS < (int)p.K;  // no-op for the gathered path
                xa[f].x = k_ok ? xa[f].x : 0u; xa[f].y = k_ok ? xa[f].y : 0u;
                xa[f].z = k_ok ? xa[f].z : 0u; xa[f].w = k_ok ? xa[f].w : 0u;
            }
            if constexpr (MODE == MODE_I8) {
                uint32_t ta[4];
                transpose4x4_bytes(xa[f].x, xa[f].y, xa[f].z, xa[f].w, ta);
                const v4i a = {(int)ta[0], (int)ta[1], (int)ta[2], (int)ta[3]};
#pragma unroll
                for (int d = 0; d < ND; d++) {
                    uint32_t G[4];
                    if constexpr (NW == 1) {
                        // one byte per row: G = {row0, row1, row2, row3}
                        G[0] = raw[f][0][0] | (raw[f][1][0] << 8) | (raw[f][2][0] << 16) | (raw[f][3][0] << 24);
                    } else {
                        transpose4x4_bytes(raw[f][0][d], raw[f][1][d], raw[f][2][d], raw[f][3][d], G);
                    }
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        if (4 * d + i < NW) {
                            const v4i b = decode16_i8(G[i]);
                            acc[4 * d + i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc[4 * d + i], 0, 0, 0);
                        }
                    }
                }
            } else {
                // natural halves h0..h7 -> dword c = { h[c], h[4+c] } (the decode's k order)
                const u32x4 au = {perm(xa[f].z, xa[f].x, 0x05040100u), perm(xa[f].z, xa[f].x, 0x07060302u),
                                  perm(xa[f].w, xa[f].y, 0x05040100u), perm(xa[f].w, xa[f].y, 0x07060302u)};
#pragma unroll
                for (int d = 0; d < ND; d++) {
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        if (4 * d + i < NW) {
                            // bytes: [zero, row0.byte i, zero, row1.byte i]
                            const uint32_t sel = ((uint32_t)(4 + i) << 24) | (0x0Cu << 16) | ((uint32_t)i << 8) | 0x0Cu;
                            const uint32_t M2 = perm(raw[f][1][d], raw[f][0][d], sel);
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
            }
        }
    }

    // ---- sum the waves' accumulators through LDS, in wave order ------------------------
    // red[w][row][t*16 + j]; lane (j, g) holds rows 4g..4g+3 of column slot t*16+j
    const int M = p.M;
#pragma unroll
    for (int t = 0; t < NW; t++) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int row = 4 * g + r;
            // copy the element out first: a bit_cast applied directly to a vector
            // element was observed to read element 0 for every r
            const auto v = acc[t][r];
            if (row < M) red[(wave * M + row) * TILE_N + t * 16 + j] = __builtin_bit_cast(uint32_t, v);
        }
    }
    __syncthreads();

    for (int idx = threadIdx.x; idx < M * TILE_N; idx += WAVES * 64) {
        const int row = idx / TILE_N;
        const int nl = idx % TILE_N;
        if (nb + nl >= p.N) continue;
        const int slot = (nl % NW) * 16 + nl / NW;
        uint32_t bits = red[row * TILE_N + slot];
#pragma unroll
        for (int w = 1; w < WAVES; w++) bits = add_bits<MODE>(bits, red[(w * M + row) * TILE_N + slot]);
        float s, b;
        if constexpr (PRE) {
            s = bits_to_f32_rt(pre_s, p.epi.scale_dtype);
            b = p.epi.bias ? bits_to_f32_rt(pre_b, p.epi.bias_dtype) : 0.0f;
        } else {
            s = epi_scale(p.epi, nb + nl);
            b = epi_bias(p.epi, nb + nl);
        }
        finish_output<MODE>(p, row, nb + nl, bits, s, b);
    }
}

// ---- host side --------------------------------------------------------------------

struct StreamPlan {
    int nw;     // bytes per lane and row: 16, 8, 4, 2 or 1 (tile = 16*nw columns)
    int waves;  // waves per workgroup
};

// the kernel addresses W_T and X with 32-bit offsets from their base pointers
bool stream_supported(int64_t N, int64_t K, const void* W_T) {
    // (rows up to 16*16*16 past the end enter the offset arithmetic before they are clamped)
    return ((uintptr_t)W_T) % 16 == 0 && N >= 1 && (ceil_div(K, 4) + 8192) * N < (1ll << 32) && K < (1ll << 26);
}

StreamPlan stream_plan(int mode, int64_t M, int64_t N, int64_t Kb) {
    StreamPlan pl;
    (void)mode;
    // optional override for tuning runs: BITTORCH_STREAM_CFG="nw,waves"
    int o_nw = 0, o_waves = 0;
    if (const char* env = getenv("BITTORCH_STREAM_CFG")) sscanf(env, "%d,%d", &o_nw, &o_waves);
    // widest lane load the row pitch allows (row starts must stay aligned to it)
    int nw = (N % 16 == 0) ? 16 : (N % 8 == 0) ? 8 : (N % 4 == 0) ? 4 : (N % 2 == 0) ? 2 : 1;
    if ((o_nw == 16 || o_nw == 8 || o_nw == 4 || o_nw == 2 || o_nw == 1) && N % o_nw == 0) {
        nw = o_nw;
    } else {
        // narrow the tile until there is at least one tile per CU
        while (nw > 1 && ceil_div(N, 16 * (int64_t)nw) < 256) nw >>= 1;
        // decode batches re-read the activations once per tile: keep tiles wider when
        // that traffic would exceed the weights' own
        (void)M;
    }
    pl.nw = nw;
    const int max_waves = 1024 / (16 * nw) < 16 ? 1024 / (16 * nw) : 16;  // LDS: WAVES*TILE_N <= 1024 words/row
    const int64_t steps = ceil_div(Kb, mode == MODE_I8 ? 16 : 8);
    int waves = (o_waves == 1 || o_waves == 2 || o_waves == 4 || o_waves == 8 || o_waves == 16) ? o_waves : 8;
    if (waves > max_waves) waves = max_waves;
    while (waves > 1 && waves > steps) waves >>= 1;
    pl.waves = waves;
    return pl;
}

size_t stream_workspace_bytes(int, int64_t, int64_t, int64_t) { return 0; }

template <int MODE, int NW, int WAVES>
static void launch_stream_k(const StreamParams& p, dim3 grid, size_t lds, hipStream_t st) {
    constexpr int PF = (NW >= 16) ? 2 : (NW == 8) ? 4 : 8;
    hipLaunchKernelGGL((stream_kernel<MODE, NW, WAVES, PF>), grid, dim3(WAVES * 64), lds, st, p);
}

template <int MODE, int NW>
static void launch_stream_w(const StreamParams& p, int waves, dim3 grid, size_t lds, hipStream_t st) {
    if constexpr (NW <= 4) {
        if (waves == 16) { launch_stream_k<MODE, NW, 16>(p, grid, lds, st); return; }
    }
    if constexpr (NW <= 8) {
        if (waves == 8) { launch_stream_k<MODE, NW, 8>(p, grid, lds, st); return; }
    }
    if (waves >= 4) { launch_stream_k<MODE, NW, 4>(p, grid, lds, st); return; }
    if (waves == 2) { launch_stream_k<MODE, NW, 2>(p, grid, lds, st); return; }
    launch_stream_k<MODE, NW, 1>(p, grid, lds, st);
}

template <int MODE>
static int launch_stream_mode(StreamParams p, const StreamPlan& pl, hipStream_t st) {
    const int64_t tile_n = 16 * (int64_t)pl.nw;
    p.tiles = (int)ceil_div(p.N, tile_n);
    p.per_xcd = (int)ceil_div(p.tiles, 8);
    const dim3 grid((unsigned)(p.per_xcd * 8));
    int waves = pl.waves;
    if (pl.nw == 16 && waves > 4) waves = 4;
    if (pl.nw == 8 && waves > 8) waves = 8;
    const size_t lds = (size_t)waves * p.M * tile_n * 4;
    switch (pl.nw) {
        case 16: launch_stream_w<MODE, 16>(p, waves, grid, lds, st); break;
        case 8: launch_stream_w<MODE, 8>(p, waves, grid, lds, st); break;
        case 4: launch_stream_w<MODE, 4>(p, waves, grid, lds, st); break;
        case 2: launch_stream_w<MODE, 2>(p, waves, grid, lds, st); break;
        default: launch_stream_w<MODE, 1>(p, waves, grid, lds, st); break;
    }
    return check_launch("stream_gemm");
}

// One launch per block of up to 16 activation rows.
int launch_stream(int mode, const void* X, int x_elem_size, const float* s_x, const uint8_t* W_T,
                  const Epilogue& epi, void* Y, int y_dtype, int32_t* acc_out, int64_t B, int64_t N,
                  int64_t K, void* workspace, size_t ws_bytes, hipStream_t st) {
    (void)workspace;
    (void)ws_bytes;
    const int64_t Kb = ceil_div(K, 4);
    const StreamPlan pl = stream_plan(mode, B, N, Kb);
    const int y_size = dtype_size(y_dtype);
    for (int64_t m0 = 0; m0 < B; m0 += 16) {
        StreamParams p;
        p.X = (const uint8_t*)X + m0 * K * x_elem_size;
        p.W_T = W_T;
        p.s_x = s_x ? s_x + m0 : nullptr;
        p.Y = (uint8_t*)Y + m0 * N * y_size;
        p.acc_out = acc_out ? acc_out + m0 * N : nullptr;
        p.epi = epi;
        p.N = N; p.K = K; p.Kb = Kb;
        p.M = (int)((B - m0 < 16) ? (B - m0) : 16);
        p.y_dtype = y_dtype;
        p.x_vec_ok = (((uintptr_t)p.X) % 16 == 0) && ((K * x_elem_size) % 16 == 0);
        int rc;
        if (mode == MODE_I8) rc = launch_stream_mode<MODE_I8>(p, pl, st);
        else if (mode == MODE_F16) rc = launch_stream_mode<MODE_F16>(p, pl, st);
        else rc = launch_stream_mode<MODE_BF16>(p, pl, st);
        if (rc != BT_OK) return rc;
    }
    return BT_OK;
}

}  // namespace bt
