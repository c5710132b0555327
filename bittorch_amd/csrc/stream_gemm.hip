// Decode-shape / small-batch packed-ternary GEMM for gfx950: streams the 2-bit
// weights W_T [Kb, N] from HBM once, decodes them in registers and feeds the
// matrix cores.  A workgroup serves one block of M <= 16 activation rows (one MFMA row block);
// grid.y walks the blocks of a taller call, which run concurrently and share the weights in L2.
//
// Arithmetic restated from the reference kernels:
//   float path (csrc/kernels/ternary_gemm_production.cu:126-141):
//       acc_f32 = sum_k x[b,k] * w[k,n];  y = acc * scale[n] + bias[n]
//   int8 path (csrc/kernels/ternary_gemm_tensor_core.cu:583-589, :652):
//       acc_i32 = sum_k q[b,k] * (127 w[k,n]);  y = (acc * s_x[b] / 127) * scale[n] + bias[n]
//
// Work decomposition.  A wave "step" covers 16 consecutive kb rows (64 values of k)
// and TILE_N output columns.  Lane (j = lane%16, g = lane/16) ends up holding, per
// column it serves, one dword G = the packed bytes of rows kb0+4g .. kb0+4g+3: the B
// operand of one 16x16x64 int8 MFMA, or of two 16x16x32 fp16/bf16 MFMAs.  The k order
// inside an MFMA is free as long as both operands agree, so the activations are
// permuted into the order the cheapest weight decode produces.
//
// How G gets into the lane depends on the tile width (template LD).  What limits a
// narrow tile is the number of vector memory instructions a CU can issue, not bytes:
//   LD_V4/8/16  lane loads 4/8/16 consecutive bytes (that many columns) from each of
//               its four rows and transposes 4x4 byte blocks in registers;
//   LD_Q1/Q2    16/32-column tiles: the four lanes of a quad load one dword each
//               (rows 4g+q, the same four columns) and exchange bytes with DPP
//               quad permutes - one load instruction per 16x16 block instead of four;
//   LD_BYTE     N not a multiple of 4: one byte per lane and row.
//   LD_T1/2/4/8 the decode-tiled copy of the weights (W_LAYOUT_TILED, see retile_kernel): the dword
//               G of every lane and step is stored as such, 256 contiguous bytes per 16-column tile
//               and step, so a wave's load covers two whole cache lines and needs no transpose
//               (a 16-column tile of the row-major W_T touches 16 bytes of 16 different lines,
//               and the seven other tiles sharing those lines sit on other compute units).
// A wave issues the loads of PF steps before it computes any of them, which is
// what keeps enough bytes in flight to cover the HBM latency.
// A workgroup owns one column tile over the WHOLE of K: there is no split-K
// across workgroups, hence no partial sums in memory, no second pass and no
// inter-workgroup synchronisation.  Tiles that share 128-byte lines of W_T are
// placed on the same XCD so the line is fetched from HBM once.  The waves of a
// workgroup take contiguous ranges of steps and their accumulators are summed
// through LDS in wave order.
// Activations: for M = 1 (XLDS) a wave fetches its whole K-slice of x with one or a
// few fully coalesced loads into LDS and reads operand fragments from there; for
// M > 1 every lane loads its own 16-element fragment per step.
#include "row_math.h"

namespace bt {

struct StreamParams {
    // what a workgroup needs before it can request its first weights comes first, so that one scalar load
    // of the kernel arguments covers it
    const void* X;        // MODE_I8: int8 [M,K]; else 16-bit activations [M,K]
    const uint8_t* W_T;   // [Kb, N]
    const void* pro_b;    // prologue operand (see pro_op below)
    int64_t N, K, Kb;     // K: length of an activation row; Kb: packed weight rows
    int wsteps;           // 16-row steps of W_T; a step index beyond it wraps (see launch_stream)
    int tiles;            // column tiles
    int per_xcd;          // tiles per XCD (grid = 8 * per_xcd)
    int tiles16;          // LD_T*: 16-column tiles of the decode-tiled weights (< 0: stored_tile16)
    int M;                // 1..16: rows of a 16-row block (of the last one when the launch covers several)
    int x_vec_ok;         // activation rows may be read with 16-byte loads
    int64_t B;            // rows of the whole call: grid.y = ceil(B / 16) blocks of 16 rows, all in one launch
    const float* s_x;     // MODE_I8: per-row activation scales [M]
    void* Y;              // [M, N] of y_dtype
    int32_t* acc_out;     // MODE_I8, optional raw accumulators [M, N]
    Epilogue epi;
    int y_dtype;
    int prehalved;        // MODE_BF16: the activations already carry the factor 1/2 of the +-2.0 weight decode
    int x_operand_order;  // MODE_I8: X is in the quantizer's operand order (16-byte groups transposed)
    // Prologue applied to the single activation row on its way into LDS (M = 1, 16-bit modes):
    //   PRO_RMSNORM  x <- rd((x * r) * w),  w = pro_b [K] or ones, r from the whole row and pro_eps
    //   PRO_SWIGLU   x <- rd(rd(silu(x)) * u),  u = pro_b [K]
    int pro_op;
    float pro_eps;
    // Output stage (16-bit modes on tiled weights whose 16-column tiles alternate gate, up, gate, up ...):
    //   EPI_SWIGLU_PAIRS  Y [M, N/2]:  Y[b, h] = rd(rd(silu(g)) * u),  g = rd(linear column h), u = rd(linear
    //                     column N/2 + h): what the SwiGLU kernel would make of the stored projections
    int epi_op;
};

enum { LD_BYTE = 0, LD_Q1 = 1, LD_Q2 = 2, LD_V4 = 4, LD_V8 = 8, LD_V16 = 16, LD_T1 = 101, LD_T2 = 102, LD_T4 = 104, LD_T8 = 108 };
constexpr int XC_MAX = 4;  // XLDS: 16-byte chunks of the x slice per lane

template <int NB> struct RawVec;
template <> struct RawVec<16> { typedef uint4 type; };
template <> struct RawVec<8> { typedef uint2 type; };
template <> struct RawVec<4> { typedef uint32_t type; };

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
        y = epi_float(__builtin_bit_cast(float, bits) * (p.prehalved ? 1.0f : 0.5f), s, b);
    }
    if (p.epi.residual) y = add_residual(y, p.epi.residual, p.y_dtype, (int64_t)row * p.N + n);
    store_out(p.Y, p.y_dtype, (int64_t)row * p.N + n, y);
}

template <int MODE>
__device__ __forceinline__ uint32_t add_bits(uint32_t a, uint32_t b) {
    if constexpr (MODE == MODE_I8) return (uint32_t)((int32_t)a + (int32_t)b);
    else return __builtin_bit_cast(uint32_t, __builtin_bit_cast(float, a) + __builtin_bit_cast(float, b));
}

// 16 bytes of activations of row i starting at element k, in natural k order.
// XV: rows are 16-byte aligned and K is a multiple of the 16-byte group, so a group that
// starts below K lies wholly inside its row; the load is unconditional on a clamped address
// (xrow = element offset of row min(i, M-1)) and the caller zeroes groups at k >= K when it
// consumes them: a load under a per-lane predicate becomes a branch with a wait behind it,
// which serialises the stream.  !XV: element-wise gather (unaligned or ragged rows), zero filled.
template <int MODE, bool XV>
__device__ __forceinline__ uint4 load_x16(const StreamParams& p, uint32_t xrow, int i, int k) {
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

__device__ __forceinline__ uint4 zero_unless(uint4 v, bool ok) {
    v.x = ok ? v.x : 0u; v.y = ok ? v.y : 0u; v.z = ok ? v.z : 0u; v.w = ok ? v.w : 0u;
    return v;
}

// d = the dword this lane loaded (row 4g+q, four columns); returns the bytes of column q of
// the dwords of quad lanes 0..3, i.e. rows 4g..4g+3 of this lane's own column.
__device__ __forceinline__ uint32_t quad_transpose(uint32_t d, uint32_t sel_q) {
    const uint32_t v0 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)d, 0x00, 0xf, 0xf, true);
    const uint32_t v1 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)d, 0x55, 0xf, 0xf, true);
    const uint32_t v2 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)d, 0xAA, 0xf, 0xf, true);
    const uint32_t v3 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)d, 0xFF, 0xf, 0xf, true);
    const uint32_t t01 = perm(v1, v0, sel_q);  // [v0.b[q], v1.b[q], -, -]
    const uint32_t t23 = perm(v3, v2, sel_q);
    return perm(t23, t01, 0x05040100u);
}

// The linear value of one output column before it is stored: the accumulator scaled, biased and
// (16-bit modes) with the decode's factor undone.
template <int MODE>
__device__ __forceinline__ float linear_value(const StreamParams& p, uint32_t bits, float s, float b) {
    if constexpr (MODE == MODE_F16) return epi_float(__builtin_bit_cast(float, bits), s, b);
    else return epi_float(__builtin_bit_cast(float, bits) * (p.prehalved ? 1.0f : 0.5f), s, b);
}

// PRO: activation prologue compiled in (PRO_NONE for all but the M = 1 variants that are launched
// with one: a run-time switch, even a uniform one, puts branches and waits around the loads of the
// plain kernel).
template <int MODE, int LD, int WAVES, int PF, bool XLDS, int PRO = 0, int EPI = 0>
__global__ __launch_bounds__(WAVES * 64) void stream_kernel(StreamParams p_in) {
    constexpr bool QUAD = (LD == LD_Q1 || LD == LD_Q2);
    constexpr bool BYTE = (LD == LD_BYTE);
    constexpr bool TILED = (LD > 100);
    constexpr int NACC = TILED ? LD - 100 : BYTE ? 1 : LD;  // output columns per lane
    constexpr int TILE_N = 16 * NACC;
    constexpr int RAWN = TILED ? NACC : BYTE ? 4 : LD;      // raw dwords per lane and step
    constexpr int ND = (!TILED && LD >= 4) ? LD / 4 : 1;    // LD_V*: dwords per lane and row
    constexpr int NCO = QUAD ? LD : TILED ? NACC : 1;       // column (LD_T*: tile) offsets per lane
    constexpr int ES = (MODE == MODE_I8) ? 1 : 2;   // bytes per activation
    constexpr int XN = (MODE == MODE_I8) ? 1 : 2;   // 16-byte pieces of x per lane and step
    constexpr bool TWO = (NACC <= 2);               // second accumulator chain
    constexpr int NACC2 = TWO ? NACC : 1;
    typedef typename std::conditional<MODE == MODE_I8, v4i, v4f>::type acc_t;

    extern __shared__ __attribute__((aligned(16))) uint32_t red[];  // [WAVES][M][TILE_N], then x slices

    // One launch covers every 16-row block of the call (grid.y): the blocks are independent, run
    // concurrently and find the weights their neighbours fetched in the XCD's L2 (the same tile of every
    // block lands on the same XCD).  This workgroup's block: rows 16*blockIdx.y .. of X, Y, s_x, ...
    StreamParams p = p_in;
    if constexpr (!XLDS) {  // (the LDS-staged variant is the single-row one)
        if (p_in.B > 16) {  // uniform
            const int64_t r0 = (int64_t)blockIdx.y * 16;
            const int64_t ny = (EPI == EPI_SWIGLU_PAIRS) ? (p_in.N >> 1) : p_in.N;
            const int ysz = (p_in.y_dtype == BT_F32) ? 4 : 2;
            p.M = (int)((p_in.B - r0 < 16) ? (p_in.B - r0) : 16);
            p.X = (const uint8_t*)p_in.X + r0 * p_in.K * ((MODE == MODE_I8) ? 1 : 2);
            p.Y = (uint8_t*)p_in.Y + r0 * ny * ysz;
            if (p_in.s_x) p.s_x = p_in.s_x + r0;
            if (p_in.acc_out) p.acc_out = p_in.acc_out + r0 * p_in.N;
            if (p_in.epi.residual) p.epi.residual = (const uint8_t*)p_in.epi.residual + r0 * p_in.N * ysz;
        }
    }

    // consecutive tiles on one XCD (workgroups are dealt round-robin over 8 XCDs)
    // (per_xcd == 0: a batch of several row blocks over few tiles; workgroups then take tiles in launch order,
    // which deals every row block's tiles round-robin over the XCDs instead of parking them all on the first few)
    const int tile = p.per_xcd ? (int)(blockIdx.x & 7) * p.per_xcd + (int)(blockIdx.x >> 3) : (int)blockIdx.x;
    if (tile >= p.tiles) return;

    const int lane = threadIdx.x & 63;
    // (wave-uniform by construction: telling the compiler so moves the K-range and address arithmetic that
    // derives from it to the scalar unit)
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int j = lane & 15;
    const int g = lane >> 4;
    const int q = lane & 3;
    const int64_t nb = (int64_t)tile * TILE_N;
    const int nsteps = (int)((p.K + 63) >> 6);
    const int spw = (nsteps + WAVES - 1) / WAVES;  // steps per wave, contiguous
    const int s_begin = wave * spw;
    const int s_end = min(nsteps, s_begin + spw);

    // 32-bit offsets from the uniform base pointers (the host checks that they fit), advanced
    // by uniform strides.  Rows past the end are clamped to the last row; their products
    // vanish because the activations at k >= K are zero.  Columns past N are computed on
    // column 0's bytes and never stored.
    const uint32_t N32 = (uint32_t)p.N;
    const uint32_t last_rowoff = (uint32_t)(p.Kb - 1) * N32;
    uint32_t coloff[NCO];
    if constexpr (TILED) {
        // byte offset of this lane's dword in step 0 of each 16-column tile; a tile past the end is
        // computed on the last tile's bytes and never stored
#pragma unroll
        for (int t = 0; t < NCO; t++)
            coloff[t] = ((uint32_t)stored_tile16(tile * NACC + t, p.tiles16) * (uint32_t)p.wsteps * 64u + (uint32_t)lane) * 4u;
    } else if constexpr (QUAD) {
#pragma unroll
        for (int cb = 0; cb < NCO; cb++) {
            const int64_t c = nb + 16 * cb + (j & ~3);
            coloff[cb] = (c < p.N) ? (uint32_t)c : 0u;
        }
    } else {
        const int64_t c = nb + (int64_t)NACC * j;
        coloff[0] = (c < p.N) ? (uint32_t)c : 0u;
    }
    const uint32_t lane_rowoff = (uint32_t)(4 * g + (QUAD ? q : 0)) * N32;
    const uint32_t step_rows = 16u * N32;
    int k0 = s_begin * 64 + 16 * g;  // first k of this lane's fragment in step s_begin
    const uint32_t xrow = (uint32_t)min(j, p.M - 1) * (uint32_t)p.K;
    const uint32_t sel_q = 0x0C0C0000u | ((uint32_t)(4 + q) << 8) | (uint32_t)q;

    // XLDS (M == 1): the wave's K-slice of x, [s_begin*64, (s_begin+spw)*64), as 16-byte
    // chunks, chunk c = lane + 64u; zero beyond K
    uint8_t* xs = (uint8_t*)(red + WAVES * p.M * TILE_N) + (size_t)wave * (XC_MAX * 64 * 16);
    uint4 xr[XLDS ? XC_MAX : 1], xb[(XLDS && PRO != 0) ? XC_MAX : 1];
    const int nchunks = spw * 64 * ES / 16;
    if constexpr (XLDS) {
        constexpr int EPC = 16 / ES;
#pragma unroll
        for (int u = 0; u < XC_MAX; u++) {
            if (u * 64 < nchunks) {  // uniform
                const int k = s_begin * 64 + (lane + 64 * u) * EPC;
                xr[u] = *(const uint4*)((const uint8_t*)p.X + (uint32_t)min(k, (int)p.K - EPC) * ES);
                if constexpr (PRO != 0) {  // second operand; RMSNorm without a weight reads X again (unused)
                    const uint8_t* bsrc = p.pro_b ? (const uint8_t*)p.pro_b : (const uint8_t*)p.X;
                    xb[u] = *(const uint4*)(bsrc + (uint32_t)min(k, (int)p.K - EPC) * ES);
                }
            }
        }
    }
    // the weight loads of the PF steps from `base` on
    auto load_weights = [&](int base, uint32_t (&raw)[PF][RAWN]) {
#pragma unroll
        for (int f = 0; f < PF; f++) {
            // weight step of activation step base+f (uniform): the activation row may hold several
            // planes of K values each, all multiplied with the same weights
            int ws = base + f;
            if (ws >= p.wsteps) ws -= p.wsteps;
            if (ws >= p.wsteps) ws -= p.wsteps;
            const uint32_t ro = lane_rowoff + (uint32_t)ws * step_rows;
            if constexpr (TILED) {
                const uint32_t so = (uint32_t)min(ws, p.wsteps - 1) * 256u;
#pragma unroll
                for (int t = 0; t < NCO; t++) raw[f][t] = ldw_nt(p.W_T + (coloff[t] + so));
            } else if constexpr (BYTE) {
#pragma unroll
                for (int r = 0; r < 4; r++)
                    raw[f][r] = (uint32_t)p.W_T[min(ro + (uint32_t)r * N32, last_rowoff) + coloff[0]];
            } else if constexpr (QUAD) {
                const uint32_t rc = min(ro, last_rowoff);
#pragma unroll
                for (int cb = 0; cb < NCO; cb++) raw[f][cb] = ldw_nt(p.W_T + (rc + coloff[cb]));
            } else {
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const typename RawVec<LD>::type v = *(const typename RawVec<LD>::type*)(
                        p.W_T + (min(ro + (uint32_t)r * N32, last_rowoff) + coloff[0]));
                    __builtin_memcpy(&raw[f][r * ND], &v, LD);
                }
            }
        }
    };
    // The single-row variant requests its first batch of weights as early as it can: the activation slice
    // first (it is needed first, and loads return in order), then the weights, then everything else; the
    // slice is transformed and parked in LDS while the weights are on their way.
    // RMSNorm prologue: the row's sum of squares, by the whole workgroup (the row is a few KiB and hot
    // in cache), accumulated in fp64 so that its fp32 value does not depend on the summation order.
    // Its loads are requested before the weights, and the sum is formed behind them: the reduction and
    // its two barriers run while the weights are on their way.
    constexpr bool PRELOAD = XLDS;
    constexpr bool PRENORM = XLDS && MODE != MODE_I8 && PRO == PRO_RMSNORM;
    constexpr int PVN = 4;  // 16-byte pieces of the row per thread (the LDS-staged variant's K limit / 8 / threads)
    uint4 pv[PRENORM ? PVN : 1];
    if constexpr (PRENORM) {
#pragma unroll
        for (int u = 0; u < PVN; u++) {
            if (u * WAVES * 64 * 8 < (int)p.K) {  // uniform
                const int k = ((int)threadIdx.x + u * WAVES * 64) * 8;
                pv[u] = *(const uint4*)((const uint16_t*)p.X + min(k, (int)p.K - 8));  // K % 8 == 0, aligned (XLDS)
            }
        }
    }
    uint32_t raw0[PRELOAD ? PF : 1][PRELOAD ? RAWN : 1];
    if constexpr (PRELOAD) load_weights(s_begin, raw0);

    // epilogue operands of this thread's output column, requested early so that their latency hides behind
    // the weight stream (raw bits now, conversion after the reduction)
    constexpr bool PRE = (WAVES * 64) % TILE_N == 0 && EPI == EPI_NONE;  // a thread finishes one column only
    uint32_t pre_s = 0u, pre_b = 0u;
    if constexpr (PRE) {
        const int64_t n = nb + (int)(threadIdx.x % TILE_N);
        if ((int)threadIdx.x < p.M * TILE_N && n < p.N) {
            pre_s = load_bits_rt(p.epi.scale, p.epi.scale_dtype, p.epi.scale_bcast ? 0 : n);
            if (p.epi.bias) pre_b = load_bits_rt(p.epi.bias, p.epi.bias_dtype, n);
        }
    }

    float rstd = 1.0f;
    if constexpr (PRENORM) {
        double ss = 0.0;
#pragma unroll
        for (int u = 0; u < PVN; u++) {
            const int k = ((int)threadIdx.x + u * WAVES * 64) * 8;
            if (u * WAVES * 64 * 8 < (int)p.K && k < (int)p.K) {
                const uint32_t d[4] = {pv[u].x, pv[u].y, pv[u].z, pv[u].w};
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const uint16_t h = (uint16_t)(d[e >> 1] >> (16 * (e & 1)));
                    const double x = (double)(MODE == MODE_F16 ? f16_bits_to_f32(h) : bf16_bits_to_f32(h));
                    ss += x * x;
                }
            }
        }
        ss = wave_sum_f64(ss);
        double* part = (double*)red;  // the reduction buffer is free until the main loop is over
        if (lane == 0) part[wave] = ss;
        __syncthreads();
        ss = 0.0;
        for (int w = 0; w < WAVES; w++) ss += part[w];
        __syncthreads();
        rstd = rms_rstd(ss, (int)p.K, p.pro_eps);
    }

    // XLDS: park the wave's x slice in LDS (transformed by the prologue) once its loads have landed
    auto park_x = [&]() {
        constexpr int EPC = 16 / ES;
#pragma unroll
        for (int u = 0; u < XC_MAX; u++) {
            if (u * 64 < nchunks) {
                const int k = s_begin * 64 + (lane + 64 * u) * EPC;
                // parked in the order the MFMA wants (each 16-byte chunk is one operand
                // fragment), so that the steps below read their A operand ready-made
                uint4 v = zero_unless(xr[u], k < (int)p.K);
                if constexpr (MODE != MODE_I8 && PRO != 0) {
                    {
                        constexpr int DT = (MODE == MODE_F16) ? BT_F16 : BT_BF16;
                        const uint32_t a[4] = {v.x, v.y, v.z, v.w};
                        const uint32_t bq[4] = {xb[u].x, xb[u].y, xb[u].z, xb[u].w};
                        uint32_t r[4];
#pragma unroll
                        for (int d = 0; d < 4; d++) {
                            uint32_t out = 0;
#pragma unroll
                            for (int e = 0; e < 2; e++) {
                                const uint16_t ha = (uint16_t)(a[d] >> (16 * e)), hb = (uint16_t)(bq[d] >> (16 * e));
                                const float fa = (DT == BT_F16) ? f16_bits_to_f32(ha) : bf16_bits_to_f32(ha);
                                const float fb = (DT == BT_F16) ? f16_bits_to_f32(hb) : bf16_bits_to_f32(hb);
                                float y;
                                if constexpr (PRO == PRO_SWIGLU) y = swiglu_value(fa, fb, DT);
                                else y = rmsnorm_value(fa, rstd, p.pro_b ? fb : 1.0f, DT);
                                const uint32_t hy = (DT == BT_F16) ? f32_to_f16_bits(y) : f32_to_bf16_bits(y);
                                out |= hy << (16 * e);
                            }
                            r[d] = out;
                        }
                        v = zero_unless(make_uint4(r[0], r[1], r[2], r[3]), k < (int)p.K);
                    }
                }
                uint4 o;
                if constexpr (MODE == MODE_I8) {
                    uint32_t t4[4] = {v.x, v.y, v.z, v.w};
                    if (!p.x_operand_order) transpose4x4_bytes(v.x, v.y, v.z, v.w, t4);  // uniform
                    o = make_uint4(t4[0], t4[1], t4[2], t4[3]);
                } else {
                    o = make_uint4(perm(v.z, v.x, 0x05040100u), perm(v.z, v.x, 0x07060302u),
                                   perm(v.w, v.y, 0x05040100u), perm(v.w, v.y, 0x07060302u));
                }
                *(uint4*)(xs + (lane + 64 * u) * 16) = o;
            }
        }
    };
    // with the prologue's reduction ahead of it, the slice is parked while the first weight batch is still on its way
    if constexpr (PRELOAD) park_x();

    acc_t acc[NACC], acc2[NACC2];
#pragma unroll
    for (int t = 0; t < NACC; t++) acc[t] = acc_t{0, 0, 0, 0};
#pragma unroll
    for (int t = 0; t < NACC2; t++) acc2[t] = acc_t{0, 0, 0, 0};

    for (int base = s_begin; base < s_end; base += PF, k0 += PF * 64) {
        uint32_t raw[PF][RAWN];
        uint4 xa[PF][XN];
        if constexpr (PRELOAD) {
            if (base == s_begin) {  // uniform: this batch was requested ahead of the prologue
#pragma unroll
                for (int f = 0; f < PF; f++)
#pragma unroll
                    for (int r = 0; r < RAWN; r++) raw[f][r] = raw0[f][r];
            } else {
                load_weights(base, raw);
            }
        } else {
            load_weights(base, raw);
        }
        if constexpr (!XLDS) {
            if (p.x_vec_ok) {
#pragma unroll
                for (int f = 0; f < PF; f++)
#pragma unroll
                    for (int h = 0; h < XN; h++) xa[f][h] = load_x16<MODE, true>(p, xrow, j, k0 + f * 64 + 8 * h);
            } else {
#pragma unroll
                for (int f = 0; f < PF; f++)
#pragma unroll
                    for (int h = 0; h < XN; h++) xa[f][h] = load_x16<MODE, false>(p, xrow, j, k0 + f * 64 + 8 * h);
            }
        } else {
            if constexpr (!PRELOAD) {
                if (base == s_begin) park_x();  // uniform
            }
        }
#pragma unroll
        for (int f = 0; f < PF; f++) {
            if (base + f >= s_end) break;  // uniform per wave
            if constexpr (XLDS) {
                // LDS accesses of one wave execute in order: the slice written above is visible
                const uint8_t* src = xs + ((base + f - s_begin) * 64 + 16 * g) * ES;
#pragma unroll
                for (int h = 0; h < XN; h++) xa[f][h] = *(const uint4*)(src + 16 * h);
            } else {
#pragma unroll
                for (int h = 0; h < XN; h++)  // no-op for the gathered path
                    xa[f][h] = zero_unless(xa[f][h], k0 + f * 64 + 8 * h < (int)p.K);
            }
            // G[t]: packed bytes of rows 4g..4g+3 of the column accumulator t serves
            uint32_t G[NACC];
            if constexpr (TILED) {
#pragma unroll
                for (int t = 0; t < NACC; t++) G[t] = raw[f][t];
            } else if constexpr (BYTE) {
                G[0] = raw[f][0] | (raw[f][1] << 8) | (raw[f][2] << 16) | (raw[f][3] << 24);
            } else if constexpr (QUAD) {
#pragma unroll
                for (int cb = 0; cb < NCO; cb++) G[cb] = quad_transpose(raw[f][cb], sel_q);
            } else {
#pragma unroll
                for (int d = 0; d < ND; d++) {
                    uint32_t Gd[4];
                    transpose4x4_bytes(raw[f][0 * ND + d], raw[f][1 * ND + d], raw[f][2 * ND + d], raw[f][3 * ND + d], Gd);
#pragma unroll
                    for (int i = 0; i < 4; i++) G[4 * d + i] = Gd[i];
                }
            }
            if constexpr (MODE == MODE_I8) {
                uint32_t ta[4];
                if constexpr (XLDS) {  // already in operand order
                    ta[0] = xa[f][0].x; ta[1] = xa[f][0].y; ta[2] = xa[f][0].z; ta[3] = xa[f][0].w;
                } else if (p.x_operand_order) {  // uniform
                    ta[0] = xa[f][0].x; ta[1] = xa[f][0].y; ta[2] = xa[f][0].z; ta[3] = xa[f][0].w;
                } else {
                    transpose4x4_bytes(xa[f][0].x, xa[f][0].y, xa[f][0].z, xa[f][0].w, ta);
                }
                const v4i a = {(int)ta[0], (int)ta[1], (int)ta[2], (int)ta[3]};
#pragma unroll
                for (int t = 0; t < NACC; t++) {
                    const v4i b = decode16_i8(G[t]);
                    if (TWO && (f & 1))
                        acc2[TWO ? t : 0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc2[TWO ? t : 0], 0, 0, 0);
                    else
                        acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc[t], 0, 0, 0);
                }
            } else {
                // natural halves h0..h7 -> dword c = { h[c], h[4+c] } (the decode's k order)
                u32x4 au[2];
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    if constexpr (XLDS)  // already in operand order
                        au[h] = u32x4{xa[f][h].x, xa[f][h].y, xa[f][h].z, xa[f][h].w};
                    else
                        au[h] = u32x4{perm(xa[f][h].z, xa[f][h].x, 0x05040100u), perm(xa[f][h].z, xa[f][h].x, 0x07060302u),
                                      perm(xa[f][h].w, xa[f][h].y, 0x05040100u), perm(xa[f][h].w, xa[f][h].y, 0x07060302u)};
                }
#pragma unroll
                for (int t = 0; t < NACC; t++) {
#pragma unroll
                    for (int h = 0; h < 2; h++) {
                        // bytes [zero, row 2h, zero, row 2h+1] of G
                        const uint32_t M2 = perm(0u, G[t], h == 0 ? 0x010C000Cu : 0x030C020Cu);
                        acc_t& dst = (TWO && h == 1) ? acc2[TWO ? t : 0] : acc[t];
                        if constexpr (MODE == MODE_F16) {
                            const u32x4 bu = decode8_16bit<LUT_F16_ONE>(M2);
                            dst = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, au[h]),
                                                                         __builtin_bit_cast(v8h, bu), dst, 0, 0, 0);
                        } else {
                            const u32x4 bu = decode8_16bit<LUT_BF16_TWO>(M2);
                            dst = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, au[h]),
                                                                          __builtin_bit_cast(v8bf, bu), dst, 0, 0, 0);
                        }
                    }
                }
            }
        }
    }
    if constexpr (TWO) {
#pragma unroll
        for (int t = 0; t < NACC; t++) acc[t] += acc2[t];
    }

    // ---- sum the waves' accumulators through LDS, in wave order ------------------------
    // red[w][row][slot]; lane (j, g) holds rows 4g..4g+3 of slot t*16 + j
    const int M = p.M;
#pragma unroll
    for (int t = 0; t < NACC; t++) {
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

    if constexpr (EPI == EPI_SWIGLU_PAIRS && TILED && (NACC % 2 == 0) && MODE != MODE_I8) {
        // tiles 2P and 2P+1 of the tiled copy hold columns 16P.. of the gate half and of the up half
        const int64_t ffn = p.N >> 1;
        for (int idx = threadIdx.x; idx < M * (TILE_N / 2); idx += WAVES * 64) {
            const int row = idx / (TILE_N / 2);
            const int hl = idx % (TILE_N / 2);
            const int64_t h = (int64_t)tile * (TILE_N / 2) + hl;
            if (h >= ffn) continue;
            const int slot_g = (hl >> 4) * 32 + (hl & 15), slot_u = slot_g + 16;
            uint32_t bg = red[row * TILE_N + slot_g], bu = red[row * TILE_N + slot_u];
#pragma unroll
            for (int w = 1; w < WAVES; w++) {
                bg = add_bits<MODE>(bg, red[(w * M + row) * TILE_N + slot_g]);
                bu = add_bits<MODE>(bu, red[(w * M + row) * TILE_N + slot_u]);
            }
            const float g = round_to_dtype(linear_value<MODE>(p, bg, epi_scale(p.epi, h), epi_bias(p.epi, h)), p.y_dtype);
            const float u = round_to_dtype(
                linear_value<MODE>(p, bu, epi_scale(p.epi, ffn + h), epi_bias(p.epi, ffn + h)), p.y_dtype);
            store_out(p.Y, p.y_dtype, (int64_t)row * ffn + h, swiglu_value(g, u, p.y_dtype));
        }
        return;
    }
    for (int idx = threadIdx.x; idx < M * TILE_N; idx += WAVES * 64) {
        const int row = idx / TILE_N;
        const int nl = idx % TILE_N;
        if (nb + nl >= p.N) continue;
        // column nl of the tile sits in slot t*16 + j: LD_V*: nl = NACC*j + t; else (LD_T* too) nl = 16*t + j
        const int slot = (LD >= 4 && !TILED) ? (nl % NACC) * 16 + nl / NACC : nl;
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
    int ld;     // LD_* tile shape (tile = 16 columns for LD_BYTE, else 16*ld)
    int waves;  // waves per workgroup: 4, 8 or 16
};

// the kernel addresses W_T and X with 32-bit offsets from their base pointers
// decode-tiled copy: whole 16-column tiles and 16-row steps, 256 bytes each
size_t tiled_bytes(int64_t N, int64_t K) { return (size_t)ceil_div(N, 16) * (size_t)ceil_div(ceil_div(K, 4), 16) * 256; }

bool stream_supported_tiled(int64_t N, int64_t K, const void* W) {
    return ((uintptr_t)W) % 256 == 0 && N >= 1 && N < (1ll << 30) && K < (1ll << 26) && tiled_bytes(N, K) < (1ull << 32);
}

bool stream_supported(int64_t N, int64_t K, const void* W_T) {
    // (rows up to 16*16*16 past the end enter the offset arithmetic before they are clamped)
    return ((uintptr_t)W_T) % 16 == 0 && N >= 1 && (ceil_div(K, 4) + 8192) * N < (1ll << 32) && K < (1ll << 26);
}

static int ld_columns(int ld) { return ld == LD_BYTE ? 16 : ld > 100 ? 16 * (ld - 100) : 16 * ld; }

StreamPlan stream_plan(int mode, int64_t M, int64_t N, int64_t Kb, int w_layout, int min_nacc = 1) {
    StreamPlan pl;
    (void)Kb;
    // optional override for tuning runs: BITTORCH_STREAM_CFG="ld,waves"
    int o_ld = -1, o_waves = 0;
    if (const char* env = option(OPT_STREAM_CFG)) sscanf(env, "%d,%d", &o_ld, &o_waves);
    int ld;
    if (layout_tiled(w_layout)) {
        // 16-column tiles, up to four per workgroup (a batch re-reads its activations once per workgroup, and so
        // does a prologue; 240 workgroups of two tiles tie with 480 of one at N = 7680 and win with a prologue)
        // (every 16-row block of the call is a grid row of the same launch: the workgroups of all blocks count)
        const int min_tiles = (M > 4) ? 160 : 224;
        const int64_t row_blocks = ceil_div(M, 16);
        // (eight tiles per workgroup only for int8 batches of several blocks, whose activation re-reads they halve:
        // 256 rows at 4096^2 16.3 -> 13.2 us; the 16-bit modes, heavier in decode, lose 5-20 % with them)
        int nacc = (row_blocks >= 2 && min_nacc == 1 && mode == MODE_I8) ? 8 : 4;
        while (nacc > min_nacc && ceil_div(N, 16 * nacc) * row_blocks < min_tiles) nacc >>= 1;
        if (o_ld == LD_T1 || o_ld == LD_T2 || o_ld == LD_T4 || (o_ld == LD_T8 && M > 1 && min_nacc == 1 && mode == MODE_I8)) nacc = o_ld - 100;
        if (nacc < min_nacc) nacc = min_nacc;
        ld = 100 + nacc;
    } else if (N % 4 != 0) {
        ld = LD_BYTE;  // row starts are not dword aligned
    } else if ((o_ld == 16 || o_ld == 8 || o_ld == 4 || o_ld == 2 || o_ld == 1) && (o_ld < 4 || N % o_ld == 0)) {
        ld = o_ld;
    } else {
        // widest lane load the row pitch allows, narrowed until there are enough tiles to
        // occupy the chip (measured: 172 tiles of 64 columns beat 344 of 32 for a 16-row
        // batch, which re-reads its activations once per tile; a single row prefers >= 256)
        // (the int8 mode, whose decode is light, does better with 128-column tiles and 8 waves than
        // with 256-column tiles and 4 on very wide layers: 23.5 -> 17.4 us at N = 65536, K = 4096)
        ld = (N % 16 == 0 && mode != MODE_I8) ? 16 : (N % 8 == 0) ? 8 : 4;
        const int min_tiles = (M > 4) ? 160 : 256;
        const int64_t row_blocks = ceil_div(M, 16);  // all blocks of the call share one launch
        while (ld > 1 && ceil_div(N, ld_columns(ld)) * row_blocks < min_tiles) ld >>= 1;
    }
    pl.ld = ld;
    const int max_waves = (ld == 16) ? 4 : (ld == 8 || ld == LD_BYTE || ld == LD_T8) ? 8 : 16;   // LDS: WAVES*TILE_N <= 1024 words per row
    int waves = (o_waves == 4 || o_waves == 8 || o_waves == 16) ? o_waves : 8;
    if (waves > max_waves) waves = max_waves;
    pl.waves = waves;
    return pl;
}

size_t stream_workspace_bytes(int, int64_t, int64_t, int64_t) { return 0; }

template <int MODE, int LD, int WAVES>
static void launch_stream_k(const StreamParams& p, bool xlds, dim3 grid, size_t lds, hipStream_t st) {
    constexpr int PF = (LD == 16) ? 2 : (LD == 8 || LD == LD_T8) ? 4 : ((LD == 4 || LD == LD_T4) && MODE != MODE_I8) ? 4 : 8;
    if constexpr ((LD == LD_T2 || LD == LD_T4) && MODE != MODE_I8) {
        if (p.epi_op == EPI_SWIGLU_PAIRS) {
            if (xlds && p.pro_op == PRO_RMSNORM)
                hipLaunchKernelGGL((stream_kernel<MODE, LD, WAVES, PF, true, PRO_RMSNORM, EPI_SWIGLU_PAIRS>), grid, dim3(WAVES * 64), lds, st, p);
            else if (xlds)
                hipLaunchKernelGGL((stream_kernel<MODE, LD, WAVES, PF, true, PRO_NONE, EPI_SWIGLU_PAIRS>), grid, dim3(WAVES * 64), lds, st, p);
            else
                hipLaunchKernelGGL((stream_kernel<MODE, LD, WAVES, PF, false, PRO_NONE, EPI_SWIGLU_PAIRS>), grid, dim3(WAVES * 64), lds, st, p);
            return;
        }
    }
    if constexpr (LD <= 4 || (LD > 100 && LD != LD_T8)) {  // decode-shape tiles: the M = 1 variant with x staged in LDS
        if (xlds) {
            if constexpr (MODE != MODE_I8) {
                if (p.pro_op == PRO_RMSNORM) {
                    hipLaunchKernelGGL((stream_kernel<MODE, LD, WAVES, PF, true, PRO_RMSNORM>), grid, dim3(WAVES * 64), lds, st, p);
                    return;
                }
                if (p.pro_op == PRO_SWIGLU) {
                    hipLaunchKernelGGL((stream_kernel<MODE, LD, WAVES, PF, true, PRO_SWIGLU>), grid, dim3(WAVES * 64), lds, st, p);
                    return;
                }
            }
            hipLaunchKernelGGL((stream_kernel<MODE, LD, WAVES, PF, true>), grid, dim3(WAVES * 64), lds, st, p);
            return;
        }
    }
    hipLaunchKernelGGL((stream_kernel<MODE, LD, WAVES, PF, false>), grid, dim3(WAVES * 64), lds, st, p);
}

template <int MODE, int LD>
static void launch_stream_w(const StreamParams& p, int waves, bool xlds, dim3 grid, size_t lds, hipStream_t st) {
    if constexpr (LD <= 4 || (LD > 100 && LD != LD_T8)) {
        if (waves == 16) { launch_stream_k<MODE, LD, 16>(p, xlds, grid, lds, st); return; }
    }
    if constexpr (LD <= 8 || LD > 100) {
        if (waves == 8) { launch_stream_k<MODE, LD, 8>(p, xlds, grid, lds, st); return; }
    }
    launch_stream_k<MODE, LD, 4>(p, xlds, grid, lds, st);
}

// x slice in LDS (the M = 1 variant): one row, aligned, at most XC_MAX 16-byte chunks per lane and
// wave, and within the default 64 KiB of dynamic LDS
static bool xlds_ok(int es, int M, bool x_vec_ok, const StreamPlan& pl, int64_t K) {
    const int64_t tile_n = ld_columns(pl.ld);
    const int64_t spw = ceil_div(ceil_div(K, 64), pl.waves);
    const size_t red_bytes = (size_t)pl.waves * M * tile_n * 4;
    const size_t xs_bytes = (size_t)pl.waves * XC_MAX * 64 * 16;
    return M == 1 && x_vec_ok && (pl.ld <= 4 || (pl.ld > 100 && pl.ld != LD_T8)) && spw * 64 * es <= XC_MAX * 64 * 16 && K >= 16 / es &&
           red_bytes + xs_bytes <= 64 * 1024 && !tuning_env("BITTORCH_STREAM_NOXLDS");
}

// Can the streaming kernel apply an RMSNorm / SwiGLU prologue to this call's activation row itself?
// (one 16-bit row that takes the LDS-staged variant; BITTORCH_NO_PROLOGUE=1 says no, for A/B runs)
bool stream_prologue_fusable(int mode, int64_t B, int64_t N, int64_t K, const void* X, const void* pro_b, int w_layout,
                             int epi_op) {
    if (mode == MODE_I8 || B != 1 || tuning_env("BITTORCH_NO_PROLOGUE")) return false;
    const bool vec = ((uintptr_t)X) % 16 == 0 && (!pro_b || ((uintptr_t)pro_b) % 16 == 0) && (K * 2) % 16 == 0;
    if (epi_op != EPI_NONE && mode == MODE_I8) return false;
    return xlds_ok(2, 1, vec, stream_plan(mode, 1, N, ceil_div(K, 4), w_layout, epi_op == EPI_SWIGLU_PAIRS ? 2 : 1), K);
}

template <int MODE>
static int launch_stream_mode(StreamParams p, const StreamPlan& pl, hipStream_t st) {
    const int64_t tile_n = ld_columns(pl.ld);
    p.tiles = (int)ceil_div(p.N, tile_n);
    p.per_xcd = (int)ceil_div(p.tiles, 8);
    unsigned grid_x = (unsigned)(p.per_xcd * 8);
    if (p.B > 16 && p.tiles % 8 != 0 && p.tiles < 64) {  // few tiles, many row blocks: balance the XCDs instead
        p.per_xcd = 0;
        grid_x = (unsigned)p.tiles;
    }
    const dim3 grid(grid_x, (unsigned)ceil_div(p.B, 16));
    const int waves = pl.waves;
    const int es = (MODE == MODE_I8) ? 1 : 2;
    const size_t red_bytes = (size_t)waves * p.M * tile_n * 4;
    const size_t xs_bytes = (size_t)waves * XC_MAX * 64 * 16;
    const bool xlds = xlds_ok(es, p.M, p.x_vec_ok != 0, pl, p.K);
    const size_t lds = red_bytes + (xlds ? xs_bytes : 0);
    if (p.epi_op == EPI_SWIGLU_PAIRS && (MODE == MODE_I8 || (pl.ld != LD_T2 && pl.ld != LD_T4) || p.N % 32 != 0 ||
                                         p.pro_op == PRO_SWIGLU || p.epi.residual)) {
        set_error("stream_gemm: the SwiGLU output stage needs 16-bit activations, pair-ordered tiled weights, N %% 32 == 0, "
                  "no SwiGLU prologue and no residual");
        return BT_ERR_INVALID;
    }
    if (p.pro_op != PRO_NONE && !xlds) {
        set_error("stream_gemm: activation prologue on a shape the callers should have routed elsewhere");
        return BT_ERR_INVALID;
    }
    switch (pl.ld) {
        case 16: launch_stream_w<MODE, 16>(p, waves, xlds, grid, lds, st); break;
        case 8: launch_stream_w<MODE, 8>(p, waves, xlds, grid, lds, st); break;
        case 4: launch_stream_w<MODE, 4>(p, waves, xlds, grid, lds, st); break;
        case 2: launch_stream_w<MODE, 2>(p, waves, xlds, grid, lds, st); break;
        case 1: launch_stream_w<MODE, 1>(p, waves, xlds, grid, lds, st); break;
        case LD_T1: launch_stream_w<MODE, LD_T1>(p, waves, xlds, grid, lds, st); break;
        case LD_T2: launch_stream_w<MODE, LD_T2>(p, waves, xlds, grid, lds, st); break;
        case LD_T4: launch_stream_w<MODE, LD_T4>(p, waves, xlds, grid, lds, st); break;
        case LD_T8:
            if constexpr (MODE == MODE_I8) launch_stream_w<MODE, LD_T8>(p, waves, false, grid, lds, st);
            break;
        default: launch_stream_w<MODE, 0>(p, waves, xlds, grid, lds, st); break;
    }
    return check_launch("stream_gemm");
}

// One launch for the whole call: grid.y walks its blocks of 16 activation rows.
// planes = 1: X is [B, K].  planes = 3: X is [B, 3*Kp], Kp = K rounded up to 64, three zero-padded planes
// of K values per row whose products with the same weights are summed (fp32 activations split into three
// bf16 terms); the kernel walks 3*Kp values of k and wraps its weight step index every Kp (weight rows past
// the matrix are clamped or zero padding, and meet zero activations).
// w_layout: W_LAYOUT_ROW_MAJOR (the reference's W_T [Kb, N]) or W_LAYOUT_TILED (retile_kernel's copy)
// q_layout: MODE_I8 only (Q_OPERAND_ORDER needs K % 16 == 0 and 16-byte aligned rows)
// pro_op / pro_b / pro_eps: activation prologue (PRO_*), only where stream_prologue_fusable() said yes
// epi_op: EPI_SWIGLU_PAIRS makes Y [B, N/2] (tiled weights in gate/up pair order, 16-bit modes)
int launch_stream(int mode, const void* X, int x_elem_size, const float* s_x, const uint8_t* W_T, int w_layout,
                  const Epilogue& epi, void* Y, int y_dtype, int32_t* acc_out, int64_t B, int64_t N,
                  int64_t K, int planes, int q_layout, int pro_op, const void* pro_b, float pro_eps, int epi_op, hipStream_t st) {
    const int64_t Kb = ceil_div(K, 4);
    const int64_t Kx = (planes == 3) ? 3 * ceil_div(K, 64) * 64 : K;
    const StreamPlan pl = stream_plan(mode, B, N, Kb, w_layout, epi_op == EPI_SWIGLU_PAIRS ? 2 : 1);
    const int64_t Ny = (epi_op == EPI_SWIGLU_PAIRS) ? N / 2 : N;  // columns of Y
    const int y_size = dtype_size(y_dtype);
    // one launch covers 65535 blocks of 16 rows; a taller call is served in slices of that many rows
    const int64_t max_rows = 65535ll * 16;
    if (B > max_rows) {
        for (int64_t r0 = 0; r0 < B; r0 += max_rows) {
            Epilogue e = epi;
            if (e.residual) e.residual = (const uint8_t*)epi.residual + r0 * N * y_size;
            const int rc = launch_stream(mode, (const uint8_t*)X + r0 * Kx * x_elem_size, x_elem_size, s_x ? s_x + r0 : nullptr, W_T,
                                         w_layout, e, (uint8_t*)Y + r0 * Ny * y_size, y_dtype, acc_out ? acc_out + r0 * N : nullptr,
                                         (B - r0 < max_rows) ? B - r0 : max_rows, N, K, planes, q_layout, pro_op, pro_b, pro_eps,
                                         epi_op, st);
            if (rc) return rc;
        }
        return BT_OK;
    }
    StreamParams p;
    p.X = X;
    p.W_T = W_T;
    p.s_x = s_x;
    p.Y = Y;
    p.acc_out = acc_out;
    p.epi = epi;
    p.N = N; p.K = Kx; p.Kb = Kb;
    p.wsteps = (int)ceil_div(Kb, 16);
    p.tiles16 = tiles16_arg(N, w_layout);
    p.prehalved = planes == 3;
    p.x_operand_order = (mode == MODE_I8 && q_layout == Q_OPERAND_ORDER) ? 1 : 0;
    p.pro_op = pro_op; p.pro_b = pro_b; p.pro_eps = pro_eps; p.epi_op = epi_op;
    p.B = B;
    p.M = (int)((B < 16) ? B : 16);
    p.y_dtype = y_dtype;
    // (a row is a multiple of 16 bytes, so every 16-row block starts as aligned as the first)
    p.x_vec_ok = (((uintptr_t)p.X) % 16 == 0) && ((Kx * x_elem_size) % 16 == 0);
    if (mode == MODE_I8) return launch_stream_mode<MODE_I8>(p, pl, st);
    if (mode == MODE_F16) return launch_stream_mode<MODE_F16>(p, pl, st);
    return launch_stream_mode<MODE_BF16>(p, pl, st);
}

}  // namespace bt
