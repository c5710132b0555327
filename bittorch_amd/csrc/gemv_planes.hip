// Decode GEMV (one activation row) for fp16 activations on the int8 matrix cores, exact.
//
// What it computes (the float path of the reference's packed kernel,
// csrc/kernels/ternary_gemm_production.cu:126-141, with the accumulation done exactly):
//     acc[n] = sum_k x[k] * w[k, n]      y[n] = acc[n] * scale[n] + bias[n]
// The reference adds the products one by one in fp32.  Here the sum is formed without any rounding:
// every finite fp16 value is an integer multiple of 2^-24 below 2^16, so X[k] = x[k] * 2^24 is an
// integer of at most 41 bits, S[n] = sum_k X[k] * w[k, n] is an exact integer, and
//     acc[n] = RN_fp32(S[n]) * 2^-24
// is the correctly rounded value of the exact dot product.  The result does not depend on how the
// kernel splits K, which is what makes the single-launch kernel, the grouped kernel and both weight
// layouts agree bit for bit.  (Rows that hold an infinity or a NaN give NaN in every column, which
// is what the reference's float arithmetic gives whenever such a value meets a zero weight.)
//
// How: X[k] is written in six base-128 digits, X = sum_p d_p 128^p with d_0..d_4 in 0..127 and d_5
// the signed top digit (two's complement), each an int8.  The six digit rows are six rows of the A
// operand of v_mfma_i32_16x16x64_i8 (a decode step has one activation row, so the other fifteen rows
// of the matrix instruction are free anyway); the B operand is the 2-bit weights decoded to int8
// {-1, 0, +1} (9 VALU operations per 16 weights, against 24 for the 16-bit decode); the int32
// accumulators of the six rows are recombined in 64-bit integer arithmetic at the end.
//
// Three kernels share the arithmetic:
//   gemv_planes_kernel        one weight matrix per launch; a workgroup owns a tile of 16 * NACC columns over the
//                             whole of K and its waves split K (deterministic integer sum through LDS).
//   gemv_planes_chunk_kernel  G independent units (own x, W, scale, bias, y; pointer tables in device memory) in ONE
//                             launch, or one very wide matrix: persistent workgroups each read a contiguous run of
//                             the (unit, 16-column tile) sequence front to back, their waves splitting K, so that
//                             the launch, set-up and drain of a 4 MiB GEMV are paid once per launch instead of once
//                             per matrix and the weights arrive in the order the memory system streams fastest.
//   gemv_planes_group_kernel  the grouped launch for the shapes the kernel above does not take (long K, few tiles per
//                             workgroup): (unit, column slab) items, a wave owns 16 * NACC columns over the whole of K
//                             (no reduction, no barrier inside an item) and keeps its weight loads running across
//                             item boundaries.
#include <cstddef>
#include <cstdlib>

#include "row_math.h"

namespace bt {

constexpr int PL_N = 6;                    // digit planes
constexpr int PL_GROUP = PL_N * 16;        // bytes of one 16-k group in LDS: six 16-byte operand fragments

enum { PL_TILED = 0, PL_ROWMAJOR = 1 };

struct PlaneParams {
    // The first 64 bytes hold what a workgroup needs before it can request its first bytes: the kernel arguments
    // come through the scalar cache one 64-byte line at a time, and every line is a round trip that a
    // latency-bound launch waits for.
    // single launch: direct pointers.  grouped launch: tables of G device pointers (bias_tab may be null).
    const void* X;
    const uint8_t* W;
    int64_t K, N;
    int wsteps;      // 16-row steps of the weights (64 k each)
    int tiles16;     // 16-column tiles
    int tiles;       // single launch: workgroup tiles of 16 * NACC columns
    int per_xcd;     // single launch: tiles per XCD (grid = 8 * per_xcd)
    int64_t Kb;
    const void* scale;
    // ---- second line
    const void* bias;
    const void* residual;
    void* Y;
    int scale_dtype, bias_dtype, scale_bcast;
    int x_dtype;     // BT_F16, or BT_BF16 (grouped launches and the contiguous walk)
    int G;
    int slabs;       // grouped launch: column slabs (8 waves x 16 * NACC columns) per unit, or tiles per workgroup
    int items;       // grouped launch: G * slabs
    float pro_eps;   // one-matrix kernel with an RMSNorm prologue
    int tiles16_signed;  // one-matrix kernel on tiled weights: tiles16, negative for a pair-ordered copy read in natural order (stored_tile16)
    int pad_;
    // ---- third line
    const void* const* X_tab;
    const uint8_t* const* W_tab;
    const void* const* scale_tab;
    const void* const* bias_tab;
    void* const* Y_tab;
    const void* pro_b;   // one-matrix kernel with a prologue: the norm weight (RMSNorm) or the second operand (SwiGLU), K values
};
static_assert(offsetof(PlaneParams, scale) == 56 && offsetof(PlaneParams, X_tab) == 128, "argument lines as laid out above");

// ---- fp16 -> six int8 digit planes ----------------------------------------------------------------
// Eight consecutive fp16 values (one 16-byte load) -> per plane the eight digit bytes, elements 0..3 in
// lo[p] and 4..7 in hi[p].  Returns true if any value is an infinity or a NaN.
__device__ __forceinline__ bool f16x8_to_planes(const uint4 v, uint32_t (&lo)[PL_N], uint32_t (&hi)[PL_N]) {
    const uint32_t d[4] = {v.x, v.y, v.z, v.w};
    bool bad = false;
#pragma unroll
    for (int p = 0; p < PL_N; p++) lo[p] = hi[p] = 0u;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const uint32_t h = (d[e >> 1] >> (16 * (e & 1))) & 0xffffu;
        const uint32_t ex = (h >> 10) & 31u, m = h & 0x3ffu;
        bad |= (ex == 31u);
        const uint32_t mag = ex ? (m | 0x400u) : m;      // 11-bit significand (subnormals: no hidden bit)
        const uint32_t sh = ex ? ex - 1u : 0u;           // x = mag * 2^(sh - 24)
        const int32_t sm = (h & 0x8000u) ? -(int32_t)mag : (int32_t)mag;
        const int64_t X = (int64_t)sm << sh;             // x * 2^24, |X| < 2^40
        const uint32_t xl = (uint32_t)X, xh = (uint32_t)((uint64_t)X >> 32);
        uint32_t dg[PL_N];
        dg[0] = xl & 127u;
        dg[1] = (xl >> 7) & 127u;
        dg[2] = (xl >> 14) & 127u;
        dg[3] = (xl >> 21) & 127u;
        dg[4] = ((xl >> 28) | (xh << 4)) & 127u;
        dg[5] = (xh >> 3) & 255u;                        // bits 35..42: the signed top digit as a byte
#pragma unroll
        for (int p = 0; p < PL_N; p++) {
            if (e < 4) lo[p] |= dg[p] << (8 * e);
            else hi[p] |= dg[p] << (8 * (e - 4));
        }
    }
    return bad;
}

// bf16 activations: the exponent range of bf16 (2^-133 .. 2^127) does not fit a fixed-point word, so the row is
// scaled by its own largest exponent.  With e1 = max(biased exponent, 1) and mag the 8-bit significand, a finite value
// is mag * 2^(e1 - 134); emax = the largest e1 of the row; X = value * 2^(166 - emax) = mag * 2^(e1 - emax + 32), an
// integer below 2^40 in magnitude for every element.  Elements more than 32 binades below the row's largest lose low
// bits (rounded half up in magnitude; more than 40 binades below: 0) -- an error of at most 2^-41 of the largest
// element each, far below what an fp32 accumulator carries; all others are represented exactly.
// The sum S of the X is exact, and acc = RN_fp32(S) * 2^(emax - 166).
__device__ __forceinline__ int bf16_e1(uint32_t h) {  // 0 for an infinity or a NaN (not part of the maximum)
    const int e = (int)((h >> 7) & 255u);
    return e == 255 ? 0 : (e ? e : 1);
}
__device__ __forceinline__ int bf16x8_max_e1(const uint4 v) {
    const uint32_t d[4] = {v.x, v.y, v.z, v.w};
    int m = 0;
#pragma unroll
    for (int e = 0; e < 8; e++) m = max(m, bf16_e1((d[e >> 1] >> (16 * (e & 1))) & 0xffffu));
    return m;
}
__device__ __forceinline__ bool bf16x8_to_planes(const uint4 v, int emax, uint32_t (&lo)[PL_N], uint32_t (&hi)[PL_N]) {
    const uint32_t d[4] = {v.x, v.y, v.z, v.w};
    bool bad = false;
#pragma unroll
    for (int p = 0; p < PL_N; p++) lo[p] = hi[p] = 0u;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const uint32_t h = (d[e >> 1] >> (16 * (e & 1))) & 0xffffu;
        const uint32_t ex = (h >> 7) & 255u, m = h & 0x7fu;
        bad |= (ex == 255u);
        const uint32_t mag = ex ? (m | 0x80u) : m;
        const int sh = (int)(ex ? ex : 1u) - emax + 32;  // <= 32
        uint64_t mg;
        if (sh >= 0) mg = (uint64_t)mag << sh;
        else if (sh >= -8) mg = (uint64_t)((mag + (1u << (-sh - 1))) >> (-sh));
        else mg = 0;
        const int64_t X = (h & 0x8000u) ? -(int64_t)mg : (int64_t)mg;
        const uint32_t xl = (uint32_t)X, xh = (uint32_t)((uint64_t)X >> 32);
        uint32_t dg[PL_N];
        dg[0] = xl & 127u;
        dg[1] = (xl >> 7) & 127u;
        dg[2] = (xl >> 14) & 127u;
        dg[3] = (xl >> 21) & 127u;
        dg[4] = ((xl >> 28) | (xh << 4)) & 127u;
        dg[5] = (xh >> 3) & 255u;
#pragma unroll
        for (int p = 0; p < PL_N; p++) {
            if (e < 4) lo[p] |= dg[p] << (8 * e);
            else hi[p] |= dg[p] << (8 * (e - 4));
        }
    }
    return bad;
}

__device__ __forceinline__ uint4 zero_unless4(uint4 v, bool ok) {
    v.x = ok ? v.x : 0u; v.y = ok ? v.y : 0u; v.z = ok ? v.z : 0u; v.w = ok ? v.w : 0u;
    return v;
}

// Chunk c of a row (elements 8c .. 8c+7) -> LDS, in matrix-core operand order.  `planes` points at the row's (or
// the wave slice's) first 16-k group; even and odd lanes hold the two halves of one group and exchange bytes, so
// every lane of a pair must call it (`write` = false for pairs outside the buffer).  v must already be zero for
// chunks beyond K.
template <int XDT = BT_F16>
__device__ __forceinline__ bool park_chunk(uint8_t* planes, int c, const uint4 v, int lane, bool write, int emax = 0) {
    uint32_t lo[PL_N], hi[PL_N];
    bool bad;
    if constexpr (XDT == BT_BF16) bad = bf16x8_to_planes(v, emax, lo, hi);
    else bad = f16x8_to_planes(v, lo, hi);
    uint8_t* dst = planes + (size_t)(c >> 1) * PL_GROUP + 8 * (c & 1);
#pragma unroll
    for (int p = 0; p < PL_N; p++) {
        const uint2 o = q_to_operand_order(lo[p], hi[p], lane & 1);
        if (write) *(uint2*)(dst + 16 * p) = o;
    }
    return bad;
}

// d = the dword this lane loaded (row 4g+q, four columns); returns the bytes of column q of the dwords of quad
// lanes 0..3, i.e. rows 4g..4g+3 of this lane's own column (row-major W_T)
__device__ __forceinline__ uint32_t pl_quad_transpose(uint32_t d, uint32_t sel_q) {
    const uint32_t v0 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)d, 0x00, 0xf, 0xf, true);
    const uint32_t v1 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)d, 0x55, 0xf, 0xf, true);
    const uint32_t v2 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)d, 0xAA, 0xf, 0xf, true);
    const uint32_t v3 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)d, 0xFF, 0xf, 0xf, true);
    const uint32_t t01 = perm(v1, v0, sel_q);
    const uint32_t t23 = perm(v3, v2, sel_q);
    return perm(t23, t01, 0x05040100u);
}

// the exact sum S (in units of 2^-24), correctly rounded to fp32 and scaled back
__device__ __forceinline__ float fixed_to_f32(int64_t S, int exp2 = -24) { return __builtin_ldexpf((float)S, exp2); }
// ... from its six plane sums
__device__ __forceinline__ float planes_to_f32(const int32_t (&s)[PL_N], int exp2 = -24) {
    int64_t S = 0;
#pragma unroll
    for (int p = PL_N - 1; p >= 0; p--) S = S * 128 + (int64_t)s[p];
    return fixed_to_f32(S, exp2);
}

template <int XDT = BT_F16>
__device__ __forceinline__ void pl_store(void* Y, const void* residual, int64_t n, float acc, float s, float b) {
    float y = epi_float(acc, s, b);
    if (residual) y = add_residual(y, residual, XDT, n);
    ((uint16_t*)Y)[n] = (XDT == BT_BF16) ? f32_to_bf16_bits(y) : f32_to_f16_bits(y);
}

// A row that holds an infinity or a NaN has no fixed-point image; its outputs are what the reference's fp32 loop
// leaves (ternary_gemm_production.cu:126-133: acc += x * w with w decoded to 0.0f or +-1.0f): the sum of x[k] * w[k, n]
// over the non-finite x[k] alone, since no finite term changes it -- NaN where a NaN, an infinity on a zero weight or
// infinities of both signs meet, otherwise the infinity with its sign.  The slow way, one thread per column scanning
// the row: such rows are not what a kernel is tuned for.  xk(k) returns the row's element k as 16-bit pattern (after
// the activation prologue, if the kernel has one).
__device__ __forceinline__ int packed_code(const uint8_t* W, bool tiled, int S, int tiles16_signed, int64_t N, int64_t n, int k) {
    size_t byte;
    if (tiled) {
        const int t = stored_tile16((int)(n >> 4), tiles16_signed);
        byte = (((size_t)t * S + (k >> 6)) * 64 + 16 * ((k >> 4) & 3) + (size_t)(n & 15)) * 4 + ((k >> 2) & 3);
    } else {
        byte = (size_t)(k >> 2) * (size_t)N + (size_t)n;
    }
    return (W[byte] >> (2 * (k & 3))) & 3;
}
template <int XDT, typename XK>
__device__ __forceinline__ float nonfinite_acc(XK xk, int K, const uint8_t* W, bool tiled, int S, int tiles16_signed, int64_t N,
                                            int64_t n) {
    float acc = 0.0f;
    for (int k = 0; k < K; k++) {
        const uint32_t h = xk(k);
        const bool nonfinite = (XDT == BT_BF16) ? ((h >> 7) & 255u) == 255u : ((h >> 10) & 31u) == 31u;
        if (!nonfinite) continue;
        const float xv = (XDT == BT_BF16) ? bf16_bits_to_f32((uint16_t)h) : f16_bits_to_f32((uint16_t)h);
        const int c = packed_code(W, tiled, S, tiles16_signed, N, n, k);
        acc = __fadd_rn(acc, __fmul_rn(xv, c == 1 ? 1.0f : c == 2 ? -1.0f : 0.0f));
    }
    return acc;
}

// The same as a call: the grouped kernels keep this path out of their loops' register allocation that way (inlined it
// cost the contiguous walk 4 % -- 87.9 -> 91.8 us at 128 units -- although it never runs there).
template <int XDT>
__device__ __noinline__ float nonfinite_acc_row(const uint16_t* xrow, int K, const uint8_t* W, int S, int tiles16, int64_t N, int64_t n) {
    return nonfinite_acc<XDT>([&](int k) -> uint32_t { return xrow[k]; }, K, W, true, S, tiles16, N, n);
}

// ---- one weight matrix per launch -------------------------------------------------------------------
// LDS: [WAVES][2][TILE_N] int64 partial sums, [WAVES] flags, then per wave the digit planes of its K slice.
// EPI = EPI_SWIGLU_PAIRS (tiled copy in gate/up pair order, NACC even): Y [N/2], Y[h] = rd(rd(silu(g)) * u) with
// g = rd(linear column h), u = rd(linear column N/2 + h), what the SwiGLU kernel makes of the stored projections.
// TAB: a few units in one launch (pointer tables, p.slabs workgroup tiles per unit).
// PRO: the activation row is produced on its way into LDS, with the row kernels' own element arithmetic (row_math.h),
// so that the result equals "row kernel, then GEMV" bit for bit: PRO_RMSNORM x <- rd((x * r) * w) with the row's
// sum of squares formed in double (exact for 16-bit values of ordinary spread, hence the same whichever way the
// waves split it; their partial sums meet in LDS, one more barrier); PRO_SWIGLU x <- rd(rd(silu(x)) * u).
template <int LAYOUT, int NACC, int WAVES, int PF, int EPI = EPI_NONE, bool TAB = false, int PRO = PRO_NONE>
__global__ __launch_bounds__(WAVES * 64) void gemv_planes_kernel(PlaneParams p) {
    constexpr int TILE_N = 16 * NACC;
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];

    int tile = (int)(blockIdx.x & 7) * p.per_xcd + (int)(blockIdx.x >> 3);  // neighbouring tiles on one XCD
    if (tile >= p.tiles) return;
    const void* Xp = p.X;
    const uint8_t* Wp = p.W;
    const void* scalep = p.scale;
    const void* biasp = p.bias;
    void* Yp = p.Y;
    if constexpr (TAB) {  // workgroup tile -> (unit, tile)
        const int unit = tile / p.slabs;
        tile -= unit * p.slabs;
        Xp = p.X_tab[unit];
        Wp = p.W_tab[unit];
        scalep = p.scale_tab[unit];
        biasp = p.bias_tab ? p.bias_tab[unit] : nullptr;
        Yp = p.Y_tab[unit];
    }
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int j = lane & 15, g = lane >> 4, q = lane & 3;
    const int nsteps = (int)((p.K + 63) >> 6);
    const int spw = (nsteps + WAVES - 1) / WAVES;  // steps per wave, contiguous
    const int s_begin = wave * spw;
    const int s_end = min(nsteps, s_begin + spw);
    const int nchunks = spw * 8;                   // 16-byte chunks of the wave's slice of x

    uint32_t* red = lds;
    uint32_t* flags = lds + WAVES * 4 * TILE_N;
    uint8_t* planes = (uint8_t*)(flags + WAVES) + (size_t)wave * spw * 4 * PL_GROUP;

    // 1. the wave's slice of x (needed first, and loads return in order), 2. its first batch of weights,
    // 3. the epilogue operands; the slice is converted while the weights are on their way
    constexpr int XC = 4;  // chunks per lane (the host keeps spw * 8 <= 64 * XC)
    uint4 xr[XC];
#pragma unroll
    for (int u = 0; u < XC; u++) {
        if (u * 64 < nchunks) {  // uniform
            const int k = s_begin * 64 + (lane + 64 * u) * 8;
            xr[u] = *(const uint4*)((const uint16_t*)Xp + (uint32_t)min(k, (int)p.K - 8));
        }
    }
    // byte offset of this lane's dword in step 0 of each of its 16-column tiles (tiled copy), resp. of its quad's
    // four columns in row 4g+q (row-major W_T); a tile / column past the end repeats valid bytes and is never stored
    uint32_t coloff[NACC];
    const uint32_t N32 = (uint32_t)p.N;
#pragma unroll
    for (int t = 0; t < NACC; t++) {
        if constexpr (LAYOUT == PL_TILED) {
            coloff[t] = ((uint32_t)stored_tile16(tile * NACC + t, p.tiles16_signed) * (uint32_t)p.wsteps * 64u + (uint32_t)lane) * 4u;
        } else {
            const int64_t c = (int64_t)tile * TILE_N + 16 * t + (j & ~3);
            coloff[t] = (c < p.N) ? (uint32_t)c : 0u;
        }
    }
    const uint32_t last_rowoff = (uint32_t)(p.Kb - 1) * N32;
    const uint32_t sel_q = 0x0C0C0000u | ((uint32_t)(4 + q) << 8) | (uint32_t)q;
    auto load_weights = [&](int base, uint32_t (&raw)[PF][NACC]) {
#pragma unroll
        for (int f = 0; f < PF; f++) {
            const int ws = min(base + f, p.wsteps - 1);  // uniform; steps past the end meet zero activations
#pragma unroll
            for (int t = 0; t < NACC; t++) {
                if constexpr (LAYOUT == PL_TILED) {
                    raw[f][t] = ldw_nt(Wp + (coloff[t] + (uint32_t)ws * 256u));
                } else {
                    const uint32_t ro = min((uint32_t)(16 * ws + 4 * g + q) * N32, last_rowoff);
                    raw[f][t] = ldw_nt(Wp + (ro + coloff[t]));
                }
            }
        }
    };
    uint32_t raw0[PF][NACC];
    load_weights(s_begin, raw0);

    // output threads: one column each; with the SwiGLU output stage one column h of the hidden vector each, made
    // of columns h (tile 2P of the pair-ordered copy) and N/2 + h (tile 2P + 1)
    uint32_t pre_s = 0u, pre_b = 0u, pre_s2 = 0u, pre_b2 = 0u;
    constexpr bool PAIRS = (EPI == EPI_SWIGLU_PAIRS);
    const int tid = (int)threadIdx.x;
    const int64_t ffn = p.N >> 1;
    const int64_t n_out = PAIRS ? (int64_t)tile * (TILE_N / 2) + tid : (int64_t)tile * TILE_N + tid;
    const bool out_thread = PAIRS ? (tid < TILE_N / 2 && n_out < ffn) : (tid < TILE_N && n_out < p.N);
    const int slot = PAIRS ? (tid >> 4) * 32 + (tid & 15) : tid;
    if (out_thread) {
        pre_s = load_bits_rt(scalep, p.scale_dtype, p.scale_bcast ? 0 : n_out);
        if (biasp) pre_b = load_bits_rt(biasp, p.bias_dtype, n_out);
        if constexpr (PAIRS) {
            pre_s2 = load_bits_rt(scalep, p.scale_dtype, p.scale_bcast ? 0 : ffn + n_out);
            if (biasp) pre_b2 = load_bits_rt(biasp, p.bias_dtype, ffn + n_out);
        }
    }

    float pro_r = 0.0f;  // RMSNorm prologue: the row's reciprocal root mean square
    if constexpr (PRO != PRO_NONE) {
        __shared__ double ss_slot[WAVES];
        uint4 br[XC];  // the second operand at the same positions
#pragma unroll
        for (int u = 0; u < XC; u++) {
            if (u * 64 < nchunks) {
                const int k = s_begin * 64 + (lane + 64 * u) * 8;
                // (RMSNorm without a weight: ones, as the row kernel multiplies by 1)
                if (p.pro_b) br[u] = *(const uint4*)((const uint16_t*)p.pro_b + (uint32_t)min(k, (int)p.K - 8));
                else br[u] = make_uint4(0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u);
            }
        }
        float r = 0.0f;
        if constexpr (PRO == PRO_RMSNORM) {
            double ss = 0.0;
#pragma unroll
            for (int u = 0; u < XC; u++) {
                if (u * 64 < nchunks) {
                    const int c = lane + 64 * u;
                    const int k = s_begin * 64 + c * 8;
                    if (k < (int)p.K && c < nchunks) {  // (a clamped chunk repeats values that another lane counts)
                        const uint32_t d[4] = {xr[u].x, xr[u].y, xr[u].z, xr[u].w};
#pragma unroll
                        for (int e = 0; e < 8; e++) {
                            const double xv = (double)f16_bits_to_f32((uint16_t)(d[e >> 1] >> (16 * (e & 1))));
                            ss += xv * xv;
                        }
                    }
                }
            }
            ss = wave_sum_f64(ss);
            if (lane == 0) ss_slot[wave] = ss;
            __syncthreads();
            ss = 0.0;
#pragma unroll
            for (int w = 0; w < WAVES; w++) ss += ss_slot[w];
            r = rms_rstd(ss, (int)p.K, p.pro_eps);
            pro_r = r;
        }
#pragma unroll
        for (int u = 0; u < XC; u++) {
            if (u * 64 < nchunks) {
                const uint32_t d[4] = {xr[u].x, xr[u].y, xr[u].z, xr[u].w};
                const uint32_t b[4] = {br[u].x, br[u].y, br[u].z, br[u].w};
                uint32_t o[4];
#pragma unroll
                for (int e2 = 0; e2 < 4; e2++) {
                    uint32_t h2 = 0u;
#pragma unroll
                    for (int hf = 0; hf < 2; hf++) {
                        const float xv = f16_bits_to_f32((uint16_t)(d[e2] >> (16 * hf)));
                        const float bv = f16_bits_to_f32((uint16_t)(b[e2] >> (16 * hf)));
                        const float hv = (PRO == PRO_RMSNORM) ? rmsnorm_value(xv, r, bv, BT_F16) : swiglu_value(xv, bv, BT_F16);
                        h2 |= (uint32_t)f32_to_f16_bits(hv) << (16 * hf);
                    }
                    o[e2] = h2;
                }
                xr[u] = make_uint4(o[0], o[1], o[2], o[3]);
            }
        }
    }
    bool bad = false;
#pragma unroll
    for (int u = 0; u < XC; u++) {
        if (u * 64 < nchunks) {
            const int c = lane + 64 * u;
            const int k = s_begin * 64 + c * 8;
            const uint4 v = zero_unless4(xr[u], k < (int)p.K && c < nchunks);
            bad |= park_chunk(planes, c, v, lane, c < nchunks);
        }
    }
    if (__builtin_amdgcn_ballot_w64(bad) != 0ull) bad = true;

    v4i acc[NACC];
#pragma unroll
    for (int t = 0; t < NACC; t++) acc[t] = v4i{0, 0, 0, 0};
    // lane (i, g) feeds digit row i of k-group g; rows 6..15 of the matrix instruction repeat rows 0..5 (unused)
    const uint8_t* a_src = planes + g * PL_GROUP + (j % PL_N) * 16;

    for (int base = s_begin; base < s_end; base += PF) {
        uint32_t raw[PF][NACC];
        if (base == s_begin) {  // uniform: this batch was requested ahead of the conversion
#pragma unroll
            for (int f = 0; f < PF; f++)
#pragma unroll
                for (int t = 0; t < NACC; t++) raw[f][t] = raw0[f][t];
        } else {
            load_weights(base, raw);
        }
#pragma unroll
        for (int f = 0; f < PF; f++) {
            if (base + f >= s_end) break;  // uniform per wave
            // LDS accesses of one wave execute in order: the slice written above is visible
            const uint4 av = *(const uint4*)(a_src + (size_t)(base + f - s_begin) * 4 * PL_GROUP);
            const v4i a = {(int)av.x, (int)av.y, (int)av.z, (int)av.w};
#pragma unroll
            for (int t = 0; t < NACC; t++) {
                uint32_t G;
                if constexpr (LAYOUT == PL_TILED) G = raw[f][t];
                else G = pl_quad_transpose(raw[f][t], sel_q);
                acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, decode16_i8(G), acc[t], 0, 0, 0);
            }
        }
    }

    // Every wave folds its digit rows into 64-bit integers first (lane (j, 0) holds rows 0..3 of column j, lane
    // (j, 1) rows 4 and 5: two partial values per column and wave), then the partial values of all waves are added
    // through LDS -- integers, so the order does not matter.
    int64_t* red64 = (int64_t*)red;  // [WAVES][2][TILE_N]
    if (g < 2) {
#pragma unroll
        for (int t = 0; t < NACC; t++) {
            const int64_t a0 = acc[t][0], a1 = acc[t][1], a2 = (g == 0) ? acc[t][2] : 0, a3 = (g == 0) ? acc[t][3] : 0;
            const int64_t part = (((a3 * 128 + a2) * 128 + a1) * 128 + a0) << (28 * g);
            red64[(wave * 2 + g) * TILE_N + t * 16 + j] = part;
        }
    }
    if (lane == 0) flags[wave] = bad ? 1u : 0u;
    __syncthreads();
    if (!out_thread) return;
    int64_t S = 0, S2 = 0;
    uint32_t any_bad = 0u;
    for (int w = 0; w < 2 * WAVES; w++) {
        S += red64[w * TILE_N + slot];
        if constexpr (PAIRS) S2 += red64[w * TILE_N + slot + 16];
    }
    for (int w = 0; w < WAVES; w++) any_bad |= flags[w];
    const float sc = bits_to_f32_rt(pre_s, p.scale_dtype);
    const float bs = biasp ? bits_to_f32_rt(pre_b, p.bias_dtype) : 0.0f;
    float acc1 = fixed_to_f32(S), acc2 = PAIRS ? fixed_to_f32(S2) : 0.0f;
    if (any_bad) {  // (uniform over the workgroup) the row as the kernel multiplied it: after the prologue, if any
        const uint16_t* xrow = (const uint16_t*)Xp;
        const uint16_t* brow = (const uint16_t*)p.pro_b;
        const float r = pro_r;
        auto xk = [&](int k) -> uint32_t {
            const float xv = f16_bits_to_f32(xrow[k]);
            if constexpr (PRO == PRO_RMSNORM) return f32_to_f16_bits(rmsnorm_value(xv, r, brow ? f16_bits_to_f32(brow[k]) : 1.0f, BT_F16));
            else if constexpr (PRO == PRO_SWIGLU) return f32_to_f16_bits(swiglu_value(xv, f16_bits_to_f32(brow[k]), BT_F16));
            else return xrow[k];
        };
        const bool tiled = LAYOUT == PL_TILED;
        const int tsig = PAIRS ? -p.tiles16 : p.tiles16_signed;  // (the output stage reads a pair-ordered copy)
        acc1 = nonfinite_acc<BT_F16>(xk, (int)p.K, Wp, tiled, p.wsteps, tsig, p.N, n_out);
        if constexpr (PAIRS) acc2 = nonfinite_acc<BT_F16>(xk, (int)p.K, Wp, tiled, p.wsteps, tsig, p.N, ffn + n_out);
    }
    if constexpr (PAIRS) {
        const float sc2 = bits_to_f32_rt(pre_s2, p.scale_dtype);
        const float bs2 = biasp ? bits_to_f32_rt(pre_b2, p.bias_dtype) : 0.0f;
        const float gv = round_to_dtype(epi_float(acc1, sc, bs), BT_F16);
        const float uv = round_to_dtype(epi_float(acc2, sc2, bs2), BT_F16);
        ((uint16_t*)Yp)[n_out] = f32_to_f16_bits(swiglu_value(gv, uv, BT_F16));
    } else {
        pl_store(Yp, p.residual, n_out, acc1, sc, bs);
    }
}

// ---- G units per launch -----------------------------------------------------------------------------
// (A single wide matrix does not run faster here than in the kernel above: 4.1-4.4 against 4.5 TB/s at
// N = 128256, K = 4096; one item per workgroup leaves nothing to overlap.)
// Persistent workgroups of 8 waves.  Item i = (unit i / slabs, slab i % slabs); wave w of the workgroup owns the
// 16-column tiles (slab * 8 + w) * NACC .. + NACC - 1 of the unit over the whole of K.  The digit planes of the
// unit's activation row are converted once per item by the whole workgroup into LDS.  The weight loads of a wave
// form one uninterrupted stream: PF steps are always in flight, and the last batch of an item already requests the
// first steps of the wave's next item.  Wave w walks the steps of its tiles in rotated order, starting at step
// (w/8 of the way through K): streams that advance in lockstep from the same step hit the same memory channels at the
// same time (a pure read of this address stream: 5.7 TB/s in lockstep, 6.7 TB/s rotated); the sums are integers, so
// the order does not change a bit of the result.
// LDS: a flag word per wave, then the digit planes of one row, padded with zero groups to a multiple of PF steps.
// XDT = BT_BF16: bf16 rows and outputs; the row is read twice per item, once for its largest exponent (the waves'
// maxima meet in LDS, one more barrier) and once for its digits (see bf16x8_to_planes).
template <int NACC, int PF, int XDT = BT_F16>
__global__ __launch_bounds__(512, 4) void gemv_planes_group_kernel(PlaneParams p) {
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    __shared__ int emax_slot[8];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int j = lane & 15, g = lane >> 4;
    const int S = p.wsteps;
    const int SP = (S + PF - 1) / PF * PF;         // steps per item, padded
    uint32_t* flags = lds;  // [8]
    uint8_t* planes = (uint8_t*)(lds + 8);
    const int nchunks = SP * 8;                    // 16-byte chunks of x, padding included
    const uint8_t* a_src = planes + g * PL_GROUP + (j % PL_N) * 16;

    // tile t of the wave within item `it`: base pointer of its first step (uniform), clamped to the last tile
    auto tile_base = [&](int it, int t) -> const uint8_t* {
        const int u = it / p.slabs, slab = it - u * p.slabs;
        const int tl = min((slab * 8 + wave) * NACC + t, p.tiles16 - 1);
        return p.W_tab[u] + (size_t)tl * (size_t)S * 256;
    };
    int it = (int)blockIdx.x;
    if (it >= p.items) return;
    const uint8_t* wcur[NACC];
#pragma unroll
    for (int t = 0; t < NACC; t++) wcur[t] = tile_base(it, t);
    const uint32_t loff = (uint32_t)lane * 4u;
    const int rot = (wave * (SP / PF)) / 8 * PF;  // first step of this wave's walk: a whole number of batches
    uint32_t raw[PF][NACC];
#pragma unroll
    for (int f = 0; f < PF; f++)
#pragma unroll
        for (int t = 0; t < NACC; t++) raw[f][t] = ldw_nt(wcur[t] + ((size_t)min(rot + f, S - 1) * 256 + loff));

    for (; it < p.items; it += (int)gridDim.x) {
        const int u = it / p.slabs, slab = it - u * p.slabs;
        const int it_next = (it + (int)gridDim.x < p.items) ? it + (int)gridDim.x : it;
        const uint8_t* wnext[NACC];
#pragma unroll
        for (int t = 0; t < NACC; t++) wnext[t] = tile_base(it_next, t);
        // the unit's activation row -> digit planes (all waves; the previous item's readers are past the barrier
        // that ended it)
        const uint16_t* xrow = (const uint16_t*)p.X_tab[u];
        int emax = 0;
        if constexpr (XDT == BT_BF16) {
            int m = 1;
            for (int c = (int)threadIdx.x; c * 8 < (int)p.K; c += 512) m = max(m, bf16x8_max_e1(*(const uint4*)(xrow + min(c * 8, (int)p.K - 8))));
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) m = max(m, __shfl_xor(m, off, 64));
            if (lane == 0) emax_slot[wave] = m;
            __syncthreads();  // (the slots' readers of the previous item are past the barrier that ended it)
            m = emax_slot[lane & 7];
#pragma unroll
            for (int off = 4; off > 0; off >>= 1) m = max(m, __shfl_xor(m, off, 64));
            emax = m;
        }
        bool bad = false;
        for (int c = (int)threadIdx.x; c < nchunks; c += 512) {
            const int k = c * 8;
            uint4 v = *(const uint4*)(xrow + min(k, (int)p.K - 8));
            v = zero_unless4(v, k < (int)p.K);
            bad |= park_chunk<XDT>(planes, c, v, lane, true, emax);
        }
        // (a word per wave, stored unconditionally: nothing to clear between items)
        const bool wave_bad = __builtin_amdgcn_ballot_w64(bad) != 0ull;
        if (lane == 0) flags[wave] = wave_bad ? 1u : 0u;
        // epilogue operands of the columns this lane will store (lanes 0..15: column j of each tile)
        const int64_t ncol0 = ((int64_t)(slab * 8 + wave) * NACC) * 16 + j;
        uint32_t pre_s[NACC], pre_b[NACC];
        const void* scale_u = p.scale_tab[u];
        const void* bias_u = p.bias_tab ? p.bias_tab[u] : nullptr;
#pragma unroll
        for (int t = 0; t < NACC; t++) {
            const int64_t n = ncol0 + 16 * t;
            pre_s[t] = pre_b[t] = 0u;
            if (g == 0 && n < p.N) {
                pre_s[t] = load_bits_rt(scale_u, p.scale_dtype, p.scale_bcast ? 0 : n);
                if (bias_u) pre_b[t] = load_bits_rt(bias_u, p.bias_dtype, n);
            }
        }
        __syncthreads();

        v4i acc[NACC];
#pragma unroll
        for (int t = 0; t < NACC; t++) acc[t] = v4i{0, 0, 0, 0};
        for (int b = 0; b < SP; b += PF) {
            // this batch covers steps base .. base + PF - 1 of the rotated walk; refill target: the same item's next
            // batch, or the first batch of the wave's next item
            const bool last = b + PF >= SP;  // uniform
            int base = b + rot;
            if (base >= SP) base -= SP;
            int sb = base + PF;
            if (sb >= SP) sb -= SP;  // (after the last batch this is `rot` again: where the next item starts)
#pragma unroll
            for (int f = 0; f < PF; f++) {
                const uint4 av = *(const uint4*)(a_src + (size_t)(base + f) * 4 * PL_GROUP);
                const v4i a = {(int)av.x, (int)av.y, (int)av.z, (int)av.w};
                const size_t so = (size_t)min(sb + f, S - 1) * 256 + loff;
#pragma unroll
                for (int t = 0; t < NACC; t++) {
                    acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, decode16_i8(raw[f][t]), acc[t], 0, 0, 0);
                    raw[f][t] = ldw_nt((last ? wnext[t] : wcur[t]) + so);
                }
            }
        }
#pragma unroll
        for (int t = 0; t < NACC; t++) wcur[t] = wnext[t];

        // lane (j, 0) holds the sums of digit rows 0..3 of column j, lane (j, 1) those of rows 4 and 5
        uint32_t fl = 0u;
#pragma unroll
        for (int w = 0; w < 8; w++) fl |= flags[w];
        const bool any_bad = fl != 0u;
        void* y_u = p.Y_tab[u];
#pragma unroll
        for (int t = 0; t < NACC; t++) {
            int32_t s[PL_N];
#pragma unroll
            for (int r = 0; r < 4; r++) s[r] = acc[t][r];
            s[4] = __shfl_down(acc[t][0], 16, 64);
            s[5] = __shfl_down(acc[t][1], 16, 64);
            const int64_t n = ncol0 + 16 * t;
            if (g == 0 && n < p.N) {
                const float sc = bits_to_f32_rt(pre_s[t], p.scale_dtype);
                const float bs = bias_u ? bits_to_f32_rt(pre_b[t], p.bias_dtype) : 0.0f;
                float av = planes_to_f32(s, (XDT == BT_BF16) ? emax - 166 : -24);
                if (any_bad) {
                    const uint16_t* xrow = (const uint16_t*)p.X_tab[u];
                    av = nonfinite_acc_row<XDT>(xrow, (int)p.K, p.W_tab[u], p.wsteps, p.tiles16, p.N, n);
                }
                pl_store<XDT>(y_u, nullptr, n, av, sc, bs);
            }
        }
        __syncthreads();  // every wave is done with the planes before the next item overwrites them
    }
}

// ---- G units per launch, K up to 8 steps per wave: contiguous walk -------------------------------------------
// The (unit, 16-column tile) pairs of the launch form one flat sequence, and the tiled copies make a unit's tiles
// contiguous in memory (16 * K / 4 bytes each).  Workgroup b owns a contiguous run of the sequence; its eight waves
// split K: wave w reads steps w * SPW .. + SPW - 1 of every tile, i.e. SPW * 256 consecutive bytes, so that the
// workgroup as a whole reads its megabyte or so front to back, 2 KiB per wave at a time -- the access pattern that
// streams fastest on this chip (a pure read: 7.2 TB/s, against 5.7-6.7 TB/s for 16 streams per workgroup that are
// 16 KiB apart).  A wave's slice of the activation digits does not change from tile to tile: it is converted once
// per unit and held in SPW * 4 registers, so the loop has no LDS reads.  The partial sums of the eight waves (six
// int32 digit-row sums per column) are added with LDS atomics into one of two accumulator arrays; every EB tiles a
// barrier ends the chunk, one thread per column finishes it (and clears the array) while the waves are already
// adding the next chunk into the other array.  TB tiles of loads are always in flight per wave, across chunk and
// unit boundaries.  Integer sums: same bits as every other split of K.
constexpr int CH_EB = 32;  // tiles per chunk (one output column per thread)
// XDT = BT_BF16: bf16 activations and outputs, the row scaled by its largest exponent (see bf16x8_to_planes): the waves
// exchange the maxima of their slices through LDS (one more barrier per unit) before they convert.
template <int SPW, int TB, int XDT = BT_F16>
__global__ __launch_bounds__(512, 4) void gemv_planes_chunk_kernel(PlaneParams p) {
    static_assert(CH_EB % TB == 0, "chunks hold whole batches");
    __shared__ int32_t accbuf[2][CH_EB][PL_N * 16];
    __shared__ uint32_t flags[2][8];
    __shared__ int emax_slot[2][8];
    __shared__ __attribute__((aligned(16))) uint8_t planes_all[8][SPW * 4 * PL_GROUP];
    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 15, g = lane >> 4;
    const int S = p.wsteps;
    const int T16 = p.tiles16;
    const int64_t total = (int64_t)p.G * T16;
    // this workgroup's run of the flat tile sequence (p.slabs = tiles per workgroup, a multiple of TB)
    const int64_t t_begin = (int64_t)blockIdx.x * p.slabs;
    const int64_t t_end = (t_begin + p.slabs < total) ? t_begin + p.slabs : total;
    if (t_begin >= t_end) return;

    for (int i = tid; i < 2 * CH_EB * PL_N * 16; i += 512) (&accbuf[0][0][0])[i] = 0;

    // byte offset of this wave's SPW steps inside a tile (steps past the end repeat the last one and meet zero digits)
    uint32_t soff[SPW];
#pragma unroll
    for (int f = 0; f < SPW; f++) soff[f] = (uint32_t)min(wave * SPW + f, S - 1) * 256u + (uint32_t)lane * 4u;
    const size_t tile_bytes = (size_t)S * 256;

    // prefetch cursor: (unit, tile) of the next tile to request, its address
    int pf_u = (int)(t_begin / T16);
    int pf_t = (int)(t_begin - (int64_t)pf_u * T16);
    int64_t pf_left = t_end - t_begin;  // tiles not yet requested
    // (one matrix per launch: direct pointers instead of tables)
    const bool tab = p.W_tab != nullptr;
    const uint8_t* pf_ptr = (tab ? p.W_tab[pf_u] : p.W) + (size_t)pf_t * tile_bytes;
    uint32_t raw[TB][SPW];
    auto request = [&](uint32_t (&dst)[SPW]) {
        // (past the end of the run: the last tile again, never used)
#pragma unroll
        for (int f = 0; f < SPW; f++) dst[f] = ldw_nt(pf_ptr + soff[f]);
        if (pf_left > 1) {
            pf_left--;
            pf_t++;
            pf_ptr += tile_bytes;
            if (pf_t == T16) {
                pf_t = 0;
                pf_u++;
                pf_ptr = tab ? p.W_tab[pf_u] : p.W;
            }
        }
    };
    // the first unit's slice of x is requested ahead of the weights (loads return in order, and it is needed first)
    const int xk = (wave * SPW * 8 + lane) * 8;
    uint4 x_first = *(const uint4*)((const uint16_t*)(tab ? p.X_tab[pf_u] : p.X) + min(xk, (int)p.K - 8));
#pragma unroll
    for (int i = 0; i < TB; i++) request(raw[i]);

    uint8_t* planes = planes_all[wave];
    const uint8_t* a_src = planes + g * PL_GROUP + (j % PL_N) * 16;
    uint4 areg[SPW];
    int cur = 0;
    int emax = 0;  // bf16: the current unit's largest exponent (every wave computes it)
    __syncthreads();  // accumulators cleared

    int64_t t0 = t_begin;
    while (t0 < t_end) {
        const int u = (int)(t0 / T16);
        const int tile0 = (int)(t0 - (int64_t)u * T16);
        // the wave's slice of the unit's activation row -> digit planes -> registers (once per unit and workgroup)
        {
            const uint16_t* xrow = (const uint16_t*)(tab ? p.X_tab[u] : p.X);
            const int c = lane;                               // chunk of eight values (SPW * 8 <= 64 chunks)
            const int k = xk;
            uint4 v = x_first;
            if (t0 != t_begin) v = *(const uint4*)(xrow + min(k, (int)p.K - 8));  // uniform
            v = zero_unless4(v, k < (int)p.K && c < SPW * 8);
            if constexpr (XDT == BT_BF16) {
                // the row's largest exponent: every wave's slice maximum meets the others' in LDS (the eight slices
                // cover the row; two sets of slots, so a wave that runs ahead into the next unit disturbs nobody)
                int m = bf16x8_max_e1(v);
#pragma unroll
                for (int off = 32; off > 0; off >>= 1) m = max(m, __shfl_xor(m, off, 64));
                if (lane == 0) emax_slot[u & 1][wave] = m;
                __syncthreads();
                m = emax_slot[u & 1][lane & 7];
#pragma unroll
                for (int off = 4; off > 0; off >>= 1) m = max(m, __shfl_xor(m, off, 64));
                emax = m;
            }
            const bool bad = park_chunk<XDT>(planes, c, v, lane, c < SPW * 8, emax);
            const bool wave_bad = __builtin_amdgcn_ballot_w64(bad) != 0ull;
            if (lane == 0) flags[u & 1][wave] = wave_bad ? 1u : 0u;
            // (LDS accesses of one wave execute in order: the slice written above is visible to its own reads)
#pragma unroll
            for (int f = 0; f < SPW; f++) areg[f] = *(const uint4*)(a_src + (size_t)f * 4 * PL_GROUP);
        }
        // chunks of this unit inside the run
        const int64_t unit_end = (int64_t)(u + 1) * T16;
        const int64_t u_stop = (unit_end < t_end) ? unit_end : t_end;
        for (int64_t c0 = t0; c0 < u_stop; c0 += CH_EB) {
            const int ntiles = (int)((u_stop - c0 < CH_EB) ? u_stop - c0 : CH_EB);  // a multiple of TB
            // this thread's output column of the chunk: its epilogue operands are requested now, a chunk ahead of their use
            const int tl = tid >> 4, jj = tid & 15;
            const int64_t n = (int64_t)(tile0 + (int)(c0 - t0) + tl) * 16 + jj;
            const bool out_col = tl < ntiles && n < p.N;
            const void* bias_u = tab ? (p.bias_tab ? p.bias_tab[u] : nullptr) : p.bias;
            uint32_t pre_s = 0u, pre_b = 0u;
            if (out_col) {
                pre_s = load_bits_rt(tab ? p.scale_tab[u] : p.scale, p.scale_dtype, p.scale_bcast ? 0 : n);
                if (bias_u) pre_b = load_bits_rt(bias_u, p.bias_dtype, n);
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
                // lane (j, 0) holds digit rows 0..3 of column j, lane (j, 1) rows 4 and 5
#pragma unroll
                for (int i = 0; i < TB; i++) {
                    int32_t* dst = &accbuf[cur][tb + i][j];
                    if (g == 0) {
#pragma unroll
                        for (int r = 0; r < 4; r++) atomicAdd(dst + 16 * r, acc[i][r]);
                    } else if (g == 1) {
                        atomicAdd(dst + 16 * 4, acc[i][0]);
                        atomicAdd(dst + 16 * 5, acc[i][1]);
                    }
                }
            }
            __syncthreads();  // every wave has added its share of this chunk
            if (tl < ntiles) {
                int32_t sums[PL_N];
#pragma unroll
                for (int r = 0; r < PL_N; r++) {
                    sums[r] = accbuf[cur][tl][16 * r + jj];
                    accbuf[cur][tl][16 * r + jj] = 0;
                }
                if (out_col) {
                    uint32_t fl = 0u;
#pragma unroll
                    for (int w = 0; w < 8; w++) fl |= flags[u & 1][w];
                    const float sc = bits_to_f32_rt(pre_s, p.scale_dtype);
                    const float bs = bias_u ? bits_to_f32_rt(pre_b, p.bias_dtype) : 0.0f;
                    const int exp2 = (XDT == BT_BF16) ? emax - 166 : -24;
                    float av = planes_to_f32(sums, exp2);
                    if (fl != 0u) {
                        const uint16_t* xrow = (const uint16_t*)(tab ? p.X_tab[u] : p.X);
                        av = nonfinite_acc_row<XDT>(xrow, (int)p.K, tab ? p.W_tab[u] : p.W, p.wsteps, p.tiles16, p.N, n);
                    }
                    pl_store<XDT>(tab ? p.Y_tab[u] : p.Y, tab ? nullptr : p.residual, n, av, sc, bs);
                }
            }
            cur ^= 1;
        }
        t0 = u_stop;
    }
}

// ---- host side ----------------------------------------------------------------------------------------
// One fp16 row, K a multiple of 16 and at most PL_MAX_K, N a multiple of 4, aligned operands: the shapes both
// weight layouts can serve, so that a layer gives the same bits whichever copy of its weights a call reads.
constexpr int64_t PL_MAX_K = 16384;

bool planes_supported(int x_dtype, int y_dtype, int64_t B, int64_t N, int64_t K, const void* X, const void* W, const void* Y,
                      int w_layout) {
    if (option(OPT_NO_PLANES)) return false;  // A/B runs: the 16-bit matrix-core path instead
    if (x_dtype != BT_F16 || y_dtype != BT_F16 || B != 1 || K % 16 != 0 || K > PL_MAX_K || K < 16 || N % 4 != 0) return false;
    if (((uintptr_t)X) % 16 != 0 || ((uintptr_t)Y) % 2 != 0) return false;
    if (layout_tiled(w_layout)) return ((uintptr_t)W) % 256 == 0;
    return ((uintptr_t)W) % 4 == 0 && (ceil_div(K, 4) + 64) * N < (1ll << 32);
}

// grouped and wide launches: 2 workgroups of 8 waves per compute unit
static int g_group_cus = 0;
static int64_t resident_wgs() {
    if (!g_group_cus) {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
        g_group_cus = cus;
    }
    return 2 * (int64_t)g_group_cus;
}

// The contiguous-walk kernel where the shape allows it: K of 3..8 steps per wave (1040 <= K <= 4096), whole batches of
// tiles, and at least `min_tiles_per_wg` tiles per resident workgroup (below that the per-chunk barrier and the one-off
// conversion weigh more than the walk gains: G = 8 units of 4096 x 4096 10.5 against 11.7 us, G = 32 equal, G = 128
// 92 against 85 us).  BITTORCH_GROUP_WALK=1 / =0 (tests, A/B runs): always / never.
// (shape only: what the kernel can serve at all)
static bool walk_shape_ok(int wsteps, int tiles16) {
    const int spw = (int)ceil_div(wsteps, 8);
    const int tb = (spw >= 5) ? 2 : 4;
    return spw >= 3 && spw <= 8 && tiles16 % tb == 0;
}
template <int XDT>
static void launch_walk_k(const PlaneParams& p, int spw, unsigned grid, hipStream_t st) {
    switch (spw) {
        case 3: hipLaunchKernelGGL((gemv_planes_chunk_kernel<3, 4, XDT>), dim3(grid), dim3(512), 0, st, p); break;
        case 4: hipLaunchKernelGGL((gemv_planes_chunk_kernel<4, 4, XDT>), dim3(grid), dim3(512), 0, st, p); break;
        case 5: hipLaunchKernelGGL((gemv_planes_chunk_kernel<5, 2, XDT>), dim3(grid), dim3(512), 0, st, p); break;
        case 6: hipLaunchKernelGGL((gemv_planes_chunk_kernel<6, 2, XDT>), dim3(grid), dim3(512), 0, st, p); break;
        case 7: hipLaunchKernelGGL((gemv_planes_chunk_kernel<7, 2, XDT>), dim3(grid), dim3(512), 0, st, p); break;
        default: hipLaunchKernelGGL((gemv_planes_chunk_kernel<8, 2, XDT>), dim3(grid), dim3(512), 0, st, p); break;
    }
}
// min_tiles_per_wg < 0: whenever the shape allows
static bool launch_walk(PlaneParams p, int64_t G, int64_t wgs, int min_tiles_per_wg, hipStream_t st) {
    const int spw = (int)ceil_div(p.wsteps, 8);
    const int tb = (spw >= 5) ? 2 : 4;
    const int64_t total = G * p.tiles16;
    const char* force = option(OPT_GROUP_WALK);
    bool want = force ? (force[0] == '1') : (total >= min_tiles_per_wg * wgs);
    if (min_tiles_per_wg < 0) want = true;
    if (!walk_shape_ok(p.wsteps, p.tiles16) || !want) return false;
    const int64_t tpw = ceil_div(ceil_div(total, wgs), tb) * tb;
    p.G = (int)G;
    p.slabs = (int)tpw;  // tiles per workgroup
    const unsigned grid = (unsigned)ceil_div(total, tpw);
    if (p.x_dtype == BT_BF16) launch_walk_k<BT_BF16>(p, spw, grid, st);
    else launch_walk_k<BT_F16>(p, spw, grid, st);
    return true;
}

template <int LAYOUT, int NACC, int EPI = EPI_NONE, bool TAB = false, int PRO = PRO_NONE, int PF = 8>
static void launch_planes_k(const PlaneParams& p, hipStream_t st) {
    // (16 or 4 waves per workgroup instead of 8: 3.72-3.74 against 3.70-3.74 us at 4096 x 4096 -- the launch is
    // bounded by its one round trip to memory, not by how the workgroup divides the work)
    constexpr int WAVES = 8;
    const int nsteps = (int)ceil_div(p.K, 64);
    const int spw = (int)ceil_div(nsteps, WAVES);
    // A wave requests PF steps of weights per batch and a batch is a round trip to memory: with more than 8 steps per wave
    // (K > 4096) the plain tiled kernel takes its whole slice in one batch of 16 or 32 (N = 2560, K = 6912: 5.6 -> 5.1 us;
    // N = 4096, K = 11008: 8.1 -> 7.9 us, where converting the 11008 activations in every workgroup is what is left).
    if constexpr (PF == 8 && LAYOUT == PL_TILED && EPI == EPI_NONE && !TAB) {
        if constexpr (NACC < 4) {  // (32 steps of four tiles would not fit the registers)
            if (spw > 16) return launch_planes_k<LAYOUT, NACC, EPI, TAB, PRO, 32>(p, st);
        }
        if (spw > 8) return launch_planes_k<LAYOUT, NACC, EPI, TAB, PRO, 16>(p, st);
    }
    const size_t lds = (size_t)WAVES * 2 * 16 * NACC * 8 + WAVES * 4 + (size_t)WAVES * spw * 4 * PL_GROUP;
    if (lds > 64 * 1024) {  // beyond the default limit of dynamic LDS (K > 10240 or so): raise it for this kernel, once
        static bool raised = false;
        if (!raised) {
            (void)hipFuncSetAttribute((const void*)gemv_planes_kernel<LAYOUT, NACC, WAVES, PF, EPI, TAB, PRO>,
                                      hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
            raised = true;
        }
    }
    hipLaunchKernelGGL((gemv_planes_kernel<LAYOUT, NACC, WAVES, PF, EPI, TAB, PRO>), dim3((unsigned)(p.per_xcd * 8)), dim3(WAVES * 64), lds, st, p);
}

// epi_op = EPI_SWIGLU_PAIRS: tiled copy in gate/up pair order, N % 32 == 0, no residual; Y is [N/2]
// pro_op / pro_b / pro_eps: activation prologue (PRO_*; pro_b 16-byte aligned, K values in the row's dtype)
int launch_planes(const void* X, const uint8_t* W, int w_layout, const Epilogue& epi, void* Y, int64_t N, int64_t K,
                  int epi_op, hipStream_t st, int pro_op, const void* pro_b, float pro_eps) {
    PlaneParams p = {};
    p.pro_b = pro_b; p.pro_eps = pro_eps;
    p.X = X; p.W = W; p.scale = epi.scale; p.bias = epi.bias; p.residual = epi.residual; p.Y = Y;
    p.scale_dtype = epi.scale_dtype; p.bias_dtype = epi.bias_dtype; p.scale_bcast = epi.scale_bcast;
    p.x_dtype = BT_F16;
    p.N = N; p.K = K; p.Kb = ceil_div(K, 4);
    p.G = 1;
    p.wsteps = (int)ceil_div(p.Kb, 16);
    p.tiles16 = (int)ceil_div(N, 16);
    // 16-column tiles per workgroup: as many as still give every compute unit a workgroup
    p.tiles16_signed = tiles16_arg(N, w_layout);
    int nacc = layout_tiled(w_layout) ? 4 : 2;
    if (const char* env = option(OPT_PLANES_NACC)) nacc = atoi(env);
    const int min_nacc = (epi_op == EPI_SWIGLU_PAIRS) ? 2 : 1;
    while (nacc > min_nacc && ceil_div(p.tiles16, nacc) < 224) nacc >>= 1;
    if (nacc != 1 && nacc != 2 && nacc != 4) nacc = min_nacc;
    if (!layout_tiled(w_layout) && nacc > 2) nacc = 2;
    if (nacc < min_nacc) nacc = min_nacc;
    p.tiles = (int)ceil_div(p.tiles16, nacc);
    p.per_xcd = (int)ceil_div(p.tiles, 8);
    if (epi_op == EPI_SWIGLU_PAIRS) {
        if (w_layout != W_LAYOUT_TILED || N % 32 != 0 || epi.residual) {
            set_error("gemv_planes: the SwiGLU output stage needs pair-ordered tiled weights, N %% 32 == 0 and no residual");
            return BT_ERR_INVALID;
        }
        if (pro_op == PRO_SWIGLU) {
            set_error("gemv_planes: a SwiGLU prologue and the SwiGLU output stage do not combine");
            return BT_ERR_INVALID;
        }
        if (pro_op == PRO_RMSNORM) {
            if (nacc == 4) launch_planes_k<PL_TILED, 4, EPI_SWIGLU_PAIRS, false, PRO_RMSNORM>(p, st);
            else launch_planes_k<PL_TILED, 2, EPI_SWIGLU_PAIRS, false, PRO_RMSNORM>(p, st);
        } else if (nacc == 4) launch_planes_k<PL_TILED, 4, EPI_SWIGLU_PAIRS>(p, st);
        else launch_planes_k<PL_TILED, 2, EPI_SWIGLU_PAIRS>(p, st);
        return check_launch("gemv_planes");
    }
    // a matrix wide enough to give every resident workgroup a dozen tiles: the grouped launch's contiguous walk
    // (N = 128256, K = 4096: 26.2 against 28.0 us; N = 32768: 11.7 against 10.9)
    if (pro_op == PRO_NONE && w_layout == W_LAYOUT_TILED && launch_walk(p, 1, resident_wgs(), 12, st)) return check_launch("gemv_planes");
#define BT_PL_LAUNCH(LAYOUT, NACC)                                                                       \
    do {                                                                                                 \
        if (pro_op == PRO_RMSNORM) launch_planes_k<LAYOUT, NACC, EPI_NONE, false, PRO_RMSNORM>(p, st);   \
        else if (pro_op == PRO_SWIGLU) launch_planes_k<LAYOUT, NACC, EPI_NONE, false, PRO_SWIGLU>(p, st); \
        else launch_planes_k<LAYOUT, NACC>(p, st);                                                       \
    } while (0)
    if (layout_tiled(w_layout)) {
        if (nacc == 4) BT_PL_LAUNCH(PL_TILED, 4);
        else if (nacc == 2) BT_PL_LAUNCH(PL_TILED, 2);
        else BT_PL_LAUNCH(PL_TILED, 1);
    } else {
        if (nacc == 2) BT_PL_LAUNCH(PL_ROWMAJOR, 2);
        else BT_PL_LAUNCH(PL_ROWMAJOR, 1);
    }
#undef BT_PL_LAUNCH
    return check_launch("gemv_planes");
}


template <int NACC, int PF, int XDT = BT_F16>
static void launch_group_k(const PlaneParams& p, unsigned grid, size_t lds, hipStream_t st) {
    if (lds > 64 * 1024) {  // the digit rows of a long activation row (K > 10240 or so): beyond the default limit of dynamic LDS
        static bool raised = false;
        if (!raised) {
            (void)hipFuncSetAttribute((const void*)gemv_planes_group_kernel<NACC, PF, XDT>,
                                      hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
            raised = true;
        }
    }
    hipLaunchKernelGGL((gemv_planes_group_kernel<NACC, PF, XDT>), dim3(grid), dim3(512), lds, st, p);
}

// A few units in one launch of the one-matrix kernel (workgroup tile -> (unit, tile) through the pointer tables): every
// workgroup converts its unit's row itself and reads 16 * NACC columns over the whole of K, as many workgroups as the
// units have tiles.  For a handful of units this beats the persistent kernels, whose workgroups each walk several
// tiles one after another (units of 4096 x 4096: G = 1 4.8 against 9.4 us, G = 2 5.8 against 9.5, G = 4 7.7 against
// 9.9, G = 6 equal, G = 8 12.6 against 10.8; units of N = 4096, K = 11008: G = 1 9.2 against 20.6, G = 4 14.9 against
// 21.6, G = 8 21.8 against 23.6, G = 16 40.6 against 38.4).  BITTORCH_GROUP_UNITS=1 / =0 (tests, A/B runs): always / never.
static bool launch_units(PlaneParams p, int64_t G, hipStream_t st) {
    const char* force = option(OPT_GROUP_UNITS);
    if (force && force[0] == '0') return false;
    if (p.K > PL_MAX_K) return false;
    if (!(force && force[0] == '1')) {
        // microseconds, fitted to launches of G units of 4096 x 4096 and 4096 x 11008 on this chip: the persistent kernel
        // has a floor that grows with K (a wave walks the whole of K for its columns) and streams at about 5 TB/s
        // beyond it; the one-matrix kernel starts lower and streams at about 4 TB/s
        const double mib = (double)G * (double)p.tiles16 * (double)p.wsteps * 256.0 / 1048576.0;
        const double k = (double)p.K;
        const double t_units = 1.4 + 0.0006 * k + 0.24 * mib;
        const double t_floor = 2.6 + 0.00162 * k + 0.04 * mib, t_stream = 4.0 + 0.2 * mib;
        if (t_units >= (t_floor > t_stream ? t_floor : t_stream)) return false;
    }
    int nacc = 4;
    while (nacc > 1 && G * ceil_div(p.tiles16, nacc) < 224) nacc >>= 1;
    p.slabs = (int)ceil_div(p.tiles16, nacc);
    if (G * p.slabs > 0x3fffffff) return false;
    p.tiles = (int)(G * p.slabs);
    p.per_xcd = (int)ceil_div(p.tiles, 8);
    if (nacc == 4) launch_planes_k<PL_TILED, 4, EPI_NONE, true>(p, st);
    else if (nacc == 2) launch_planes_k<PL_TILED, 2, EPI_NONE, true>(p, st);
    else launch_planes_k<PL_TILED, 1, EPI_NONE, true>(p, st);
    return true;
}

static int launch_group_params(PlaneParams p, int64_t G, hipStream_t st) {
    const int64_t wgs = resident_wgs();
    const bool bf16 = p.x_dtype == BT_BF16;
    if (!bf16) {
        const char* force = option(OPT_GROUP_UNITS);
        if (force && force[0] == '1' && launch_units(p, G, st)) return check_launch("gemv_planes_group");
    }
    // (bf16 units have no one-matrix kernel: the walk wherever the shape allows it, which is also the faster of their
    // two kernels for a handful of units)
    if (launch_walk(p, G, wgs, bf16 ? -1 : 16, st)) return check_launch("gemv_planes_group");
    if (!bf16 && launch_units(p, G, st)) return check_launch("gemv_planes_group");
    // columns per wave: 32 (two tiles) streams best (5.3 TB/s against 4.8 with four tiles and 4.4-5.0 with one at
    // G = 128, 4096 x 4096); another width only where it fills the resident workgroups markedly more evenly
    int nacc = 2;
    if (const char* env = option(OPT_GROUP_NACC)) {
        nacc = atoi(env);
        if (nacc != 1 && nacc != 2 && nacc != 4) nacc = 2;
    } else {
        double best = -1.0;
        const int order[3] = {2, 4, 1};
        for (int i = 0; i < 3; i++) {
            const int c = order[i];
            const int64_t items = G * ceil_div(p.tiles16, 8 * c);
            const double eff = (double)items / (double)(ceil_div(items, wgs) * wgs) *
                               ((double)p.tiles16 / (double)(ceil_div(p.tiles16, 8 * c) * 8 * c));
            if (eff > best * 1.15) { best = eff; nacc = c; }
        }
    }
    p.slabs = (int)ceil_div(p.tiles16, 8 * nacc);
    p.items = (int)(G * p.slabs);
    const unsigned grid = (unsigned)((p.items < wgs) ? p.items : wgs);
    int pf = 8;
    if (const char* env = tuning_env("BITTORCH_GROUP_PF")) pf = bf16 ? 8 : atoi(env);
    const int SP = (int)ceil_div(p.wsteps, pf) * pf;
    const size_t lds = 32 + (size_t)SP * 4 * PL_GROUP;
    if (bf16) {
        if (nacc == 4) launch_group_k<4, 8, BT_BF16>(p, grid, lds, st);
        else if (nacc == 2) launch_group_k<2, 8, BT_BF16>(p, grid, lds, st);
        else launch_group_k<1, 8, BT_BF16>(p, grid, lds, st);
    } else if (pf == 16) {
        if (nacc == 4) launch_group_k<4, 16>(p, grid, lds, st);
        else if (nacc == 2) launch_group_k<2, 16>(p, grid, lds, st);
        else launch_group_k<1, 16>(p, grid, lds, st);
    } else {
        if (nacc == 4) launch_group_k<4, 8>(p, grid, lds, st);
        else if (nacc == 2) launch_group_k<2, 8>(p, grid, lds, st);
        else launch_group_k<1, 8>(p, grid, lds, st);
    }
    return check_launch("gemv_planes_group");
}

// the shapes of the contiguous-walk kernel: K of 3..8 steps of 64 per wave (1040 <= K <= 4096, K % 16 == 0) and
// whole batches of 16-column tiles (N % 32 == 0 for K > 2048, N % 64 == 0 below)
bool planes_bf16_shape_ok(int64_t N, int64_t K) {
    if (K % 16 != 0 || N % 4 != 0 || N <= 0 || K <= 0) return false;
    return walk_shape_ok((int)ceil_div(ceil_div(K, 4), 16), (int)ceil_div(N, 16));
}

// One very wide bf16 matrix (a vocabulary projection) through the contiguous walk, direct pointers; the caller has
// checked planes_bf16_shape_ok, the alignment of the operands (as planes_supported does for fp16) and that the
// matrix gives every resident workgroup a dozen tiles (planes_bf16_wide).
bool planes_bf16_wide(int64_t N, int64_t K) {
    const char* force = option(OPT_GROUP_WALK);
    if (force && force[0] == '0') return false;
    return planes_bf16_shape_ok(N, K) && ((force && force[0] == '1') || ceil_div(N, 16) >= 12 * resident_wgs());
}
int launch_planes_bf16_wide(const void* X, const uint8_t* W, const Epilogue& epi, void* Y, int64_t N, int64_t K, hipStream_t st) {
    PlaneParams p = {};
    p.X = X; p.W = W; p.scale = epi.scale; p.bias = epi.bias; p.residual = epi.residual; p.Y = Y;
    p.scale_dtype = epi.scale_dtype; p.bias_dtype = epi.bias_dtype; p.scale_bcast = epi.scale_bcast;
    p.x_dtype = BT_BF16;
    p.N = N; p.K = K; p.Kb = ceil_div(K, 4);
    p.G = 1;
    p.wsteps = (int)ceil_div(p.Kb, 16);
    p.tiles16 = (int)ceil_div(N, 16);
    p.tiles16_signed = p.tiles16;
    if (!launch_walk(p, 1, resident_wgs(), -1, st)) return BT_ERR_INVALID;
    return check_launch("gemv_planes");
}

int launch_planes_group(const void* const* X_tab, int x_dtype, const uint8_t* const* W_tab, const void* const* scale_tab,
                        int scale_dtype, int scale_bcast, const void* const* bias_tab, int bias_dtype, void* const* Y_tab,
                        int64_t G, int64_t N, int64_t K, hipStream_t st) {
    PlaneParams p = {};
    p.X_tab = X_tab; p.W_tab = W_tab; p.scale_tab = scale_tab; p.bias_tab = bias_tab; p.Y_tab = Y_tab;
    p.scale_dtype = scale_dtype; p.bias_dtype = bias_dtype; p.scale_bcast = scale_bcast;
    p.x_dtype = x_dtype;
    p.N = N; p.K = K; p.Kb = ceil_div(K, 4);
    p.G = (int)G;
    p.wsteps = (int)ceil_div(p.Kb, 16);
    p.tiles16 = (int)ceil_div(N, 16);
    p.tiles16_signed = p.tiles16;
    return launch_group_params(p, G, st);
}

}  // namespace bt
