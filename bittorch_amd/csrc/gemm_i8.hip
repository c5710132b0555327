// Prefill-shape int8 x packed-ternary GEMM for gfx950 on the int8 matrix cores.
//
// Arithmetic restated from the reference's experimental tensor-core kernel with
// the whole-row activation scale (csrc/kernels/ternary_gemm_tensor_core.cu:73-75,
// :343-347, :439, :583-589, :652):
//   acc_i32[m,n] = sum_k q[m,k] * 127*w[k,n]
//   y[m,n]       = (float(acc) * s_x[m] / 127) * scale[n] + bias[n]
// (the MFMA runs on +-1 weights; the accumulators are multiplied by 127 exactly
// in the epilogue, which is the same integer).
//
// Tiling: a 512-thread workgroup (8 waves) owns a 128 x 256 output tile.  Wave w works on
// columns 64*(w&3) .. +63 of the tile and on k64 sub-step (w>>2) of every 128-wide K stage,
// walking all 128 rows, so every weight is decoded exactly once per workgroup and the decode
// cost (about 0.7 VALU operations per weight) is shared by 128 rows of MFMA work; the two K
// halves are added through LDS once after the main loop.
//   * Activations (int8, row-major [M,K]) go through LDS, double buffered, 128 k
//     per stage, stored in MFMA operand order: slot (sub, mb, lane) is the 16
//     bytes lane (i = lane%16, g = lane/16) feeds to v_mfma_i32_16x16x64_i8 for
//     row block mb and k64 sub-step sub.
//   * Weights never touch LDS: lane (j, g) loads one dword (four output columns
//     nb + 64*(w&3) + 4j .. +3) from each of the four rows kb + 4g .. 4g+3, transposes
//     the 4x4 bytes and decodes them in registers into the B operands of four MFMAs
//     (one per column).
//   * The stage is software-pipelined inside the wave (see the main loop).
#include <algorithm>
#include <cstddef>
#include <cstdlib>

#include "bt_common.h"

namespace bt {

constexpr int G_BM = 128;
constexpr int G_BN = 256;
constexpr int G_BK = 128;           // k per LDS stage (two k64 MFMA sub-steps)
constexpr int G_MB = G_BM / 16;     // 16-row blocks per tile
constexpr int G_STAGE_BYTES = G_BM * G_BK;  // 16 KiB

struct GemmParams {
    // The first 64 bytes hold what a workgroup needs to find its tile and request its first operands: the kernel
    // arguments come through the scalar cache a 64-byte line at a time.
    const int8_t* Q;      // [M, K]
    const uint8_t* W_T;   // [Kb, N]
    int64_t K, M, N;
    int tiles_m, tiles_n;
    int per_xcd;          // workgroups per XCD (grid = 8 * per_xcd)
    int wsteps, tiles16;  // WT: 16-row steps and 16-column tiles of the decode-tiled weight copy (tiles16 < 0: stored_tile16)
    int tile_n0;          // first column tile of this launch (tiles_n counts the launch's own column tiles)
    // ---- needed later
    const float* s_x;     // [M]
    void* Y;              // [M, N]
    int32_t* acc_out;     // optional [M, N]
    int64_t Kb;
    int y_dtype;
    int long_epilogue;    // A/B runs and tests (option GEMM_LONG_EPILOGUE): never the short epilogue
    const int32_t* q_rowsum;  // FL kernels: sum of each row of Q over K (what the codes w + 1 of the field layout add)
    Epilogue epi;
};
static_assert(offsetof(GemmParams, s_x) == 64, "first argument line as laid out above");

__device__ __forceinline__ void store4(void* Y, int dt, int64_t idx, const float (&v)[4]) {
    if (dt == BT_F32) {
        st4_nt((float*)Y + idx, __builtin_bit_cast(uint32_t, v[0]), __builtin_bit_cast(uint32_t, v[1]),
               __builtin_bit_cast(uint32_t, v[2]), __builtin_bit_cast(uint32_t, v[3]));
    } else {
        uint16_t h[4];
#pragma unroll
        for (int i = 0; i < 4; i++) h[i] = (dt == BT_F16) ? f32_to_f16_bits(v[i]) : f32_to_bf16_bits(v[i]);
        st2_nt((uint16_t*)Y + idx, (uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16));
    }
}

// Finishes NB 16-row blocks (acc[MB0 .. MB0+NB-1]) of the tile: NB = 4 in a tile of 128 rows, 2 or 1 in the tiles of
// 64 and 32 rows a launch's remainder is cut into.
// The epilogue's operands (row scales of the wave's rows, column scales and biases as raw bits)
// are requested before the K-half exchange, whose LDS round trips cover their latency.
template <int NB>
struct EpiOperands {
    float sx[NB][4];  // [row block within the half][r]
    uint32_t ws_bits[4], bs_bits[4];
    uint2 res[NB][4]; // 16-bit residual of the lane's four columns in each of its rows (short epilogue only)
};
// The residual of a 16-bit output for the short epilogue (full tile): all 16 rows requested at once, next to the
// other epilogue operands, so that the hand-over of the K halves covers their latency.  (One load per row right
// before its use, as the long epilogue does, leaves a memory round trip per row exposed: 5 us per tile.)
template <int NB>
__device__ __forceinline__ void load_epi_residual(const GemmParams& p, int64_t m0, int mb0, int g, int64_t ncol, EpiOperands<NB>& e) {
    const uint16_t* base = (const uint16_t*)p.epi.residual + (m0 + 16 * mb0 + 4 * g) * p.N + ncol;
#pragma unroll
    for (int mbi = 0; mbi < NB; mbi++)
#pragma unroll
        for (int r = 0; r < 4; r++) e.res[mbi][r] = *(const uint2*)(base + (int64_t)(16 * mbi + r) * p.N);
}
template <int NB>
__device__ __forceinline__ void load_epi_operands(const GemmParams& p, int64_t m0, int mb0, int g, int64_t ncol,
                                                  bool col_ok, EpiOperands<NB>& e) {
#pragma unroll
    for (int mbi = 0; mbi < NB; mbi++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int64_t m = m0 + 16 * (mb0 + mbi) + 4 * g + r;
            e.sx[mbi][r] = p.s_x[m < p.M ? m : p.M - 1];
        }
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const int64_t n = col_ok ? ncol + t : 0;
        e.ws_bits[t] = load_bits_rt(p.epi.scale, p.epi.scale_dtype, p.epi.scale_bcast ? 0 : n);
        e.bs_bits[t] = p.epi.bias ? load_bits_rt(p.epi.bias, p.epi.bias_dtype, n) : 0u;
    }
}

// The field layout (W_LAYOUT_TILED_FIELDS, FL = true) leaves column block t of a lane scaled by 4^t (64 for t = 3):
// float(acc) * (127 / 4^t) is the same real number as float(acc / 4^t) * 127 -- the scaled accumulator has the
// significant bits of the true one and the factor is a power of two apart from 127 -- so the epilogue takes the
// scale out in the multiplication it already has.
template <bool FL>
__device__ __forceinline__ constexpr float k127(int t) {
    return FL ? (t == 0 ? 127.0f : t == 1 ? 127.0f / 4.0f : t == 2 ? 127.0f / 16.0f : 127.0f / 64.0f) : 127.0f;
}
template <bool FL>
__device__ __forceinline__ constexpr int field_shift(int t) { return FL ? 2 * t : 0; }

template <int YDT, int MB0, int NB, bool FL = false>
__device__ __forceinline__ void gemm_epilogue(const GemmParams& p, const v4i (&acc)[2 * NB][4], int64_t m0, int g,
                                              int64_t ncol, const EpiOperands<NB>& e) {
    float ws[4], bs[4];
#pragma unroll
    for (int t = 0; t < 4; t++) {
        ws[t] = bits_to_f32_rt(e.ws_bits[t], p.epi.scale_dtype);
        bs[t] = p.epi.bias ? bits_to_f32_rt(e.bs_bits[t], p.epi.bias_dtype) : 0.0f;
    }
#pragma unroll
    for (int mbi = 0; mbi < NB; mbi++) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int64_t m = m0 + 16 * (MB0 + mbi) + 4 * g + r;
            if (m >= p.M) continue;
            const float sx = e.sx[mbi][r];
            float y[4];
#pragma unroll
            for (int t = 0; t < 4; t++) {
                // float(127 a) = float(a) * 127 rounded once: |a| <= 127 K < 2^24 (checked by the host), so float(a)
                // is exact and the product rounds the same integer the reference converts (one operation less than
                // 127 a in integers first)
                const float a127f = __fmul_rn((float)acc[MB0 + mbi][t][r], k127<FL>(t));
                y[t] = epi_int8_f(a127f, sx, ws[t], bs[t]);
            }
            if (p.epi.residual) add_residual4(y, p.epi.residual, YDT, m * p.N + ncol);
            store4(p.Y, YDT, m * p.N + ncol, y);
            if (p.acc_out) {
                uint32_t a127[4];
#pragma unroll
                for (int t = 0; t < 4; t++) a127[t] = (uint32_t)times127(acc[MB0 + mbi][t][r] >> field_shift<FL>(t));
                st4_nt(p.acc_out + m * p.N + ncol, a127[0], a127[1], a127[2], a127[3]);
            }
        }
    }
}
// The same for the common case, with the bookkeeping taken out of the per-row work: every row of the tile exists,
// no residual, no accumulator output, and every row scale large enough for the two-operation division
// (all wave-uniform, checked by the caller).  A row's address is a uniform base plus a 32-bit lane offset fixed
// for the whole epilogue.  Same bits as gemm_epilogue.
template <int YDT, int MB0, int NB, bool RES = false, bool FL = false>
__device__ __forceinline__ void gemm_epilogue_fast(const GemmParams& p, const v4i (&acc)[2 * NB][4], int64_t m0, int g,
                                                   int64_t ncol, const EpiOperands<NB>& e) {
    float ws[4], bs[4];
#pragma unroll
    for (int t = 0; t < 4; t++) {
        ws[t] = bits_to_f32_rt(e.ws_bits[t], p.epi.scale_dtype);
        bs[t] = p.epi.bias ? bits_to_f32_rt(e.bs_bits[t], p.epi.bias_dtype) : 0.0f;
    }
    constexpr int ES = (YDT == BT_F32) ? 4 : 2;
    const int64_t ncol0 = (int64_t)__builtin_amdgcn_readfirstlane((int)(ncol / G_BN)) * G_BN;  // the tile's first column
    const uint32_t lane_off = ((uint32_t)(4 * g) * (uint32_t)p.N + (uint32_t)(ncol - ncol0)) * ES;
    char* const base = (char*)p.Y + ((m0 + 16 * MB0) * p.N + ncol0) * ES;  // uniform
    const int64_t row_bytes = p.N * ES;
#pragma unroll
    for (int mbi = 0; mbi < NB; mbi++) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const float sx = e.sx[mbi][r];
            float y[4];
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const float a127f = __fmul_rn((float)acc[MB0 + mbi][t][r], k127<FL>(t));
                const float q = div127_fast(__fmul_rn(a127f, sx));
                y[t] = __fadd_rn(__fmul_rn(q, ws[t]), bs[t]);
            }
            if constexpr (RES && YDT != BT_F32) {  // linear rounded to the output's dtype, then + residual (add_residual4)
                const uint32_t d[2] = {e.res[mbi][r].x, e.res[mbi][r].y};
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const uint32_t h = (d[t >> 1] >> (16 * (t & 1))) & 0xffffu;
                    const float rv = (YDT == BT_F16) ? f16_bits_to_f32((uint16_t)h) : bf16_bits_to_f32((uint16_t)h);
                    y[t] = sum_in_dtype(round_to_dtype(y[t], YDT), rv, YDT);
                }
            }
            char* const dst = base + (int64_t)(16 * mbi + r) * row_bytes + lane_off;
            if constexpr (YDT == BT_F32) {
                st4_nt((float*)dst, __builtin_bit_cast(uint32_t, y[0]), __builtin_bit_cast(uint32_t, y[1]),
                       __builtin_bit_cast(uint32_t, y[2]), __builtin_bit_cast(uint32_t, y[3]));
            } else {
                uint16_t h[4];
#pragma unroll
                for (int i = 0; i < 4; i++) h[i] = (YDT == BT_F16) ? f32_to_f16_bits(y[i]) : f32_to_bf16_bits(y[i]);
                st2_nt((uint16_t*)dst, (uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16));
            }
        }
    }
}
template <int MB0, int NB, bool FL = false>
__device__ __forceinline__ void gemm_epilogue_dt(const GemmParams& p, const v4i (&acc)[2 * NB][4], int64_t m0, int g,
                                                 int64_t ncol, const EpiOperands<NB>& e) {
    if (p.y_dtype == BT_BF16) gemm_epilogue<BT_BF16, MB0, NB, FL>(p, acc, m0, g, ncol, e);
    else if (p.y_dtype == BT_F16) gemm_epilogue<BT_F16, MB0, NB, FL>(p, acc, m0, g, ncol, e);
    else gemm_epilogue<BT_F32, MB0, NB, FL>(p, acc, m0, g, ncol, e);
}
template <int MB0, int NB, bool FL = false>
__device__ __forceinline__ void gemm_epilogue_dt(const GemmParams& p, const v4i (&acc)[2 * NB][4], int64_t m0, int g,
                                                 int64_t ncol, const EpiOperands<NB>& e, bool fast) {
    if (fast) {  // wave-uniform
        if (p.epi.residual) {  // (16-bit outputs only: checked by the caller)
            if (p.y_dtype == BT_BF16) gemm_epilogue_fast<BT_BF16, MB0, NB, true, FL>(p, acc, m0, g, ncol, e);
            else gemm_epilogue_fast<BT_F16, MB0, NB, true, FL>(p, acc, m0, g, ncol, e);
        } else if (p.y_dtype == BT_BF16) gemm_epilogue_fast<BT_BF16, MB0, NB, false, FL>(p, acc, m0, g, ncol, e);
        else if (p.y_dtype == BT_F16) gemm_epilogue_fast<BT_F16, MB0, NB, false, FL>(p, acc, m0, g, ncol, e);
        else gemm_epilogue_fast<BT_F32, MB0, NB, false, FL>(p, acc, m0, g, ncol, e);
        return;
    }
    gemm_epilogue_dt<MB0, NB, FL>(p, acc, m0, g, ncol, e);
}

// Adding the two K halves: waves (wn, 0) and (wn, 1) hold partial sums of the same outputs.  K half 1 hands over row
// blocks 0..3 and finishes 4..7, K half 0 the other way round, through one 64 KiB area of LDS (the stage buffers, dead
// by then): word (q, wn, lane) is register q of that lane.  Moving 64 KiB into LDS and out again is bandwidth, not
// latency (most of a microsecond), so the order matters: K half 1, which ends the K loop half a stage ahead of K half 0,
// writes its share while K half 0 still runs its last MFMAs; behind the barrier that ends the loop K half 0 takes that
// share and puts its own into the same slots (a lane overwrites only words it has just read itself, and the LDS
// operations of a wave execute in order), and one more barrier later K half 1 takes it: two barriers, and one of the
// two writes out of the way.
template <int NB>
__device__ __forceinline__ void give_blocks(const v4i (&acc)[2 * NB][4], int mb0, uint8_t* area, int wn, int lane) {
    int32_t* xch = (int32_t*)area;
    const int slot = wn * 64 + lane;
#pragma unroll
    for (int mb = 0; mb < NB; mb++)
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const v4i v = acc[mb0 + mb][t];
            *(int4*)(xch + ((mb * 4 + t) * 256 + slot) * 4) = make_int4(v[0], v[1], v[2], v[3]);
        }
}
template <int NB>
__device__ __forceinline__ void take_blocks(v4i (&acc)[2 * NB][4], int mb0, const uint8_t* area, int wn, int lane) {
    const int32_t* xch = (const int32_t*)area;
    const int slot = wn * 64 + lane;
#pragma unroll
    for (int mb = 0; mb < NB; mb++)
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const int4 v = *(const int4*)(xch + ((mb * 4 + t) * 256 + slot) * 4);
            acc[mb0 + mb][t] += v4i{v.x, v.y, v.z, v.w};
        }
}

// TAIL = false: K is a multiple of the 128-wide stage and the main loop is branch free.
// TAIL = true: any K % 16 == 0; the last, partial stage is masked (slower bookkeeping).
//
// 512 threads = 8 waves: wave w works on columns 64*(w&3) .. +63 of the tile and on
// k64 sub-step (w>>2) of every 128-wide stage, so the two waves that share a SIMD
// split K between them (each weight is still decoded once per workgroup) and one
// wave's LDS / barrier / decode latency hides behind the other's MFMAs.  The two
// K halves are added through LDS once, after the main loop, and each half of the
// workgroup finishes 64 of the 128 rows.
// QOO = true: Q is in operand order (16-byte groups already transposed by the quantizer), and
// the staging copies them to LDS untouched.
// WT = true: W_T is the decode-tiled copy (W_LAYOUT_TILED): the four dwords a lane decodes per stage
// (16 consecutive k of its four columns) are 16 contiguous bytes there, one load and no transpose.
// ANTIPHASE = false (A/B runs of experiment builds, BITTORCH_GEMM_INPHASE=1, benchmarked variant only): both K halves run the stage in
// the same order.
// NB: 16-row blocks per K half and wave: 4 is the 128-row tile; 2 and 1 are the tiles of 64 and 32 rows (same columns,
// same staging and LDS layout with rows past the tile clamped, a quarter to half of the MFMAs per decoded weight) that a
// launch's remainder is cut into when whole tiles would leave most compute units idle (launch_gemm_i8).
// FL = true (with WT): W_T is the field-layout copy (W_LAYOUT_TILED_FIELDS, retile_fields_kernel): the same 16 bytes
// per lane and stage, but byte b of dword c holds, in its four 2-bit fields, the weights of the lane's FOUR columns at
// k = 4 b + c -- field t (columns 4 j + t) as w + 1 for t < 3 and as a two's-complement w for t = 3.  The B operand of
// column block t and operand dword c is then `raw[c] & (0x03030303 << 2 t)`: one AND instead of a mask and a byte
// permute, an int8 value 4^t (w + 1) resp. 64 w.  The sum over k of q (w + 1) is the wanted sum plus the row's sum of
// q, which the accumulators of K half 0 start from with the opposite sign (p.q_rowsum), and the factor 4^t leaves in
// the epilogue's multiplication by 127 (k127).  Integer sums throughout: the same accumulators, the same outputs.
template <bool TAIL, bool QOO, bool WT = false, bool ANTIPHASE = true, int NB = 4, bool FL = false>
__global__ __launch_bounds__(512) void gemm_i8_kernel(GemmParams p) {
    static_assert(!FL || (WT && !TAIL), "the field layout is a tiled layout; K in whole stages");
    __shared__ __attribute__((aligned(16))) uint8_t lds[65536];  // 2 A stages; reused for the K-half exchange
    constexpr int BM = 32 * NB;  // rows of the tile

    // XCD-aware tile order: the 8 XCDs each take a contiguous run of tiles, and
    // runs are walked in groups of four row tiles so that one XCD's L2 holds a
    // compact block of activation rows and weight columns.
    // (32-bit arithmetic: the host keeps the number of tiles below 2^31, and 64-bit divisions are long
    // instruction sequences ahead of a workgroup's first load)
    const uint32_t lin = (blockIdx.x & 7u) * (uint32_t)p.per_xcd + (blockIdx.x >> 3);
    const uint32_t tiles_m = (uint32_t)p.tiles_m, tiles_n = (uint32_t)p.tiles_n;
    if (lin >= tiles_m * tiles_n) return;
    constexpr uint32_t GM = 4;
    const uint32_t group = lin / (GM * tiles_n);
    const uint32_t first_m = group * GM;
    const uint32_t gm = (tiles_m - first_m < GM) ? tiles_m - first_m : GM;
    const uint32_t in_group = lin - group * GM * tiles_n;
    const uint32_t tn = (gm == GM) ? in_group / GM : in_group / gm;  // (the common divisor is a shift)
    const int tile_m = (int)(first_m + (in_group - tn * gm));
    const int tile_n = (int)tn + p.tile_n0;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wn = wave & 3;     // column quarter
    const int kgrp = wave >> 2;  // k64 sub-step of each stage
    const int j = lane & 15;
    const int g = lane >> 4;
    const int64_t m0 = (int64_t)tile_m * BM;
    const int64_t ncol = (int64_t)tile_n * G_BN + 64 * wn + 4 * j;
    const bool col_ok = ncol < p.N;

    // Addresses are a wave-uniform base (advanced once per stage) plus a 32-bit
    // per-lane offset fixed for the whole kernel.  Loads are unconditional with
    // clamped rows / columns: rows past M and columns past N only feed outputs that
    // are never stored; the K tail is zeroed in the A operand of the last stage.
    // (The host guarantees K % 16 == 0, N % 4 == 0, aligned bases, 32-bit offsets.)
    // A staging role: one row, 32 of its 128 stage bytes.  A wave stages one 16-row block:
    // its 64 lanes touch 16 cache lines per load (four 32-byte parts of each row's line), and
    // eight consecutive lanes write 128 contiguous bytes of LDS.
    const int a_row = 16 * wave + (lane & 15);
    const int a_part = lane >> 4;  // bytes 32*a_part .. +31 -> sub-step a_part>>1, chunks 2*(a_part&1), +1
    const int64_t rows_left = (p.M - m0 < BM) ? p.M - m0 : BM;  // (a tile of fewer than 128 rows: the other waves stage its last row again)
    const uint32_t a_row_c = (uint32_t)((a_row < rows_left) ? a_row : rows_left - 1);
    const uint32_t a_off = a_row_c * (uint32_t)p.K + 32u * a_part;
    uint32_t b_off;
    if constexpr (WT) {
        const int tt = stored_tile16((int)(ncol >> 4), p.tiles16);
        b_off = ((uint32_t)tt * (uint32_t)p.wsteps * 64u + (uint32_t)(16 * g + 4 * (j & 3))) * 4u;
    } else {
        b_off = (uint32_t)(col_ok ? ncol : 0) + (uint32_t)(16 * kgrp + 4 * g) * (uint32_t)p.N;
    }
    const int8_t* a_base = p.Q + m0 * p.K;  // uniform
    const uint8_t* b_base = p.W_T;          // uniform
    const int64_t N = p.N;
    const int nfull = (int)(p.K / G_BK);
    const int nstages = (int)((p.K + G_BK - 1) / G_BK);

    // two stages of operands in flight: set s%2 holds stage s until it is written to LDS
    uint4 a_set[2][2];
    uint32_t b_set[2][4];

    // part: 1 = activations, 2 = weights, 3 = both
    auto load_full = [&](int64_t k0, int part, uint4 (&a_reg)[2], uint32_t (&b_reg)[4]) {
        if (part & 1) {
            const int8_t* ab = a_base + k0;
            a_reg[0] = *(const uint4*)(ab + a_off);
            a_reg[1] = *(const uint4*)(ab + 16 + a_off);
        }
        if (part & 2) {
            if constexpr (WT) {
                const int step = min((int)(k0 >> 6) + kgrp, p.wsteps - 1);  // uniform per wave
                const uint4 v = *(const uint4*)(b_base + (size_t)step * 256 + b_off);
                b_reg[0] = v.x; b_reg[1] = v.y; b_reg[2] = v.z; b_reg[3] = v.w;
            } else {
                const uint8_t* bb = b_base + (k0 >> 2) * N;
#pragma unroll
                for (int r = 0; r < 4; r++) b_reg[r] = *(const uint32_t*)(bb + r * N + b_off);
            }
        }
    };
    auto load_tail = [&](int64_t k0, int part, uint4 (&a_reg)[2], uint32_t (&b_reg)[4]) {
        // last, partial stage: k beyond K reads a clamped address and is zeroed in A
        if (part & 1) {
            const int8_t* ab = a_base + k0;
#pragma unroll
            for (int c = 0; c < 2; c++) {
                const bool in = (k0 + 32 * a_part + 16 * c) < p.K;
                const uint4 v = *(const uint4*)(ab + (in ? 16 * c : 0) + (in ? a_off : a_row_c * (uint32_t)p.K));
                const uint32_t m = in ? 0xFFFFFFFFu : 0u;
                a_reg[c] = make_uint4(v.x & m, v.y & m, v.z & m, v.w & m);
            }
        }
        if constexpr (WT) {
            if (part & 2) {  // the copy is zero-padded to whole steps; a step past the end meets zeroed activations
                const int step = min((int)(k0 >> 6) + kgrp, p.wsteps - 1);
                const uint4 v = *(const uint4*)(b_base + (size_t)step * 256 + b_off);
                b_reg[0] = v.x; b_reg[1] = v.y; b_reg[2] = v.z; b_reg[3] = v.w;
            }
        } else if (part & 2) {
#pragma unroll
            for (int r = 0; r < 4; r++) {
                int64_t kb = (k0 >> 2) + 16 * kgrp + r + 4 * g;
                kb = kb < p.Kb ? kb : p.Kb - 1;
                b_reg[r] = *(const uint32_t*)(b_base + kb * N + (col_ok ? ncol : 0));
            }
        }
    };
    auto load_stage = [&](int st, int part, uint4 (&a_reg)[2], uint32_t (&b_reg)[4]) {  // st, part uniform
        if constexpr (TAIL) {
            if (st >= nstages) st = nstages - 1;
            if (st < nfull) load_full((int64_t)st * G_BK, part, a_reg, b_reg);
            else load_tail((int64_t)st * G_BK, part, a_reg, b_reg);
        } else {
            // past the end: reload the last stage (never consumed) instead of branching
            load_full((int64_t)(st < nstages ? st : nstages - 1) * G_BK, part, a_reg, b_reg);
        }
    };
    auto store_a = [&](int buf, const uint4 (&a_reg)[2]) {
        // slot (sub, mb, lane = c*16 + i) holds the 16 bytes MFMA lane (i, g = c) reads
        uint8_t* base = lds + buf * G_STAGE_BYTES;
        const int mb = a_row >> 4, i = a_row & 15, sub = a_part >> 1;
#pragma unroll
        for (int e = 0; e < 2; e++) {
            const int c = 2 * (a_part & 1) + e;
            uint32_t t[4];
            if constexpr (QOO) {
                t[0] = a_reg[e].x; t[1] = a_reg[e].y; t[2] = a_reg[e].z; t[3] = a_reg[e].w;
            } else {
                transpose4x4_bytes(a_reg[e].x, a_reg[e].y, a_reg[e].z, a_reg[e].w, t);
            }
            *(uint4*)(base + ((size_t)((sub * G_MB + mb) * 64 + c * 16 + i) << 4)) = make_uint4(t[0], t[1], t[2], t[3]);
        }
    };

    v4i acc[2 * NB][4];
#pragma unroll
    for (int mb = 0; mb < 2 * NB; mb++)
#pragma unroll
        for (int t = 0; t < 4; t++) acc[mb][t] = v4i{0, 0, 0, 0};
    if constexpr (FL) {
        if (kgrp == 0) {  // (wave-uniform) lane (j, g) holds rows 16 mb + 4 g + r of its columns
#pragma unroll
            for (int mb = 0; mb < 2 * NB; mb++) {
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int64_t m = m0 + 16 * mb + 4 * g + r;
                    const int32_t rs = p.q_rowsum[m < p.M ? m : p.M - 1];
                    acc[mb][0][r] = -rs;
                    acc[mb][1][r] = -(rs << 2);
                    acc[mb][2][r] = -(rs << 4);
                }
            }
        }
    }

    // ---- main loop --------------------------------------------------------------------
    // Stage s is computed from LDS buffer s%2 and is software-pipelined inside the wave so
    // that the matrix cores never wait for the stage's own operand preparation:
    //   * on entry the wave already holds the decoded weights of stage s (b_dec) and the
    //     activation fragments of row blocks 0..3 (a_lo);
    //   * it writes its piece of stage s+1 into the other LDS buffer, re-uses those registers
    //     for the global loads of stage s+3 (two full stages to arrive), requests row blocks
    //     4..7 (a_hi), and issues the 16 MFMAs of row blocks 0..3 while the weights of stage
    //     s+1 are being decoded in the shadow of those MFMAs;
    //   * the one barrier of the stage publishes buffer (s+1)%2; row blocks 0..3 of stage
    //     s+1 are requested right behind it and arrive under the 16 MFMAs of row blocks 4..7.
    // Stages past the end are clamped (loaded, never consumed) instead of branched around;
    // the loop handles two stages per trip so that the register sets are indexed statically.
    v4i b_dec[2][4];
    uint4 a_lo[NB], a_hi[NB];
    const uint32_t a_lds_off = (uint32_t)(kgrp * (G_MB * 1024)) + ((uint32_t)lane << 4);
    auto decode_b = [&](const uint32_t (&raw)[4], v4i (&out)[4]) {
        if constexpr (FL) {
#pragma unroll
            for (int t = 0; t < 4; t++)
#pragma unroll
                for (int c = 0; c < 4; c++) out[t][c] = (int)(raw[c] & (0x03030303u << (2 * t)));
            return;
        }
        uint32_t G[4];
        if constexpr (WT) { G[0] = raw[0]; G[1] = raw[1]; G[2] = raw[2]; G[3] = raw[3]; }
        else transpose4x4_bytes(raw[0], raw[1], raw[2], raw[3], G);
#pragma unroll
        for (int t = 0; t < 4; t++) out[t] = decode16_i8(G[t]);
    };
    auto read_a = [&](int buf, int mb0, uint4 (&dst)[NB]) {
        const uint8_t* a_lds = lds + buf * G_STAGE_BYTES + a_lds_off;
        // in this order, one by one: LDS returns in order, and the first MFMA of a run needs the first row block only
        // (left alone, the scheduler issues the reads in descending order and the run waits for all of them)
#pragma unroll
        for (int i = 0; i < NB; i++) {
            dst[i] = *(const uint4*)(a_lds + (mb0 + i) * 1024);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto mfma_half = [&](int mb0, const uint4 (&av)[NB], const v4i (&b)[4]) {
#pragma unroll
        for (int i = 0; i < NB; i++) {
            const v4i a = {(int)av[i].x, (int)av[i].y, (int)av[i].z, (int)av[i].w};
#pragma unroll
            for (int t = 0; t < 4; t++)
                acc[mb0 + i][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b[t], acc[mb0 + i][t], 0, 0, 0);
        }
    };

    load_stage(0, 3, a_set[0], b_set[0]);
    load_stage(1, 3, a_set[1], b_set[1]);
    store_a(0, a_set[0]);
    decode_b(b_set[0], b_dec[0]);
    load_stage(2, 3, a_set[0], b_set[0]);
    __syncthreads();
    read_a(0, 0, a_lo);

    // decode of the next stage's weights cut into slices of at most five VALU operations,
    // one slice issued behind each of the later MFMAs of row blocks 0..3 (an MFMA occupies the matrix pipe
    // for 16 cycles; the VALU operations of the same wave behind it run in its shadow)
    uint32_t d_t[4], d_G[4], d_H[4];
    auto decode_slice = [&](int c, const uint32_t (&raw)[4], v4i (&out)[4]) {
        if constexpr (FL) {  // one operation per slice: operand dword c & 3 of column block c >> 2
            if (c < 16) out[c >> 2][c & 3] = (int)(raw[c & 3] & (0x03030303u << (2 * (c >> 2))));
            return;
        }
        const uint32_t lutA_lo = 0x00FF0100u, lutB_lo = 0x0000FF00u, lutB_hi = 0x00000001u;
        auto partA = [&](int t) {
            d_H[t] = d_G[t] >> 4;
            out[t][0] = (int)perm(0u, lutA_lo, d_G[t] & 0x03030303u);
        };
        auto partB = [&](int t) {
            out[t][1] = (int)perm(lutB_hi, lutB_lo, d_G[t] & 0x0C0C0C0Cu);
            out[t][2] = (int)perm(0u, lutA_lo, d_H[t] & 0x03030303u);
        };
        auto partC = [&](int t) { out[t][3] = (int)perm(lutB_hi, lutB_lo, d_H[t] & 0x0C0C0C0Cu); };
        if constexpr (WT) {
            // tiled weights need no transpose: the nine operations of each column are cut into four slices of at
            // most three, one behind every one of the 16 MFMAs, so that no MFMA has to wait for the wave's own VALU work
            const int t = c >> 2;
            switch (c & 3) {
                case 0: d_G[t] = raw[t]; partA(t); break;
                case 1: out[t][1] = (int)perm(lutB_hi, lutB_lo, d_G[t] & 0x0C0C0C0Cu); break;
                case 2: out[t][2] = (int)perm(0u, lutA_lo, d_H[t] & 0x03030303u); break;
                default: partC(t); break;
            }
            return;
        }
        switch (c) {
            case 4:
                if constexpr (!WT) {
                    d_t[0] = perm(raw[1], raw[0], 0x05010400u);
                    d_t[1] = perm(raw[1], raw[0], 0x07030602u);
                    d_t[2] = perm(raw[3], raw[2], 0x05010400u);
                    d_t[3] = perm(raw[3], raw[2], 0x07030602u);
                }
                break;
            case 5:
                if constexpr (WT) {
                    d_G[0] = raw[0]; d_G[1] = raw[1]; d_G[2] = raw[2]; d_G[3] = raw[3];
                } else {
                    d_G[0] = perm(d_t[2], d_t[0], 0x05040100u);
                    d_G[1] = perm(d_t[2], d_t[0], 0x07060302u);
                    d_G[2] = perm(d_t[3], d_t[1], 0x05040100u);
                    d_G[3] = perm(d_t[3], d_t[1], 0x07060302u);
                }
                break;
            case 6: partA(0); break;
            case 7: partB(0); break;
            case 8: partC(0); partA(1); break;
            case 9: partB(1); break;
            case 10: partC(1); partA(2); break;
            case 11: partB(2); break;
            case 12: partC(2); partA(3); break;
            case 13: partB(3); break;
            case 14: partC(3); break;
            default: break;
        }
    };

    auto stage = [&](int s, uint4 (&a_reg)[2], uint32_t (&b_reg)[4], const v4i (&b_cur)[4], v4i (&b_nxt)[4]) {
        // a_reg / b_reg hold stage s+1 on entry and are reloaded with stage s+3
        const int cur = s & 1;
        store_a(cur ^ 1, a_reg);
        load_stage(s + 3, 1, a_reg, b_reg);
        read_a(cur, NB, a_hi);
        __builtin_amdgcn_sched_barrier(0);
        // the wave that issues matrix instructions goes first on its SIMD; the other wave's staging, loads
        // and LDS traffic fill the gaps (same-run A/B: 1-3 % on every shape)
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int c = 0; c < 4 * NB; c++) {
            const int i = c >> 2, t = c & 3;
            const v4i a = {(int)a_lo[i].x, (int)a_lo[i].y, (int)a_lo[i].z, (int)a_lo[i].w};
            acc[i][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b_cur[t], acc[i][t], 0, 0, 0);
#pragma unroll
            for (int q = 0; q < 4 / NB; q++) decode_slice(c * (4 / NB) + q, b_reg, b_nxt);  // (NB = 4: one slice)
            __builtin_amdgcn_sched_barrier(0);  // keep the slice behind its MFMA
        }
        // the raw weights are dead now: their registers take the loads of stage s+3 directly
        // (a copy of a register with a load in flight would have to wait for that load)
        load_stage(s + 3, 2, a_reg, b_reg);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_setprio(0);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        read_a(cur ^ 1, 0, a_lo);
        mfma_half(NB, a_hi, b_cur);
        __builtin_amdgcn_sched_barrier(0);
        // The fragments just requested for the next stage arrived during these MFMAs: saying so here (lgkmcnt(0), vmcnt
        // and expcnt untouched) costs nothing, and keeps the wait the compiler otherwise puts in front of the next stage's
        // first MFMA -- for everything outstanding across the loop edge, the four reads issued right before it included --
        // out of the way.
        __builtin_amdgcn_s_waitcnt(0xC07F);
        __builtin_amdgcn_sched_barrier(0);
    };
    // The two waves that share a SIMD (the K halves of one column quarter) run the stage in different orders, so
    // that one of them is inside a run of MFMAs while the other stages, loads and reads LDS: K half 1 reads all
    // eight row blocks of stage s right behind the barrier that published them, then does both MFMA halves in a
    // row and arrives at the next barrier with stage s finished, while K half 0 (above) is half a stage behind it
    // and has its second MFMA half on the far side of the barrier.  Same barriers, same buffers: stage s+1 goes to
    // the buffer whose readers all finished before the last barrier.
    auto stage_y = [&](int s, uint4 (&a_reg)[2], uint32_t (&b_reg)[4], const v4i (&b_cur)[4], v4i (&b_nxt)[4]) {
        const int cur = s & 1;
        read_a(cur, 0, a_lo);
        read_a(cur, NB, a_hi);
        store_a(cur ^ 1, a_reg);
        load_stage(s + 3, 1, a_reg, b_reg);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < 4 * NB; c++) {
            const int i = c >> 2, t = c & 3;
            const v4i a = {(int)a_lo[i].x, (int)a_lo[i].y, (int)a_lo[i].z, (int)a_lo[i].w};
            acc[i][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b_cur[t], acc[i][t], 0, 0, 0);
#pragma unroll
            for (int q = 0; q < 4 / NB; q++) decode_slice(c * (4 / NB) + q, b_reg, b_nxt);
            __builtin_amdgcn_sched_barrier(0);
        }
        load_stage(s + 3, 2, a_reg, b_reg);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_setprio(1);
        mfma_half(NB, a_hi, b_cur);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_setprio(0);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
    };
    // (an odd last stage is peeled: with a conditional second half inside the loop the two
    // paths to the loop header leave different loads outstanding, and the wait the compiler
    // puts at the top of the loop then drains the whole queue, freshly issued loads included)
    int s = 0;
    if (kgrp == 0 || !ANTIPHASE) {  // wave-uniform
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the first fragments, so that the loop is entered as it is re-entered
        __builtin_amdgcn_sched_barrier(0);
        for (; s + 1 < nstages; s += 2) {
            stage(s, a_set[1], b_set[1], b_dec[0], b_dec[1]);
            stage(s + 1, a_set[0], b_set[0], b_dec[1], b_dec[0]);
        }
        if (s < nstages) stage(s, a_set[1], b_set[1], b_dec[0], b_dec[1]);
    } else {
        for (; s + 1 < nstages; s += 2) {
            stage_y(s, a_set[1], b_set[1], b_dec[0], b_dec[1]);
            stage_y(s + 1, a_set[0], b_set[0], b_dec[1], b_dec[0]);
        }
        if (s < nstages) stage_y(s, a_set[1], b_set[1], b_dec[0], b_dec[1]);
    }
    // K half 1 leaves the loop with nothing left to read from the stage buffers, and K half 0 holds the fragments of its
    // last MFMAs in registers (what it still reads behind the last barrier of the loop belongs to a stage that does not
    // exist and is never used): the hand-over may overwrite the buffers from here on.
    if (kgrp == 1) give_blocks<NB>(acc, 0, lds, wn, lane);  // wave-uniform branches
    __syncthreads();

    EpiOperands<NB> epi_ops;
    load_epi_operands<NB>(p, m0, NB * kgrp, g, ncol, col_ok, epi_ops);
    // what can take the short epilogue as far as the launch and the tile decide (uniform); the row scales have their say below
    const bool short_ok = !p.long_epilogue && m0 + BM <= p.M && !p.acc_out && (!p.epi.residual || p.y_dtype != BT_F32);
    if (short_ok && p.epi.residual && col_ok) load_epi_residual<NB>(p, m0, NB * kgrp, g, ncol, epi_ops);

    if (kgrp == 0) {
        take_blocks<NB>(acc, 0, lds, wn, lane);   // K half 1's sums of my row blocks 0..3 (0..NB-1)
        give_blocks<NB>(acc, NB, lds, wn, lane);  // my sums of its row blocks 4..7 (NB..2NB-1), into the slots just read
    }
    __syncthreads();
    if (kgrp == 1) take_blocks<NB>(acc, NB, lds, wn, lane);

    // the short epilogue where nothing needs the long one (every condition uniform over the wave)
    bool small_sx = false;
#pragma unroll
    for (int mbi = 0; mbi < NB; mbi++)
#pragma unroll
        for (int r = 0; r < 4; r++) small_sx |= !(__builtin_fabsf(epi_ops.sx[mbi][r]) >= DIV127_FAST_MIN_SX);
    const bool fast = short_ok && __builtin_amdgcn_ballot_w64(small_sx) == 0ull;
    if (!col_ok) return;
    if (kgrp == 0) gemm_epilogue_dt<0, NB, FL>(p, acc, m0, g, ncol, epi_ops, fast);  // wave-uniform branch
    else gemm_epilogue_dt<NB, NB, FL>(p, acc, m0, g, ncol, epi_ops, fast);
}


// the same kernel on the decode-tiled weight copy (256-byte aligned, below 4 GiB: checked by the caller)
bool gemm_i8_supported_tiled(int64_t N, int64_t K, const void* Q) {
    return N % 4 == 0 && K % 16 == 0 && ((uintptr_t)Q) % 16 == 0 && (G_BM + 1) * K < (1ll << 32);
}

// the tiled kernel reads Q with 16-byte loads and W_T / Y with 4-column vectors
bool gemm_i8_supported(int64_t N, int64_t K, const void* Q, const void* W_T) {
    // 32-bit per-lane offsets: a row tile of Q and the whole of W_T stay below 4 GiB
    return N % 4 == 0 && K % 16 == 0 && ((uintptr_t)W_T) % 4 == 0 && ((uintptr_t)Q) % 16 == 0 &&
           (G_BM + 1) * K < (1ll << 32) && ceil_div(K, 4) * N < (1ll << 32);
}

// One launch over column tiles [tile_n0, tile_n0 + tiles_n) in tiles of 32 * NB rows.
template <int NB>
static int launch_gemm_i8_part(GemmParams p, int tile_n0, int tiles_n, bool qoo, bool tiled, bool fields, hipStream_t st) {
    p.tile_n0 = tile_n0;
    p.tiles_n = tiles_n;
    p.tiles_m = (int)ceil_div(p.M, 32 * NB);
    const int64_t total = (int64_t)p.tiles_m * p.tiles_n;
    if (total >= (1ll << 31) - 8) {
        set_error("bt_ternary_gemm_i8: %lld tiles of %d x 256 outputs are more than one launch takes", (long long)total, 32 * NB);
        return BT_ERR_INVALID;
    }
    p.per_xcd = (int)ceil_div(total, 8);
    const dim3 grid((unsigned)(p.per_xcd * 8)), block(512);
    const bool tail = p.K % G_BK != 0;
    if (fields) {  // (the caller has checked: K in whole stages)
        if (qoo) hipLaunchKernelGGL((gemm_i8_kernel<false, true, true, true, NB, true>), grid, block, 0, st, p);
        else hipLaunchKernelGGL((gemm_i8_kernel<false, false, true, true, NB, true>), grid, block, 0, st, p);
    } else if constexpr (NB != 4) {  // (only where launch_gemm_i8 cuts finer: tiled weights, whole stages)
        if (qoo) hipLaunchKernelGGL((gemm_i8_kernel<false, true, true, true, NB>), grid, block, 0, st, p);
        else hipLaunchKernelGGL((gemm_i8_kernel<false, false, true, true, NB>), grid, block, 0, st, p);
    } else if (tiled) {
        if (!tail) {
            if (qoo && tuning_env("BITTORCH_GEMM_INPHASE")) hipLaunchKernelGGL((gemm_i8_kernel<false, true, true, false>), grid, block, 0, st, p);
            else if (qoo) hipLaunchKernelGGL((gemm_i8_kernel<false, true, true>), grid, block, 0, st, p);
            else hipLaunchKernelGGL((gemm_i8_kernel<false, false, true>), grid, block, 0, st, p);
        } else {
            if (qoo) hipLaunchKernelGGL((gemm_i8_kernel<true, true, true>), grid, block, 0, st, p);
            else hipLaunchKernelGGL((gemm_i8_kernel<true, false, true>), grid, block, 0, st, p);
        }
    } else if (!tail) {
        if (qoo) hipLaunchKernelGGL((gemm_i8_kernel<false, true>), grid, block, 0, st, p);
        else hipLaunchKernelGGL((gemm_i8_kernel<false, false>), grid, block, 0, st, p);
    } else {
        if (qoo) hipLaunchKernelGGL((gemm_i8_kernel<true, true>), grid, block, 0, st, p);
        else hipLaunchKernelGGL((gemm_i8_kernel<true, false>), grid, block, 0, st, p);
    }
    return check_launch("bt_ternary_gemm_i8");
}

// q_rowsum: the rows' sums of Q, needed (and only read) with a field-layout copy
int launch_gemm_i8(const int8_t* Q, int q_layout, const float* s_x, const int32_t* q_rowsum, const uint8_t* W_T, int w_layout,
                   const Epilogue& epi, void* Y, int y_dtype, int32_t* acc_out, int64_t M, int64_t N, int64_t K,
                   hipStream_t st) {
    GemmParams p = {};
    p.Q = Q; p.s_x = s_x; p.W_T = W_T; p.Y = Y; p.acc_out = acc_out; p.epi = epi; p.q_rowsum = q_rowsum;
    p.M = M; p.N = N; p.K = K; p.Kb = ceil_div(K, 4);
    p.y_dtype = y_dtype;
    p.long_epilogue = option(OPT_GEMM_LONG_EPILOGUE) != nullptr;
    p.wsteps = (int)ceil_div(p.Kb, 16);
    p.tiles16 = tiles16_arg(N, w_layout);
    const bool qoo = q_layout == Q_OPERAND_ORDER, tiled = layout_tiled(w_layout), fields = layout_fields(w_layout);
    const int64_t tiles_n = ceil_div(N, G_BN);
    // the column tiles of a mostly empty last round in finer tiles, a launch of their own behind the whole tiles
    // (gemm_split; same sums, same bits)
    const GemmSplit sp = gemm_split(M, N, tiled && K % G_BK == 0 && !tuning_env("BITTORCH_GEMM_INPHASE"));
    if (sp.nb != 4) {
        if (sp.cols < tiles_n) {
            const int rc = launch_gemm_i8_part<4>(p, 0, (int)(tiles_n - sp.cols), qoo, tiled, fields, st);
            if (rc) return rc;
        }
        return sp.nb == 1 ? launch_gemm_i8_part<1>(p, (int)(tiles_n - sp.cols), (int)sp.cols, qoo, tiled, fields, st)
                          : launch_gemm_i8_part<2>(p, (int)(tiles_n - sp.cols), (int)sp.cols, qoo, tiled, fields, st);
    }
    return launch_gemm_i8_part<4>(p, 0, (int)tiles_n, qoo, tiled, fields, st);
}

}  // namespace bt
