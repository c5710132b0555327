// Large-batch fp16 / bf16 x packed-ternary GEMM for gfx950 on the 16-bit matrix cores:
// the float path of the packed forward for batches too tall for the streaming kernel.
//
// Arithmetic restated from the reference's large-batch packed kernel
// (csrc/kernels/ternary_gemm_production.cu:158-250, accumulate :226-235, epilogue :244-247):
//   acc_f32[m,n] = sum_k x[m,k] * w[k,n];   y[m,n] = acc * scale[n] + bias[n]
// (fp32 accumulation of exact products; the summation order differs from the reference's
// sequential loop, which the 16-bit output tolerance covers).
//
// Same structure as the int8 prefill kernel: a 512-thread workgroup (8 waves) owns a
// 128 x 256 output tile; wave w works on columns 64*(w&3) .. +63 and on k32 sub-step (w>>2)
// of every 64-wide K stage over all 128 rows; the two K halves are added through LDS once.
//   * Activations (16-bit, row-major [M,K]) go through LDS, double buffered, 64 k per stage,
//     stored in MFMA operand order: slot (sub, mb, lane) is the 16 bytes (8 values) lane
//     (i = lane%16, g = lane/16) feeds to v_mfma_f32_16x16x32_{f16,bf16} for row block mb and
//     k32 sub-step sub, with the values already in the k order the weight decode produces.
//   * Weights never touch LDS: lane (j, g) loads one dword (four output columns) from each of
//     the two rows kb + 2g, 2g+1 and decodes each column's two bytes into eight 16-bit weights
//     with v_perm table lookups (fp16 +-1.0; bf16 +-2.0 with the sum halved exactly).
//   * The stage is software-pipelined inside the wave like the int8 kernel's.
#include <algorithm>
#include <cstddef>
#include <cstdlib>

#include "bt_common.h"

namespace bt {

constexpr int F_BM = 128;
constexpr int F_BN = 256;
constexpr int F_BK = 64;            // k per LDS stage (two k32 MFMA sub-steps)
constexpr int F_MB = F_BM / 16;     // 16-row blocks per tile
constexpr int F_STAGE_BYTES = F_BM * F_BK * 2;  // 16 KiB

struct GemmFParams {
    // The first 64 bytes hold what a workgroup needs to find its tile and request its first operands: the kernel
    // arguments come through the scalar cache a 64-byte line at a time.
    const uint16_t* X;    // [M, K] fp16 or bf16 bits
    const uint8_t* W_T;   // [Kb, N]
    int64_t K, M, N;      // K: length of an activation row
    int tiles_m, tiles_n;
    int per_xcd;          // workgroups per XCD (grid = 8 * per_xcd)
    int wstages;          // 64-wide stages of W_T; a stage index beyond it wraps (see launch_gemm_f16)
    int tiles16;          // WT: 16-column tiles of the decode-tiled weight copy (its 16-row steps are the stages; < 0: stored_tile16)
    int tile_n0;          // first column tile of this launch (tiles_n counts the launch's own column tiles)
    // ---- needed later
    void* Y;              // [M, N]
    int64_t Kb;           // packed weight rows
    int y_dtype;
    int prehalved;        // MODE_BF16: the activations already carry the factor 1/2 of the +-2.0 weight decode
    Epilogue epi;
};
static_assert(offsetof(GemmFParams, Y) == 64, "first argument line as laid out above");

__device__ __forceinline__ void store4f(void* Y, int dt, int64_t idx, const float (&v)[4]) {
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

// Finishes NB 16-row blocks (acc[MB0 .. MB0+NB-1]) of the tile: NB = 4 in a tile of 128 rows, 2 or 1 in the tiles of 64
// and 32 rows a launch's remainder is cut into.
// RES: the 16-bit residual of the lane's 16 rows was requested ahead of the hand-over of the K halves (full tiles
// only); one load per row right before its use leaves a memory round trip per row exposed, 5 us per tile.
// FULL: every row of the tile exists: no per-row bounds checks, and a row's address is a lane offset fixed for the whole
// epilogue plus a uniform row term (the general form pays two quarter-rate 64-bit multiplies per row).
template <int MODE, int YDT, int MB0, int NB, bool RES = false, bool FULL = false>
__device__ __forceinline__ void gemm_f_epilogue(const GemmFParams& p, const v4f (&acc)[2 * NB][4], int64_t m0, int g,
                                                int64_t ncol, const uint32_t (&ws_bits)[4], const uint32_t (&bs_bits)[4],
                                                const uint2 (&res)[NB][4]) {
    float ws[4], bs[4];
#pragma unroll
    for (int t = 0; t < 4; t++) {
        ws[t] = bits_to_f32_rt(ws_bits[t], p.epi.scale_dtype);
        bs[t] = p.epi.bias ? bits_to_f32_rt(bs_bits[t], p.epi.bias_dtype) : 0.0f;
    }
#pragma unroll
    for (int mbi = 0; mbi < NB; mbi++) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int64_t m = m0 + 16 * (MB0 + mbi) + 4 * g + r;
            if constexpr (!FULL) {
                if (m >= p.M) continue;
            }
            float y[4];
#pragma unroll
            for (int t = 0; t < 4; t++) {
                float a = acc[MB0 + mbi][t][r];
                if constexpr (MODE == MODE_BF16) a *= (p.prehalved ? 1.0f : 0.5f);  // weights were decoded as +-2.0
                y[t] = epi_float(a, ws[t], bs[t]);
            }
            if constexpr (RES && YDT != BT_F32) {  // what add_residual4 does, on the bits already here
                const uint32_t d[2] = {res[mbi][r].x, res[mbi][r].y};
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const uint32_t h = (d[t >> 1] >> (16 * (t & 1))) & 0xffffu;
                    const float rv = (YDT == BT_F16) ? f16_bits_to_f32((uint16_t)h) : bf16_bits_to_f32((uint16_t)h);
                    y[t] = sum_in_dtype(round_to_dtype(y[t], YDT), rv, YDT);
                }
            } else if (p.epi.residual) {
                add_residual4(y, p.epi.residual, YDT, m * p.N + ncol);
            }
            if constexpr (FULL) {
                constexpr int ES = (YDT == BT_F32) ? 4 : 2;
                const int64_t ncol0 = (int64_t)__builtin_amdgcn_readfirstlane((int)(ncol / F_BN)) * F_BN;  // the tile's first column
                const uint32_t lane_off = ((uint32_t)(4 * g) * (uint32_t)p.N + (uint32_t)(ncol - ncol0)) * ES;
                char* const dst = (char*)p.Y + ((m0 + 16 * (MB0 + mbi) + r) * p.N + ncol0) * ES + lane_off;  // uniform + lane
                if constexpr (YDT == BT_F32) {
                    st4_nt((float*)dst, __builtin_bit_cast(uint32_t, y[0]), __builtin_bit_cast(uint32_t, y[1]),
                           __builtin_bit_cast(uint32_t, y[2]), __builtin_bit_cast(uint32_t, y[3]));
                } else {
                    uint16_t h[4];
#pragma unroll
                    for (int i = 0; i < 4; i++) h[i] = (YDT == BT_F16) ? f32_to_f16_bits(y[i]) : f32_to_bf16_bits(y[i]);
                    st2_nt((uint16_t*)dst, (uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16));
                }
            } else {
                store4f(p.Y, YDT, m * p.N + ncol, y);
            }
        }
    }
}
template <int MODE, int MB0, int NB>
__device__ __forceinline__ void gemm_f_epilogue_dt(const GemmFParams& p, const v4f (&acc)[2 * NB][4], int64_t m0,
                                                   int g, int64_t ncol, const uint32_t (&ws_bits)[4],
                                                   const uint32_t (&bs_bits)[4], const uint2 (&res)[NB][4], bool res_here) {
    if (res_here) {  // uniform; 16-bit outputs of a full tile
        if (p.y_dtype == BT_BF16) gemm_f_epilogue<MODE, BT_BF16, MB0, NB, true, true>(p, acc, m0, g, ncol, ws_bits, bs_bits, res);
        else gemm_f_epilogue<MODE, BT_F16, MB0, NB, true, true>(p, acc, m0, g, ncol, ws_bits, bs_bits, res);
        return;
    }
    if (!p.epi.residual && m0 + 32 * NB <= p.M) {  // uniform: a full tile without residual
        if (p.y_dtype == BT_BF16) gemm_f_epilogue<MODE, BT_BF16, MB0, NB, false, true>(p, acc, m0, g, ncol, ws_bits, bs_bits, res);
        else if (p.y_dtype == BT_F16) gemm_f_epilogue<MODE, BT_F16, MB0, NB, false, true>(p, acc, m0, g, ncol, ws_bits, bs_bits, res);
        else gemm_f_epilogue<MODE, BT_F32, MB0, NB, false, true>(p, acc, m0, g, ncol, ws_bits, bs_bits, res);
        return;
    }
    if (p.y_dtype == BT_BF16) gemm_f_epilogue<MODE, BT_BF16, MB0, NB>(p, acc, m0, g, ncol, ws_bits, bs_bits, res);
    else if (p.y_dtype == BT_F16) gemm_f_epilogue<MODE, BT_F16, MB0, NB>(p, acc, m0, g, ncol, ws_bits, bs_bits, res);
    else gemm_f_epilogue<MODE, BT_F32, MB0, NB>(p, acc, m0, g, ncol, ws_bits, bs_bits, res);
}

// TAIL = false: K is a multiple of the 64-wide stage and the main loop is branch free.
// TAIL = true: any K % 8 == 0; the last, partial stage is masked.
// WT = true: W_T is the decode-tiled copy (W_LAYOUT_TILED): the dwords of a lane's four columns in its step are
// 16 contiguous bytes (one load instead of two), of which the k32 sub-step uses two bytes each.
// NB: 16-row blocks per K half and wave: 4 is the 128-row tile; 2 and 1 are the tiles of 64 and 32 rows (same columns,
// same staging and LDS layout with rows past the tile clamped) that a launch's remainder is cut into when whole tiles
// would leave most compute units idle (launch_gemm_f16).
template <int MODE, bool TAIL, bool WT = false, int NB = 4>
__global__ __launch_bounds__(512) void gemm_f16_kernel(GemmFParams p) {
    constexpr int BR = WT ? 4 : 2;  // raw weight dwords per lane and stage
    constexpr int BM = 32 * NB;     // rows of the tile
    __shared__ __attribute__((aligned(16))) uint8_t lds[65536];  // 2 A stages; reused for the K-half exchange

    // XCD-aware tile order: the 8 XCDs each take a contiguous run of tiles, walked in groups
    // of four row tiles so that one XCD's L2 holds a compact block of rows and columns
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
    const int kgrp = wave >> 2;  // k32 sub-step of each stage
    const int j = lane & 15;
    const int g = lane >> 4;
    const int64_t m0 = (int64_t)tile_m * BM;
    const int64_t ncol = (int64_t)tile_n * F_BN + 64 * wn + 4 * j;
    const bool col_ok = ncol < p.N;

    // Addresses are a wave-uniform base (advanced once per stage) plus a 32-bit per-lane
    // offset fixed for the whole kernel.  Loads are unconditional with clamped rows / columns:
    // rows past M and columns past N only feed outputs that are never stored; the K tail is
    // zeroed in the A operand of the last stage.
    // A staging role: one row, 32 of its 128 stage bytes (16 values).  A wave stages one 16-row
    // block: its 64 lanes touch 16 cache lines per load, eight consecutive lanes write 128
    // contiguous bytes of LDS.
    const int a_row = 16 * wave + (lane & 15);
    const int a_part = lane >> 4;  // values 16*a_part .. +15 -> sub-step a_part>>1, groups 2*(a_part&1), +1
    const int64_t rows_left = (p.M - m0 < BM) ? p.M - m0 : BM;  // (a tile of fewer than 128 rows: the other waves stage its last row again)
    const uint32_t a_row_c = (uint32_t)((a_row < rows_left) ? a_row : rows_left - 1);
    const uint32_t a_off = (a_row_c * (uint32_t)p.K + 16u * a_part) * 2u;  // bytes
    uint32_t b_off;
    if constexpr (WT) {
        const int tt = stored_tile16((int)(ncol >> 4), p.tiles16);
        b_off = ((uint32_t)tt * (uint32_t)p.wstages * 64u + (uint32_t)(16 * (2 * kgrp + (g >> 1)) + 4 * (j & 3))) * 4u;
    } else {
        b_off = (uint32_t)(col_ok ? ncol : 0) + (uint32_t)(8 * kgrp + 2 * g) * (uint32_t)p.N;
    }
    // WT: bytes [zero, row 2(g&1), zero, row 2(g&1)+1] of a column's dword
    const uint32_t sel_wt = ((uint32_t)(2 * (g & 1) + 1) << 24) | (0x0Cu << 16) | ((uint32_t)(2 * (g & 1)) << 8) | 0x0Cu;
    const uint8_t* a_base = (const uint8_t*)(p.X + m0 * p.K);  // uniform
    const uint8_t* b_base = p.W_T;                              // uniform
    const int64_t N = p.N;
    const int nfull = (int)(p.K / F_BK);
    const int nstages = (int)((p.K + F_BK - 1) / F_BK);

    // two stages of operands in flight: set s%2 holds stage s until it is written to LDS
    uint4 a_set[2][2];
    uint32_t b_set[2][BR];

    // part: 1 = activations, 2 = weights, 3 = both
    auto load_full = [&](int st, int part, uint4 (&a_reg)[2], uint32_t (&b_reg)[BR]) {
        if (part & 1) {
            const uint8_t* ab = a_base + 2 * (int64_t)st * F_BK;
            a_reg[0] = *(const uint4*)(ab + a_off);
            a_reg[1] = *(const uint4*)(ab + 16 + a_off);
        }
        if (part & 2) {
            // the activation row may hold several planes of K values, all multiplied with the
            // same weights: the weight stage wraps (uniform)
            int ws = st;
            if (ws >= p.wstages) ws -= p.wstages;
            if (ws >= p.wstages) ws -= p.wstages;
            if constexpr (WT) {
                const uint4 v = *(const uint4*)(b_base + (size_t)ws * 256 + b_off);
                b_reg[0] = v.x; b_reg[1] = v.y; b_reg[2] = v.z; b_reg[BR - 1] = v.w;
            } else if constexpr (TAIL) {
                // zero-padded activation planes with K % 64 != 0: the last weight stage of a plane runs past W_T
#pragma unroll
                for (int r = 0; r < 2; r++) {
                    int64_t kb = (int64_t)ws * (F_BK / 4) + 8 * kgrp + 2 * g + r;
                    kb = kb < p.Kb ? kb : p.Kb - 1;
                    b_reg[r] = *(const uint32_t*)(b_base + kb * N + (col_ok ? ncol : 0));
                }
            } else {
                const uint8_t* bb = b_base + (int64_t)ws * (F_BK / 4) * N;
                b_reg[0] = *(const uint32_t*)(bb + b_off);
                b_reg[1] = *(const uint32_t*)(bb + N + b_off);
            }
        }
    };
    auto load_tail = [&](int64_t k0, int part, uint4 (&a_reg)[2], uint32_t (&b_reg)[BR]) {
        // last, partial stage: k beyond K reads a clamped address and is zeroed in A
        if (part & 1) {
            const uint8_t* ab = a_base + 2 * k0;
#pragma unroll
            for (int c = 0; c < 2; c++) {
                const bool in = (k0 + 16 * a_part + 8 * c) < p.K;
                const uint4 v = *(const uint4*)(ab + (in ? 16 * c : 0) + (in ? a_off : a_row_c * (uint32_t)p.K * 2u));
                const uint32_t m = in ? 0xFFFFFFFFu : 0u;
                a_reg[c] = make_uint4(v.x & m, v.y & m, v.z & m, v.w & m);
            }
        }
        if constexpr (WT) {
            if (part & 2) {  // the copy is zero-padded to whole steps; this is the last step (no planes with a tail)
                const uint4 v = *(const uint4*)(b_base + (size_t)min((int)(k0 >> 6), p.wstages - 1) * 256 + b_off);
                b_reg[0] = v.x; b_reg[1] = v.y; b_reg[2] = v.z; b_reg[BR - 1] = v.w;
            }
        } else if (part & 2) {
#pragma unroll
            for (int r = 0; r < 2; r++) {
                int64_t kb = (k0 >> 2) + 8 * kgrp + 2 * g + r;
                kb = kb < p.Kb ? kb : p.Kb - 1;
                b_reg[r] = *(const uint32_t*)(b_base + kb * N + (col_ok ? ncol : 0));
            }
        }
    };
    auto load_stage = [&](int st, int part, uint4 (&a_reg)[2], uint32_t (&b_reg)[BR]) {  // st, part uniform
        if constexpr (TAIL) {
            if (st >= nstages) st = nstages - 1;
            if (st < nfull) load_full(st, part, a_reg, b_reg);
            else load_tail((int64_t)st * F_BK, part, a_reg, b_reg);
        } else {
            // past the end: reload the last stage (never consumed) instead of branching
            load_full(st < nstages ? st : nstages - 1, part, a_reg, b_reg);
        }
    };
    auto store_a = [&](int buf, const uint4 (&a_reg)[2]) {
        // slot (sub, mb, lane = c*16 + i) holds the 16 bytes MFMA lane (i, g = c) reads:
        // natural values h0..h7 -> dword d = { h[d], h[4+d] } (the decode's k order)
        uint8_t* base = lds + buf * F_STAGE_BYTES;
        const int mb = a_row >> 4, i = a_row & 15, sub = a_part >> 1;
#pragma unroll
        for (int e = 0; e < 2; e++) {
            const int c = 2 * (a_part & 1) + e;
            const uint4 v = a_reg[e];
            *(uint4*)(base + ((size_t)((sub * F_MB + mb) * 64 + c * 16 + i) << 4)) =
                make_uint4(perm(v.z, v.x, 0x05040100u), perm(v.z, v.x, 0x07060302u), perm(v.w, v.y, 0x05040100u),
                           perm(v.w, v.y, 0x07060302u));
        }
    };

    v4f acc[2 * NB][4];
#pragma unroll
    for (int mb = 0; mb < 2 * NB; mb++)
#pragma unroll
        for (int t = 0; t < 4; t++) acc[mb][t] = v4f{0.f, 0.f, 0.f, 0.f};

    // ---- main loop (see the int8 kernel: same pipeline) ------------------------------------
    // Stage s is computed from LDS buffer s%2.  On entry the wave holds the decoded weights of
    // stage s and the activation fragments of row blocks 0..3; it writes its piece of stage s+1
    // into the other buffer, reloads those registers with stage s+3, requests row blocks 4..7,
    // and issues the MFMAs of row blocks 0..3 with the decode of stage s+1 sliced in behind
    // them; the stage's one barrier publishes buffer (s+1)%2, whose row blocks 0..3 are
    // requested right behind it and arrive under the MFMAs of row blocks 4..7.
    u32x4 b_dec[2][4];
    uint4 a_lo[NB], a_hi[NB];
    const uint32_t a_lds_off = (uint32_t)(kgrp * (F_MB * 1024)) + ((uint32_t)lane << 4);
    constexpr uint32_t LUT = (MODE == MODE_F16) ? LUT_F16_ONE : LUT_BF16_TWO;
    auto decode_col = [&](const uint32_t (&raw)[BR], int t, u32x4& out) {
        if constexpr (WT) {
            out = decode8_16bit<LUT>(perm(0u, raw[t], sel_wt));
        } else {
            // bytes [zero, row0.byte t, zero, row1.byte t]
            const uint32_t sel = ((uint32_t)(4 + t) << 24) | (0x0Cu << 16) | ((uint32_t)t << 8) | 0x0Cu;
            out = decode8_16bit<LUT>(perm(raw[1], raw[0], sel));
        }
    };
    auto read_a = [&](int buf, int mb0, uint4 (&dst)[NB]) {
        const uint8_t* a_lds = lds + buf * F_STAGE_BYTES + a_lds_off;
        // in this order, one by one: LDS returns in order, and the first MFMA of a run needs the first row block only
#pragma unroll
        for (int i = 0; i < NB; i++) {
            dst[i] = *(const uint4*)(a_lds + (mb0 + i) * 1024);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto mfma = [&](const uint4& av, const u32x4& bv, v4f& c) {
        const u32x4 a = {av.x, av.y, av.z, av.w};
        if constexpr (MODE == MODE_F16)
            c = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, bv), c, 0, 0, 0);
        else
            c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, bv), c, 0, 0, 0);
    };

    load_stage(0, 3, a_set[0], b_set[0]);
    load_stage(1, 3, a_set[1], b_set[1]);
    store_a(0, a_set[0]);
#pragma unroll
    for (int t = 0; t < 4; t++) decode_col(b_set[0], t, b_dec[0][t]);
    load_stage(2, 3, a_set[0], b_set[0]);
    __syncthreads();
    read_a(0, 0, a_lo);

    auto stage = [&](int s, uint4 (&a_reg)[2], uint32_t (&b_reg)[BR], const u32x4 (&b_cur)[4], u32x4 (&b_nxt)[4]) {
        // a_reg / b_reg hold stage s+1 on entry and are reloaded with stage s+3
        const int cur = s & 1;
        store_a(cur ^ 1, a_reg);
        load_stage(s + 3, 1, a_reg, b_reg);
        read_a(cur, NB, a_hi);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < 4 * NB; c++) {
            mfma(a_lo[c >> 2], b_cur[c & 3], acc[c >> 2][c & 3]);
            if (c % NB == (NB > 1 ? 1 : 0)) decode_col(b_reg, c / NB, b_nxt[c / NB]);  // one column behind every fourth MFMA (NB = 4)
            __builtin_amdgcn_sched_barrier(0);
        }
        // the raw weights are dead now: their registers take the loads of stage s+3 directly
        load_stage(s + 3, 2, a_reg, b_reg);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        read_a(cur ^ 1, 0, a_lo);
#pragma unroll
        for (int c = 0; c < 4 * NB; c++) mfma(a_hi[c >> 2], b_cur[c & 3], acc[NB + (c >> 2)][c & 3]);
        __builtin_amdgcn_sched_barrier(0);
        // the fragments requested for the next stage arrived during these MFMAs: saying so here (lgkmcnt(0) alone) is free,
        // and keeps the compiler's wait for everything outstanding across the loop edge away from the next stage's first MFMA
        __builtin_amdgcn_s_waitcnt(0xC07F);
        __builtin_amdgcn_sched_barrier(0);
    };
    // The two waves that share a SIMD (the K halves of one column quarter) run the stage in different orders, so
    // that one of them is inside a run of MFMAs while the other stages, loads and reads LDS: K half 1 reads all
    // eight row blocks of stage s right behind the barrier that published them, does both MFMA halves in a row and
    // arrives at the next barrier with stage s finished; K half 0 (above) has its second half beyond the barrier.
    auto stage_y = [&](int s, uint4 (&a_reg)[2], uint32_t (&b_reg)[BR], const u32x4 (&b_cur)[4], u32x4 (&b_nxt)[4]) {
        const int cur = s & 1;
        read_a(cur, 0, a_lo);
        read_a(cur, NB, a_hi);
        store_a(cur ^ 1, a_reg);
        load_stage(s + 3, 1, a_reg, b_reg);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < 4 * NB; c++) {
            mfma(a_lo[c >> 2], b_cur[c & 3], acc[c >> 2][c & 3]);
            if (c % NB == (NB > 1 ? 1 : 0)) decode_col(b_reg, c / NB, b_nxt[c / NB]);
            __builtin_amdgcn_sched_barrier(0);
        }
        load_stage(s + 3, 2, a_reg, b_reg);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < 4 * NB; c++) mfma(a_hi[c >> 2], b_cur[c & 3], acc[NB + (c >> 2)][c & 3]);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
    };
    // (an odd last stage is peeled so that both paths into the loop header leave the same
    // loads outstanding)
    int s = 0;
    if (kgrp == 0) {  // wave-uniform
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
    // ---- add the two K halves through the stage buffers (64 KiB; word (q, wn, lane) is register q of that lane): K half 1
    // hands over row blocks 0..3 and finishes 4..7, K half 0 the other way round.  K half 1 leaves the loop half a stage
    // ahead and writes its share while K half 0 runs its last MFMAs (nobody reads live data from the buffers any more:
    // K half 0 holds the fragments of those MFMAs in registers); behind the barrier K half 0 takes that share and puts
    // its own into the slots it has just read (the LDS operations of a wave execute in order); one more barrier and
    // K half 1 takes it.  (a + b == b + a in floating point: same bits whichever half adds.) ----
    float* xch = (float*)lds;
    const int slot = wn * 64 + lane;
    auto give = [&](int mb0) {
#pragma unroll
        for (int mb = 0; mb < NB; mb++)
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const v4f v = acc[mb0 + mb][t];
                *(float4*)(xch + ((mb * 4 + t) * 256 + slot) * 4) = make_float4(v[0], v[1], v[2], v[3]);
            }
    };
    auto take = [&](int mb0) {
#pragma unroll
        for (int mb = 0; mb < NB; mb++)
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const float4 v = *(const float4*)(xch + ((mb * 4 + t) * 256 + slot) * 4);
                acc[mb0 + mb][t] += v4f{v.x, v.y, v.z, v.w};
            }
    };
    if (kgrp == 1) give(0);  // wave-uniform branches
    __syncthreads();

    // column scales and biases (raw bits) requested ahead of the rest of the hand-over, which covers their latency
    uint32_t ws_bits[4], bs_bits[4];
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const int64_t n = col_ok ? ncol + t : 0;
        ws_bits[t] = load_bits_rt(p.epi.scale, p.epi.scale_dtype, p.epi.scale_bcast ? 0 : n);
        bs_bits[t] = p.epi.bias ? load_bits_rt(p.epi.bias, p.epi.bias_dtype, n) : 0u;
    }

    // the residual of a full tile's 16-bit output: all 16 rows of the lane at once, under the rest of the hand-over
    uint2 res_pre[NB][4] = {};
    const bool res_here = p.epi.residual && p.y_dtype != BT_F32 && m0 + BM <= p.M;  // uniform
    if (res_here && col_ok) {
        const uint16_t* rb = (const uint16_t*)p.epi.residual + (m0 + 16 * (NB * kgrp) + 4 * g) * p.N + ncol;
#pragma unroll
        for (int mbi = 0; mbi < NB; mbi++)
#pragma unroll
            for (int r = 0; r < 4; r++) res_pre[mbi][r] = *(const uint2*)(rb + (int64_t)(16 * mbi + r) * p.N);
    }

    if (kgrp == 0) {
        take(0);
        give(NB);
    }
    __syncthreads();
    if (kgrp == 1) take(NB);

    if (!col_ok) return;
    if (kgrp == 0) gemm_f_epilogue_dt<MODE, 0, NB>(p, acc, m0, g, ncol, ws_bits, bs_bits, res_pre, res_here);  // wave-uniform branch
    else gemm_f_epilogue_dt<MODE, NB, NB>(p, acc, m0, g, ncol, ws_bits, bs_bits, res_pre, res_here);
}

// the tiled kernel reads X with 16-byte loads and W_T / Y with 4-column vectors
// the same kernel on the decode-tiled weight copy (256-byte aligned, below 4 GiB: checked by the caller)
bool gemm_f16_supported_tiled(int64_t N, int64_t K, const void* X, const void* Y) {
    return N % 4 == 0 && K % 8 == 0 && K >= 8 && ((uintptr_t)X) % 16 == 0 && ((uintptr_t)Y) % 16 == 0 &&
           (F_BM + 1) * K * 2 < (1ll << 32);
}

bool gemm_f16_supported(int64_t N, int64_t K, const void* X, const void* W_T, const void* Y) {
    return N % 4 == 0 && K % 8 == 0 && K >= 8 && ((uintptr_t)W_T) % 4 == 0 && ((uintptr_t)X) % 16 == 0 &&
           ((uintptr_t)Y) % 16 == 0 && (F_BM + 1) * K * 2 < (1ll << 32) && ceil_div(K, 4) * N < (1ll << 32);
}

// planes = 1: X is [M, K].  planes = 3: X is [M, 3*Kp], Kp = K rounded up to 64, three zero-padded planes of K
// values per row whose products with the same weights are summed (fp32 activations split into three bf16 terms).
// With K % 64 != 0 the last weight stage of every plane runs past W_T's rows: the TAIL instantiation clamps them.
// One launch over column tiles [tile_n0, tile_n0 + tiles_n) in tiles of 32 * NB rows.
template <int NB>
static int launch_gemm_f16_part(GemmFParams p, int mode, int tile_n0, int tiles_n, bool tiled, bool tail, hipStream_t st) {
    p.tile_n0 = tile_n0;
    p.tiles_n = tiles_n;
    p.tiles_m = (int)ceil_div(p.M, 32 * NB);
    const int64_t total = (int64_t)p.tiles_m * p.tiles_n;
    if (total >= (1ll << 31) - 8) {
        set_error("gemm_f16: %lld tiles of %d x 256 outputs are more than one launch takes", (long long)total, 32 * NB);
        return BT_ERR_INVALID;
    }
    p.per_xcd = (int)ceil_div(total, 8);
    const dim3 grid((unsigned)(p.per_xcd * 8)), block(512);
    if constexpr (NB != 4) {  // (only where launch_gemm_f16 cuts finer: tiled weights, whole stages)
        if (mode == MODE_F16) hipLaunchKernelGGL((gemm_f16_kernel<MODE_F16, false, true, NB>), grid, block, 0, st, p);
        else hipLaunchKernelGGL((gemm_f16_kernel<MODE_BF16, false, true, NB>), grid, block, 0, st, p);
        return check_launch("bt_ternary_linear_tiled_forward");
    } else if (tiled) {
        if (mode == MODE_F16) {
            if (tail) hipLaunchKernelGGL((gemm_f16_kernel<MODE_F16, true, true>), grid, block, 0, st, p);
            else hipLaunchKernelGGL((gemm_f16_kernel<MODE_F16, false, true>), grid, block, 0, st, p);
        } else {
            if (tail) hipLaunchKernelGGL((gemm_f16_kernel<MODE_BF16, true, true>), grid, block, 0, st, p);
            else hipLaunchKernelGGL((gemm_f16_kernel<MODE_BF16, false, true>), grid, block, 0, st, p);
        }
        return check_launch("bt_ternary_linear_tiled_forward");
    }
    if (mode == MODE_F16) {
        if (tail) hipLaunchKernelGGL((gemm_f16_kernel<MODE_F16, true>), grid, block, 0, st, p);
        else hipLaunchKernelGGL((gemm_f16_kernel<MODE_F16, false>), grid, block, 0, st, p);
    } else {
        if (tail) hipLaunchKernelGGL((gemm_f16_kernel<MODE_BF16, true>), grid, block, 0, st, p);
        else hipLaunchKernelGGL((gemm_f16_kernel<MODE_BF16, false>), grid, block, 0, st, p);
    }
    return check_launch("bt_ternary_linear_packed_forward");
}

int launch_gemm_f16(int mode, const void* X, const uint8_t* W_T, int w_layout, const Epilogue& epi, void* Y, int y_dtype,
                    int64_t M, int64_t N, int64_t K, int planes, hipStream_t st) {
    GemmFParams p = {};
    p.X = (const uint16_t*)X; p.W_T = W_T; p.Y = Y; p.epi = epi;
    p.M = M; p.N = N; p.K = (planes == 3) ? 3 * ceil_div(K, F_BK) * F_BK : K; p.Kb = ceil_div(K, 4);
    p.wstages = (int)ceil_div(K, F_BK);
    p.prehalved = planes == 3;
    p.y_dtype = y_dtype;
    p.tiles16 = tiles16_arg(N, w_layout);
    const bool tail = K % F_BK != 0, tiled = layout_tiled(w_layout);
    const int64_t tiles_n = ceil_div(N, F_BN);
    // the remainder of a launch in tiles of 64 or 32 rows, as in the int8 GEMM (gemm_split: same rule, same prices; fp32
    // sums in the same order, so the same bits)
    const GemmSplit sp = gemm_split(M, N, tiled && !tail);
    if (sp.nb != 4) {
        if (sp.cols < tiles_n) {
            const int rc = launch_gemm_f16_part<4>(p, mode, 0, (int)(tiles_n - sp.cols), tiled, tail, st);
            if (rc) return rc;
        }
        return sp.nb == 1 ? launch_gemm_f16_part<1>(p, mode, (int)(tiles_n - sp.cols), (int)sp.cols, tiled, tail, st)
                          : launch_gemm_f16_part<2>(p, mode, (int)(tiles_n - sp.cols), (int)sp.cols, tiled, tail, st);
    }
    return launch_gemm_f16_part<4>(p, mode, 0, (int)tiles_n, tiled, tail, st);
}

}  // namespace bt
