// Internal helpers shared by the gfx950 kernels of libbittorch_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include <algorithm>
#include <type_traits>

#include "../../include/bittorch_hip.h"

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

namespace bt {

// operand modes of the streaming kernel
enum { MODE_I8 = 0, MODE_F16 = 1, MODE_BF16 = 2 };

// ---- host side: error text + launch check --------------------------------
void set_error(const char* fmt, ...);
int check_launch(const char* what);

static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---- run-time options -------------------------------------------------------------------------------------------------
// The documented switches of the library.  Each is read from the environment (BITTORCH_<NAME>) once per process, on the
// first call that asks for any of them, and can be overridden afterwards with bt_set_option (tests and benchmarks choose a
// code path that way); asking for one on a call is an array lookup, not a getenv.  BITTORCH_KERNEL is not among them:
// the reference re-reads it on every call (ternary_gemm_production.cu:262-273) and so does this library.
enum Option {
    OPT_STREAM_MAX_ROWS,     // n: batches of up to n rows take the streaming kernel, larger ones the tiled GEMM
    OPT_GEMM_LONG_EPILOGUE,  // 1: the tiled int8 GEMM never takes its short epilogue
    OPT_GEMM_TAIL_SPLIT,     // 0: the remainder of a tiled GEMM launch is not cut into finer tiles
    OPT_GROUP_WALK,          // grouped GEMV: 1 / chunk / 0 force a kernel
    OPT_GROUP_NACC,          // grouped GEMV: 16-column blocks per wave of the slab kernel
    OPT_GROUP_UNITS,         // grouped GEMV: 1 forces the one-matrix kernel over (unit, tile) workgroups, 0 forbids it
    OPT_PLANES_NACC,         // exact GEMV, one matrix per launch: 16-column blocks per workgroup
    OPT_ROWOP_GENERIC,       // 1: SwiGLU / RMSNorm rows on the shape-generic kernel
    OPT_STREAM_CFG,          // "ld,waves": tile width and wave count of the streaming kernel
    OPT_NO_PLANES,           // 1: a single fp16 row takes the 16-bit streaming kernel instead of the exact GEMV
    OPT_COUNT
};
const char* option(Option o);  // the option's text, or nullptr when it is not set (capi.hip)

// A/B switches of experiment builds (-DBT_TUNING): compiled out of the product library.
#ifdef BT_TUNING
static inline const char* tuning_env(const char* name) { return getenv(name); }
#else
static inline const char* tuning_env(const char*) { return nullptr; }
#endif

// ---- the remainder of a tiled GEMM launch (gemm_i8.hip, gemm_f16.hip, and the rule that routes a batch to them) ------
// Workgroups take 128 x 256 tiles in rounds of one per compute unit.  When the last round holds tiles for at most half
// of the compute units, the column tiles of that remainder are computed in tiles of 64 or 32 rows instead (nb = 2 or 1
// row blocks per K half and wave), two or four workgroups where there was one, in a launch of their own behind the
// whole tiles.  A finer tile does fewer MFMAs per decoded weight and its stage is bound by the chain LDS read -> decode
// -> barrier, so it only pays where the alternative is idle compute units.  Prices in rounds of whole tiles, as measured
// (int8; M = 4096, N = 2560: K = 2560 36.5 -> 32.8 us, K = 6912 74.9 -> 67.3 us; N = K = 4096: M = 1024 23.9 -> 19.8 us,
// M = 512 23.5 -> 15.6 us): a round of half tiles 0.85, of quarter tiles 0.75, the second launch 0.1.
struct GemmSplit {
    int nb;          // 4: no finer tiles
    int64_t cols;    // column tiles (of 256) cut finer, the last ones of the matrix
    double rounds;   // price of the launch(es) in rounds of whole tiles
};
static inline int64_t gemm_compute_units() {  // of the current device (asked once per process)
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
// allowed: the caller's kernel has finer tiles for this call (decode-tiled weights, K in whole stages);
// option GEMM_TAIL_SPLIT = 0 (tests, A/B runs): never.
static inline GemmSplit gemm_split(int64_t M, int64_t N, bool allowed) {
    const int64_t C = gemm_compute_units();
    const int64_t tiles_m = ceil_div(M, 128), tiles_n = ceil_div(N, 256), total = tiles_m * tiles_n;
    GemmSplit r = {4, 0, (double)ceil_div(total, C)};
    const char* env = option(OPT_GEMM_TAIL_SPLIT);
    if (!allowed || (env && env[0] == '0')) return r;
    const int64_t rem = total % C;
    if (rem == 0 || 2 * rem > C) return r;
    const int nb = (4 * rem <= C) ? 1 : 2;
    const int64_t cols = std::min(tiles_n, ceil_div(rem, tiles_m));
    const int64_t whole = tiles_m * (tiles_n - cols), fine = ceil_div(M, 32 * nb) * cols;
    const double split = (double)ceil_div(whole, C) + (double)ceil_div(fine, C) * (nb == 1 ? 0.75 : 0.85) + (whole ? 0.1 : 0.0);
    if (split < r.rounds - 0.04) r = {nb, cols, split};
    return r;
}

// ---- element access by dtype tag (BT_F32 / BT_F16 / BT_BF16) --------------
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) {
    return __builtin_bit_cast(float, (uint32_t)h << 16);
}
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    return __builtin_bit_cast(uint16_t, (__bf16)f);  // v_cvt_pk_bf16_f32, RNE
}
__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
    return (float)__builtin_bit_cast(_Float16, h);
}
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
    // The empty asm keeps the conversion a conversion of the fp32 value: without it the compiler
    // folds "(half)(a * b + c)" into v_fma_mixlo_f16, which rounds the exact result once, where
    // the reference (and the CPU restatement) round to fp32 first and to fp16 second.
    asm("" : "+v"(f));
    return __builtin_bit_cast(uint16_t, (_Float16)f);  // v_cvt_f16_f32, RNE
}

template <int DT>
__device__ __forceinline__ float load_elem(const void* p, int64_t i) {
    if constexpr (DT == BT_F32) return ((const float*)p)[i];
    else if constexpr (DT == BT_F16) return f16_bits_to_f32(((const uint16_t*)p)[i]);
    else if constexpr (DT == BT_I8) return (float)((const int8_t*)p)[i];
    else return bf16_bits_to_f32(((const uint16_t*)p)[i]);
}
template <int DT>
__device__ __forceinline__ void store_elem(void* p, int64_t i, float v) {
    if constexpr (DT == BT_F32) ((float*)p)[i] = v;
    else if constexpr (DT == BT_F16) ((uint16_t*)p)[i] = f32_to_f16_bits(v);
    else ((uint16_t*)p)[i] = f32_to_bf16_bits(v);
}
// run-time dtype (scale / bias vectors: a handful of loads per thread)
__device__ __forceinline__ float load_elem_rt(const void* p, int dt, int64_t i) {
    if (dt == BT_F32) return ((const float*)p)[i];
    if (dt == BT_F16) return f16_bits_to_f32(((const uint16_t*)p)[i]);
    return bf16_bits_to_f32(((const uint16_t*)p)[i]);
}
// The same in two halves, so that a caller can issue the load early and convert late:
// the load leaves raw bits in a register (no use, hence no wait, inside the dtype branch).
__device__ __forceinline__ uint32_t load_bits_rt(const void* p, int dt, int64_t i) {
    if (dt == BT_F32) return ((const uint32_t*)p)[i];
    return (uint32_t)((const uint16_t*)p)[i];
}
__device__ __forceinline__ float bits_to_f32_rt(uint32_t bits, int dt) {
    if (dt == BT_F32) return __builtin_bit_cast(float, bits);
    if (dt == BT_F16) return f16_bits_to_f32((uint16_t)bits);
    return bf16_bits_to_f32((uint16_t)bits);
}
// round a float to the grid of dtype dt and widen it again
__device__ __forceinline__ float round_to_dtype(float v, int dt) {
    if (dt == BT_F16) return f16_bits_to_f32(f32_to_f16_bits(v));
    if (dt == BT_BF16) return bf16_bits_to_f32(f32_to_bf16_bits(v));
    return v;
}
static inline int dtype_size(int dt) { return dt == BT_F32 ? 4 : 2; }

// Epilogue operand bundle (scale / bias vectors and their element types).
struct Epilogue {
    const void* scale;
    const void* bias;  // may be null
    int scale_dtype;
    int bias_dtype;
    int scale_bcast;  // 1: scale has one entry that applies to every column
    const void* residual;  // optional [B, N] in the output's dtype, added to the finished output
};
__device__ __forceinline__ float epi_scale(const Epilogue& e, int64_t n) {
    return load_elem_rt(e.scale, e.scale_dtype, e.scale_bcast ? 0 : n);
}
__device__ __forceinline__ float epi_bias(const Epilogue& e, int64_t n) {
    return e.bias ? load_elem_rt(e.bias, e.bias_dtype, n) : 0.0f;
}
// Residual connection folded into the epilogue: y is first rounded to the output dtype, then the
// residual is added in fp32 and the sum rounded again by the store -- the two roundings of an
// unfused "linear, then add" in that dtype, so fusing does not change a bit.  (The fp32 sum of two
// 16-bit values is exact unless their exponents are more than 13 apart, and then the smaller one
// cannot move the larger across a rounding boundary: rounding the fp32 sum equals rounding the
// exact sum.)
__device__ __forceinline__ float sum_in_dtype(float y_rounded, float r, int dt) {
    (void)dt;
    return __fadd_rn(y_rounded, r);
}
__device__ __forceinline__ float add_residual(float y, const void* res, int dt, int64_t idx) {
    return sum_in_dtype(round_to_dtype(y, dt), load_elem_rt(res, dt, idx), dt);
}
// four consecutive outputs (idx % 4 == 0, residual 16-byte aligned for fp32, 8-byte for 16-bit)
__device__ __forceinline__ void add_residual4(float (&y)[4], const void* res, int dt, int64_t idx) {
    float r[4];
    if (dt == BT_F32) {
        const float4 v = *(const float4*)((const float*)res + idx);
        r[0] = v.x; r[1] = v.y; r[2] = v.z; r[3] = v.w;
    } else {
        const uint2 v = *(const uint2*)((const uint16_t*)res + idx);
        const uint32_t d[2] = {v.x, v.y};
#pragma unroll
        for (int i = 0; i < 4; i++) r[i] = bits_to_f32_rt((d[i >> 1] >> (16 * (i & 1))) & 0xffffu, dt);
    }
#pragma unroll
    for (int i = 0; i < 4; i++) y[i] = sum_in_dtype(round_to_dtype(y[i], dt), r[i], dt);
}
// fp32 accumulate path: one multiply, one add, each rounded (no fma contraction)
__device__ __forceinline__ float epi_float(float acc, float s, float b) {
    return __fadd_rn(__fmul_rn(acc, s), b);
}
// x / 127.0f, correctly rounded, in three operations: q0 = x * RN(1/127), one fused
// residual and one fused correction.  Checked exhaustively against IEEE division for
// every finite fp32 x; the only difference is the sign of the result for x = -0.0,
// which the int8 epilogue cannot produce (float(int) * positive scale is never -0).
__device__ __forceinline__ float div127(float x) {
    const float y = 1.0f / 127.0f;
    const float q0 = x * y;
    const float r = __builtin_fmaf(-127.0f, q0, x);
    return __builtin_fmaf(r, y, q0);
}
// x / 127.0f in two operations: x * zh + RN(x * zl) with zh + zl = 1/127 to 48 bits, one fused multiply-add.
// Checked exhaustively against IEEE division for every finite fp32 x: correctly rounded except for
// 2^-122 <= |x| < 2^-113, where x * zl is subnormal and loses the bits that decide the rounding.  The caller
// rules that range out (see DIV127_FAST_MIN_SX) or uses div127.
__device__ __forceinline__ float div127_fast(float x) {
    const float zh = 0x1.020408p-7f, zl = 0x1.020408p-35f;
    return __builtin_fmaf(x, zh, __fmul_rn(x, zl));
}
// The dividend of the int8 epilogue is float(127 a) * s_x with an integer a: zero, or at least 127 |s_x| (1 - 2^-24)
// in magnitude.  With |s_x| >= 2^-119 it is zero or above 2^-113, so div127_fast is exact for it.
constexpr float DIV127_FAST_MIN_SX = 0x1p-119f;
// int8 path: ((float(acc) * s_x) / 127) * w_scale + bias, left to right
__device__ __forceinline__ float epi_int8_f(float acc127, float sx, float ws, float b) {
    float r = __fmul_rn(acc127, sx);
    r = div127(r);
    r = __fmul_rn(r, ws);
    return __fadd_rn(r, b);
}
__device__ __forceinline__ float epi_int8(int32_t acc127, float sx, float ws, float b) {
    return epi_int8_f((float)acc127, sx, ws, b);
}
// 127 * a without the quarter-rate 32-bit multiply
__device__ __forceinline__ int32_t times127(int32_t a) { return (int32_t)(((uint32_t)a << 7) - (uint32_t)a); }

// Packed weights are read once per call: the loads carry the non-temporal hint, which keeps the stream out of
// the way of the cached operands and, measured on this chip, raises the read rate of a pure stream from 6.1 to
// 6.9 TB/s.
__device__ __forceinline__ uint32_t ldw_nt(const void* p) {
#ifdef BT_NO_NT
    return *(const uint32_t*)p;
#else
    return __builtin_nontemporal_load((const uint32_t*)p);
#endif
}
__device__ __forceinline__ uint2 ldw2_nt(const void* p) {
#ifdef BT_NO_NT
    return *(const uint2*)p;
#else
    typedef uint32_t u32x2_nt __attribute__((ext_vector_type(2)));
    const u32x2_nt v = __builtin_nontemporal_load((const u32x2_nt*)p);
    return make_uint2(v[0], v[1]);
#endif
}
__device__ __forceinline__ uint4 ldw4_nt(const void* p) {
#ifdef BT_NO_NT
    return *(const uint4*)p;
#else
    typedef uint32_t u32x4_nt __attribute__((ext_vector_type(4)));
    const u32x4_nt v = __builtin_nontemporal_load((const u32x4_nt*)p);
    return make_uint4(v[0], v[1], v[2], v[3]);
#endif
}

// Outputs of the tall GEMMs (16 MiB and more per launch) leave with the non-temporal hint: written through as they are
// produced instead of sitting dirty in the XCD's L2 until the end-of-kernel write-back (2048 x 4096 x 4096 int8 GEMM:
// 30.3 -> 28.7 us in same-run A/Bs).
__device__ __forceinline__ void st2_nt(void* p, uint32_t a, uint32_t b) {
    typedef uint32_t u32x2_st __attribute__((ext_vector_type(2)));
    u32x2_st o;
    o[0] = a; o[1] = b;
    __builtin_nontemporal_store(o, (u32x2_st*)p);
}
__device__ __forceinline__ void st4_nt(void* p, uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    typedef uint32_t u32x4_st __attribute__((ext_vector_type(4)));
    u32x4_st o;
    o[0] = a; o[1] = b; o[2] = c; o[3] = d;
    __builtin_nontemporal_store(o, (u32x4_st*)p);
}

// ---- 2-bit decode in registers -------------------------------------------
// v_perm_b32: result byte i = byte sel[i] of the 8-byte value {hi,lo}
// (0..3 -> lo, 4..7 -> hi); sel 8 -> 0xFF if bit 15 of lo is set else 0x00;
// sel 12 -> 0x00.
__device__ __forceinline__ uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel) {
    return __builtin_amdgcn_perm(hi, lo, sel);
}

// g[i] = { r0.byte[i], r1.byte[i], r2.byte[i], r3.byte[i] }  (byte 0 first)
__device__ __forceinline__ void transpose4x4_bytes(uint32_t r0, uint32_t r1, uint32_t r2,
                                                   uint32_t r3, uint32_t (&g)[4]) {
    const uint32_t a_lo = perm(r1, r0, 0x05010400u);  // r0.b0 r1.b0 r0.b1 r1.b1
    const uint32_t a_hi = perm(r1, r0, 0x07030602u);  // r0.b2 r1.b2 r0.b3 r1.b3
    const uint32_t b_lo = perm(r3, r2, 0x05010400u);
    const uint32_t b_hi = perm(r3, r2, 0x07030602u);
    g[0] = perm(b_lo, a_lo, 0x05040100u);
    g[1] = perm(b_lo, a_lo, 0x07060302u);
    g[2] = perm(b_hi, a_hi, 0x05040100u);
    g[3] = perm(b_hi, a_hi, 0x07060302u);
}

// G holds four packed bytes (four consecutive kb rows of one output column).
// Returns 16 int8 weights in {-1,0,+1}: dword c, byte r = weight (row r, slot c),
// i.e. k = 4*(kb0 + r) + c.  Codes: 1 -> +1, 2 -> -1, 0 and 3 -> 0.
// Slots 0 and 2 index a 4-entry byte table with the code itself; slots 1 and 3
// use the code still shifted left by two (0,4,8,12) as the selector, which the
// table {lo.byte0 = 0, hi.byte0 = +1, "8" = 0xFF via lo bit 15, "12" = 0} decodes
// without a shift.
__device__ __forceinline__ v4i decode16_i8(uint32_t G) {
    const uint32_t lutA_lo = 0x00FF0100u;  // sel 0..3 -> 0, +1, -1, 0
    const uint32_t lutB_lo = 0x0000FF00u;  // byte0 = 0 (sel 0); bit 15 set (sel 8 -> 0xFF)
    const uint32_t lutB_hi = 0x00000001u;  // sel 4 -> +1
    const uint32_t H = G >> 4;
    v4i out;
    out[0] = (int)perm(0u, lutA_lo, G & 0x03030303u);
    out[1] = (int)perm(lutB_hi, lutB_lo, G & 0x0C0C0C0Cu);
    out[2] = (int)perm(0u, lutA_lo, H & 0x03030303u);
    out[3] = (int)perm(lutB_hi, lutB_lo, H & 0x0C0C0C0Cu);
    return out;
}

// M.byte1 / M.byte3 hold the packed bytes of two consecutive kb rows of one
// output column.  Returns eight 16-bit floats: dword c = { w(row0, slot c),
// w(row1, slot c) }, where the non-zero weights have high byte HI_POS / HI_NEG
// and low byte 0 (fp16: +-1.0 = 0x3C00 / 0xBC00; bf16: +-2.0 = 0x4000 / 0xC000).
template <uint32_t LUT>
__device__ __forceinline__ u32x4 decode8_16bit(uint32_t M) {
    u32x4 out;
    out[0] = perm(0u, LUT, M & 0x03000300u);
    out[1] = perm(0u, LUT, (M >> 2) & 0x03000300u);
    out[2] = perm(0u, LUT, (M >> 4) & 0x03000300u);
    out[3] = perm(0u, LUT, (M >> 6) & 0x03000300u);
    return out;
}
constexpr uint32_t LUT_F16_ONE = 0x00BC3C00u;   // sel 0..3 -> 0x00, 0x3C, 0xBC, 0x00
constexpr uint32_t LUT_BF16_TWO = 0x00C04000u;  // sel 0..3 -> 0x00, 0x40, 0xC0, 0x00

// ---- layout of quantized activations ----------------------------------------
// Q_ROW_MAJOR: int8 [B, K] as is.  Q_OPERAND_ORDER (K % 16 == 0): the same rows, but every aligned
// 16-byte group stored as the 4x4 byte transpose of its natural order (byte 4c+r holds element
// 4r+c): the k order in which the in-register weight decode lays out an MFMA operand, so that the
// GEMMs feed activations to the matrix cores without permuting them first.
// roundf (halves away from zero) in three operations: add the largest float below one half, with the sign of
// x, and truncate.  Exact for every float: below 2^23 the sum rounds to the next integer precisely when the
// fraction is at least one half (x + 0.5 - 2^-25 lies at most half a grid step below that integer, and the
// tie at 1 - 2^-25 goes to the even 1.0); from 2^23 on x is an integer and the sum is x.
__device__ __forceinline__ float round_half_away(float x) {
    return truncf(__fadd_rn(x, copysignf(0.49999997f, x)));
}

enum { Q_ROW_MAJOR = 0, Q_OPERAND_ORDER = 1 };

// Layouts of the packed weights the streaming kernel reads.
//   W_LAYOUT_ROW_MAJOR  the reference's W_T [Kb, N] (bittorch/quant/ternary_packed.py:174-206)
//   W_LAYOUT_TILED      decode-tiled copy: dword ((t * S + s) * 64 + 16 g + j), S = ceil(Kb / 16), holds
//                       the bytes W_T[16 s + 4 g + r, 16 t + j], r = 0..3 (low byte first), zero where the
//                       row or the column lies outside the matrix
//   W_LAYOUT_TILED_PAIRS_AS_NATURAL  a decode-tiled copy whose tiles are stored in gate/up pair order (tile t of the
//                       left half of the columns at 2t, tile t of the right half at 2t + 1: BT_TILES_GATE_UP_PAIRS), read
//                       by a kernel that works in the matrix's natural column order
//   W_LAYOUT_TILED_FIELDS  prefill-only variant of the decode-tiled copy (the tiled int8 GEMM alone reads it): the same
//                       position for every aligned group of four dwords -- columns 4 q .. 4 q + 3 of a tile at one
//                       16-row step and row group -- but inside the group field t (bits 2 t, 2 t + 1) of byte b of
//                       dword c holds column 4 q + t at k = 4 b + c: w + 1 for t < 3, w in two's complement for t = 3
//                       (retile_fields_kernel); _PAIRS_AS_NATURAL as above
enum { W_LAYOUT_ROW_MAJOR = 0, W_LAYOUT_TILED = 1, W_LAYOUT_TILED_PAIRS_AS_NATURAL = 2, W_LAYOUT_TILED_FIELDS = 3,
       W_LAYOUT_TILED_FIELDS_PAIRS_AS_NATURAL = 4 };
static inline bool layout_tiled(int w_layout) { return w_layout != W_LAYOUT_ROW_MAJOR; }
static inline bool layout_fields(int w_layout) {
    return w_layout == W_LAYOUT_TILED_FIELDS || w_layout == W_LAYOUT_TILED_FIELDS_PAIRS_AS_NATURAL;
}
// The kernels' `tiles16` argument: the number of 16-column tiles, negative for W_LAYOUT_TILED_PAIRS_AS_NATURAL.
static inline int tiles16_arg(int64_t N, int w_layout) {
    const int t = (int)ceil_div(N, 16);
    return (w_layout == W_LAYOUT_TILED_PAIRS_AS_NATURAL || w_layout == W_LAYOUT_TILED_FIELDS_PAIRS_AS_NATURAL) ? -t : t;
}
// Where 16-column tile t of the matrix (natural column order) sits in the copy; a tile past the end repeats the last
// one (it only feeds outputs that are never stored).
__device__ __forceinline__ int stored_tile16(int t, int tiles16) {
    if (tiles16 >= 0) return min(t, tiles16 - 1);
    const int n = -tiles16, half = n >> 1;
    t = min(t, n - 1);
    return t < half ? 2 * t : 2 * (t - half) + 1;
}

// activation prologues and output stages of the streaming kernel (BT_PRO_*, BT_EPI_* of the C ABI)
enum { PRO_NONE = 0, PRO_RMSNORM = 1, PRO_SWIGLU = 2 };
enum { EPI_NONE = 0, EPI_SWIGLU_PAIRS = 1, EPI_NATURAL_FROM_PAIRS = 2 /* at the C ABI only: becomes a weight layout */ };

// Two neighbouring lanes hold the 16 quantized bytes of one group (even lane: elements 0..7 as
// lo, hi; odd lane: elements 8..15).  Returns this lane's 8 bytes of the transposed group.
// Both lanes of a pair must call it (it exchanges registers between them).
__device__ __forceinline__ uint2 q_to_operand_order(uint32_t lo, uint32_t hi, int lane_parity) {
    // the neighbour's two dwords through a DPP quad permute [1,0,3,2] (no LDS round trip)
    const uint32_t plo = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)lo, 0xB1, 0xf, 0xf, true);
    const uint32_t phi = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)hi, 0xB1, 0xf, 0xf, true);
    // rows r0..r3 of the 4x4 byte block = elements 0-3, 4-7, 8-11, 12-15
    const bool odd = lane_parity != 0;
    const uint32_t r0 = odd ? plo : lo, r1 = odd ? phi : hi, r2 = odd ? lo : plo, r3 = odd ? hi : phi;
    // the even lane keeps columns 0,1 of the block (transposed rows 0,1), the odd lane columns 2,3
    const uint32_t sel = odd ? 0x07030602u : 0x05010400u;
    const uint32_t ta = perm(r1, r0, sel), tb = perm(r3, r2, sel);
    return make_uint2(perm(tb, ta, 0x05040100u), perm(tb, ta, 0x07060302u));
}
// position of element k of a row in the operand-order layout
__device__ __forceinline__ int64_t q_operand_order_pos(int64_t k) {
    return (k & ~(int64_t)15) | ((k & 3) << 2) | ((k >> 2) & 3);
}

__device__ __forceinline__ int decode2(uint32_t code) { return (int)(code == 1u) - (int)(code == 2u); }

// ---- wave64 reductions ------------------------------------------------------
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}
__device__ __forceinline__ int wave_sum_i32(int v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

}  // namespace bt
