/*
 * CPU oracle for the ternary-linear hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain scalar C, the arithmetic of the reference
 * implementation so that the HIP kernels can be diffed against it.  It is
 * never linked into, imported by or called from the shipped package; only the
 * tests, the smoke check and the benchmark's cpu_baseline leg may use it.
 *
 * Every function names the reference lines it follows (paths relative to the
 * reference checkout).  Parity status of each function:
 *
 *   bto_quantize        pinned   (reference-held known answers, torch CPU ops
 *                                 executing the same formula, brute force)
 *   bto_pack / unpack   pinned   (reference-held byte known answers 0x49, 85,
 *                                 170, 0; round trip; K%4 != 0 padding)
 *   bto_linear_packed   pinned   (textbook x @ (w*s).T + b in float64, all-zero
 *                                 and all-ones weights, the reference's JS
 *                                 known-answer vectors)
 *   bto_linear_unpacked pinned   (same checks as bto_linear_packed)
 *   bto_linear_packed_exact_f16  pinned (the same linear with the sum formed exactly and
 *                                 rounded once: float64 dot product, exact for fp16
 *                                 operands, rounded to fp32; ties and subnormals)
 *   bto_linear_packed_rowscaled_bf16  this library's own arithmetic for bf16 rows (the
 *                                 reference's packed kernel takes fp16 / fp32): pinned by
 *                                 the float64 dot product rounded once to fp32 wherever
 *                                 the row spans at most 32 binades (then the scaling is
 *                                 exact), by hand-made rows that exercise the half-up
 *                                 rounding and the flush of far smaller elements, and by
 *                                 the NaN / Inf rule
 *   bto_act_quant_i8    parity unpinned by the reference (no reference test
 *   bto_gemm_i8         touches the int8 path); pinned here only by brute
 *                       force on tiny inputs, exact integer identities and
 *                       agreement with the float path inside the int8
 *                       quantisation error bound.
 *   bto_swiglu          no counterpart in the reference's Python/CUDA code (the
 *   bto_rmsnorm         block glue lives in its JS runtime, in float64 maths):
 *   bto_exp_fixed       these restate THIS library's fused row operations so
 *                       that the kernels can be diffed bit for bit; pinned by
 *                       float64 closed forms (silu, exp, rms) to a stated
 *                       tolerance and by torch's own ops in the tests.
 *
 * Build: gcc -O2 -fPIC -shared -ffp-contract=off -fopenmp (see Makefile).
 * -ffp-contract=off keeps every multiply and add separately rounded, which is
 * what the comments below mean by "one fp32 multiply, then one fp32 add".
 */
#include <math.h>
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#include <stdlib.h>

/* dtype tags shared with include/bittorch_hip.h */
enum { BTO_F32 = 0, BTO_F16 = 1, BTO_BF16 = 2 };

/* ---- rounding helpers: float -> (fp16|bf16) -> float, round-nearest-even -- */

static float round_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return f; /* NaN */
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    u &= 0xffff0000u;
    memcpy(&f, &u, 4);
    return f;
}

static float round_to_f16(float f) {
    /* IEEE binary16 round-to-nearest-even, done by hand (no _Float16 in gcc 11/x86):
     * scale into the half grid with exact power-of-two multiplies so that the
     * fp32 adder performs the rounding, including the subnormal range. */
    if (!(fabsf(f) <= 3.4e38f)) return f;          /* NaN / Inf pass through */
    if (fabsf(f) >= 65520.0f) return copysignf(INFINITY, f);
    float a = fabsf(f);
    float r;
    if (a < 6.103515625e-05f) {
        /* subnormal half: multiples of 2^-24 */
        const float magic = 12582912.0f; /* 1.5 * 2^23: adds round to integer, RNE */
        float t = a * 16777216.0f;       /* / 2^-24, exact */
        t = (t + magic) - magic;
        r = t * 5.9604644775390625e-08f; /* * 2^-24, exact */
    } else {
        /* normal half: keep 11 significant bits */
        uint32_t u;
        memcpy(&u, &a, 4);
        uint32_t lsb = (u >> 13) & 1u;
        u += 0xfffu + lsb;
        u &= 0xffffe000u;
        memcpy(&r, &u, 4);
    }
    return copysignf(r, f);
}

static float round_to_dtype(float f, int dtype) {
    if (dtype == BTO_F16) return round_to_f16(f);
    if (dtype == BTO_BF16) return round_to_bf16(f);
    return f;
}

/* threads the OpenMP loops below will use (reported with the CPU baseline) */
#ifdef _OPENMP
#include <omp.h>
int bto_num_threads(void) { return omp_get_max_threads(); }
#else
int bto_num_threads(void) { return 1; }
#endif

/* exported so tests can check the helpers against torch's casts */
float bto_round_to_dtype(float f, int dtype) { return round_to_dtype(f, dtype); }

/*
 * Ternary quantizer.  Follows bittorch/quant/ternary.py:100-150.
 *
 *   per_channel: scale[n] = max_k |W[n,k]|, clamped below at 1e-8   (:122-127)
 *   per tensor : scale    = max_{n,k} |W[n,k]|, clamped             (:130-131)
 *   threshold  = threshold_factor * scale                            (:134)
 *   w_tern     = sign(W) where |W| > threshold (strict), else 0     (:137-142)
 *
 * W holds the master weights already widened to float; `dtype` says which
 * type the reference tensor had, because torch evaluates `0.05 * scale` and
 * the clamp in float and then rounds the result back to that type.  The
 * Python scalar threshold_factor reaches the multiply as a float
 * (`(float)0.05`), so the threshold is fl(tf_f32 * scale) rounded to dtype.
 *
 * scale has N entries (per_channel) or 1 entry.  w_tern may be NULL.
 */
void bto_quantize(const float* W, int64_t N, int64_t K, double threshold_factor,
                  int per_channel, int dtype, int8_t* w_tern, float* scale) {
    const float tf = (float)threshold_factor;
    const float clamp_min = round_to_dtype(1e-8f, dtype);
    float gmax = 0.0f;
    if (!per_channel) {
        for (int64_t i = 0; i < N * K; i++) {
            float a = fabsf(W[i]);
            if (a > gmax) gmax = a;
        }
        if (gmax < clamp_min) gmax = clamp_min;
        scale[0] = gmax;
    }
    for (int64_t n = 0; n < N; n++) {
        const float* row = W + n * K;
        float s;
        if (per_channel) {
            s = 0.0f;
            for (int64_t k = 0; k < K; k++) {
                float a = fabsf(row[k]);
                if (a > s) s = a;
            }
            if (s < clamp_min) s = clamp_min;
            scale[n] = s;
        } else {
            s = gmax;
        }
        const float thr = round_to_dtype(tf * s, dtype);
        if (w_tern) {
            for (int64_t k = 0; k < K; k++) {
                float w = row[k];
                int8_t t = 0;
                if (fabsf(w) > thr) t = (w > 0.0f) ? 1 : -1;
                w_tern[n * K + k] = t;
            }
        }
    }
}

/*
 * 2-bit codec.  Follows bittorch/quant/ternary_packed.py:22-75.
 *   code: +1 -> 1, -1 -> 2, 0 -> 0                                   (:59-61)
 *   byte = c0 | c1<<2 | c2<<4 | c3<<6, c_i = element k = 4*kb + i    (:68-73)
 *   K is zero-padded up to a multiple of four                        (:51-55)
 * packed is [N, Kb] row-major, Kb = ceil(K/4).
 */
void bto_pack(const int8_t* w_tern, int64_t N, int64_t K, uint8_t* packed) {
    const int64_t Kb = (K + 3) / 4;
    for (int64_t n = 0; n < N; n++) {
        for (int64_t kb = 0; kb < Kb; kb++) {
            unsigned byte = 0;
            for (int i = 0; i < 4; i++) {
                int64_t k = 4 * kb + i;
                int8_t w = (k < K) ? w_tern[n * K + k] : 0;
                unsigned c = (w == 1) ? 1u : (w == -1) ? 2u : 0u;
                byte |= c << (2 * i);
            }
            packed[n * Kb + kb] = (uint8_t)byte;
        }
    }
}

/*
 * Transposed layout.  Follows bittorch/quant/ternary_packed.py:174-206:
 * packed_T = pack_ternary(w).T.contiguous(), shape [Kb, N]; byte [kb, n]
 * holds W[n, 4kb .. 4kb+3].
 */
void bto_pack_transposed(const int8_t* w_tern, int64_t N, int64_t K, uint8_t* packed_T) {
    const int64_t Kb = (K + 3) / 4;
    for (int64_t n = 0; n < N; n++) {
        for (int64_t kb = 0; kb < Kb; kb++) {
            unsigned byte = 0;
            for (int i = 0; i < 4; i++) {
                int64_t k = 4 * kb + i;
                int8_t w = (k < K) ? w_tern[n * K + k] : 0;
                unsigned c = (w == 1) ? 1u : (w == -1) ? 2u : 0u;
                byte |= c << (2 * i);
            }
            packed_T[kb * N + n] = (uint8_t)byte;
        }
    }
}

/* code -> value; 3 ("reserved") decodes to 0.
 * bittorch/quant/ternary_packed.py:112-115,
 * csrc/kernels/ternary_gemm_production.cu:37-39 */
static inline int decode2(unsigned code) { return (int)(code == 1u) - (int)(code == 2u); }

/* Follows bittorch/quant/ternary_packed.py:78-120 (slices the K padding off). */
void bto_unpack(const uint8_t* packed, int64_t N, int64_t K, int8_t* w_tern) {
    const int64_t Kb = (K + 3) / 4;
    for (int64_t n = 0; n < N; n++)
        for (int64_t k = 0; k < K; k++)
            w_tern[n * K + k] = (int8_t)decode2((packed[n * Kb + k / 4] >> (2 * (k % 4))) & 3u);
}

/* Follows bittorch/quant/ternary_packed.py:209-223. */
void bto_unpack_transposed(const uint8_t* packed_T, int64_t N, int64_t K, int8_t* w_tern) {
    for (int64_t n = 0; n < N; n++)
        for (int64_t k = 0; k < K; k++)
            w_tern[n * K + k] = (int8_t)decode2((packed_T[(k / 4) * N + n] >> (2 * (k % 4))) & 3u);
}

/*
 * Packed float-accumulate linear.  Follows
 * csrc/kernels/ternary_gemm_production.cu:53-142 (and :158-250):
 *   acc (fp32) += X[b,k] * decode(W_T[k/4, n], k%4), k ascending      (:126-133)
 *   Y[b,n] = cast(acc * scale[n] + bias[n])                           (:139-141)
 * x*w is exact for w in {-1,0,+1}, so fused or unfused multiply-add give the
 * same accumulator.  The epilogue here is one fp32 multiply then one fp32 add.
 * X is [B,K] widened to float; scale has scale_len entries (N, or 1 = broadcast);
 * bias may be NULL.  Y is the fp32 value before the cast to the output dtype.
 */
void bto_linear_packed(const float* X, const uint8_t* W_T, const float* scale,
                       int64_t scale_len, const float* bias, float* Y, int64_t B,
                       int64_t N, int64_t K) {
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; n++) {
        const float s = scale[scale_len == 1 ? 0 : n];
        const float bv = bias ? bias[n] : 0.0f;
        for (int64_t b = 0; b < B; b++) {
            float acc = 0.0f;
            for (int64_t k = 0; k < K; k++) {
                int w = decode2((W_T[(k / 4) * N + n] >> (2 * (k % 4))) & 3u);
                acc += X[b * K + k] * (float)w;
            }
            float r = acc * s;
            r = r + bv;
            Y[b * N + n] = r;
        }
    }
}

/* The same with the epilogue as one fused multiply-add, acc * s + b rounded once: what a compiler that contracts
 * floating-point expressions (nvcc's default for ternary_gemm_production.cu:139-141) makes of the reference's source
 * line.  The library and bto_linear_packed round the product first (the reading of the line as written); this variant
 * exists so that the tests can bound the distance between the two readings: at most one unit in the last place of
 * the fp32 result. */
void bto_linear_packed_fused_epilogue(const float* X, const uint8_t* W_T, const float* scale,
                                      int64_t scale_len, const float* bias, float* Y, int64_t B,
                                      int64_t N, int64_t K) {
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; n++) {
        const float s = scale[scale_len == 1 ? 0 : n];
        const float bv = bias ? bias[n] : 0.0f;
        for (int64_t b = 0; b < B; b++) {
            float acc = 0.0f;
            for (int64_t k = 0; k < K; k++) {
                int w = decode2((W_T[(k / 4) * N + n] >> (2 * (k % 4))) & 3u);
                acc += X[b * K + k] * (float)w;
            }
            Y[b * N + n] = fmaf(acc, s, bv);
        }
    }
}

/* Same contraction in float64 throughout: the high-precision truth that the
 * tolerance tests measure both the oracle and the kernels against. */
void bto_linear_packed_f64(const float* X, const uint8_t* W_T, const float* scale,
                           int64_t scale_len, const float* bias, double* Y, int64_t B,
                           int64_t N, int64_t K) {
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; n++) {
        const double s = scale[scale_len == 1 ? 0 : n];
        const double bv = bias ? bias[n] : 0.0;
        for (int64_t b = 0; b < B; b++) {
            double acc = 0.0;
            for (int64_t k = 0; k < K; k++) {
                int w = decode2((W_T[(k / 4) * N + n] >> (2 * (k % 4))) & 3u);
                acc += (double)X[b * K + k] * (double)w;
            }
            Y[b * N + n] = acc * s + bv;
        }
    }
}

/*
 * The same linear with the dot product summed exactly (what the library's single-row fp16 GEMV does on
 * the int8 matrix cores): the reference's loop (ternary_gemm_production.cu:126-133) adds one rounded
 * fp32 term at a time; here X[k] = x[k] * 2^24 is an integer for every finite fp16 x (|X| < 2^40), the
 * sum S = sum_k X[k] * w[k,n] is an exact 64-bit integer, and acc = RN_fp32(S) * 2^-24 is the correctly
 * rounded dot product.  Epilogue as above (:139-141): one fp32 multiply, one fp32 add.
 * X must hold fp16 values widened to float (checked: anything else returns -1); a row with an
 * infinity or a NaN gets, column by column, what the reference's loop leaves (nonfinite_acc below).  Returns 0.
 * Pinned by the float64 dot product, which is exact for these operands while |S| < 2^53, rounded once
 * to fp32 (tests/test_oracle.py).
 */
/* A row that holds an infinity or a NaN has no fixed-point image: its accumulator is what the reference's fp32 loop
 * leaves (ternary_gemm_production.cu:126-133, acc += x * w with w decoded to 0.0f or +-1.0f), i.e. the sum of
 * x[k] * w[k, n] over the non-finite x[k] alone, since no finite term changes it: NaN where a NaN, an infinity on a
 * zero weight or infinities of both signs meet, otherwise the infinity with its sign. */
static float nonfinite_acc(const float* xrow, const uint8_t* W_T, int64_t N, int64_t K, int64_t n) {
    float acc = 0.0f;
    for (int64_t k = 0; k < K; k++) {
        const float x = xrow[k];
        if (fabsf(x) <= 3.4028234663852886e38f) continue;
        acc = acc + x * (float)decode2((W_T[(k / 4) * N + n] >> (2 * (k % 4))) & 3u);
    }
    return acc;
}

int bto_linear_packed_exact_f16(const float* X, const uint8_t* W_T, const float* scale,
                                int64_t scale_len, const float* bias, float* Y, int64_t B,
                                int64_t N, int64_t K) {
    int64_t* XI = (int64_t*)malloc((size_t)B * K * sizeof(int64_t));
    uint8_t* bad = (uint8_t*)calloc((size_t)B, 1);
    if (!XI || !bad) { free(XI); free(bad); return -2; }
    int status = 0;
    for (int64_t b = 0; b < B; b++)
        for (int64_t k = 0; k < K; k++) {
            const float x = X[b * K + k];
            if (!(fabsf(x) <= 65504.0f)) { bad[b] = 1; XI[b * K + k] = 0; continue; }
            if (round_to_f16(x) != x) status = -1; /* not an fp16 value */
            XI[b * K + k] = (int64_t)((double)x * 16777216.0); /* exact: fp16 values are multiples of 2^-24 */
        }
    if (status == 0) {
#pragma omp parallel for schedule(static)
        for (int64_t n = 0; n < N; n++) {
            const float s = scale[scale_len == 1 ? 0 : n];
            const float bv = bias ? bias[n] : 0.0f;
            for (int64_t b = 0; b < B; b++) {
                int64_t S = 0;
                for (int64_t k = 0; k < K; k++)
                    S += XI[b * K + k] * (int64_t)decode2((W_T[(k / 4) * N + n] >> (2 * (k % 4))) & 3u);
                float acc = (float)S * 5.9604644775390625e-08f; /* RN(S) * 2^-24, the scaling exact */
                if (bad[b]) acc = nonfinite_acc(X + b * K, W_T, N, K, n);
                float r = acc * s;
                r = r + bv;
                Y[b * N + n] = r;
            }
        }
    }
    free(XI);
    free(bad);
    return status;
}

/*
 * The same for bf16 activations (this library's own arithmetic for one bf16 row times a very wide matrix and for
 * bf16 units of a grouped launch; no counterpart in the reference, whose packed kernel takes fp16 / fp32).  The
 * exponent range of bf16 does not fit one fixed-point word, so each row is scaled by its own largest exponent:
 * a finite bf16 value is mag * 2^(e1 - 134) with mag its 8-bit significand and e1 = max(biased exponent, 1);
 * emax = the largest e1 of the row; X[k] = mag * 2^(e1 - emax + 32), an integer below 2^40 in magnitude, where an
 * element more than 32 binades below the largest is rounded to an integer half-up in magnitude (more than 40 binades
 * below: 0).  S = sum_k X[k] * w[k, n] exactly; acc = RN_fp32(S) * 2^(emax - 166); then the reference's epilogue.
 * X holds bf16 values widened to float; returns -1 if one is not a bf16 value.  Rows with an infinity or a NaN:
 * nonfinite_acc above.
 */
int bto_linear_packed_rowscaled_bf16(const float* X, const uint8_t* W_T, const float* scale,
                                     int64_t scale_len, const float* bias, float* Y, int64_t B,
                                     int64_t N, int64_t K) {
    int64_t* XI = (int64_t*)malloc((size_t)B * K * sizeof(int64_t));
    uint8_t* bad = (uint8_t*)calloc((size_t)B, 1);
    int* emax = (int*)malloc((size_t)B * sizeof(int));
    if (!XI || !bad || !emax) { free(XI); free(bad); free(emax); return -2; }
    int status = 0;
    for (int64_t b = 0; b < B; b++) {
        int em = 1;
        for (int64_t k = 0; k < K; k++) {
            uint32_t u;
            memcpy(&u, &X[b * K + k], 4);
            if (u & 0xffffu) status = -1; /* not a bf16 value */
            const int e = (int)((u >> 23) & 255u);
            if (e == 255) { bad[b] = 1; continue; }
            const int e1 = e ? e : 1;
            if (e1 > em) em = e1;
        }
        emax[b] = em;
        for (int64_t k = 0; k < K; k++) {
            uint32_t u;
            memcpy(&u, &X[b * K + k], 4);
            const int e = (int)((u >> 23) & 255u);
            if (e == 255) { XI[b * K + k] = 0; continue; }
            const uint32_t m = (u >> 16) & 0x7fu;
            const uint64_t mag = e ? (m | 0x80u) : m;
            const int sh = (e ? e : 1) - em + 32;
            uint64_t mg;
            if (sh >= 0) mg = mag << sh;
            else if (sh >= -8) mg = (mag + (1ull << (-sh - 1))) >> (-sh);
            else mg = 0;
            XI[b * K + k] = (u >> 31) ? -(int64_t)mg : (int64_t)mg;
        }
    }
    if (status == 0) {
#pragma omp parallel for schedule(static)
        for (int64_t n = 0; n < N; n++) {
            const float s = scale[scale_len == 1 ? 0 : n];
            const float bv = bias ? bias[n] : 0.0f;
            for (int64_t b = 0; b < B; b++) {
                int64_t S = 0;
                for (int64_t k = 0; k < K; k++)
                    S += XI[b * K + k] * (int64_t)decode2((W_T[(k / 4) * N + n] >> (2 * (k % 4))) & 3u);
                float acc = ldexpf((float)S, emax[b] - 166);
                if (bad[b]) acc = nonfinite_acc(X + b * K, W_T, N, K, n);
                float r = acc * s;
                r = r + bv;
                Y[b * N + n] = r;
            }
        }
    }
    free(XI);
    free(bad);
    free(emax);
    return status;
}

/*
 * Unpacked (dense int8 weights) float-accumulate linear.  Follows
 * csrc/kernels/ternary_gemm.cu:41-73: acc += float(X)*float(W), k ascending
 * (:59-63), acc *= scale[n] (:65-66), acc += bias[n] (:68-70).
 */
void bto_linear_unpacked(const float* X, const int8_t* W, const float* scale,
                         int64_t scale_len, const float* bias, float* Y, int64_t B,
                         int64_t N, int64_t K) {
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; n++) {
        const float s = scale[scale_len == 1 ? 0 : n];
        for (int64_t b = 0; b < B; b++) {
            float acc = 0.0f;
            for (int64_t k = 0; k < K; k++) acc += X[b * K + k] * (float)W[n * K + k];
            acc = acc * s;
            if (bias) acc = acc + bias[n];
            Y[b * N + n] = acc;
        }
    }
}

/*
 * Per-row int8 activation quantizer.  Follows
 * csrc/kernels/ternary_gemm_tensor_core.cu:431-441 and :343-347,:456-457 with
 * the scale taken over the WHOLE row (the reference recomputes it per 32-wide
 * K tile and keeps only the last one for the epilogue, which is only
 * self-consistent for K <= 32; the whole-row form is the intended one):
 *   amax = max_k |x|;  s_x = amax > 1e-6 ? amax / 127 : 1            (:439)
 *   inv  = 1.0f / s_x                                                 (:456)
 *   q    = (int8) clamp(roundf(x * inv), -127, 127)                   (:343-347)
 * roundf rounds halfway cases away from zero.
 */
void bto_act_quant_i8(const float* X, int64_t B, int64_t K, int8_t* Q, float* s_x) {
    for (int64_t b = 0; b < B; b++) {
        const float* row = X + b * K;
        float amax = 0.0f;
        for (int64_t k = 0; k < K; k++) amax = fmaxf(amax, fabsf(row[k]));
        const float s = (amax > 1e-6f) ? (amax / 127.0f) : 1.0f;
        const float inv = 1.0f / s;
        s_x[b] = s;
        for (int64_t k = 0; k < K; k++) {
            float v = row[k] * inv;
            v = fmaxf(-127.0f, fminf(127.0f, roundf(v)));
            Q[b * K + k] = (int8_t)v;
        }
    }
}

/*
 * int8 x ternary GEMM with int32 accumulators.  Follows
 * csrc/kernels/ternary_gemm_tensor_core.cu:73-75 (weights decode to +-127),
 * :583-589 (int8*int8 -> int32 accumulate) and :652
 *   y = (float(acc) * s_x / 127.0f) * w_scale + bias
 * evaluated left to right, each operation rounded to fp32.
 * acc (nullable) receives the raw int32 accumulators [B,N]; Y the fp32 result.
 */
void bto_gemm_i8(const int8_t* Q, const float* s_x, const uint8_t* W_T, const float* scale,
                 int64_t scale_len, const float* bias, int32_t* acc_out, float* Y, int64_t B,
                 int64_t N, int64_t K) {
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; n++) {
        const float ws = scale[scale_len == 1 ? 0 : n];
        const float bv = bias ? bias[n] : 0.0f;
        for (int64_t b = 0; b < B; b++) {
            int32_t acc = 0;
            for (int64_t k = 0; k < K; k++) {
                int w = 127 * decode2((W_T[(k / 4) * N + n] >> (2 * (k % 4))) & 3u);
                acc += (int32_t)Q[b * K + k] * w;
            }
            if (acc_out) acc_out[b * N + n] = acc;
            float r = (float)acc * s_x[b];
            r = r / 127.0f;
            r = r * ws;
            r = r + bv;
            Y[b * N + n] = r;
        }
    }
}

/* ---- fused row operations (restating bittorch_amd/csrc/row_ops.hip) -------------------- */

/* exp(a) by a fixed sequence of correctly rounded fp32 operations: +inf above 88.7228, a clamped to -87 below,
 * n = rint(a*log2(e)), r = a - n*ln2 (two-part ln2, fused), degree-7 Taylor polynomial in Horner
 * form with fused multiply-adds, then the exact scaling by 2^n. */
float bto_exp_fixed(float a) {
    if (!(a == a)) return a;
    if (a > 88.7228f) return INFINITY;  /* exp overflows fp32 */
    a = fmaxf(a, -87.0f);
    const float n = rintf(a * 1.44269504088896341f);
    float r = fmaf(n, -0.693145751953125f, a);
    r = fmaf(n, -1.42860682030941723212e-6f, r);
    float p = 1.0f / 5040.0f;
    p = fmaf(p, r, 1.0f / 720.0f);
    p = fmaf(p, r, 1.0f / 120.0f);
    p = fmaf(p, r, 1.0f / 24.0f);
    p = fmaf(p, r, 1.0f / 6.0f);
    p = fmaf(p, r, 0.5f);
    p = fmaf(p, r, 1.0f);
    p = fmaf(p, r, 1.0f);
    return ldexpf(p, (int)n);
}

static void quant_row_i8(const float* v, int64_t K, int8_t* q, float* s_out) {
    float amax = 0.0f;
    for (int64_t k = 0; k < K; k++) amax = fmaxf(amax, fabsf(v[k]));
    const float s = (amax > 1e-6f) ? (amax / 127.0f) : 1.0f;
    const float inv = 1.0f / s;
    *s_out = s;
    for (int64_t k = 0; k < K; k++) q[k] = (int8_t)fmaxf(-127.0f, fminf(127.0f, roundf(v[k] * inv)));
}

/* SwiGLU of the block's MLP (js/src/models/TernaryTransformer.ts:366-423: silu(gate) * up):
 *   h = rd( rd( g / (1 + exp_fixed(-g)) ) * u ),  rd = round to dtype
 * gate / up are fp32 arrays holding values already on the dtype's grid.  H (nullable) receives h
 * as fp32; Q / s_x (nullable) the per-row int8 quantisation of h (same formulas as
 * bto_act_quant_i8). */
void bto_swiglu(const float* gate, const float* up, int dtype, int64_t B, int64_t K, float* H, int8_t* Q,
                float* s_x) {
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < B; b++) {
        float* v = (float*)malloc((size_t)K * sizeof(float));
        for (int64_t k = 0; k < K; k++) {
            const float g = gate[b * K + k];
            const float e = bto_exp_fixed(-g);
            const float sl = round_to_dtype(g / (1.0f + e), dtype);
            v[k] = round_to_dtype(sl * up[b * K + k], dtype);
        }
        if (H) memcpy(H + b * K, v, (size_t)K * sizeof(float));
        if (Q) quant_row_i8(v, K, Q + b * K, s_x + b);
        free(v);
    }
}

/* RMSNorm of the pre-norm block (TernaryTransformer.ts:489-521):
 *   ss = float( sum_k double(x_k)^2 );  r = 1 / sqrtf(ss / K + eps);  y_k = rd( (x_k * r) * w_k )
 * weight may be null (all ones). */
void bto_rmsnorm(const float* X, const float* weight, float eps, int dtype, int64_t B, int64_t K, float* Y,
                 int8_t* Q, float* s_x) {
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < B; b++) {
        float* v = (float*)malloc((size_t)K * sizeof(float));
        double ss = 0.0;
        for (int64_t k = 0; k < K; k++) ss += (double)X[b * K + k] * (double)X[b * K + k];
        const float ms = (float)ss / (float)K;
        const float r = 1.0f / sqrtf(ms + eps);
        for (int64_t k = 0; k < K; k++)
            v[k] = round_to_dtype((X[b * K + k] * r) * (weight ? weight[k] : 1.0f), dtype);
        if (Y) memcpy(Y + b * K, v, (size_t)K * sizeof(float));
        if (Q) quant_row_i8(v, K, Q + b * K, s_x + b);
        free(v);
    }
}
