// extern "C" entry points of libbittorch_hip.so: validation and kernel choice.
// Replaces the host dispatch of the reference (csrc/core/dispatch.cpp:52-142).
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "bt_common.h"

namespace bt {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int check_launch(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: HIP launch failed: %s", what, hipGetErrorString(e));
        return BT_ERR_LAUNCH;
    }
    return BT_OK;
}

// ---- run-time options (bt_common.h) -----------------------------------------------------------------------------------
static const char* const kOptionNames[OPT_COUNT] = {
    "STREAM_MAX_ROWS", "GEMM_LONG_EPILOGUE", "GEMM_TAIL_SPLIT", "GROUP_WALK", "GROUP_NACC",
    "GROUP_UNITS", "PLANES_NACC", "ROWOP_GENERIC", "STREAM_CFG", "NO_PLANES",
};
struct OptionSlot {
    char text[2][48];              // two buffers, so that a reader never sees one being rewritten by the next override
    std::atomic<const char*> cur;  // nullptr: not set
    int next;
};
static OptionSlot g_options[OPT_COUNT];
static std::once_flag g_options_once;
static void options_from_environment() {
    for (int o = 0; o < OPT_COUNT; o++) {
        char name[64];
        snprintf(name, sizeof(name), "BITTORCH_%s", kOptionNames[o]);
        const char* env = getenv(name);
        if (env && strlen(env) < sizeof(g_options[o].text[0])) {
            strcpy(g_options[o].text[0], env);
            g_options[o].cur.store(g_options[o].text[0], std::memory_order_release);
            g_options[o].next = 1;
        }
    }
}
const char* option(Option o) {
    std::call_once(g_options_once, options_from_environment);
    return g_options[o].cur.load(std::memory_order_acquire);
}

// kernels in the other translation units
bool stream_supported(int64_t N, int64_t K, const void* W_T);
size_t stream_workspace_bytes(int mode, int64_t M, int64_t N, int64_t Kb);
bool stream_supported_tiled(int64_t N, int64_t K, const void* W);
size_t tiled_bytes(int64_t N, int64_t K);
int launch_stream(int mode, const void* X, int x_elem_size, const float* s_x, const uint8_t* W_T, int w_layout,
                  const Epilogue& epi, void* Y, int y_dtype, int32_t* acc_out, int64_t B, int64_t N,
                  int64_t K, int planes, int q_layout, int pro_op, const void* pro_b, float pro_eps, int epi_op,
                  hipStream_t st);
bool stream_prologue_fusable(int mode, int64_t B, int64_t N, int64_t K, const void* X, const void* pro_b, int w_layout,
                             int epi_op);
int launch_retile(const uint8_t* W_T, int64_t N, int64_t K, int pairs, void* T, bool inverse, uint8_t* W_out,
                  hipStream_t st);
int launch_split_f32_planes(const void* X, int64_t B, int64_t K, int64_t Kp, void* P, hipStream_t st);
int launch_packed_generic(const void* X, int x_dtype, const uint8_t* W_T, const Epilogue& epi, void* Y,
                          int64_t B, int64_t N, int64_t K, hipStream_t st);
int launch_unpacked(const void* X, int x_dtype, const int8_t* W, const Epilogue& epi, void* Y, int64_t B,
                    int64_t N, int64_t K, hipStream_t st);
int launch_act_quant(const void* X, int x_dtype, int64_t B, int64_t K, int8_t* Q, float* s_x, int q_layout,
                     int32_t* rowsum, hipStream_t st);
int launch_retile_fields(const uint8_t* W_tiled, int64_t N, int64_t K, uint8_t* W_fields, hipStream_t st);
bool gemm_i8_supported(int64_t N, int64_t K, const void* Q, const void* W_T);
int launch_row_op(int op, int dtype, const void* A, int64_t lda, const void* Bv, int64_t ldb, float eps, int64_t B,
                  int64_t K, void* H, int8_t* Q, float* s_x, int q_layout, int32_t* rowsum, hipStream_t st,
                  const char* who);
bool gemm_f16_supported(int64_t N, int64_t K, const void* X, const void* W_T, const void* Y);
bool gemm_f16_supported_tiled(int64_t N, int64_t K, const void* X, const void* Y);
int launch_gemm_f16(int mode, const void* X, const uint8_t* W_T, int w_layout, const Epilogue& epi, void* Y, int y_dtype,
                    int64_t M, int64_t N, int64_t K, int planes, hipStream_t st);
bool planes_supported(int x_dtype, int y_dtype, int64_t B, int64_t N, int64_t K, const void* X, const void* W, const void* Y,
                      int w_layout);
int launch_planes(const void* X, const uint8_t* W, int w_layout, const Epilogue& epi, void* Y, int64_t N, int64_t K,
                  int epi_op, hipStream_t st, int pro_op = 0, const void* pro_b = nullptr, float pro_eps = 0.0f);
int launch_planes_group(const void* const* X_tab, int x_dtype, const uint8_t* const* W_tab, const void* const* scale_tab,
                        int scale_dtype, int scale_bcast, const void* const* bias_tab, int bias_dtype, void* const* Y_tab,
                        int64_t G, int64_t N, int64_t K, hipStream_t st);
bool i8_group_supported(int64_t K);
int launch_i8_group(const int8_t* const* Q_tab, int q_layout, const float* const* sx_tab, const uint8_t* const* W_tab,
                    const void* const* scale_tab, int scale_dtype, int scale_bcast, const void* const* bias_tab,
                    int bias_dtype, void* const* Y_tab, int y_dtype, int32_t* const* acc_tab, int64_t G, int64_t M,
                    int64_t N, int64_t K, hipStream_t st);
bool planes_bf16_shape_ok(int64_t N, int64_t K);
bool planes_bf16_wide(int64_t N, int64_t K);
int launch_planes_bf16_wide(const void* X, const uint8_t* W, const Epilogue& epi, void* Y, int64_t N, int64_t K, hipStream_t st);
bool gemm_i8_supported_tiled(int64_t N, int64_t K, const void* Q);
int launch_gemm_i8(const int8_t* Q, int q_layout, const float* s_x, const int32_t* q_rowsum, const uint8_t* W_T, int w_layout,
                   const Epilogue& epi, void* Y, int y_dtype, int32_t* acc_out, int64_t M, int64_t N, int64_t K,
                   hipStream_t st);

static bool valid_dtype(int dt) { return dt == BT_F32 || dt == BT_F16 || dt == BT_BF16; }

static int make_epilogue(const char* who, const void* scale, int scale_dtype, int64_t scale_len,
                         const void* bias, int bias_dtype, int64_t N, Epilogue* e) {
    if (!scale) {
        set_error("%s: scale is null", who);
        return BT_ERR_INVALID;
    }
    if (scale_len != N && scale_len != 1) {
        set_error("%s: scale size doesn't match N (%lld entries, N=%lld)", who, (long long)scale_len,
                  (long long)N);
        return BT_ERR_INVALID;
    }
    if (!valid_dtype(scale_dtype) || (bias && !valid_dtype(bias_dtype))) {
        set_error("%s: unsupported scale/bias dtype", who);
        return BT_ERR_INVALID;
    }
    e->scale = scale;
    e->bias = bias;
    e->scale_dtype = scale_dtype;
    e->bias_dtype = bias_dtype;
    e->scale_bcast = (scale_len == 1 && N != 1) ? 1 : 0;
    e->residual = nullptr;
    return BT_OK;
}

static int check_shape(const char* who, const void* X, const void* W, const void* Y, int x_dtype,
                       int64_t B, int64_t N, int64_t K) {
    if (!X || !W || !Y) {
        set_error("%s: null tensor pointer", who);
        return BT_ERR_INVALID;
    }
    if (B <= 0 || N <= 0 || K <= 0) {
        set_error("%s: empty shape (B=%lld N=%lld K=%lld)", who, (long long)B, (long long)N, (long long)K);
        return BT_ERR_INVALID;
    }
    if (!valid_dtype(x_dtype)) {
        set_error("%s: unsupported activation dtype %d", who, x_dtype);
        return BT_ERR_INVALID;
    }
    return BT_OK;
}

// The matrix-core paths write Y with vector stores and use 32-bit indices
// inside a 16-row block.
static bool fast_path_ok(const void* Y, int64_t N, int64_t K) {
    return ((uintptr_t)Y) % 16 == 0 && N < (1ll << 30) && K < (1ll << 30);
}

// int32 accumulators hold sum_k q*127w with |q| <= 127; the matrix cores sum q*w (|sum| <= 127 K), which the prefill
// GEMM's epilogue converts to fp32 before it multiplies by 127: exact while 127 K < 2^24
static const int64_t kMaxKInt8 = 132096;

// batches up to this many rows go through the streaming (decode-shape) kernel
// Streaming kernel or tiled GEMM?  The streaming kernel runs the 16-row blocks of a call concurrently in one
// launch and its time grows with the work, B * N * K; a tiled GEMM takes the time of one 128 x 256 tile, which
// grows with K only, for every round of 256 tiles.  Both are priced with times fitted to measurements on this
// chip (five layer shapes, narrow and shallow ones besides, both weight layouts), in microseconds:
//   streaming  4 + B N K * 2.2e-9 + 0.003 workgroups (int8),  4 + B N K * 5.0e-9 + 0.004 workgroups (16-bit),
//              workgroups = 16-row blocks x 128- resp. 64-column tiles
//   GEMM       rounds * (8.6 + 0.0044 K) (int8),  rounds * (6.9 + 0.010 K) (16-bit)
// which puts the crossover at 1.5 .. 2 M outputs for K = 2560 .. 4096 (the GEMM would occupy under a fifth of
// the compute units there) and later for shallow layers.  The option STREAM_MAX_ROWS = n replaces the rule by
// "B <= n" (tuning and test runs).
static bool prefers_stream(int64_t B, int64_t N, int64_t K, bool int8, bool tiled = false) {
    if (const char* env = option(OPT_STREAM_MAX_ROWS)) {
        const long v = atol(env);
        if (v >= 1) return B <= v;
    }
    if (B <= 32) return true;
    const double work = (double)B * (double)N * (double)K;
    // (rounds of whole tiles, or what the finer tiles of a small launch's remainder cost in them)
    const double rounds = gemm_split(B, N, tiled && K % (int8 ? 128 : 64) == 0).rounds;
    const double wgs = (double)(ceil_div(B, 16) * ceil_div(N, int8 ? 128 : 64));
    const double t_stream = 4.0 + work * (int8 ? 2.2e-9 : 5.0e-9) + wgs * (int8 ? 0.003 : 0.004);
    const double t_gemm = rounds * (int8 ? 8.6 + 0.0044 * (double)K : 6.9 + 0.010 * (double)K);
    return t_stream < t_gemm;
}

static size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

}  // namespace bt

using namespace bt;

extern "C" int bt_abi_version(void) { return BT_ABI_VERSION; }

extern "C" const char* bt_last_error(void) { return g_err; }

extern "C" int bt_set_option(const char* name, const char* value) {
    std::call_once(g_options_once, options_from_environment);
    if (!name) {  // back to "not set", every option
        for (int o = 0; o < OPT_COUNT; o++) g_options[o].cur.store(nullptr, std::memory_order_release);
        return BT_OK;
    }
    if (!strncmp(name, "BITTORCH_", 9)) name += 9;
    for (int o = 0; o < OPT_COUNT; o++) {
        if (strcmp(name, kOptionNames[o])) continue;
        OptionSlot& s = g_options[o];
        if (!value) {
            s.cur.store(nullptr, std::memory_order_release);
            return BT_OK;
        }
        if (strlen(value) >= sizeof(s.text[0])) {
            set_error("bt_set_option: value of %s is longer than %zu characters", name, sizeof(s.text[0]) - 1);
            return BT_ERR_INVALID;
        }
        strcpy(s.text[s.next], value);
        s.cur.store(s.text[s.next], std::memory_order_release);
        s.next ^= 1;
        return BT_OK;
    }
    set_error("bt_set_option: unknown option '%s'", name);
    return BT_ERR_INVALID;
}

extern "C" int bt_ternary_linear_forward(const void* X, int x_dtype, const int8_t* W_tern, const void* scale,
                                         int scale_dtype, int64_t scale_len, const void* bias, int bias_dtype,
                                         void* Y, int64_t B, int64_t N, int64_t K, void* stream) {
    const char* who = "bt_ternary_linear_forward";
    int rc = check_shape(who, X, W_tern, Y, x_dtype, B, N, K);
    if (rc) return rc;
    Epilogue epi;
    rc = make_epilogue(who, scale, scale_dtype, scale_len, bias, bias_dtype, N, &epi);
    if (rc) return rc;
    return launch_unpacked(X, x_dtype, W_tern, epi, Y, B, N, K, (hipStream_t)stream);
}

static bool generic_forced() {
    const char* env = getenv("BITTORCH_KERNEL");
    return env && !strcmp(env, "generic");
}

static bool packed_uses_stream(int x_dtype, const void* W_T, const void* Y, int64_t N, int64_t K) {
    if (generic_forced()) return false;
    return x_dtype != BT_F32 && stream_supported(N, K, W_T) && fast_path_ok(Y, N, K);
}

// fp32 activations run on the bf16 matrix-core kernels as three exact bf16 planes (hi, mid, lo), each
// zero-padded to the kernels' 64-wide step; the planes live in the workspace.
static int64_t plane_len(int64_t K) { return ceil_div(K, 64) * 64; }
static size_t f32_planes_bytes(int64_t B, int64_t K) { return align256((size_t)B * 3 * plane_len(K) * 2); }
static bool packed_uses_f32_planes(const void* W_T, const void* Y, int64_t N, int64_t K) {
    if (generic_forced()) return false;
    return stream_supported(N, 3 * plane_len(K), W_T) && fast_path_ok(Y, N, 3 * plane_len(K));
}

extern "C" size_t bt_packed_forward_workspace_bytes(int64_t B, int64_t N, int64_t K, int x_dtype) {
    if (B <= 0 || N <= 0 || K <= 0) return 0;
    if (x_dtype == BT_F32) return f32_planes_bytes(B, K);
    return stream_workspace_bytes(x_dtype == BT_F16 ? MODE_F16 : MODE_BF16, B, N, ceil_div(K, 4));
}

// residual (optional): [B, N] in Y's dtype, 16-byte aligned; Y = round(round(linear) + residual)
static int set_residual(const char* who, const void* residual, Epilogue* e) {
    if (residual && ((uintptr_t)residual) % 16 != 0) {
        set_error("%s: residual must be 16-byte aligned", who);
        return BT_ERR_INVALID;
    }
    e->residual = residual;
    return BT_OK;
}

static int packed_forward_impl(const char* who, const void* X, int x_dtype, const uint8_t* W_T, int w_layout, int epi_op,
                               const void* scale, int scale_dtype, int64_t scale_len, const void* bias, int bias_dtype,
                               const void* residual, void* Y, int64_t B, int64_t N, int64_t K, void* workspace,
                               size_t workspace_bytes, void* stream) {
    int rc = check_shape(who, X, W_T, Y, x_dtype, B, N, K);
    if (rc) return rc;
    Epilogue epi;
    rc = make_epilogue(who, scale, scale_dtype, scale_len, bias, bias_dtype, N, &epi);
    if (rc) return rc;
    rc = set_residual(who, residual, &epi);
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    if (epi_op != 0 && (epi_op != EPI_SWIGLU_PAIRS || w_layout != W_LAYOUT_TILED || N % 32 != 0 || residual)) {
        set_error("%s: the SwiGLU output stage needs pair-ordered tiled weights, N %% 32 == 0 and no residual", who);
        return BT_ERR_INVALID;
    }
    if (w_layout == W_LAYOUT_TILED_PAIRS_AS_NATURAL && (N % 32 != 0 || epi_op != 0)) {
        set_error("%s: a pair-ordered tiled copy has N %% 32 == 0; its natural-order output takes no output stage", who);
        return BT_ERR_INVALID;
    }
    if (layout_tiled(w_layout)) {
        // the decode-tiled copy is read by the streaming kernel only, once per 16 rows
        if (!stream_supported_tiled(N, K, W_T) || !fast_path_ok(Y, N, 3 * K) || 3 * K >= (1ll << 26)) {
            set_error("%s: tiled weights must be 256-byte aligned and below 4 GiB, Y 16-byte aligned", who);
            return BT_ERR_INVALID;
        }
        // one fp16 row: the exact GEMV on the int8 matrix cores
        if (planes_supported(x_dtype, x_dtype, B, N, K, X, W_T, Y, w_layout))
            return launch_planes(X, W_T, w_layout, epi, Y, N, K, epi_op, st);
        // one bf16 row times a very wide matrix (a vocabulary projection): the same kernel family, the row scaled by
        // its largest exponent
        if (x_dtype == BT_BF16 && B == 1 && epi_op == 0 && ((uintptr_t)X) % 16 == 0 && !option(OPT_NO_PLANES) &&
            w_layout == W_LAYOUT_TILED && planes_bf16_wide(N, K))
            return launch_planes_bf16_wide(X, W_T, epi, Y, N, K, st);
        if (x_dtype != BT_F32) {
            const int mode = (x_dtype == BT_F16) ? MODE_F16 : MODE_BF16;
            // tall batches: the tiled matrix-core GEMM reads the copy too (not with the SwiGLU output stage)
            if (!prefers_stream(B, N, K, false, true) && epi_op == 0 && gemm_f16_supported_tiled(N, K, X, Y))
                return launch_gemm_f16(mode, X, W_T, w_layout, epi, Y, x_dtype, B, N, K, 1, st);
            return launch_stream(mode, X, 2, nullptr, W_T, w_layout, epi, Y, x_dtype, nullptr, B, N, K, 1,
                                 Q_ROW_MAJOR, 0, nullptr, 0.0f, epi_op, st);
        }
        if (!workspace || workspace_bytes < f32_planes_bytes(B, K) || ((uintptr_t)workspace) % 256 != 0) {
            set_error("%s: fp32 activations on tiled weights need a workspace of %zu bytes (256-byte aligned)", who,
                      f32_planes_bytes(B, K));
            return BT_ERR_INVALID;
        }
        const int64_t Kp = plane_len(K);
        rc = launch_split_f32_planes(X, B, K, Kp, workspace, st);
        if (rc) return rc;
        if (!prefers_stream(B, N, 3 * Kp, false, K % 64 == 0) && epi_op == 0 && gemm_f16_supported_tiled(N, 3 * Kp, workspace, Y))
            return launch_gemm_f16(MODE_BF16, workspace, W_T, w_layout, epi, Y, BT_F32, B, N, K, 3, st);
        return launch_stream(MODE_BF16, workspace, 2, nullptr, W_T, w_layout, epi, Y, BT_F32, nullptr, B, N, K, 3,
                             Q_ROW_MAJOR, 0, nullptr, 0.0f, epi_op, st);
    }
    if (packed_uses_stream(x_dtype, W_T, Y, N, K)) {
        if (planes_supported(x_dtype, x_dtype, B, N, K, X, W_T, Y, W_LAYOUT_ROW_MAJOR))
            return launch_planes(X, W_T, W_LAYOUT_ROW_MAJOR, epi, Y, N, K, 0, st);
        const int mode = (x_dtype == BT_F16) ? MODE_F16 : MODE_BF16;
        // tall batches go to the tiled matrix-core kernel, decode shapes stream the weights
        if (!prefers_stream(B, N, K, false) && gemm_f16_supported(N, K, X, W_T, Y))
            return launch_gemm_f16(mode, X, W_T, W_LAYOUT_ROW_MAJOR, epi, Y, x_dtype, B, N, K, 1, st);
        return launch_stream(mode, X, 2, nullptr, W_T, W_LAYOUT_ROW_MAJOR, epi, Y, x_dtype, nullptr, B, N, K, 1, Q_ROW_MAJOR, 0, nullptr, 0.0f, 0, st);
    }
    if (x_dtype == BT_F32 && packed_uses_f32_planes(W_T, Y, N, K) && workspace &&
        workspace_bytes >= f32_planes_bytes(B, K) && ((uintptr_t)workspace) % 256 == 0) {
        // (without a workspace the call still succeeds, on the generic kernel)
        const int64_t Kp = plane_len(K);
        rc = launch_split_f32_planes(X, B, K, Kp, workspace, st);
        if (rc) return rc;
        if (!prefers_stream(B, N, 3 * Kp, false) && gemm_f16_supported(N, 3 * Kp, workspace, W_T, Y))
            return launch_gemm_f16(MODE_BF16, workspace, W_T, W_LAYOUT_ROW_MAJOR, epi, Y, BT_F32, B, N, K, 3, st);
        return launch_stream(MODE_BF16, workspace, 2, nullptr, W_T, W_LAYOUT_ROW_MAJOR, epi, Y, BT_F32, nullptr, B, N, K, 3, Q_ROW_MAJOR, 0, nullptr, 0.0f, 0, st);
    }
    return launch_packed_generic(X, x_dtype, W_T, epi, Y, B, N, K, st);
}

extern "C" int bt_ternary_linear_packed_forward(const void* X, int x_dtype, const uint8_t* W_T,
                                                const void* scale, int scale_dtype, int64_t scale_len,
                                                const void* bias, int bias_dtype, void* Y, int64_t B,
                                                int64_t N, int64_t K, void* workspace, size_t workspace_bytes,
                                                void* stream) {
    return packed_forward_impl("bt_ternary_linear_packed_forward", X, x_dtype, W_T, W_LAYOUT_ROW_MAJOR, 0, scale, scale_dtype, scale_len, bias,
                               bias_dtype, nullptr, Y, B, N, K, workspace, workspace_bytes, stream);
}

extern "C" int bt_ternary_linear_packed_forward_res(const void* X, int x_dtype, const uint8_t* W_T,
                                                    const void* scale, int scale_dtype, int64_t scale_len,
                                                    const void* bias, int bias_dtype, const void* residual,
                                                    void* Y, int64_t B, int64_t N, int64_t K, void* workspace,
                                                    size_t workspace_bytes, void* stream) {
    return packed_forward_impl("bt_ternary_linear_packed_forward_res", X, x_dtype, W_T, W_LAYOUT_ROW_MAJOR, 0, scale, scale_dtype, scale_len,
                               bias, bias_dtype, residual, Y, B, N, K, workspace, workspace_bytes, stream);
}

extern "C" int bt_act_quant_i8(const void* X, int x_dtype, int64_t B, int64_t K, int8_t* Q, float* s_x,
                               void* stream) {
    if (!X || !Q || !s_x || B <= 0 || K <= 0 || !valid_dtype(x_dtype)) {
        set_error("bt_act_quant_i8: null pointer, empty shape or bad dtype");
        return BT_ERR_INVALID;
    }
    return launch_act_quant(X, x_dtype, B, K, Q, s_x, Q_ROW_MAJOR, nullptr, (hipStream_t)stream);
}

// q_layout: BT_Q_ROW_MAJOR or BT_Q_OPERAND_ORDER (K % 16 == 0, X 16-byte and Q 16-byte aligned)
static int check_q_layout(const char* who, int q_layout, int64_t K, const void* Q, const void* X) {
    if (q_layout == Q_ROW_MAJOR) return BT_OK;
    if (q_layout != Q_OPERAND_ORDER) {
        set_error("%s: unknown q_layout %d", who, q_layout);
        return BT_ERR_INVALID;
    }
    if (K % 16 != 0 || ((uintptr_t)Q) % 16 != 0 || (X && ((uintptr_t)X) % 16 != 0)) {
        set_error("%s: the operand-order layout needs K %% 16 == 0 and 16-byte aligned buffers (K=%lld)", who,
                  (long long)K);
        return BT_ERR_INVALID;
    }
    return BT_OK;
}

extern "C" int bt_act_quant_i8_layout(const void* X, int x_dtype, int64_t B, int64_t K, int8_t* Q, float* s_x,
                                      int q_layout, void* stream) {
    const char* who = "bt_act_quant_i8_layout";
    if (!X || !Q || !s_x || B <= 0 || K <= 0 || !valid_dtype(x_dtype)) {
        set_error("%s: null pointer, empty shape or bad dtype", who);
        return BT_ERR_INVALID;
    }
    const int rc = check_q_layout(who, q_layout, K, Q, X);
    if (rc) return rc;
    return launch_act_quant(X, x_dtype, B, K, Q, s_x, q_layout, nullptr, (hipStream_t)stream);
}

extern "C" int bt_act_quant_i8_rowsum(const void* X, int x_dtype, int64_t B, int64_t K, int8_t* Q, float* s_x,
                                      int32_t* q_rowsum, int q_layout, void* stream) {
    const char* who = "bt_act_quant_i8_rowsum";
    if (!X || !Q || !s_x || !q_rowsum || B <= 0 || K <= 0 || !valid_dtype(x_dtype)) {
        set_error("%s: null pointer, empty shape or bad dtype", who);
        return BT_ERR_INVALID;
    }
    const int rc = check_q_layout(who, q_layout, K, Q, X);
    if (rc) return rc;
    return launch_act_quant(X, x_dtype, B, K, Q, s_x, q_layout, q_rowsum, (hipStream_t)stream);
}

extern "C" size_t bt_gemm_i8_workspace_bytes(int64_t B, int64_t N, int64_t K) {
    if (B <= 0 || N <= 0 || K <= 0) return 0;
    return stream_workspace_bytes(MODE_I8, B, N, ceil_div(K, 4));
}

static int gemm_i8_impl(const char* who, const int8_t* Q, int q_layout, const float* s_x, const uint8_t* W_T, int w_layout,
                        const void* scale,
                        int scale_dtype, int64_t scale_len, const void* bias, int bias_dtype, const void* residual,
                        void* Y, int y_dtype, int32_t* acc_out, int64_t B, int64_t N, int64_t K, void* stream) {
    int rc = check_shape(who, Q, W_T, Y, y_dtype, B, N, K);
    if (rc) return rc;
    if (!s_x) {
        set_error("%s: s_x is null", who);
        return BT_ERR_INVALID;
    }
    rc = check_q_layout(who, q_layout, K, Q, nullptr);
    if (rc) return rc;
    if (K > kMaxKInt8) {
        set_error("%s: K=%lld could overflow the int32 accumulators (limit %lld)", who, (long long)K,
                  (long long)kMaxKInt8);
        return BT_ERR_INVALID;
    }
    if (((uintptr_t)W_T) % 16 != 0 || !fast_path_ok(Y, N, K) || (acc_out && ((uintptr_t)acc_out) % 16 != 0)) {
        set_error("%s: W_T, Y and acc_out must be 16-byte aligned", who);
        return BT_ERR_INVALID;
    }
    Epilogue epi;
    rc = make_epilogue(who, scale, scale_dtype, scale_len, bias, bias_dtype, N, &epi);
    if (rc) return rc;
    rc = set_residual(who, residual, &epi);
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    if (layout_tiled(w_layout)) {
        if (!stream_supported_tiled(N, K, W_T)) {
            set_error("%s: tiled weights must be 256-byte aligned and below 4 GiB", who);
            return BT_ERR_INVALID;
        }
        if (!prefers_stream(B, N, K, true, true) && gemm_i8_supported_tiled(N, K, Q))
            return launch_gemm_i8(Q, q_layout, s_x, nullptr, W_T, w_layout, epi, Y, y_dtype, acc_out, B, N, K, st);
        return launch_stream(MODE_I8, Q, 1, s_x, W_T, w_layout, epi, Y, y_dtype, acc_out, B, N, K, 1, q_layout, 0, nullptr,
                             0.0f, 0, st);
    }
    // decode-shape batches, and any batch whose N the tiled kernel's 4-column
    // vector accesses cannot take, stream the weights once per 16 rows
    if (prefers_stream(B, N, K, true) || !gemm_i8_supported(N, K, Q, W_T)) {
        if (!stream_supported(N, K, W_T)) {
            set_error("%s: packed weight matrix of %lld x %lld bytes exceeds the 4 GiB the kernels address", who,
                      (long long)ceil_div(K, 4), (long long)N);
            return BT_ERR_INVALID;
        }
        return launch_stream(MODE_I8, Q, 1, s_x, W_T, w_layout, epi, Y, y_dtype, acc_out, B, N, K, 1, q_layout, 0, nullptr, 0.0f, 0, st);
    }
    return launch_gemm_i8(Q, q_layout, s_x, nullptr, W_T, W_LAYOUT_ROW_MAJOR, epi, Y, y_dtype, acc_out, B, N, K, st);
}

extern "C" int bt_ternary_gemm_i8(const int8_t* Q, const float* s_x, const uint8_t* W_T, const void* scale,
                                  int scale_dtype, int64_t scale_len, const void* bias, int bias_dtype,
                                  void* Y, int y_dtype, int32_t* acc_out, int64_t B, int64_t N, int64_t K,
                                  void* workspace, size_t workspace_bytes, void* stream) {
    (void)workspace; (void)workspace_bytes;
    return gemm_i8_impl("bt_ternary_gemm_i8", Q, Q_ROW_MAJOR, s_x, W_T, W_LAYOUT_ROW_MAJOR, scale, scale_dtype, scale_len, bias, bias_dtype, nullptr, Y,
                        y_dtype, acc_out, B, N, K, stream);
}

extern "C" int bt_ternary_gemm_i8_res(const int8_t* Q, int q_layout, const float* s_x, const uint8_t* W_T, const void* scale,
                                      int scale_dtype, int64_t scale_len, const void* bias, int bias_dtype,
                                      const void* residual, void* Y, int y_dtype, int32_t* acc_out, int64_t B,
                                      int64_t N, int64_t K, void* stream) {
    return gemm_i8_impl("bt_ternary_gemm_i8_res", Q, q_layout, s_x, W_T, W_LAYOUT_ROW_MAJOR, scale, scale_dtype, scale_len, bias, bias_dtype, residual,
                        Y, y_dtype, acc_out, B, N, K, stream);
}

extern "C" size_t bt_tensor_core_workspace_bytes(int64_t B, int64_t N, int64_t K) {
    if (B <= 0 || N <= 0 || K <= 0) return 0;
    // [GEMM scratch (none at present)] [Q int8 B*K] [s_x fp32 B]
    return align256(bt_gemm_i8_workspace_bytes(B, N, K)) + align256((size_t)B * K) + align256((size_t)B * 4);
}

extern "C" int bt_ternary_linear_tensor_core_forward(const void* X, int x_dtype, const uint8_t* W_T,
                                                     const void* scale, int scale_dtype, int64_t scale_len,
                                                     const void* bias, int bias_dtype, void* Y, int64_t B,
                                                     int64_t N, int64_t K, void* workspace,
                                                     size_t workspace_bytes, void* stream) {
    const char* who = "bt_ternary_linear_tensor_core_forward";
    int rc = check_shape(who, X, W_T, Y, x_dtype, B, N, K);
    if (rc) return rc;
    const size_t need = bt_tensor_core_workspace_bytes(B, N, K);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace) % 256 != 0) {
        set_error("%s: workspace of %zu bytes (256-byte aligned) needed, %zu given", who, need, workspace_bytes);
        return BT_ERR_WORKSPACE;
    }
    const size_t gemm_bytes = align256(bt_gemm_i8_workspace_bytes(B, N, K));
    int8_t* Q = (int8_t*)((uint8_t*)workspace + gemm_bytes);
    float* s_x = (float*)((uint8_t*)Q + align256((size_t)B * K));
    // Q is private to this call: written in operand order whenever the layout applies, so that
    // neither GEMM kernel has to permute activations
    // (BITTORCH_Q_LAYOUT=rowmajor keeps the row-major layout, for A/B runs)
    const char* lay = tuning_env("BITTORCH_Q_LAYOUT");
    const int q_layout = (K % 16 == 0 && ((uintptr_t)X) % 16 == 0 && !(lay && !strcmp(lay, "rowmajor")))
                             ? Q_OPERAND_ORDER : Q_ROW_MAJOR;
    rc = launch_act_quant(X, x_dtype, B, K, Q, s_x, q_layout, nullptr, (hipStream_t)stream);
    if (rc) return rc;
    (void)gemm_bytes;
    return gemm_i8_impl(who, Q, q_layout, s_x, W_T, W_LAYOUT_ROW_MAJOR, scale, scale_dtype, scale_len, bias, bias_dtype, nullptr,
                        Y, x_dtype, nullptr, B, N, K, stream);
}

// ---- the matrix-core forward for callers that cannot allocate ----------------------------------
// The int8 activations Q and their row scales, which bt_ternary_linear_tensor_core_forward keeps in the caller's
// workspace, live in a device array of this library instead.  Host code must never hand the array's
// name to a kernel (there it is a host-side stand-in, not a device address): the device address is
// asked for once per device with hipGetSymbolAddress and only that pointer is used afterwards.
namespace bt {
constexpr size_t kStaticQBytes = BT_STATIC_SCRATCH_ACTIVATION_BYTES;  // int8 activations: B * K bytes at most
constexpr size_t kStaticRows = BT_STATIC_SCRATCH_ROWS;               // row scales: B at most
constexpr size_t kStaticBytes = kStaticQBytes + kStaticRows * sizeof(float);
constexpr int kStaticMaxDevices = 64;
}  // namespace bt
static __device__ __align__(256) unsigned char scratch[bt::kStaticBytes];
static void* g_scratch_ptr[bt::kStaticMaxDevices];  // per device: each GPU holds its own copy of the array
static std::mutex g_scratch_mutex;

// device address of `scratch` on the current device (looked up on the first call per device)
static int static_scratch_ptr(const char* who, unsigned char** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kStaticMaxDevices) {
        set_error("%s: cannot identify the current device (%s, device %d)", who, hipGetErrorString(e), dev);
        return BT_ERR_LAUNCH;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            set_error("%s: hipGetSymbolAddress(scratch) failed on device %d: %s", who, dev, hipGetErrorString(e));
            return BT_ERR_LAUNCH;
        }
        g_scratch_ptr[dev] = ptr;
    }
    *out = (unsigned char*)g_scratch_ptr[dev];
    return BT_OK;
}

extern "C" int bt_ternary_linear_tensor_core_forward_static(const void* X, int x_dtype, const uint8_t* W_T,
                                                            const void* scale, int scale_dtype, int64_t scale_len,
                                                            const void* bias, int bias_dtype, void* Y, int64_t B,
                                                            int64_t N, int64_t K, void* stream) {
    const char* who = "bt_ternary_linear_tensor_core_forward_static";
    int rc = check_shape(who, X, W_T, Y, x_dtype, B, N, K);
    if (rc) return rc;
    if ((uint64_t)B > kStaticRows || (uint64_t)K > kStaticQBytes || (uint64_t)B * (uint64_t)K > kStaticQBytes) {
        set_error("%s: B*K = %lld x %lld exceeds the library's static scratch (B*K <= %zu bytes, B <= %zu rows); "
                  "use bt_ternary_linear_tensor_core_forward with a workspace", who, (long long)B, (long long)K,
                  kStaticQBytes, kStaticRows);
        return BT_ERR_WORKSPACE;
    }
    unsigned char* base = nullptr;
    rc = static_scratch_ptr(who, &base);
    if (rc) return rc;
    int8_t* Q = (int8_t*)base;
    float* s_x = (float*)(base + kStaticQBytes);
    // both are written in full by the quantizer before the GEMM reads them: nothing has to start at zero
    const int q_layout = (K % 16 == 0 && ((uintptr_t)X) % 16 == 0) ? Q_OPERAND_ORDER : Q_ROW_MAJOR;
    rc = launch_act_quant(X, x_dtype, B, K, Q, s_x, q_layout, nullptr, (hipStream_t)stream);
    if (rc) return rc;
    return gemm_i8_impl(who, Q, q_layout, s_x, W_T, W_LAYOUT_ROW_MAJOR, scale, scale_dtype, scale_len, bias, bias_dtype,
                        nullptr, Y, x_dtype, nullptr, B, N, K, stream);
}

// ---- G decode GEMVs in one launch ---------------------------------------------------------------
extern "C" int bt_ternary_gemv_grouped(const void* const* X_tab, int x_dtype, const uint8_t* const* W_tiled_tab,
                                       const void* const* scale_tab, int scale_dtype, int64_t scale_len,
                                       const void* const* bias_tab, int bias_dtype, void* const* Y_tab, int64_t G,
                                       int64_t N, int64_t K, void* stream) {
    const char* who = "bt_ternary_gemv_grouped";
    if (!X_tab || !W_tiled_tab || !scale_tab || !Y_tab) {
        set_error("%s: null pointer table", who);
        return BT_ERR_INVALID;
    }
    if (G <= 0 || N <= 0 || K <= 0 || G > (1 << 20)) {
        set_error("%s: empty shape or too many units (G=%lld N=%lld K=%lld)", who, (long long)G, (long long)N, (long long)K);
        return BT_ERR_INVALID;
    }
    if (x_dtype != BT_F16 && x_dtype != BT_BF16) {
        set_error("%s: activations must be fp16 or bf16 (dtype tag %d given)", who, x_dtype);
        return BT_ERR_INVALID;
    }
    if (K % 16 != 0 || K > 16384) {
        set_error("%s: K must be a multiple of 16 and at most 16384 (K=%lld)", who, (long long)K);
        return BT_ERR_INVALID;
    }
    if ((scale_len != N && scale_len != 1) || !valid_dtype(scale_dtype) || (bias_tab && !valid_dtype(bias_dtype))) {
        set_error("%s: scale size doesn't match N, or unsupported scale/bias dtype", who);
        return BT_ERR_INVALID;
    }
    if (tiled_bytes(N, K) >= (1ull << 32) || G * ceil_div(N, 128) >= (1ll << 31)) {
        set_error("%s: a unit's tiled weights must stay below 4 GiB", who);
        return BT_ERR_INVALID;
    }
    return launch_planes_group(X_tab, x_dtype, W_tiled_tab, scale_tab, scale_dtype, (scale_len == 1 && N != 1) ? 1 : 0, bias_tab,
                               bias_dtype, Y_tab, G, N, K, (hipStream_t)stream);
}

// ---- G small-batch int8 units in one launch ------------------------------------------------------
extern "C" int bt_ternary_gemm_i8_grouped(const int8_t* const* Q_tab, int q_layout, const float* const* sx_tab,
                                          const uint8_t* const* W_tiled_tab, const void* const* scale_tab,
                                          int scale_dtype, int64_t scale_len, const void* const* bias_tab,
                                          int bias_dtype, void* const* Y_tab, int y_dtype, int32_t* const* acc_tab,
                                          int64_t G, int64_t M, int64_t N, int64_t K, void* stream) {
    const char* who = "bt_ternary_gemm_i8_grouped";
    if (!Q_tab || !sx_tab || !W_tiled_tab || !scale_tab || !Y_tab) {
        set_error("%s: null pointer table", who);
        return BT_ERR_INVALID;
    }
    if (G <= 0 || N <= 0 || K <= 0 || M <= 0 || G > (1 << 20)) {
        set_error("%s: empty shape or too many units (G=%lld M=%lld N=%lld K=%lld)", who, (long long)G, (long long)M,
                  (long long)N, (long long)K);
        return BT_ERR_INVALID;
    }
    if (M > 16) {
        set_error("%s: a unit has at most 16 activation rows (M=%lld)", who, (long long)M);
        return BT_ERR_INVALID;
    }
    if (!i8_group_supported(K)) {
        set_error("%s: K must be a multiple of 16 and at most 11264 (K=%lld)", who, (long long)K);
        return BT_ERR_INVALID;
    }
    if (q_layout != Q_ROW_MAJOR && q_layout != Q_OPERAND_ORDER) {
        set_error("%s: q_layout must be BT_Q_ROW_MAJOR or BT_Q_OPERAND_ORDER (got %d)", who, q_layout);
        return BT_ERR_INVALID;
    }
    if ((scale_len != N && scale_len != 1) || !valid_dtype(scale_dtype) || (bias_tab && !valid_dtype(bias_dtype)) ||
        !valid_dtype(y_dtype)) {
        set_error("%s: scale size doesn't match N, or unsupported scale/bias/output dtype", who);
        return BT_ERR_INVALID;
    }
    if (tiled_bytes(N, K) >= (1ull << 32) || G * ceil_div(N, 16) >= (1ll << 31) || 17 * K >= (1ll << 31)) {
        set_error("%s: a unit's tiled weights must stay below 4 GiB", who);
        return BT_ERR_INVALID;
    }
    return launch_i8_group(Q_tab, q_layout, sx_tab, W_tiled_tab, scale_tab, scale_dtype, (scale_len == 1 && N != 1) ? 1 : 0,
                           bias_tab, bias_dtype, Y_tab, y_dtype, acc_tab, G, M, N, K, (hipStream_t)stream);
}

// ---- fused producers of the GEMM activations (row_ops.hip) ----------------------------------
static int check_row_op(const char* who, const void* A, int dtype, int64_t B, int64_t K, int64_t lda, void* H,
                        int8_t* Q, float* s_x) {
    if (!A || B <= 0 || K <= 0 || !valid_dtype(dtype)) {
        set_error("%s: null pointer, empty shape or bad dtype", who);
        return BT_ERR_INVALID;
    }
    if (lda < K || K > 0x7fffffff || B > 0x7fffffff) {
        set_error("%s: row stride %lld below K=%lld, or shape beyond 2^31", who, (long long)lda, (long long)K);
        return BT_ERR_INVALID;
    }
    if (!H && !Q) {
        set_error("%s: no output requested (H and Q both null)", who);
        return BT_ERR_INVALID;
    }
    if (Q && !s_x) {
        set_error("%s: Q given without s_x", who);
        return BT_ERR_INVALID;
    }
    return BT_OK;
}

extern "C" int bt_swiglu(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up, int dtype, int64_t B,
                         int64_t K, void* H, int8_t* Q, float* s_x, int q_layout, void* stream) {
    const char* who = "bt_swiglu";
    int rc = check_row_op(who, gate, dtype, B, K, ld_gate, H, Q, s_x);
    if (rc) return rc;
    if (!up || ld_up < K) {
        set_error("%s: up is null or its row stride is below K", who);
        return BT_ERR_INVALID;
    }
    if (Q && (rc = check_q_layout(who, q_layout, K, Q, nullptr))) return rc;
    return launch_row_op(0, dtype, gate, ld_gate, up, ld_up, 0.0f, B, K, H, Q, s_x, q_layout, nullptr, (hipStream_t)stream, who);
}

extern "C" int bt_swiglu_rowsum(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up, int dtype, int64_t B,
                                int64_t K, void* H, int8_t* Q, float* s_x, int32_t* q_rowsum, int q_layout, void* stream) {
    const char* who = "bt_swiglu_rowsum";
    int rc = check_row_op(who, gate, dtype, B, K, ld_gate, H, Q, s_x);
    if (rc) return rc;
    if (!up || ld_up < K || !Q || !q_rowsum) {
        set_error("%s: up, Q or q_rowsum is null, or up's row stride is below K", who);
        return BT_ERR_INVALID;
    }
    if ((rc = check_q_layout(who, q_layout, K, Q, nullptr))) return rc;
    return launch_row_op(0, dtype, gate, ld_gate, up, ld_up, 0.0f, B, K, H, Q, s_x, q_layout, q_rowsum, (hipStream_t)stream, who);
}

extern "C" int bt_rmsnorm(const void* X, int64_t ld_x, const void* weight, float eps, int dtype, int64_t B,
                          int64_t K, void* Y, int8_t* Q, float* s_x, int q_layout, void* stream) {
    const char* who = "bt_rmsnorm";
    int rc = check_row_op(who, X, dtype, B, K, ld_x, Y, Q, s_x);
    if (rc) return rc;
    if (Q && (rc = check_q_layout(who, q_layout, K, Q, nullptr))) return rc;
    return launch_row_op(1, dtype, X, ld_x, weight, 0, eps, B, K, Y, Q, s_x, q_layout, nullptr, (hipStream_t)stream, who);
}

extern "C" int bt_rmsnorm_rowsum(const void* X, int64_t ld_x, const void* weight, float eps, int dtype, int64_t B,
                                 int64_t K, void* Y, int8_t* Q, float* s_x, int32_t* q_rowsum, int q_layout, void* stream) {
    const char* who = "bt_rmsnorm_rowsum";
    int rc = check_row_op(who, X, dtype, B, K, ld_x, Y, Q, s_x);
    if (rc) return rc;
    if (!Q || !q_rowsum) {
        set_error("%s: Q or q_rowsum is null", who);
        return BT_ERR_INVALID;
    }
    if ((rc = check_q_layout(who, q_layout, K, Q, nullptr))) return rc;
    return launch_row_op(1, dtype, X, ld_x, weight, 0, eps, B, K, Y, Q, s_x, q_layout, q_rowsum, (hipStream_t)stream, who);
}

// ---- packed forward with an activation prologue -----------------------------------------------
extern "C" size_t bt_packed_forward_fused_workspace_bytes(int64_t B, int64_t N, int64_t K, int x_dtype) {
    if (B <= 0 || N <= 0 || K <= 0 || !valid_dtype(x_dtype)) return 0;
    // [the prologue's output, B x K in x_dtype, when it runs as its own kernel][the forward's own scratch]
    return align256((size_t)B * K * dtype_size(x_dtype)) + bt_packed_forward_workspace_bytes(B, N, K, x_dtype);
}

static int fused_forward_impl(const char* who, const void* X, int64_t ld_x, int x_dtype, int pro_op, const void* pro_b,
                              int64_t ld_b, float eps, const uint8_t* W_T, int w_layout, int epi_op, const void* scale,
                              int scale_dtype, int64_t scale_len, const void* bias, int bias_dtype,
                              const void* residual, void* Y, int64_t B, int64_t N, int64_t K, void* workspace,
                              size_t workspace_bytes, void* stream) {
    int rc = check_shape(who, X, W_T, Y, x_dtype, B, N, K);
    if (rc) return rc;
    if (pro_op != 1 && pro_op != 2) {
        set_error("%s: prologue must be BT_PRO_RMSNORM or BT_PRO_SWIGLU (got %d)", who, pro_op);
        return BT_ERR_INVALID;
    }
    if (pro_op == PRO_SWIGLU && epi_op != EPI_NONE) {
        set_error("%s: a SwiGLU prologue and the SwiGLU output stage do not combine", who);
        return BT_ERR_INVALID;
    }
    if (ld_x < K || (pro_op == 2 && (!pro_b || ld_b < K))) {
        set_error("%s: row stride below K, or SwiGLU without its second operand", who);
        return BT_ERR_INVALID;
    }
    hipStream_t st = (hipStream_t)stream;
    // one 16-bit row on the streaming kernel: the prologue runs inside the GEMV, on the row's way into LDS
    const bool streams = layout_tiled(w_layout) ? (stream_supported_tiled(N, K, W_T) && fast_path_ok(Y, N, K))
                                                      : packed_uses_stream(x_dtype, W_T, Y, N, K);
    // a row that takes the exact fp16 GEMV gets its prologue inside that kernel (same element arithmetic as the row
    // kernel, so the result equals the unfused sequence bit for bit), or from the row kernel where that is switched off
    if (B == 1 && !tuning_env("BITTORCH_NO_PROLOGUE") && ((uintptr_t)pro_b) % 16 == 0 && (pro_b || pro_op == PRO_RMSNORM) &&
        streams && planes_supported(x_dtype, x_dtype, B, N, K, X, W_T, Y, w_layout)) {
        if (epi_op != 0 && (epi_op != EPI_SWIGLU_PAIRS || w_layout != W_LAYOUT_TILED || N % 32 != 0 || residual)) {
            set_error("%s: the SwiGLU output stage needs pair-ordered tiled weights, N %% 32 == 0 and no residual", who);
            return BT_ERR_INVALID;
        }
        Epilogue epi;
        rc = make_epilogue(who, scale, scale_dtype, scale_len, bias, bias_dtype, N, &epi);
        if (rc) return rc;
        rc = set_residual(who, residual, &epi);
        if (rc) return rc;
        return launch_planes(X, W_T, w_layout, epi, Y, N, K, epi_op, st, pro_op, pro_b, eps);
    }
    const size_t h_need = align256((size_t)B * K * dtype_size(x_dtype));
    const bool two_step_ok = workspace && workspace_bytes >= h_need && ((uintptr_t)workspace) % 256 == 0;
    const bool exact_row = two_step_ok && planes_supported(x_dtype, x_dtype, B, N, K, workspace, W_T, Y, w_layout);
    if (x_dtype != BT_F32 && B == 1 && streams && !exact_row) {
        const int mode = (x_dtype == BT_F16) ? MODE_F16 : MODE_BF16;
        if (stream_prologue_fusable(mode, B, N, K, X, pro_b, w_layout, epi_op)) {
            Epilogue epi;
            rc = make_epilogue(who, scale, scale_dtype, scale_len, bias, bias_dtype, N, &epi);
            if (rc) return rc;
            rc = set_residual(who, residual, &epi);
            if (rc) return rc;
            return launch_stream(mode, X, 2, nullptr, W_T, w_layout, epi, Y, x_dtype, nullptr, B, N, K, 1, Q_ROW_MAJOR, pro_op,
                                 pro_b, eps, epi_op, st);
        }
    }
    // otherwise: the prologue as its own kernel into the workspace, then the plain forward
    const size_t h_bytes = align256((size_t)B * K * dtype_size(x_dtype));
    if (!workspace || workspace_bytes < h_bytes || ((uintptr_t)workspace) % 256 != 0) {
        set_error("%s: workspace of %zu bytes (256-byte aligned) needed, %zu given", who,
                  bt_packed_forward_fused_workspace_bytes(B, N, K, x_dtype), workspace_bytes);
        return BT_ERR_WORKSPACE;
    }
    rc = launch_row_op(pro_op == 2 ? 0 : 1, x_dtype, X, ld_x, pro_b, ld_b, eps, B, K, workspace, nullptr, nullptr,
                       Q_ROW_MAJOR, nullptr, st, who);
    if (rc) return rc;
    return packed_forward_impl(who, workspace, x_dtype, W_T, w_layout, epi_op, scale, scale_dtype, scale_len, bias, bias_dtype,
                               residual, Y, B, N, K, (uint8_t*)workspace + h_bytes, workspace_bytes - h_bytes, stream);
}

extern "C" int bt_ternary_linear_packed_forward_fused(const void* X, int64_t ld_x, int x_dtype, int pro_op,
                                                      const void* pro_b, int64_t ld_b, float eps,
                                                      const uint8_t* W_T, const void* scale, int scale_dtype,
                                                      int64_t scale_len, const void* bias, int bias_dtype,
                                                      const void* residual, void* Y, int64_t B, int64_t N,
                                                      int64_t K, void* workspace, size_t workspace_bytes,
                                                      void* stream) {
    return fused_forward_impl("bt_ternary_linear_packed_forward_fused", X, ld_x, x_dtype, pro_op, pro_b, ld_b, eps, W_T,
                              W_LAYOUT_ROW_MAJOR, 0, scale, scale_dtype, scale_len, bias, bias_dtype, residual, Y, B, N, K,
                              workspace, workspace_bytes, stream);
}

// ---- decode-tiled copy of the packed weights ---------------------------------------------------
extern "C" size_t bt_tiled_weights_bytes(int64_t N, int64_t K) {
    if (N <= 0 || K <= 0) return 0;
    return tiled_bytes(N, K);
}

static int check_retile(const char* who, const void* a, const void* b, int64_t N, int64_t K, const void* tiled) {
    if (!a || !b || N <= 0 || K <= 0) {
        set_error("%s: null pointer or empty shape", who);
        return BT_ERR_INVALID;
    }
    if (((uintptr_t)tiled) % 256 != 0 || tiled_bytes(N, K) >= (1ull << 32)) {
        set_error("%s: the tiled copy must be 256-byte aligned and below 4 GiB", who);
        return BT_ERR_INVALID;
    }
    return BT_OK;
}

static int check_tile_order(const char* who, int order, int64_t N) {
    if (order == 0 || (order == 1 && N % 32 == 0)) return BT_OK;
    set_error("%s: tile order must be BT_TILES_NATURAL, or BT_TILES_GATE_UP_PAIRS with N %% 32 == 0 (order=%d, N=%lld)",
              who, order, (long long)N);
    return BT_ERR_INVALID;
}

extern "C" int bt_retile_weights(const uint8_t* W_T, int64_t N, int64_t K, int order, uint8_t* W_tiled, void* stream) {
    int rc = check_retile("bt_retile_weights", W_T, W_tiled, N, K, W_tiled);
    if (rc) return rc;
    if ((rc = check_tile_order("bt_retile_weights", order, N))) return rc;
    return launch_retile(W_T, N, K, order, W_tiled, false, nullptr, (hipStream_t)stream);
}

extern "C" int bt_untile_weights(const uint8_t* W_tiled, int64_t N, int64_t K, int order, uint8_t* W_T, void* stream) {
    int rc = check_retile("bt_untile_weights", W_tiled, W_T, N, K, W_tiled);
    if (rc) return rc;
    if ((rc = check_tile_order("bt_untile_weights", order, N))) return rc;
    return launch_retile(nullptr, N, K, order, (void*)W_tiled, true, W_T, (hipStream_t)stream);
}

extern "C" int bt_ternary_linear_tiled_forward(const void* X, int64_t ld_x, int x_dtype, int pro_op,
                                               const void* pro_b, int64_t ld_b, float eps, const uint8_t* W_tiled,
                                               const void* scale, int scale_dtype, int64_t scale_len,
                                               const void* bias, int bias_dtype, const void* residual, int epi_op,
                                               void* Y, int64_t B, int64_t N, int64_t K, void* workspace,
                                               size_t workspace_bytes, void* stream) {
    const char* who = "bt_ternary_linear_tiled_forward";
    int w_layout = W_LAYOUT_TILED;
    if (epi_op == EPI_NATURAL_FROM_PAIRS) {  // a copy in gate/up pair order, the plain linear output in natural column order
        if (N % 32 != 0) {
            set_error("%s: a pair-ordered tiled copy has N %% 32 == 0 (N=%lld)", who, (long long)N);
            return BT_ERR_INVALID;
        }
        w_layout = W_LAYOUT_TILED_PAIRS_AS_NATURAL;
        epi_op = EPI_NONE;
    }
    if (pro_op != 0)
        return fused_forward_impl(who, X, ld_x, x_dtype, pro_op, pro_b, ld_b, eps, W_tiled, w_layout, epi_op, scale,
                                  scale_dtype, scale_len, bias, bias_dtype, residual, Y, B, N, K, workspace,
                                  workspace_bytes, stream);
    if (ld_x != K) {
        set_error("%s: without a prologue the activation rows must be contiguous (ld_x=%lld, K=%lld)", who,
                  (long long)ld_x, (long long)K);
        return BT_ERR_INVALID;
    }
    return packed_forward_impl(who, X, x_dtype, W_tiled, w_layout, epi_op, scale, scale_dtype, scale_len, bias, bias_dtype,
                               residual, Y, B, N, K, workspace, workspace_bytes, stream);
}

extern "C" int bt_ternary_gemm_i8_tiled(const int8_t* Q, int q_layout, const float* s_x, const uint8_t* W_tiled,
                                        const void* scale, int scale_dtype, int64_t scale_len, const void* bias,
                                        int bias_dtype, const void* residual, void* Y, int y_dtype, int32_t* acc_out,
                                        int64_t B, int64_t N, int64_t K, void* stream) {
    return gemm_i8_impl("bt_ternary_gemm_i8_tiled", Q, q_layout, s_x, W_tiled, W_LAYOUT_TILED, scale, scale_dtype,
                        scale_len, bias, bias_dtype, residual, Y, y_dtype, acc_out, B, N, K, stream);
}

// ---- the prefill-only field layout of the tiled copy ----------------------------------------------------------------
extern "C" int bt_retile_fields(const uint8_t* W_tiled, int64_t N, int64_t K, uint8_t* W_fields, void* stream) {
    int rc = check_retile("bt_retile_fields", W_tiled, W_fields, N, K, W_tiled);
    if (rc) return rc;
    if (((uintptr_t)W_fields) % 256 != 0) {
        set_error("bt_retile_fields: W_fields must be 256-byte aligned");
        return BT_ERR_INVALID;
    }
    return launch_retile_fields(W_tiled, N, K, W_fields, (hipStream_t)stream);
}

extern "C" int bt_ternary_gemm_i8_fields(const int8_t* Q, int q_layout, const float* s_x, const int32_t* q_rowsum,
                                         const uint8_t* W_fields, int tile_order, const void* scale, int scale_dtype,
                                         int64_t scale_len, const void* bias, int bias_dtype, const void* residual,
                                         void* Y, int y_dtype, int32_t* acc_out, int64_t B, int64_t N, int64_t K,
                                         void* stream) {
    const char* who = "bt_ternary_gemm_i8_fields";
    int rc = check_shape(who, Q, W_fields, Y, y_dtype, B, N, K);
    if (rc) return rc;
    if (!s_x || !q_rowsum) {
        set_error("%s: s_x or q_rowsum is null", who);
        return BT_ERR_INVALID;
    }
    rc = check_q_layout(who, q_layout, K, Q, nullptr);
    if (rc) return rc;
    if ((rc = check_tile_order(who, tile_order, N))) return rc;
    if (K % 128 != 0 || K > kMaxKInt8) {
        set_error("%s: K must be a multiple of 128 and at most %lld (K=%lld); other shapes take the decode-tiled copy", who,
                  (long long)kMaxKInt8, (long long)K);
        return BT_ERR_INVALID;
    }
    if (!fast_path_ok(Y, N, K) || (acc_out && ((uintptr_t)acc_out) % 16 != 0) || !stream_supported_tiled(N, K, W_fields) ||
        !gemm_i8_supported_tiled(N, K, Q)) {
        set_error("%s: N %% 4 == 0, 16-byte aligned Q, Y and acc_out and a 256-byte aligned copy below 4 GiB are needed", who);
        return BT_ERR_INVALID;
    }
    Epilogue epi;
    rc = make_epilogue(who, scale, scale_dtype, scale_len, bias, bias_dtype, N, &epi);
    if (rc) return rc;
    rc = set_residual(who, residual, &epi);
    if (rc) return rc;
    return launch_gemm_i8(Q, q_layout, s_x, q_rowsum, W_fields,
                          tile_order ? W_LAYOUT_TILED_FIELDS_PAIRS_AS_NATURAL : W_LAYOUT_TILED_FIELDS, epi, Y, y_dtype, acc_out,
                          B, N, K, (hipStream_t)stream);
}
