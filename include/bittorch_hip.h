/*
 * C ABI of libbittorch_hip.so: the MI355X (gfx950) ternary-linear backend.
 *
 * Plain pointers and sizes only; no C++ or torch types cross this boundary.
 * All pointers except the optional ones are DEVICE pointers owned by the
 * caller; the library never allocates or frees device memory and keeps no
 * mutable global state besides the option table of bt_set_option, so calls on
 * different streams are independent.
 * Kernels are enqueued on `stream` (a hipStream_t passed as void*; NULL is
 * the default stream) and the call returns without synchronising.
 *
 * Every function returns 0 on success or a negative bt_status; the text of
 * the last failure on the calling thread is available from bt_last_error().
 *
 * Entry points replace the reference's pybind11 module `bittorch._C`
 * (csrc/bindings/bittorch_bindings.cpp:34-88) and the host dispatch behind it
 * (csrc/core/dispatch.cpp:52-142); each declaration cites what it replaces.
 */
#ifndef BITTORCH_HIP_H
#define BITTORCH_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BT_ABI_VERSION 2

/* element types of activations / scales / biases / outputs */
typedef enum { BT_F32 = 0, BT_F16 = 1, BT_BF16 = 2, BT_I8 = 3 /* bt_unpack_dequant output only */ } bt_dtype;

typedef enum {
    BT_OK = 0,
    BT_ERR_INVALID = -1,   /* bad shape / dtype / null pointer */
    BT_ERR_WORKSPACE = -2, /* workspace too small */
    BT_ERR_LAUNCH = -3     /* HIP reported a launch error */
} bt_status;

/*
 * Workspaces.  The library allocates nothing: an entry point that needs device
 * scratch takes a caller-provided `workspace` of at least the number of bytes its
 * *_workspace_bytes() query returns for the same shape (0 means none is needed and
 * NULL may be passed).  A workspace needs no initialisation and carries nothing
 * from one call to the next; two calls that may run concurrently (different
 * streams) need different workspaces.  Workspaces must be 256-byte aligned.
 * At present bt_ternary_linear_tensor_core_forward uses one (the int8 activations
 * and their row scales) and bt_ternary_linear_packed_forward uses one for fp32
 * activations (three bf16 planes); bt_ternary_gemm_i8 keeps the argument so that a
 * kernel that needs scratch can be introduced without an ABI change.
 */
/* ABI version of the loaded library (BT_ABI_VERSION at build time). */
int bt_abi_version(void);

/* Message of the last failure on this thread ("" if none). */
const char* bt_last_error(void);

/*
 * Run-time options.  The library has a small set of documented switches (kernel choice for tests, benchmarks and
 * tuning runs): STREAM_MAX_ROWS, GEMM_LONG_EPILOGUE, GEMM_TAIL_SPLIT, GROUP_WALK, GROUP_NACC, GROUP_UNITS,
 * PLANES_NACC, ROWOP_GENERIC, STREAM_CFG, NO_PLANES.  Each takes its initial value from the environment variable
 * BITTORCH_<NAME>, read once per process on the first call that consults an option; bt_set_option overrides it from
 * then on (value NULL: not set; name NULL: every option not set).  `name` may carry the BITTORCH_ prefix.  Not to be
 * called while another thread is inside the library.  BITTORCH_KERNEL (auto | generic) is not one of them: like the
 * reference (csrc/kernels/ternary_gemm_production.cu:262-273) the library reads it from the environment on every
 * call.  No counterpart in the reference, which has that one switch only.
 */
int bt_set_option(const char* name, const char* value);

/*
 * Fused ternary quantize + 2-bit pack.
 * Replaces the torch op chains of bittorch/quant/ternary.py:122-142
 * (absmax scale, threshold, sign) and bittorch/quant/ternary_packed.py:50-73,
 * :202-206 (encode, pack, transpose) with one pass over the master weights.
 *
 *   W          [N,K] row-major master weights of type w_dtype
 *   packed_T   [ceil(K/4), N] uint8 out, byte [kb,n] = W[n,4kb..4kb+3] codes
 *              (+1 -> 1, -1 -> 2, 0 -> 0; element i in bits 2i..2i+1)
 *   scale      fp32 out: [N] row absmax (per_channel != 0) or [1] tensor absmax,
 *              floored at 1e-8 rounded to w_dtype
 *   w_tern     optional [N,K] int8 out with the ternary values (may be NULL)
 *   packed_T may be NULL if only scale / w_tern are wanted.
 */
int bt_quantize_pack(const void* W, int w_dtype, int64_t N, int64_t K, double threshold_factor,
                     int per_channel, uint8_t* packed_T, float* scale, int8_t* w_tern,
                     void* stream);

/*
 * Unpacked-weight forward: Y = X @ (W_tern * scale).T + bias, fp32 accumulate.
 * Replaces bittorch._C.ternary_linear_forward (bittorch_bindings.cpp:41-46,
 * dispatch.cpp:52-87, csrc/kernels/ternary_gemm.cu:206-279).
 *   X [B,K] x_dtype, W_tern [N,K] int8, Y [B,N] x_dtype.
 *   scale: scale_len entries (N, or 1 = broadcast) of scale_dtype.
 *   bias: NULL or N entries of bias_dtype.
 */
int bt_ternary_linear_forward(const void* X, int x_dtype, const int8_t* W_tern, const void* scale,
                              int scale_dtype, int64_t scale_len, const void* bias, int bias_dtype,
                              void* Y, int64_t B, int64_t N, int64_t K, void* stream);

/*
 * Packed-weight forward with fp32 accumulation (decode GEMV / small batch / any B).
 * Replaces bittorch._C.ternary_linear_packed_forward (bittorch_bindings.cpp:48-63,
 * dispatch.cpp:105-142, csrc/kernels/ternary_gemm_production.cu:286-362).
 *   X [B,K] x_dtype; W_T [ceil(K/4),N] uint8; Y [B,N] x_dtype.
 *   A cost model fitted to measurements picks the kernel: the streaming kernel (weights read once
 *   per 16 rows, all 16-row blocks of the call in one launch) while B*N*K is small, the tiled 16-bit
 *   matrix-core GEMM beyond (crossover near 1.5-2 M outputs for K = 2560..4096;
 *   the option STREAM_MAX_ROWS = n replaces the rule by "B <= n").  A single fp16 row (K % 16 == 0,
 *   K <= 16384, N % 4 == 0) runs the exact GEMV on the int8 matrix cores: the dot products are summed
 *   without rounding and rounded to fp32 once.  fp32 activations (any K) are first split into
 *   three bf16 planes (x = hi + mid + lo exactly), each zero-padded to a multiple of 64 values, in
 *   the workspace and run on the same bf16 kernels with exact products and fp32 accumulation.
 *   Unaligned operands, a missing workspace and BITTORCH_KERNEL=generic run a generic
 *   kernel that accumulates in the reference's k order.
 *   workspace: at least bt_packed_forward_workspace_bytes(B,N,K,x_dtype) bytes
 *   (6*B*Kp rounded up to 256 for fp32, Kp = K rounded up to 64; 0 otherwise: may be NULL).
 */
size_t bt_packed_forward_workspace_bytes(int64_t B, int64_t N, int64_t K, int x_dtype);
int bt_ternary_linear_packed_forward(const void* X, int x_dtype, const uint8_t* W_T,
                                     const void* scale, int scale_dtype, int64_t scale_len,
                                     const void* bias, int bias_dtype, void* Y, int64_t B,
                                     int64_t N, int64_t K, void* workspace, size_t workspace_bytes,
                                     void* stream);

/*
 * Per-row int8 activation quantizer (whole-row absmax scale).
 * Restates the activation stage of kernel_v2_tensor_core
 * (csrc/kernels/ternary_gemm_tensor_core.cu:431-459, :343-347):
 *   s_x[b] = amax > 1e-6 ? amax/127 : 1;  Q = clamp(roundf(X * (1/s_x)), -127, 127)
 *   X [B,K] x_dtype -> Q [B,K] int8, s_x [B] fp32.
 */
int bt_act_quant_i8(const void* X, int x_dtype, int64_t B, int64_t K, int8_t* Q, float* s_x,
                    void* stream);

/*
 * Layout of quantized activations between a quantizing kernel and an int8 GEMM (no counterpart in
 * the reference, whose kernel quantizes inside its own shared memory):
 *   BT_Q_ROW_MAJOR      int8 [B,K] as is (what bt_act_quant_i8 writes and bt_ternary_gemm_i8 reads);
 *   BT_Q_OPERAND_ORDER  the same rows with every aligned 16-byte group stored as the 4x4 byte
 *                       transpose of its natural order (byte 4c+r = element 4r+c): the k order the
 *                       in-register weight decode gives the matrix-core operands, so the GEMMs copy
 *                       activations to the matrix cores without permuting them (4 % faster at
 *                       2048x4096x4096).  Needs K % 16 == 0 and 16-byte aligned buffers.
 * A buffer must be read with the layout it was written in; bt_ternary_linear_tensor_core_forward
 * picks the operand order by itself for its private Q.
 */
enum { BT_Q_ROW_MAJOR = 0, BT_Q_OPERAND_ORDER = 1 };
int bt_act_quant_i8_layout(const void* X, int x_dtype, int64_t B, int64_t K, int8_t* Q, float* s_x,
                           int q_layout, void* stream);
/* The same, and q_rowsum [B] int32: the sum of each quantized row over K, which bt_ternary_gemm_i8_fields needs
 * (same arithmetic for Q and s_x: csrc/kernels/ternary_gemm_tensor_core.cu:343-347, :439; the sums have no
 * counterpart in the reference). */
int bt_act_quant_i8_rowsum(const void* X, int x_dtype, int64_t B, int64_t K, int8_t* Q, float* s_x, int32_t* q_rowsum,
                           int q_layout, void* stream);

/*
 * int8 x packed-ternary GEMM on the matrix cores, int32 accumulators.
 * Restates the MMA stage and epilogue of kernel_v2_tensor_core
 * (ternary_gemm_tensor_core.cu:583-589, :652): weights decode to +-127,
 *   y = (float(acc) * s_x[b] / 127.0f) * scale[n] + bias[n].
 *   Q [B,K] int8, s_x [B] fp32, W_T [ceil(K/4),N] uint8, Y [B,N] y_dtype.
 *   acc_out: optional [B,N] int32 copy of the raw accumulators (may be NULL).
 *   workspace: at least bt_gemm_i8_workspace_bytes(B,N,K) bytes (currently 0: may be NULL).
 *   K <= 132096 (the int8 entry points all refuse a longer K: 127*127*K must fit the int32 accumulators and
 *   127*K the 24 significand bits of the accumulator's conversion to fp32).
 */
size_t bt_gemm_i8_workspace_bytes(int64_t B, int64_t N, int64_t K);
int bt_ternary_gemm_i8(const int8_t* Q, const float* s_x, const uint8_t* W_T, const void* scale,
                       int scale_dtype, int64_t scale_len, const void* bias, int bias_dtype,
                       void* Y, int y_dtype, int32_t* acc_out, int64_t B, int64_t N, int64_t K,
                       void* workspace, size_t workspace_bytes, void* stream);

/*
 * The two GEMM entry points above with a residual connection folded into the epilogue:
 *   Y = rd( rd(linear) + residual ),   rd = round to Y's dtype
 * i.e. exactly the two roundings of "y = linear(x); y = y + residual" in that dtype.  They have no
 * counterpart in the reference's Python/CUDA code; they serve the pre-norm block of its JS
 * runtime (js/src/models/TernaryTransformer.ts:489-521: x = x + attn(norm(x)); x = x + mlp(norm(x))).
 *   residual: [B,N] in Y's dtype, 16-byte aligned; NULL = no residual (the plain entry point).
 *   q_layout (int8 variant): layout Q was written in.
 *   It may be Y itself (every output element is read once, by the thread that then writes it).
 */
int bt_ternary_linear_packed_forward_res(const void* X, int x_dtype, const uint8_t* W_T,
                                         const void* scale, int scale_dtype, int64_t scale_len,
                                         const void* bias, int bias_dtype, const void* residual,
                                         void* Y, int64_t B, int64_t N, int64_t K, void* workspace,
                                         size_t workspace_bytes, void* stream);
int bt_ternary_gemm_i8_res(const int8_t* Q, int q_layout, const float* s_x, const uint8_t* W_T, const void* scale,
                           int scale_dtype, int64_t scale_len, const void* bias, int bias_dtype,
                           const void* residual, void* Y, int y_dtype, int32_t* acc_out, int64_t B,
                           int64_t N, int64_t K, void* stream);

/*
 * Fused producers of the GEMMs' activations (no counterpart in the reference's Python/CUDA code;
 * block structure of its JS runtime, TernaryTransformer.ts:366-423 and :489-521).  One pass over
 * the rows computes the value, optionally stores it in the input dtype (H / Y) and optionally
 * quantizes it per row exactly as bt_act_quant_i8 would quantize the stored tensor (Q, s_x): at
 * least one of the two outputs must be requested.  rd = round to dtype, fp32 arithmetic, every
 * operation rounded on its own:
 *   bt_swiglu:  h = rd( rd( g / (1 + exp(-g)) ) * u )       gate, up [B,K] with row strides
 *               ld_gate, ld_up (elements; lets both halves of one [B,2K] GEMM output be read in
 *               place); exp is a fixed fp32 polynomial (0.85 ulp), restated by the CPU oracle.
 *   bt_rmsnorm: y = rd( (x * r) * w ),  r = 1/sqrt(float(sum double(x)^2)/K + eps)
 *               weight [K] in the same dtype or NULL (ones).
 *   q_layout: layout of Q (BT_Q_ROW_MAJOR / BT_Q_OPERAND_ORDER, see bt_act_quant_i8_layout).
 */
int bt_swiglu(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up, int dtype, int64_t B,
              int64_t K, void* H, int8_t* Q, float* s_x, int q_layout, void* stream);
int bt_rmsnorm(const void* X, int64_t ld_x, const void* weight, float eps, int dtype, int64_t B,
               int64_t K, void* Y, int8_t* Q, float* s_x, int q_layout, void* stream);
/* The same with Q required and q_rowsum [B] int32, the rows' sums of Q, as a further output (for
 * bt_ternary_gemm_i8_fields; see bt_act_quant_i8_rowsum). */
int bt_swiglu_rowsum(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up, int dtype, int64_t B,
                     int64_t K, void* H, int8_t* Q, float* s_x, int32_t* q_rowsum, int q_layout, void* stream);
int bt_rmsnorm_rowsum(const void* X, int64_t ld_x, const void* weight, float eps, int dtype, int64_t B,
                      int64_t K, void* Y, int8_t* Q, float* s_x, int32_t* q_rowsum, int q_layout, void* stream);

/*
 * Packed forward with an activation prologue (no counterpart in the reference's Python/CUDA code;
 * pre-norm block and SwiGLU MLP of its JS runtime, TernaryTransformer.ts:489-521, :366-423):
 *   Y = linear( pro(X) ) [+ residual],   pro = BT_PRO_RMSNORM: rmsnorm(X; weight = pro_b or ones, eps)
 *                                        pro = BT_PRO_SWIGLU:  silu(X) * pro_b   (X = gate, pro_b = up)
 * with exactly the values bt_rmsnorm / bt_swiglu would store in x_dtype.  For a single 16-bit row
 * (one decode token) the prologue runs inside the GEMV kernel (the exact fp16 GEMV or the streaming kernel,
 * whichever the plain forward would take), on the row's way into LDS, and saves a launch; every other
 * shape runs the prologue kernel into the workspace and then the plain forward.
 *   X [B,K] with row stride ld_x, pro_b [K] (RMSNorm, may be NULL) or [B,K] with row stride ld_b (SwiGLU).
 *   workspace: at least bt_packed_forward_fused_workspace_bytes(B,N,K,x_dtype) bytes.
 */
enum { BT_PRO_NONE = 0, BT_PRO_RMSNORM = 1, BT_PRO_SWIGLU = 2 };
size_t bt_packed_forward_fused_workspace_bytes(int64_t B, int64_t N, int64_t K, int x_dtype);
int bt_ternary_linear_packed_forward_fused(const void* X, int64_t ld_x, int x_dtype, int pro_op,
                                           const void* pro_b, int64_t ld_b, float eps,
                                           const uint8_t* W_T, const void* scale, int scale_dtype,
                                           int64_t scale_len, const void* bias, int bias_dtype,
                                           const void* residual, void* Y, int64_t B, int64_t N,
                                           int64_t K, void* workspace, size_t workspace_bytes,
                                           void* stream);

/*
 * Decode-tiled copy of the packed weights (no counterpart in the reference, whose kernels read
 * W_T [Kb, N] of bittorch/quant/ternary_packed.py:174-206 only).  A decode-shape kernel gives every
 * compute unit a 16-column tile; in the row-major W_T such a tile touches 16 bytes of each 128-byte
 * line.  The tiled copy stores, for tile t = n / 16 and step s = kb / 16 (S = ceil(Kb / 16) steps), 64
 * dwords: dword ((t * S + s) * 64 + 16 g + j) holds the bytes W_T[16 s + 4 g + r, 16 t + j], r = 0..3,
 * low byte first (= 16 consecutive k of one output column), zero outside the matrix.  It is built
 * once from W_T (bt_retile_weights, exact inverse bt_untile_weights) and holds
 * bt_tiled_weights_bytes(N, K) = ceil(N/16) * S * 256 bytes, 256-byte aligned, below 4 GiB.
 *   order: BT_TILES_NATURAL, or BT_TILES_GATE_UP_PAIRS (N % 32 == 0) for a layer whose columns are
 *     [gate | up] of a SwiGLU MLP: tile 2P of the copy is tile P of the matrix, tile 2P + 1 is tile
 *     N/32 + P, so that one workgroup holds column h of both halves.
 *   bt_ternary_linear_tiled_forward: bt_ternary_linear_packed_forward_fused on the tiled copy, with
 *     pro_op = BT_PRO_NONE allowed (then ld_x must equal K); the weights are streamed once per 16
 *     rows of X, so it is meant for decode shapes; fp32 X needs the workspace.
 *     Results equal those of the row-major entry points bit for bit wherever both layouts take the same kernel
 *     (always up to 32 rows); a larger batch near the crossover between the streaming kernel and the tiled GEMM
 *     may be routed differently on the tiled copy (its remainder tiles are cheaper), and the two kernels add the
 *     fp32 partial sums in different orders.
 *     epi_op = BT_EPI_SWIGLU_PAIRS (pair-ordered copy, no residual, no SwiGLU prologue): Y is [B, N/2],
 *     Y[b, h] = what bt_swiglu makes of the stored projections, rd(rd(silu(g)) * u) with g = rd(linear
 *     column h), u = rd(linear column N/2 + h): the SwiGLU MLP's hidden vector leaves the gate|up kernel
 *     itself (structure: TernaryTransformer.ts:366-423).
 *     epi_op = BT_EPI_NATURAL_FROM_PAIRS (pair-ordered copy): Y is the plain linear output [B, N] in the matrix's
 *     natural column order, every kernel looking its column tiles up where the pair order put them; bit-identical
 *     to the same call on a natural-order copy.  With the two, one pair-ordered copy serves every call of a fused
 *     [gate | up] layer in 16-bit and fp32 activations (the int8 entry point reads natural-order copies only).
 *   bt_ternary_gemm_i8_tiled: bt_ternary_gemm_i8_res on the tiled copy (same remark).
 *   A tall batch on the tiled copy may take two kernel launches on the stream instead of one (the column tiles of
 *   a mostly empty last round of 128 x 256 tiles run as tiles of 64 or 32 rows behind the whole tiles): same
 *   results, nothing for the caller to do; both launches are captured by a HIP graph like any other.
 */
enum { BT_TILES_NATURAL = 0, BT_TILES_GATE_UP_PAIRS = 1 };
enum { BT_EPI_NONE = 0, BT_EPI_SWIGLU_PAIRS = 1, BT_EPI_NATURAL_FROM_PAIRS = 2 };
size_t bt_tiled_weights_bytes(int64_t N, int64_t K);
int bt_retile_weights(const uint8_t* W_T, int64_t N, int64_t K, int order, uint8_t* W_tiled, void* stream);
int bt_untile_weights(const uint8_t* W_tiled, int64_t N, int64_t K, int order, uint8_t* W_T, void* stream);
int bt_ternary_linear_tiled_forward(const void* X, int64_t ld_x, int x_dtype, int pro_op, const void* pro_b,
                                    int64_t ld_b, float eps, const uint8_t* W_tiled, const void* scale,
                                    int scale_dtype, int64_t scale_len, const void* bias, int bias_dtype,
                                    const void* residual, int epi_op, void* Y, int64_t B, int64_t N, int64_t K,
                                    void* workspace, size_t workspace_bytes, void* stream);
int bt_ternary_gemm_i8_tiled(const int8_t* Q, int q_layout, const float* s_x, const uint8_t* W_tiled,
                             const void* scale, int scale_dtype, int64_t scale_len, const void* bias,
                             int bias_dtype, const void* residual, void* Y, int y_dtype, int32_t* acc_out,
                             int64_t B, int64_t N, int64_t K, void* stream);

/*
 * A prefill-only second form of the tiled copy, for the matrix-core int8 GEMM alone (no counterpart in the
 * reference; the arithmetic is its int8 kernel's, csrc/kernels/ternary_gemm_tensor_core.cu:343-347, :439, :583-589,
 * :652, and the results equal bt_ternary_gemm_i8_tiled bit for bit, int32 accumulators included).  Same size and
 * alignment as the tiled copy (bt_tiled_weights_bytes); inside every aligned 16 bytes the 2-bit fields are
 * transposed so that a byte holds one k of FOUR columns, three of them as w + 1 and one in two's complement, and
 * the GEMM's operand of a column block is one AND of a loaded dword instead of a mask and a byte permute.  What
 * the codes w + 1 add to a dot product is the row's sum of q, which the caller supplies (bt_act_quant_i8_rowsum).
 *   bt_retile_fields: W_tiled (natural or pair-ordered, the order is kept) -> W_fields.
 *   bt_ternary_gemm_i8_fields: always the tiled GEMM kernel (meant for prefill batches: hundreds of rows and more);
 *     K % 128 == 0; tile_order BT_TILES_GATE_UP_PAIRS reads a pair-ordered copy and writes Y in the matrix's natural
 *     column order; otherwise the arguments of bt_ternary_gemm_i8_tiled.
 */
int bt_retile_fields(const uint8_t* W_tiled, int64_t N, int64_t K, uint8_t* W_fields, void* stream);
int bt_ternary_gemm_i8_fields(const int8_t* Q, int q_layout, const float* s_x, const int32_t* q_rowsum,
                              const uint8_t* W_fields, int tile_order, const void* scale, int scale_dtype,
                              int64_t scale_len, const void* bias, int bias_dtype, const void* residual, void* Y,
                              int y_dtype, int32_t* acc_out, int64_t B, int64_t N, int64_t K, void* stream);

/*
 * G independent decode GEMVs in ONE launch (no counterpart in the reference, whose packed kernel
 * csrc/kernels/ternary_gemm_production.cu:53-142 serves one matrix per launch): unit u computes
 *   Y_tab[u] [N] = X_tab[u] [K] (fp16) x W_tiled_tab[u] (decode-tiled copy of a W_T [ceil(K/4), N]) * scale + bias
 * exactly as a single bt_ternary_linear_tiled_forward call on one row would (bit-identical outputs).  A
 * 4 MiB weight matrix takes less time to stream than a kernel takes to start and drain; this entry point
 * pays launch, set-up and drain once for G matrices: persistent workgroups each read a contiguous run
 * of the (unit, 16-column tile) sequence front to back, their waves splitting K (1040 <= K <= 4096 and
 * at least 16 tiles per workgroup; other shapes: (unit, column slab) items, a wave per tile column),
 * and keep their weight loads running from one unit into the next.  A handful of units (where a cost model
 * prices it lower) run the one-matrix kernel with one workgroup per (unit, column tile) instead.
 *   The five tables are DEVICE arrays of G device pointers, caller-owned (bias_tab may be NULL: no
 *   bias; its entries may not be NULL otherwise).  Every unit has the same N, K, scale length
 *   (N, or 1 = per-tensor) and element types.  x_dtype BT_F16: Y is fp16; K % 16 == 0, K <= 16384;
 *   each W_tiled 256-byte aligned, each X 16-byte aligned.  Units may share operands (one x for many
 *   matrices, one matrix for many rows) but not outputs.
 *   x_dtype BT_BF16 (Y bf16): the same shapes.  A bf16 row spans more binades than a fixed-point sum can hold, so each row is
 *   scaled by its own largest exponent: with E the (unbiased) exponent of the row's largest magnitude,
 *   element x becomes the integer round_half_up(|x| * 2^(39 - E)) with its sign (exact for every element
 *   whose exponent is within 32 of E, zero for those more than 40 below it), the integers are summed
 *   exactly on the int8 matrix cores as six base-128 digit rows, and acc = fp32(S) * 2^(E - 39) enters
 *   the usual epilogue y = bf16(fp32(acc * scale) + bias).  The result
 *   does not depend on the order of summation; against the fp32 sums of the other bf16 kernels it differs
 *   by the rounding of those sums (a few units of fp32 spacing), never by more.  A row holding Inf or NaN
 *   gives NaN outputs.  bt_ternary_linear_tiled_forward takes the same route for ONE bf16 row (B = 1, no
 *   prologue, epi_op = BT_EPI_NONE) times a matrix of at least 6144 column tiles of 16 (N >= 98304) within
 *   the same K range: a vocabulary projection.
 */
int bt_ternary_gemv_grouped(const void* const* X_tab, int x_dtype, const uint8_t* const* W_tiled_tab,
                            const void* const* scale_tab, int scale_dtype, int64_t scale_len,
                            const void* const* bias_tab, int bias_dtype, void* const* Y_tab, int64_t G,
                            int64_t N, int64_t K, void* stream);

/*
 * G independent small-batch int8 units in ONE launch (no counterpart in the reference, as above): unit u computes
 *   Y_tab[u] [M, N] = Q_tab[u] [M, K] (int8, row scales sx_tab[u] [M]) x W_tiled_tab[u] -> ((acc * s_x) / 127) * scale + bias
 * exactly as bt_ternary_gemm_i8_tiled would for that unit: int32 accumulators and outputs bit-identical (the
 * arithmetic of csrc/kernels/ternary_gemm_tensor_core.cu:343-347, :439, :583-589, :652 with the whole-row scale).
 * M <= 16 rows per unit, the same M, N, K, layouts and element types for every unit: batched decode steps through
 * several same-shaped layers (BASELINE config 3's shapes: 16 x 4096 -> 11008 and 16 x 11008 -> 4096).  Persistent
 * workgroups read the flat (unit, 16-column tile) sequence of the tiled copies front to back, their waves splitting
 * K; a wave keeps its K slice of the unit's 16 rows in registers for all of the unit's tiles, so the activations are
 * read once per workgroup and unit instead of once per workgroup and tile.
 *   The tables are DEVICE arrays of G device pointers, caller-owned; bias_tab and acc_tab may be NULL (no bias; no
 *   accumulator output), their entries may not be NULL otherwise.  q_layout as in bt_ternary_gemm_i8_res.
 *   K % 16 == 0, K <= 11264; each Q 16-byte aligned, each W_tiled 256-byte aligned; acc_tab[u] [M, N] int32 receives
 *   the accumulators (sum q * 127 w).  Units may share operands but not outputs.
 */
int bt_ternary_gemm_i8_grouped(const int8_t* const* Q_tab, int q_layout, const float* const* sx_tab,
                               const uint8_t* const* W_tiled_tab, const void* const* scale_tab, int scale_dtype,
                               int64_t scale_len, const void* const* bias_tab, int bias_dtype, void* const* Y_tab,
                               int y_dtype, int32_t* const* acc_tab, int64_t G, int64_t M, int64_t N, int64_t K,
                               void* stream);

/*
 * Matrix-core forward from float activations: bt_act_quant_i8 followed by
 * bt_ternary_gemm_i8.  Replaces bittorch._C.ternary_linear_tensor_core_forward
 * (bittorch_bindings.cpp:65-87, ternary_gemm_tensor_core.cu:663-727) for
 * version == 2; version == 1 (the reference's float-compute validation kernel,
 * :120-271) is served by bt_ternary_linear_packed_forward.
 *   workspace: at least bt_tensor_core_workspace_bytes(B,N,K) bytes; holds Q and s_x.
 */
size_t bt_tensor_core_workspace_bytes(int64_t B, int64_t N, int64_t K);
int bt_ternary_linear_tensor_core_forward(const void* X, int x_dtype, const uint8_t* W_T,
                                          const void* scale, int scale_dtype, int64_t scale_len,
                                          const void* bias, int bias_dtype, void* Y, int64_t B,
                                          int64_t N, int64_t K, void* workspace,
                                          size_t workspace_bytes, void* stream);

/*
 * bt_ternary_linear_tensor_core_forward for callers that cannot allocate device memory or pass a
 * workspace: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * It has no counterpart in the reference.  Same arguments and bit-identical results; the int8
 * activations and their row scales live in a device array inside the library
 * (BT_STATIC_SCRATCH_ACTIVATION_BYTES + 4 * BT_STATIC_SCRATCH_ROWS bytes, held by every GPU the
 * library runs on until the process ends) instead of a workspace.  The call allocates and frees
 * nothing.  Limits: B * K <= BT_STATIC_SCRATCH_ACTIVATION_BYTES and B <= BT_STATIC_SCRATCH_ROWS,
 * otherwise BT_ERR_WORKSPACE.  All calls on one GPU share the array: calls that may overlap on one
 * GPU (different streams, different host threads) race; the array needs no clearing between calls
 * (the quantizer writes everything the GEMM reads).  The first call on a device looks the array's
 * device address up (hipGetSymbolAddress): make that call outside a stream capture.
 */
#define BT_STATIC_SCRATCH_ACTIVATION_BYTES (16u << 20)
#define BT_STATIC_SCRATCH_ROWS 65536
int bt_ternary_linear_tensor_core_forward_static(const void* X, int x_dtype, const uint8_t* W_T,
                                                 const void* scale, int scale_dtype, int64_t scale_len,
                                                 const void* bias, int bias_dtype, void* Y, int64_t B,
                                                 int64_t N, int64_t K, void* stream);

/*
 * Packed weights -> dense ternary or effective weights, for the training
 * backward (grad_x = grad_y @ (w_tern * scale)) without keeping a dense copy
 * alive between forward and backward (the reference saves one,
 * bittorch/nn/ternary_linear_cuda.py:62-66).
 *   out [N,K] of out_dtype = decode(W_T) * scale[n]   (scale NULL -> plain decode;
 *   out_dtype BT_I8 -> the ternary values themselves, scale ignored)
 */
int bt_unpack_dequant(const uint8_t* W_T, const float* scale, int64_t scale_len, void* out,
                      int out_dtype, int64_t N, int64_t K, void* stream);

/*
 * Dense ternary weights -> packed transposed layout, on the device.
 * Replaces pack_ternary_transposed (bittorch/quant/ternary_packed.py:174-206) for weights
 * that are already ternary: W_tern [N,K] int8 in {-1,0,+1} -> packed_T [ceil(K/4),N] uint8.
 * The host side uses it to serve bittorch._C.ternary_linear_forward (dense int8 weights)
 * with the packed matrix-core kernels.
 */
int bt_pack_ternary_i8(const int8_t* W_tern, int64_t N, int64_t K, uint8_t* packed_T, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* BITTORCH_HIP_H */
