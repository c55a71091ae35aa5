/* C ABI of libspark_shim_hip.so: the MI355X (gfx950) build of spark-engine's quantized MoE expert path.
 *
 * Every entry point keeps the reference shim's contract (engine-rs/shim): plain device pointers, a trailing stream, `int` return
 * with 0 = success (a small positive / negative code for argument errors, otherwise the hipError_t of the launch), no allocation and
 * no synchronisation inside, every scratch buffer passed in by the caller and sized by the matching *_ws_bytes, fixed grids with
 * device-side counts so a call can be recorded into a HIP graph.  Results are deterministic and independent of the number of rows in
 * the call.  `hipStream_t` replaces `cudaStream_t` in the position the reference has it.
 *
 * Names that start with `qwen_`, `glm`, `ds41_` are the reference's own symbols (same parameter order and meaning); each comment
 * names the reference definition it replaces.  Names that start with `spark_` are run-time-sized forms of the same kernels that the
 * reference does not export (its dimensions are compile-time traits).
 */
#ifndef SPARK_SHIM_H
#define SPARK_SHIM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#ifndef SPARK_API
#define SPARK_API
#endif
#ifndef HIP_INCLUDE_HIP_HIP_RUNTIME_API_H
typedef struct ihipStream_t* hipStream_t;
#endif

/* ---------------------------------------------------------------- dequantisation surfaces (bit-exact) ------------------------ */

/* EXL3 trellis [K/16, N/16, 16*bits] int16 -> the inner matrix [K, N] fp16 (no Hadamard, no scales); bits 3..6;
 * codebook 1 = mcg, 2 = mul1.  Replaces engine-rs/shim/qwen_exl3.cu:221 (qwen_exl3_reconstruct, mul1 only). */
SPARK_API int spark_exl3_reconstruct(const void* trellis, void* w_f16, int K, int N, int bits, int codebook, hipStream_t st);
SPARK_API int qwen_exl3_reconstruct(const void* trellis, void* w_f16, int K, int N, int bits, hipStream_t st);
/* Effective weight W = diag(suh) H inner H diag(svh), written transposed [N, K] fp16 with row stride ldo.
 * Replaces engine-rs/shim/qwen_exl3.cu:208 (qwen_exl3_fold). */
SPARK_API int spark_exl3_fold(const void* trellis, const void* suh, const void* svh, int K, int N, int bits, int codebook, void* out_f16,
                              int64_t ldo, hipStream_t st);
SPARK_API int qwen_exl3_fold(const void* trellis, const void* suh, const void* svh, int K, int N, int bits, void* out_f16, int64_t ldo,
                             hipStream_t st);
/* Dense EXL3 linears for M <= 64 rows, trellis widths 3..6 bits, mul1 codebook: y = had128(had128(x * suh) @ inner) * svh in three
 * steps or at once.  xh [M, K] fp16, part [S, M, N] fp32 (S = K slices, summed in order), cnt unused (may be NULL; left as it is).  qwen_exl3_multi: up to 4
 * linears on the same x (silu bit 0 with n = 2: y[0] = silu(linear 0) * linear 1); with mg / mn (fp32 [M, 4, K]) the input is
 * (1/4) sum_s mn[m][s][k] * sigmoid(mg[m][s][k]), also written to xout fp32 [M, K]; silu bits 1 and 2 (separate launches, fork
 * onto the reference runtime's side stream) are accepted and change nothing here: everything runs on st.
 * Replace engine-rs/shim/qwen_exl3.cu:70-206. */
SPARK_API int qwen_exl3_had_in(const void* x, int x_f32, int64_t ldx, const void* suh, void* xh, int M, int K, hipStream_t st);
SPARK_API int qwen_exl3_had_multi(const void* x, int64_t ldx, int M, int K, int n, const void* const* suh, void* const* xh, hipStream_t st);
SPARK_API int qwen_exl3_gemv(const void* xh, const void* trellis, void* part, int M, int K, int N, int bits, int S, hipStream_t st);
SPARK_API int qwen_exl3_finish(const void* part, int S, const void* svh, void* y, int y_f32, int64_t ldy, int M, int N, hipStream_t st);
SPARK_API int qwen_exl3_finish_h(const void* part, const void* svh, void* y, int64_t ldy, int M, int N, hipStream_t st);
SPARK_API int qwen_exl3_linear(const void* x, int64_t ldx, const void* suh, const void* trellis, const void* svh, void* part, void* y,
                               int64_t ldy, void* cnt, int M, int K, int N, int bits, int S, hipStream_t st);
SPARK_API int qwen_exl3_multi(const void* x, int64_t ldx, const void* mg, const void* mn, void* xout, int M, int K, int n,
                              const void* const* suh, void* const* xh, const void* const* trellis, void* const* part, const int* N,
                              const int* S, const void* const* svh, void* const* y, const int64_t* ldy, const int* bits, int silu,
                              hipStream_t st);
/* MXFP4: w [N, K/2] bytes (low nibble = even k), s [N, K/32] E8M0 -> fp32 [N, K].
 * Restates reference/ds41/kernel.py:122-131 (dequant_fp4_weight) and engine-rs/src/ds41/load.rs:338-349. */
SPARK_API int spark_mxfp4_dequant(const void* w, const void* s, float* out, int N, int K, hipStream_t st);
/* FP8 E4M3 [N, K] with one fp32 scale per bs x bs block -> fp32.  Restates reference/ds41/kernel.py:96-99. */
SPARK_API int spark_fp8_block_dequant(const void* w, const float* s, float* out, int N, int K, int bs, hipStream_t st);
/* FP8 E4M3 [N, K] with one E8M0 scale per 32 x 32 block (the engine's dense layout, engine-rs/shim/ds41.cu:28-73) -> fp32. */
SPARK_API int spark_fp8_e8m0_dequant(const void* w, const void* s, float* out, int N, int K, hipStream_t st);

/* ---------------------------------------------------------------- activation quantisation and glue -------------------------- */

/* x bf16 -> per 32: power-of-two scale from the block maximum, E4M3 round-to-nearest-even saturating, dequantised back to bf16.
 * Replaces engine-rs/shim/ds41.cu:274 (ds41_act_quant32); bit-exact with engine-rs/src/ds41/ops.rs:26-35. */
SPARK_API int ds41_act_quant32(const void* x, void* out, long long numel, hipStream_t st);
/* Same quantiser, leaving the E4M3 bytes q [numel] and the E8M0 scale bytes s [numel/32].  Replaces ds41_mx.cu:1406. */
SPARK_API int ds41_act_quant_fp8(const void* x, void* q, void* s, long long numel, hipStream_t st);
/* The same bytes for rows that are stored as E4M3 bytes wq [numel] with an E8M0 byte per 32 ws [numel/32]: act_quant of their bf16
 * dequantisation (byte x 2^(scale - 127) rounded to bf16; scale byte 0 gives 0) without writing it out.  Replaces
 * engine-rs/shim/ds41_mx.cu:1400 (ds41_requant_fp8; kernel :333-353), which feeds stored FP8 rows to the FP8 products. */
SPARK_API int ds41_requant_fp8(const void* wq, const void* ws, void* q, void* s, long long numel, hipStream_t st);
/* gu fp32 [T, 2I] (gate | up) -> act_quant(bf16(silu(min(g, lim)) * clamp(u, +-lim))) bf16 [T, I].  Replaces ds41_ops.cu:615. */
SPARK_API int ds41_swiglu_quant(const float* gu, void* out, int T, int I, float lim, hipStream_t st);
/* h = silu(g) * u over n fp32 values.  Replaces engine-rs/shim/qwen_moe.cu:101. */
SPARK_API int qwen_moe_silu_mul(const void* g, const void* u, void* h, int n, hipStream_t st);
/* out[r, :] = sigmoid(gl[r * ldg + col]) * d[r, :] (the shared expert's scalar gate).  Replaces qwen_moe.cu:106. */
SPARK_API int qwen_moe_gate_scale(const void* gl, int64_t ldg, int col, const void* d, void* out, int R, int N, hipStream_t st);

/* ---------------------------------------------------------------- routers ---------------------------------------------------- */

/* softmax over E fp32 logits (row stride ld), top-k by repeated argmax with ties to the lower index, weights renormalised to sum 1.
 * idx int32 [R, topk], w fp32 [R, topk].  E <= 1024, topk <= 16.  Replaces engine-rs/shim/qwen_moe.cu:10-66,90-99. */
SPARK_API int spark_softmax_route(const void* logits, int64_t ld, int R, int E, int topk, void* idx, void* w, hipStream_t st);
SPARK_API int qwen_moe_route(const void* logits, int R, void* idx, void* w, hipStream_t st);
SPARK_API int qwen_moe_route_ld(const void* logits, int64_t ld, int R, void* idx, void* w, hipStream_t st);
/* s = sqrt(softplus(x)), top-K of s + bias, w = s / (sum + 1e-20) * scale for K > 1.  idx int64 [T, K].
 * Replaces engine-rs/shim/ds41_ops.cu:376-419,609. */
SPARK_API int ds41_route(const float* logits, const float* bias, int64_t* idx, float* w, int T, int E, int K, float scale, hipStream_t st);
/* score = sigmoid(x), top-K of score + bias, w = score / max(sum, 1e-20) * scaling.  Restates dataflow.cu:433-448,489-513. */
SPARK_API int spark_sigmoid_route(const float* logits, const float* bias, int64_t* idx, float* w, int T, int E, int K, float scaling,
                                  hipStream_t st);
/* GLM router: logits = h [rows, k] fp32 x w [experts, k] (fp32 or bf16), then the sigmoid selection above.
 * `partial` is scratch of rows * experts * glm53_router_split() floats.  Replaces engine-rs/shim/dataflow.cu:519-546. */
SPARK_API int glm53_router_split(void);
SPARK_API int glm53_router_fused_cuda(const float* h, const void* w, int w_bf16, const float* bias, float* partial, long long* ids,
                                      float* weights, int rows, int experts, int k, float scaling, hipStream_t st);
/* The same, and wh [rows, 8] binary16 receives the round-to-nearest-even copy of the weights (what glm_moe_experts takes as w).
 * Replaces engine-rs/shim/dataflow.cu:549-574 (GLM53_ROUTER_HALF_W=1; Rust caller engine-rs/src/moe.rs:66-67). */
SPARK_API int glm53_router_fused_h_cuda(const float* h, const void* w, int w_bf16, const float* bias, float* partial, long long* ids,
                                        float* weights, void* wh, int rows, int experts, int k, float scaling, hipStream_t st);

/* ---------------------------------------------------------------- dense quantised GEMVs (m <= 8 rows) ----------------------- */

/* y [m, n] fp32 = x [m, k] bf16 . w^T, w [n, k/2] MXFP4 codes, ws [n, k/32] E8M0.  Replaces engine-rs/shim/ds41.cu:75-110,236. */
SPARK_API int ds41_mxfp4_gemv(const void* x, const void* w, const void* ws, float* y, int m, int n, int k, hipStream_t st);
/* w [n, k] E4M3 with E8M0 scales per 32 x 32 block; xs = row stride of x in elements; rpg = rows per scale group of a stacked
 * weight (0 = one matrix).  Replaces engine-rs/shim/ds41.cu:28-73,240,248. */
SPARK_API int ds41_fp8_gemv_ex(const void* x, const void* w, const void* ws, float* y, int m, int n, int k, int xs, int rpg, hipStream_t st);
SPARK_API int ds41_fp8_gemv(const void* x, const void* w, const void* ws, float* y, int m, int n, int k, hipStream_t st);
/* The same product for up to 16 rows.  Replaces engine-rs/shim/ds41_mx.cu:1385-1393 (ds41_fp8_gemv_bx). */
SPARK_API int ds41_fp8_gemv_bx(const void* x, const void* w, const void* ws, float* y, int m, int n, int k, int xs, int rpg, hipStream_t st);
/* FP8 weights times act-quantised activations, m <= 32: x bf16 [m, k] (quantised inside when aq is NULL) or aq E4M3 + as_ UE8M0
 * per 32; y fp32, or bf16 when ob16.  Replace engine-rs/shim/ds41_mx.cu:1348-1382. */
SPARK_API int ds41_fp8_gemv_mx_init(void);
SPARK_API size_t ds41_fp8_gemv_mx_smem_max(void);
SPARK_API int ds41_fp8_gemv_mx_q(const void* x, const void* aq, const void* as_, const void* w, const void* ws, void* y, int m, int n, int k,
                                 int ob16, hipStream_t st);
/* w [n, k] E4M3 with fp32 scales [ceil(n/128), ceil(k/128)]; the projection of reference/ds41/kernel.py:96-119 (fp8_gemm) with bf16
 * activations used as given. */
SPARK_API int spark_fp8_block128_gemv(const void* x, const void* w, const float* scales, float* y, int m, int n, int k, hipStream_t st);
/* The same projection on weights packed once at load into the matrix unit's operand order (tiles of 16 rows x 128 k; the layout is
 * written out in csrc/fp8_packed.hip), for 1-16 activation rows at one cost: no counterpart symbol in the reference, whose dense FP8
 * kernels (engine-rs/shim/ds41.cu:75-110, 236-250) read the row-major matrix; it stands to them as moe_pack (engine-rs/src/ds41/kern.rs:718-770)
 * stands to the checkpoint's expert matrices.  n a multiple of 16, k a multiple of 128 (gemv: up to 8192); `out` holds n * k bytes;
 * scales as for spark_fp8_block128_gemv.  Returns 1 for shapes outside these. */
SPARK_API int spark_fp8_t16_pack(const void* w, void* out, int n, int k, hipStream_t st);
SPARK_API int spark_fp8_block128_gemv_t16(const void* x, const void* wt, const float* scales, float* y, int m, int n, int k, hipStream_t st);
/* the same packed matrix with E8M0 scales per 32 x 32 ([n / 32, k / 32] bytes): the product of ds41_fp8_gemv (engine-rs/shim/ds41.cu:28-73,
 * bf16 activations used as given) at one cost for 1-16 rows; n a multiple of 32 */
SPARK_API int spark_fp8_e8m0_gemv_t16(const void* x, const void* wt, const void* scales, float* y, int m, int n, int k, hipStream_t st);
/* w [n, k] bf16 (router logits).  Replaces engine-rs/shim/ds41.cu:252. */
SPARK_API int ds41_bf16_gemv(const void* x, const void* w, float* y, int m, int n, int k, hipStream_t st);
/* the same for up to 16 rows (k a multiple of 32, n of 8).  Replaces engine-rs/shim/ds41_mx.cu:1394 (ds41_bf16_gemv_mx). */
SPARK_API int ds41_bf16_gemv_mx(const void* x, const void* w, float* y, int m, int n, int k, hipStream_t st);

/* ---------------------------------------------------------------- MXFP4 expert layer ---------------------------------------- */

/* y[r] = add[r] + sum over shared experts + sum_k (slot order) w2_e . q(bf16(silu(min(bf16(w1_e . xq), 10)) * clamp(bf16(w3_e . xq), +-10)
 * * rw[r, k])), q = the act_quant above, products against E4M3 activations with E8M0 scales exact in fp32
 * (engine-rs/shim/ds41_moe.cu:1-24, ds41_mx.cu:129-292).
 * layout: 0 = streaming records made by spark_mxfp4_prepack, 1 = checkpoint layout w [E, rows, K/2] + s [E, rows, K/32],
 *         2 = the reference's moe_pack layout (engine-rs/src/ds41/kern.rs:718-726), 3 = its moe_pack_mx layout (kern.rs:728-734).
 * Shared experts (n_shared of them, weight 1, every row) are experts E .. E + n_shared - 1 of the same stacked tensors. */
SPARK_API size_t spark_mxfp4_packed_bytes(long long rows_total, int K);
SPARK_API int spark_mxfp4_prepack(const void* w, const void* s, void* packed, long long rows_total, int K, hipStream_t st);
SPARK_API size_t spark_mxfp4_moe_ws_bytes(int R, int H, int I, int topk, int E, int n_shared);
/* xq E4M3 [R, H], xs E8M0 [R, H/32] */
SPARK_API int spark_mxfp4_moe_q(const void* xq, const void* xs, int R, const int64_t* idx, const float* rw, const void* w1, const void* s1,
                                const void* w3, const void* s3, const void* w2, const void* s2, int layout, int H, int I, int topk, int E,
                                int n_shared, const float* add, float* y, void* ws, hipStream_t st);
/* x bf16 [R, H]; xq / xs are caller scratch of R*H and R*H/32 bytes */
SPARK_API int spark_mxfp4_moe(const void* x, void* xq, void* xs, int R, const int64_t* idx, const float* rw, const void* w1, const void* s1,
                              const void* w3, const void* s3, const void* w2, const void* s2, int layout, int H, int I, int topk, int E,
                              int n_shared, const float* add, float* y, void* ws, hipStream_t st);
/* Decode entry (R <= 8 token rows, topk + n_shared <= 16): the whole layer as ONE launch.  x is bf16 [R, H] when xs is NULL (act_quant
 * runs inside the kernel) or E4M3 [R, H] with its E8M0 scales xs.  flags bit 0: the caller promises that ws was prepared by
 * spark_mxfp4_moe_ws_init and only used by these entry points since.  A workspace the library itself saw prepared (see
 * spark_mxfp4_moe_ws_init) is recognised by its address without the flag; any other one is prepared first by one more launch.
 * flags bit 1: use the several-kernel path (xs required).  Same values, bit for bit, as the several-kernel path.
 * flags bit 4 (16): y is bf16 [R, H] - the binary32 result rounded to nearest even - instead of binary32.
 * spark_mxfp4_moe_ws_init(ws, bytes, st): call once after allocating ws, outside stream capture (its one-time workgroup placement
 * check synchronises the device; until it has run the kernels exchange through device-coherent accesses only).  It puts every
 * exchanged word into its idle state and records the address: decode-sized calls through spark_mxfp4_moe_x, spark_mxfp4_moe(_q),
 * ds41_moe_mx(_ex) and ds41_moe that use this workspace then run as one launch.  Call spark_moe_ws_release(ws) before freeing it. */
SPARK_API int spark_mxfp4_moe_ws_init(void* ws, size_t bytes, hipStream_t st);
SPARK_API int spark_mxfp4_moe_x(const void* x, const void* xs, int R, const int64_t* idx, const float* rw, const void* w1, const void* s1,
                                const void* w3, const void* s3, const void* w2, const void* s2, int layout, int H, int I, int topk, int E,
                                int n_shared, const float* add, float* y, void* ws, int flags, hipStream_t st);
/* The reference's DeepSeek entry points (H = 5120 as compiled there, weights in the moe_pack_mx layout with raw scale bytes).
 * Replace engine-rs/shim/ds41_mx.cu:1426-1523.  ds41_moe_mx_ws_ptrs hands out the per-pair down output [P, H] fp32 and pairmap [P]
 * inside ws (out row pairmap[r * topk + k] belongs to token row r, slot k), valid after ds41_moe_mx_ex(skip_combine = 1).
 * ds41_moe_mx_col_passes: the reference caps the per-pair output at 512 MiB and runs down + combine in 2 or 4 column passes beyond
 * (engine-rs/shim/ds41_mx.cu:1416-1425); the same rule here (prefill-sized calls; no skip_combine with more than one pass).
 * ds41_moe_mx_pair_b16: 1 when the call's per-pair outputs are bf16: with DS41_MOE_PAIR_BF16=1 in the environment (off by default,
 * as in the reference, ds41_mx.cu:1243-1255) calls of more than 64 rows keep every pair's down output as the bf16 rounding of its
 * binary32 sum (half the bytes the down product writes and the sum over the pairs reads); the sums over the pairs stay binary32 in
 * slot order.  ds41_moe_mx_ws_ptrs then hands out uint16 [P, H] behind its float** argument.
 * ds41_moe_gr16_max: accepted and ignored.  In the reference it moves the row count at which 16-row items give way to 32-row
 * items; here one kernel family serves every row count and a row's bits never depend on the rows around it. */
SPARK_API void ds41_moe_mx_set_s2(int on);
SPARK_API int ds41_moe_mx_get_s2(void);
SPARK_API void ds41_moe_gr16_max(int v);
SPARK_API int ds41_moe_mx_col_passes(int R, int topk, int E);
SPARK_API int ds41_moe_mx_pair_b16(int R, int topk, int E);
SPARK_API size_t ds41_moe_mx_ws_bytes(int R, int I, int topk, int E);
SPARK_API int ds41_moe_mx_ex(const void* xq, const void* xs, int R, const int64_t* idx, const float* rw, const void* w1, const void* s1,
                             const void* w3, const void* s3, const void* w2, const void* s2, int I, const float* add, float* y, void* ws,
                             int topk, int E, int skip_combine, hipStream_t st);
SPARK_API int ds41_moe_mx(const void* xq, const void* xs, int R, const int64_t* idx, const float* rw, const void* w1, const void* s1,
                          const void* w3, const void* s3, const void* w2, const void* s2, int I, const float* add, float* y, void* ws, int topk,
                          int E, hipStream_t st);
SPARK_API int ds41_moe_mx_combine_rows(void* ws, int R, int I, int topk, int E, const float* add, float* y, int r0, int nr, hipStream_t st);
SPARK_API int ds41_moe_mx_combine(void* ws, int R, int I, int topk, int E, const float* add, float* y, hipStream_t st);
SPARK_API int ds41_moe_mx_ws_ptrs(void* ws, int R, int I, int topk, int E, float** out, int** pairmap);
/* Weight-only FP8 with one binary32 scale per output row (the GLM dense / shared-expert projections; quantiser
 * engine-rs/src/dense_fp8.rs:59-62: scale = row amax / 448):  y[r, n] = (sum_k a(x[r, k]) * e4m3(w[n, k])) * scales[n].
 * x binary32 [m, k], w E4M3 [n, k], scales binary32 [n], y binary32 [m, n]; exact products, binary32 sums; a row's value does not
 * depend on the rows beside it.  Return 0, or 1 (the reference's cudaErrorInvalidValue) for a shape outside the stated limits.
 * glm53_fp8_dense_cuda: a = round to binary16, m 1..16, n and k multiples of 64; rounded != 0: every output rounded to binary16.
 *   scratch, mode and split_override pick among the reference's kernels and feed its split-K forms: accepted, not used (one kernel
 *   family here, K split by the shape).  Replaces engine-rs/shim/fp8.cu:110-128.
 * glm53_fp8_bf16_cuda: a = round to bf16, no output rounding; splits must be 1, 2, 4, 8 or 16 and is otherwise unused.
 *   Replaces engine-rs/shim/fp8.cu:143-151.
 * glm53_fp8_bf16_skinny_cuda: bf16 activations read as they are, m 2..32, n a multiple of 16.  Replaces engine-rs/shim/fp8.cu:134-141. */
SPARK_API int glm53_fp8_dense_cuda(const float* x, const void* w, const float* scales, float* y, float* scratch, int m, int n, int k, int rounded,
                                   int mode, int split_override, hipStream_t st);
SPARK_API int glm53_fp8_bf16_cuda(const float* x, const void* w, const float* scales, float* y, float* scratch, int m, int n, int k, int splits,
                                  hipStream_t st);
SPARK_API int glm53_fp8_bf16_skinny_cuda(const void* x_bf16, const void* w, const float* scales, float* y, int m, int n, int k, hipStream_t st);

/* bf16 activations (already act-quantised), weights in the moe_pack layout.  Replaces engine-rs/shim/ds41_moe.cu:259-292. */
SPARK_API size_t ds41_moe_ws_bytes(int R, int I, int topk, int E);
SPARK_API int ds41_moe(const void* xq, int R, const int64_t* idx, const float* rw, const void* w1, const void* s1, const void* w3,
                       const void* s3, const void* w2, const void* s2, int I, const float* add, float* y, void* ws, int topk, int E,
                       hipStream_t st);

/* ---------------------------------------------------------------- EXL3 expert layer ----------------------------------------- */

/* out[r] = add[r] + sum_k (slot order) w[r, k] * down_e(act(gate_e(x_r), up_e(x_r))), every matrix an EXL3 4-bit trellis with its
 * own Hadamard sign vector suh [K] and channel scale svh [N] (fp16).  tab = uint64 [9][E] device pointers: gate, up, down trellis;
 * gate, up, down suh; gate, up, down svh (engine-rs/shim/moe_exl3.cuh:8-9).  xtype / wtype: 0 fp32, 1 fp16, 2 bf16; itype: 0 int32,
 * 1 int64; act: 0 silu(g) * u, 1 the same after clamping g <= 10 and |u| <= 10; codebook 1 mcg, 2 mul1.  out fp32 [R, H].
 * flags bit 0: the caller promises that ws was prepared by spark_exl3_moe_ws_init and only ever used by these entry points (skips the
 * preparing launch); a workspace the library saw prepared is recognised by its address without the flag;
 * flags bit 1: force the several-kernel path (the comparison path of the tests).
 * flags bit 2: tab has a tenth row, uint64 [E], with each expert's trellis width (3..6 bits, engine-rs/shim/moe_exl3.cuh:239-252); all
 * three matrices of an expert share it.
 * flags bit 3: tab has an eleventh row with each expert's own intermediate width (a multiple of 128, at most I; I is then the stride
 * of the intermediates); gate / up have that many columns, down that many rows.
 * Both table forms take the paths of uniform tables: one launch up to 8 rows, the grouped GEMM beyond.
 * flags bit 4 (16): out is bf16 [R, H] - the binary32 result rounded to nearest even - instead of binary32 (any path, any row count).
 * spark_exl3_moe_ws_init(ws, bytes, st): call once after allocating ws, outside stream capture (its one-time workgroup placement
 * check synchronises the device; until it has run the kernels exchange through device-coherent accesses only).  It puts every
 * exchanged word into its idle state and records the address: decode-sized calls through spark_exl3_moe, qwen_moe_experts and
 * glm_moe*_experts that use this workspace then run as one launch.  ws NULL: only the one-time set-up (placement check, device
 * address of the array behind spark_exl3_moe_static).  Call
 * spark_moe_ws_release(ws) before freeing the memory.
 * Replaces engine-rs/shim/moe_exl3.cuh:1512-1691 (moex::experts). */
SPARK_API size_t spark_exl3_moe_ws_bytes(int R, int H, int I, int E, int topk);
SPARK_API int spark_exl3_moe_ws_init(void* ws, size_t bytes, hipStream_t st);
SPARK_API int spark_exl3_moe(const void* x, int xtype, int64_t ldx, int R, const void* idx, int itype, const void* w, int wtype, const void* tab,
                             const void* add, void* out, void* ws, int H, int I, int E, int topk, int codebook, int act, int flags,
                             hipStream_t st);
/* spark_exl3_moe without the workspace argument, for callers that cannot allocate (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): the exchange words of the single-launch kernel live in a 16 MiB array of the library's own
 * (one per GPU, held until the process ends).  It has no counterpart in the reference, whose callers always own their scratch.  Decode
 * sizes only: returns -5 for calls the single-launch path does not take (more than 8 rows, more than 128 pairs, tables with
 * per-expert widths), -7 when the call's exchange words exceed the array, -1 for shapes no path takes.  Calls nothing that
 * allocates; every call first puts the words it uses into their idle state with a fill kernel, so nothing is assumed of the last
 * call's leftovers.  All calls on one GPU share the array: calls that overlap on one GPU race. */
SPARK_API int spark_exl3_moe_static(const void* x, int xtype, int64_t ldx, int R, const void* idx, int itype, const void* w, int wtype, const void* tab,
                                    const void* add, void* out, int H, int I, int E, int topk, int codebook, int act, hipStream_t st);
/* The error flag of that array after the last spark_exl3_moe_static call on the current device (each call clears it as it starts):
 * waits for the stream, then 0 = every wait of the call was served, 1 = a wait expired or the routes broke the contract (the rows
 * concerned hold NaN), negative = not set up / the read failed.  Synchronises: a diagnostic, never on a capturing stream. */
SPARK_API int spark_exl3_moe_static_status(hipStream_t st);
/* Qwen: E 512, top-10, H 2560, I 640, x / w fp32, idx int32, mul1.  Replaces engine-rs/shim/qwen_moe.cu:111-117.
 * S (here and in the glm_* forms) is the reference's K-slice count, a tuning hint there: accepted and ignored, the slices follow the
 * shape alone so that a row's bits do not depend on the call. */
SPARK_API size_t qwen_moe_ws_bytes(int R, int S);
SPARK_API int qwen_moe_experts(const void* x, int64_t ldx, int R, const void* idx, const void* w, const void* tab, const void* add, void* out,
                               void* ws, int S, hipStream_t st);
/* GLM: E 288, top-8, H 4096, I 1024, x / w fp16, idx int64, mcg, clamped activation.  kmask = set of trellis widths present (bit b = some
 * expert has b bits, 3..6): 1 << 4 reads a nine-row table of 4-bit experts, anything else a ten-row table (see spark_exl3_moe flags bit 2).
 * Replaces engine-rs/shim/glm_moe.cu:8-16. */
SPARK_API size_t glm_moe_ws_bytes(int R, int S);
SPARK_API int glm_moe_experts(const void* x, int64_t ldx, int R, const void* idx, const void* w, const void* tab, const void* add, void* out,
                              void* ws, int S, const void* suh0, int kmask, hipStream_t st);
/* GLM under a three-way split of every expert: each expert 768 or 640 wide (6 or 5 of its 128-wide Hadamard blocks).  tab = uint64
 * [11][288]: rows 0-8 as above, row 9 the trellis width in bits (read when kmask is not 1 << 4), row 10 the expert's intermediate
 * width; gate / up trellis [H/16, width/16, 16 bits] int16, down [width/16, H/16, 16 bits].  Everything else as glm_moe_experts.
 * Replaces engine-rs/shim/glm_moe.cu:17-24 (moex::GlmMoe3, engine-rs/shim/moe_exl3.cuh:63-67,132-136). */
SPARK_API size_t glm_moe3_ws_bytes(int R, int S);
SPARK_API int glm_moe3_experts(const void* x, int64_t ldx, int R, const void* idx, const void* w, const void* tab, const void* add, void* out,
                               void* ws, int S, int kmask, hipStream_t st);

/* ---------------------------------------------------------------- single-launch workspaces (not part of the reference ABI) ---- */

/* The single-launch decode kernels (spark_exl3_moe, spark_mxfp4_moe_x and the reference-named forms at up to 8 rows) pass data
 * between the workgroups of one launch through words of ws that are all-ones while idle; every wait is bounded.  If a wait ever
 * expires (it never should: a block only waits for blocks dispatched before it), or a token row names an expert twice (an item
 * would outgrow the kernels' arrays: it is cut at what they hold), the kernel sets the first 32-bit word of ws (sticky), stores NaN
 * into every output element whose sum it could not complete and still runs to its end; the launch returns 0 like the reference's
 * launchers, which cannot see device state either, so the failure is in the data for a caller that only checks return codes.  While
 * the flag is set every later call on that workspace stores NaN too (the words a failed call left behind are not idle), until the
 * workspace is prepared again.  spark_moe_ws_status(ws, st) waits for st and returns the flag: 0 = clear, 1 = set - and ws is then
 * no longer known as prepared, so the next call that does not pass "prepared" (flags bit 0) prepares it again itself; a caller that
 * passes the bit calls the matching *_ws_init first -, negative = the read failed.  It synchronises: a diagnostic for tests,
 * benchmarks and a serving loop's periodic health check, not for captured streams.
 * spark_moe_ws_release(ws): forget that ws was prepared (before freeing or reusing the memory). */
SPARK_API int spark_moe_ws_status(const void* ws, hipStream_t st);
SPARK_API void spark_moe_ws_release(const void* ws);

/* ---------------------------------------------------------------- diagnostics (not part of the reference ABI) ---------------- */

/* buf = device memory of 16 * gridDim int64 the single-launch kernels fill with per-block wall-clock stamps (NULL = off).  Only
 * libraries built with -DSPK_EXL3_TRACE / -DSPK_MX_TRACE record stamps; the release build ignores the buffer. */
SPARK_API void spark_debug_exl3_trace(long long* buf);
SPARK_API void spark_debug_mx_trace(long long* buf);
/* what the one-time workgroup placement check found: 1 = workgroup b of a 1-D grid runs on XCD b % 8, 0 = not so, -1 = not run yet */
SPARK_API int spark_debug_placement(void);
/* exchange mode of the single-launch EXL3 kernel: 1 = same-XCD through L2, 0 = device-coherent, -1 = as the placement check found */
SPARK_API void spark_debug_exl3_local(int v);
/* the same switch for the single-launch MXFP4 kernel */
SPARK_API void spark_debug_mx_local(int v);
/* tile height of the dense row-tile GEMV: 16 or 8 weight rows per workgroup, 0 = chosen by the number of activation rows (same values either way) */
SPARK_API void spark_debug_gemv_rows(int v);
/* 0: ds41_fp8_gemv_mx_q, spark_fp8_block128_gemv and ds41_fp8_gemv(_ex, _bx) run their dot-product / transposing kernels for every
 * shape; 1 (default): the row-major matrix-unit kernel with every weight load of a wave in flight where the dispatch rules choose
 * it; 2: the FP8 GEMVs with bf16 activations take it wherever it applies (for comparing on one machine; the forms differ in the
 * order of the binary32 sums only) */
SPARK_API void spark_debug_fp8q_rowmajor(int on);
/* 256-wide chunks of a wave's K span in that kernel: 1, 2 or 4, 0 = chosen by the shape (a value that does not fit K is ignored) */
SPARK_API void spark_debug_rm_span(int ch);
/* the bf16 per-pair outputs of the ds41_* prefill calls: 1 / 0 = on / off, negative = as DS41_MOE_PAIR_BF16 in the environment says */
SPARK_API void spark_debug_mx_pair_b16(int on);
/* the cap on the per-pair output buffer of the ds41_* prefill calls in bytes (0 = back to DS41_MOE_OUT_MB or 512 MiB) */
SPARK_API void spark_debug_mx_out_cap(size_t bytes);
/* Opt-in check of every expert call's routes on the host before anything is launched (for bringing up an integration): on with 1
 * or with SPARK_VALIDATE_ROUTES=1 in the environment, off with 0.  A call whose routes break the contract - an index outside [0, E),
 * an expert repeated within a token row - then returns -6 (spark_exl3_moe*, qwen_moe_experts, glm_moe*_experts) or 6 (spark_mxfp4_moe*,
 * ds41_moe*) and launches nothing; -8 / 8 = the check itself failed.  It waits for the stream and copies the indices to the host:
 * never on a capturing stream, never in production. */
SPARK_API void spark_debug_validate_routes(int on);
/* Host-side queries (nothing is launched, no GPU needed): the path a call of this shape takes.  0 = one launch, 1 = the grouped GEMM,
 * 2 = the several-kernel path (EXL3: the item kernels), -1 = a shape no entry point takes.  layout: 0 T16 records, 1 checkpoint
 * layout, 2 / 3 / 4 = the reference's moe_pack / moe_pack_mx / moe_pack_mx with 2-bit coded scales (the ds41_* entry points, H 5120);
 * flags as spark_exl3_moe's. */
SPARK_API int spark_mxfp4_moe_path(int layout, int R, int H, int I, int topk, int E, int n_shared);
SPARK_API int spark_exl3_moe_path(int R, int H, int I, int E, int topk, int flags);
/* diagnostics: the most rows (0..8) a call may have to run as the single launch where the MXFP4 grouped GEMM could take it too;
 * negative = the built-in rule (8 on T16 records; 2 on the reference's tile layouts, 4 from an intermediate width of 1536 on) */
SPARK_API void spark_debug_mx_fused_rows(int rows);
/* Where the several-kernel MXFP4 path (flags bit 1 of spark_mxfp4_moe_x; every call of more than 8 rows) left the act-quantised
 * intermediate of its last call inside a spark_mxfp4_moe* workspace: E4M3 codes hq [P, I] and UE8M0 scale bytes hs [P, I / 32] in
 * grouped order, prow [P] = the pair (row * (topk + n_shared) + slot) of each grouped row.  For tests that compare the
 * intermediate with the CPU oracle's; returns 1 on a shape the entry points refuse. */
SPARK_API int spark_debug_mx_ws_h(void* ws, int R, int H, int I, int topk, int E, int n_shared, void** hq, void** hs, int** prow);
/* The stream floor: reads `bytes` bytes (rounded down to 16) at src (device memory, 16-byte aligned) with non-temporal 16-byte loads
 * and stores one word a wave into out (device memory of 4096 bytes): the time it takes bounds from below every kernel that must
 * fetch that many bytes from memory.  The benchmark times it in the same graph of instances as the layers.  1 = bad arguments. */
SPARK_API int spark_debug_stream_read(const void* src, size_t bytes, void* out, hipStream_t st);
/* k-tiles per wave of a stage-1 block of the single-launch EXL3 kernel: 4 or 8 forces it, 0 = chosen by the shape (the default) */
SPARK_API void spark_debug_exl3_twa(int v);

#ifdef __cplusplus
}
#endif
#endif
