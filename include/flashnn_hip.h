/*
 * flashnn_hip.h - C ABI of libflashnn_hip.so: the gfx950 (MI355X) kernels behind the
 * FLASHNN quantized-GEMM operators.
 *
 * The reference has no FFI: its operators call Python launcher functions that start
 * Triton kernels.  Every entry point below replaces one of those launchers and keeps
 * its contract: the caller owns and allocates all tensors (device pointers), the call
 * enqueues work on the given HIP stream and returns without waiting, and every output
 * element is overwritten (no pre-zeroing is needed).
 *
 * Conventions
 *   - all pointers are device pointers unless stated; sizes/strides are in ELEMENTS;
 *   - matrices are row-major with an explicit leading dimension (row stride);
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *   - a call with no rows (M = 0) or no output channels (N = 0) is valid, launches nothing and
 *     may pass NULL for its tensors (an empty tensor has no address);
 *   - return value: 0 ok, FNN_ERR_ARG (-1) bad argument, FNN_ERR_UNSUPPORTED (-2)
 *     shape/dtype not handled, FNN_ERR_HIP (-3) HIP runtime error.  After a non-zero
 *     return fnn_last_error() gives a thread-local, human-readable message.
 *   - calls are re-entrant (fnn_gemm_a8w8_static excepted: see there) and never allocate, free or
 *     synchronise.  State kept between calls:
 *     per thread the last error message and the name of the last kernel launched; per
 *     process, set once and never changed again, which devices have had a kernel's LDS
 *     limit raised and (only with FLASHNN_HIP_LOG=1) which kernel variants have been
 *     logged.  No call reads a setting that another call can change.
 *   - an error the calling thread's own HIP calls left pending before a call is neither
 *     reported by the call nor cleared by it.
 *   - FLASHNN_HIP_LOG=1 in the environment (read once): one line on stderr the first time
 *     each kernel variant is launched in the process.
 */
#ifndef FLASHNN_HIP_H_
#define FLASHNN_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element type codes used by the *_dtype arguments */
enum fnn_dtype { FNN_F16 = 0, FNN_BF16 = 1, FNN_F32 = 2 };

enum fnn_status { FNN_OK = 0, FNN_ERR_ARG = -1, FNN_ERR_UNSUPPORTED = -2, FNN_ERR_HIP = -3 };

/* ABI version of this header (bumped on any signature change): 2 since fnn_gemm_a8w8_tiled names the waves and the workspace entry points exist. */
int fnn_version(void);

/* Message describing the last failure on the calling thread ("" if none). */
const char* fnn_last_error(void);

/*
 * Name of the kernel that the calling thread's last call launched, with the numbers that tell
 * its variants apart, e.g. "gemm_a8w8_ring_kernel<256,192,4>" (tile rows, tile columns, waves);
 * "" before the first launch.  A call that launches two kernels (a column split) names the
 * last.  The pointer stays valid until the thread's next call of this function.  The reference
 * logs the chosen configuration through loguru (flashnn/triton_kernels/triton_utils.py:112,139).
 */
const char* fnn_last_kernel(void);

/*
 * Per-token symmetric int8 quantisation.
 * Replaces triton_dynamic_quantize(out, input, scale)
 *   (flashnn/triton_kernels/dynamic_quant.py:73-97), with the arithmetic of
 *   DynamicQuantize._torch_impl (flashnn/quant_gemm.py:53-57): everything is computed
 *   in the input type, scale = absmax/127, q = round_half_even(x/scale).
 * q        [M,K] int8, row stride ldq
 * scale    [M]   fp16 (always fp16, also for bf16 input)
 * x        [M,K] fp16/bf16 (x_dtype), row stride ldx
 */
int fnn_dynamic_quant(void* q, void* scale, const void* x, int64_t M, int64_t K,
                      int64_t ldx, int64_t ldq, int x_dtype, void* stream);

/*
 * Fused RMSNorm + per-token int8 quantisation.
 * Replaces triton_rmsnorm_dquant_forward(x, weight, eps)
 *   (flashnn/triton_kernels/rms_norm_dquant.py:80-96), with the arithmetic of
 *   RMSNormDquant._torch_impl (flashnn/norm.py:45-60): fp32 throughout,
 *   q = clamp(round_half_even(n/scale)), scale = max|n|/127 stored in the input type.
 * q        [M,K] int8, row stride ldq
 * scale    [M]   same type as x
 * x        [M,K] fp16/bf16 (x_dtype), row stride ldx
 * gamma    [K]   fp16/bf16/fp32 (gamma_dtype)
 */
int fnn_rmsnorm_dquant(void* q, void* scale, const void* x, const void* gamma, float eps,
                       int64_t M, int64_t K, int64_t ldx, int64_t ldq, int x_dtype,
                       int gamma_dtype, void* stream);

/*
 * out[m,n] = (sum_k a[m,k]*b[n,k])_int32 * alpha_row[m] * alpha_col[n]  -> fp16/bf16.
 * Replaces triton_gemm_a8w8_forward(out, a, b, alpha_row, alpha_col)
 *   (flashnn/triton_kernels/gemm_a8w8.py:182-221; kernel :74-179): int32 accumulation,
 *   both scales widened to fp32 and multiplied in turn.
 * a [M,K] int8 (lda), b [N,K] int8 (ldb), out [M,N] (ldc),
 * alpha_row [M], alpha_col [N] of the given scale types.
 */
int fnn_gemm_a8w8(void* out, const void* a, const void* b, const void* alpha_row,
                  const void* alpha_col, int64_t M, int64_t N, int64_t K, int64_t lda,
                  int64_t ldb, int64_t ldc, int out_dtype, int alpha_row_dtype,
                  int alpha_col_dtype, void* stream);

/*
 * Raw int32 accumulators of the same contraction, acc[m,n] = sum_k a[m,k]*b[n,k].
 * No counterpart in the reference API: it exposes the integer result that the Triton
 * kernel keeps in registers (gemm_a8w8.py:135-150) so that it can be checked bit for
 * bit against an integer matmul.
 */
int fnn_gemm_a8w8_i32(int32_t* acc, const void* a, const void* b, int64_t M, int64_t N,
                      int64_t K, int64_t lda, int64_t ldb, int64_t ldc, void* stream);

/*
 * Weight-only GEMM with int8 weights:
 *   out[m,n] = sum_k act[m,k] * (qw[n,k] - zp[g(k),n]) * scale[g(k),n]  (+ bias[n]).
 * Replaces triton_gemm_a16w8_forward(out, act, quant_w, scale_w, bias, zero_points)
 *   (flashnn/triton_kernels/gemm_a16w8.py:275-338), semantics of
 *   GemmWeightOnly._torch_impl (flashnn/quant_gemm.py:156-173).
 * act   [M,K] fp16/bf16 (act_dtype), row stride lda
 * qw    [N,K] int8, row stride ldw
 * scale group == 0: [N] per channel;  group > 0: [K/group, N] (row stride N)
 * zp    NULL or same shape as scale (float values, zp_dtype)
 * bias  NULL or [N] (bias_dtype)
 * out   [M,N] fp16/bf16 (out_dtype), row stride ldc
 */
int fnn_gemm_a16w8(void* out, const void* act, const void* qw, const void* scale,
                   const void* bias, const void* zp, int64_t M, int64_t N, int64_t K,
                   int64_t lda, int64_t ldw, int64_t ldc, int64_t group, int act_dtype,
                   int out_dtype, int scale_dtype, int zp_dtype, int bias_dtype,
                   void* stream);

/*
 * Weight-only GEMM with packed signed int4 weights.
 * Replaces triton_gemm_a16w4_forward(...) (flashnn/triton_kernels/gemm_a16w4.py:336-406),
 *   semantics of GemmWeightOnly._torch_impl (flashnn/quant_gemm.py:174-204).
 * qw is [N/2,K] bytes (row stride ldw): byte [j,k] holds channel n=2j in its low
 * nibble and n=2j+1 in its high nibble, each a two's-complement value in [-8,7].
 * N is the number of OUTPUT channels (even).  Other arguments as fnn_gemm_a16w8.
 */
int fnn_gemm_a16w4(void* out, const void* act, const void* qw, const void* scale,
                   const void* bias, const void* zp, int64_t M, int64_t N, int64_t K,
                   int64_t lda, int64_t ldw, int64_t ldc, int64_t group, int act_dtype,
                   int out_dtype, int scale_dtype, int zp_dtype, int bias_dtype,
                   void* stream);

/*
 * fnn_gemm_a16w8 / fnn_gemm_a16w4 with scratch memory for the activations.  The reference's torch path
 * rounds every dequantised weight to fp16 before the dot product, (q - zp) * s with both operations rounded
 * (flashnn/quant_gemm.py:14-36); the tiled kernel for more than 64 rows does the same where activations and
 * tables are fp16 (so do the few-row kernels with per-channel tables), and the result then differs from the
 * reference's only by the order of the fp32 additions.  (The tiled kernel takes the calls for which it has
 * more than 128 tiles of 128 rows x 128 channels; narrower problems run as 64-row passes of the few-row
 * kernel, faster there, and need no workspace.)  bf16 activations (more than 64 rows, fp16 tables
 * per channel or per group of 128, 256, 512 .. values) reach that form through
 * one conversion pass: every row becomes an fp16 row in the workspace, scaled by a power of two that makes
 * every value representable (undone exactly on the output).  Without a workspace, or with less than
 *   fnn_gemm_weight_only_workspace_bytes(M, N, K, group, act_dtype, scale_dtype)   (0: the call would not use one)
 * the call is fnn_gemm_a16w8 / fnn_gemm_a16w4: the same kernels scaling group sums in fp32, which agrees with
 * the reference within rtol = atol = 1e-2 on the configured shapes but is not its rounding.  The workspace
 * needs no initialisation, is 16-byte aligned, and belongs to the call while it runs (calls that overlap
 * in time need one each).
 */
size_t fnn_gemm_weight_only_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t group, int act_dtype,
                                            int scale_dtype);
int fnn_gemm_a16w8_ws(void* out, const void* act, const void* qw, const void* scale, const void* bias,
                      const void* zp, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw, int64_t ldc,
                      int64_t group, int act_dtype, int out_dtype, int scale_dtype, int zp_dtype, int bias_dtype,
                      void* workspace, size_t ws_bytes, void* stream);
int fnn_gemm_a16w4_ws(void* out, const void* act, const void* qw, const void* scale, const void* bias,
                      const void* zp, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw, int64_t ldc,
                      int64_t group, int act_dtype, int out_dtype, int scale_dtype, int zp_dtype, int bias_dtype,
                      void* workspace, size_t ws_bytes, void* stream);

/*
 * fnn_gemm_a16w8 / fnn_gemm_a16w4 with the blocks of the few-row kernel named by the caller: block_m activation
 * rows per pass over the weights (16, 32 or 64) and block_n output channels per workgroup (16, 32 or 64 weight
 * rows: int8 16 / 32 / 64 channels, int4 32 / 64 / 128), block_m not above the weight rows of a workgroup.  The
 * counterpart of the BLOCK_M / BLOCK_N of the reference's autotune lists for these kernels
 * (flashnn/triton_kernels/gemm_a16w8.py:15-80, gemm_a16w4.py:15-80), for a tuned-configuration cache to time and
 * record; up to 64 rows.  FNN_ERR_UNSUPPORTED where the pair is not built, the shape does not divide into such
 * blocks, or the library's own choice for the call rounds every weight as the reference does and this kernel
 * would not: a named block never changes the rounding of the result, only the order of the fp32 additions.
 */
int fnn_gemm_a16w8_tiled(void* out, const void* act, const void* qw, const void* scale, const void* bias,
                         const void* zp, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw, int64_t ldc,
                         int64_t group, int act_dtype, int out_dtype, int scale_dtype, int zp_dtype, int bias_dtype,
                         int block_m, int block_n, void* stream);
int fnn_gemm_a16w4_tiled(void* out, const void* act, const void* qw, const void* scale, const void* bias,
                         const void* zp, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw, int64_t ldc,
                         int64_t group, int act_dtype, int out_dtype, int scale_dtype, int zp_dtype, int bias_dtype,
                         int block_m, int block_n, void* stream);

/*
 * fnn_gemm_a16w4 on weights repacked once by the caller (made for the decode of one or a few tokens).  The
 * reference keeps int4 weights as [N/2, K] bytes with [K/group, N] tables beside them
 * (flashnn/quant_gemm.py:174-204; its Triton launcher, flashnn/triton_kernels/gemm_a16w4.py:336-406, reads
 * that layout as it is); a decode kernel then fetches rows K bytes apart plus two side tables.  The packed
 * form is one stream: everything 16 channels need for 1024 values of K - 8 KB of nibbles, then the 8 x 16
 * scales and the 8 x 16 zero points of those eight groups - is one contiguous unit of 8704 bytes, units in the
 * order [channel tile][K range].  The bytes are exactly the reference layout's with fp16 tables,
 * N K / 2 + 2 (K / 128) N 2; nothing is dropped or merged, zero points stay the caller's fp16 values.
 * The unit's inner order is written out in flashnn_amd/csrc/gemm_wo_prepacked.hip and restated, with its
 * inverse, in oracle/flashnn_oracle.py (prepack_a16w4 / unpack_prepacked_a16w4).
 *   fnn_a16w4_prepacked_bytes(N, K, group)  size of the packed form; 0 if the shape has none (it needs
 *                                           group = 128, N % 16 == 0, K % 1024 == 0 and K / 1024 in
 *                                           {1, 2, 4} or at least 8)
 *   fnn_a16w4_prepack(packed, qw, scale, zp, ...)   packed <- the reference layout (qw [N/2, K] with row stride
 *                                           ldw, scale and zp [K/128, N] fp16, zp may be NULL = zeros);
 *                                           a device-side copy, asynchronous on `stream`
 *   fnn_gemm_a16w4_prepacked(out, act, packed, bias, ...)   out[m, n] as fnn_gemm_a16w4 computes it, within
 *                                           rtol = atol = 1e-2 of the reference (group scales are applied in
 *                                           fp32 to group sums).  M = 1: a kernel that streams the packed
 *                                           form at the rate of a bare load stream; M > 1: a kernel for 16,
 *                                           32 or 64 rows per pass over the weights (more rows: more passes;
 *                                           from about 100 rows on the reference layout's tiled kernel is
 *                                           faster on large matrices).  act rows lda elements apart (lda % 8
 *                                           == 0 for M > 1, 64 rows within 4 GB), out rows ldc apart.
 * Nothing repacks implicitly: fnn_gemm_a16w4 always reads the reference layout.
 */
size_t fnn_a16w4_prepacked_bytes(int64_t N, int64_t K, int64_t group);
int fnn_a16w4_prepack(void* packed, const void* qw, const void* scale, const void* zp, int64_t N, int64_t K,
                      int64_t ldw, int64_t group, int scale_dtype, int zp_dtype, void* stream);
int fnn_gemm_a16w4_prepacked(void* out, const void* act, const void* packed, const void* bias, int64_t M,
                             int64_t N, int64_t K, int64_t lda, int64_t ldc, int64_t group, int act_dtype,
                             int out_dtype, int bias_dtype, void* stream);

/* RMSNorm: out[m,k] = round_T(round_T(x[m,k] * rsqrt(mean_k(x^2) + eps)) * gamma[k]), T = x_dtype.
 * Replaces triton_rmsnorm_forward(x, weight, eps) (flashnn/triton_kernels/rms_norm.py:68-83) behind
 * RMSNorm (flashnn/norm.py:19-36); semantics of _torch_impl (:31-33) with the result in the input
 * type, as _triton_impl returns it (:28-29).  x, out: [M,K] fp16/bf16 with row strides ldx, ldo
 * (elements); gamma: [K] fp16/bf16/fp32. */
int fnn_rmsnorm(void* out, const void* x, const void* gamma, float eps, int64_t M, int64_t K,
                int64_t ldx, int64_t ldo, int x_dtype, int gamma_dtype, void* stream);

/* LayerNorm over the last dimension: out = round_T(((x - mean) * rstd) * gamma + beta).
 * Replaces triton_layer_norm_forward(x, weight, bias, eps) (flashnn/triton_kernels/layer_norm.py:84-101)
 * behind LayerNorm (flashnn/norm.py:69-94; _torch_impl = torch.nn.functional.layer_norm, :82-85).
 * gamma and beta: [K], both of type gb_dtype (fp16/bf16/fp32). */
int fnn_layernorm(void* out, const void* x, const void* gamma, const void* beta, float eps, int64_t M,
                  int64_t K, int64_t ldx, int64_t ldo, int x_dtype, int gb_dtype, void* stream);

/* LayerNorm + per-token int8 quantisation: y = layernorm(x) rounded to T, scale[m] = max|y| / 127 and
 * q = clamp(round(y / scale), -128, 127), the last three evaluated in T as torch evaluates them.
 * Replaces triton_layer_norm_dquant_forward(x, weight, bias, eps)
 * (flashnn/triton_kernels/layer_norm_dquant.py:91-105) behind LayernormDquant (flashnn/norm.py:97-124;
 * semantics of _torch_impl, :112-119).  q: int8 [M,K] with row stride ldq; scale: [M] of type x_dtype. */
int fnn_layernorm_dquant(void* q, void* scale, const void* x, const void* gamma, const void* beta,
                         float eps, int64_t M, int64_t K, int64_t ldx, int64_t ldq, int x_dtype,
                         int gb_dtype, void* stream);

/*
 * fnn_gemm_a8w8 with the output tile of the MFMA kernel chosen by the caller: (tile_m, tile_n, waves) with
 * waves = 4 (or 0: the tile's default) and the tile one of 256x256, 256x192, 256x128, 128x128, 64x128; (0, 0, 0)
 * is the library's own choice.  A named tile also bypasses the few-row kernels.  This is what a shape-keyed
 * tuned-configuration cache calls - the role that compile_and_cache_kernels and its JSON file play in the
 * reference (flashnn/triton_kernels/triton_utils.py:84-151; method name "gemm_a8w8_M_N_K",
 * gemm_a8w8.py:199; `waves` is the num_warps of its launch options, gemm_a8w8.py:17-50).
 * Results are bit-identical for every tile.
 */
int fnn_gemm_a8w8_tiled(void* out, const void* a, const void* b, const void* alpha_row,
                        const void* alpha_col, int64_t M, int64_t N, int64_t K, int64_t lda,
                        int64_t ldb, int64_t ldc, int out_dtype, int alpha_row_dtype,
                        int alpha_col_dtype, int tile_m, int tile_n, int waves, void* stream);

/*
 * fnn_gemm_a8w8 with a workspace: where few tiles would leave most CUs idle over a long K (at most 256
 * tiles of 128x128, K of 6144 and more), K is cut into parts that run as separate workgroups; the parts' int32 accumulators
 * meet in the workspace and the last part to finish a tile adds them up and writes the scaled output.
 * Integer addition does not depend on the order, so the result equals fnn_gemm_a8w8's bit for bit.  Shapes
 * that do not gain run exactly as in fnn_gemm_a8w8.  The role of the SPLIT_K meta-parameter of the
 * reference's kernel (flashnn/triton_kernels/gemm_a8w8.py:17-50, 74-179), whose parts meet through
 * tl.atomic_add on an output the caller has zeroed.
 *
 * workspace  device memory, 16-byte aligned; its first 4096 bytes are counters that must be zero when a
 *            call starts and are zero again when it ends: zero them once after allocation
 *            (fnn_workspace_init, or hipMemset / a zero-filled tensor) and never again - except after a
 *            call on it failed with FNN_ERR_HIP or its kernel was aborted: counters may then be left
 *            behind, and every later split on that workspace would be wrong until it is initialised
 *            again.  The rest needs no initialisation.  Calls that overlap in time (other streams, other
 *            threads, a captured graph replayed on several streams at once) need a workspace each.
 *            fnn_workspace_init(NULL, 0, stream) clears the counters of the library's own workspace
 *            on the current device (the one fnn_gemm_a8w8_static uses).
 * ws_bytes   its size.  fnn_gemm_a8w8_workspace_bytes(M, N, K) is what the call would use for a shape (0:
 *            the shape is not split); 32 MiB + 4096 bytes hold every shape.  With less than a shape needs
 *            the call takes the largest split that fits (16 MiB hold all but the splits into more units
 *            than there are CUs), and with none that fits (at least the 4096 bytes of counters; or
 *            workspace = NULL with ws_bytes = 0) it runs unsplit.
 */
size_t fnn_gemm_a8w8_workspace_bytes(int64_t M, int64_t N, int64_t K);
int fnn_workspace_init(void* workspace, size_t ws_bytes, void* stream);
int fnn_gemm_a8w8_ws(void* out, const void* a, const void* b, const void* alpha_row,
                     const void* alpha_col, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                     int64_t ldc, int out_dtype, int alpha_row_dtype, int alpha_col_dtype,
                     void* workspace, size_t ws_bytes, void* stream);

/*
 * fnn_gemm_a8w8_ws with the tile and the number of parts named: tiles 256x128, 256x192 and 128x128, kparts
 * from 2 up as long as a part holds four slabs of 128 bytes of K; kparts 0 or 1 is fnn_gemm_a8w8_tiled.
 * FNN_ERR_ARG if the shape cannot be split so or the workspace is too small (the message says what is
 * needed).  For tests and tuning; results are bit-identical for every choice.
 */
int fnn_gemm_a8w8_ws_tiled(void* out, const void* a, const void* b, const void* alpha_row,
                           const void* alpha_col, int64_t M, int64_t N, int64_t K, int64_t lda,
                           int64_t ldb, int64_t ldc, int out_dtype, int alpha_row_dtype,
                           int alpha_col_dtype, int tile_m, int tile_n, int kparts, void* workspace,
                           size_t ws_bytes, void* stream);

/*
 * fnn_gemm_a8w8_ws_tiled without the workspace argument: the workspace is an array of 16 MiB that the
 * library holds on every GPU it runs on (part of its code object, from load to the end of the process).
 * No counterpart in the reference.  It is for callers that cannot allocate: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc - the call allocates and frees nothing (the device
 * address of the array is looked up once per device, on the first call there).
 *   tile_m = tile_n = kparts = 0: the library's choice, as fnn_gemm_a8w8_ws with a workspace of 16 MiB.
 *   a named split that needs more than the array holds: FNN_ERR_UNSUPPORTED, and the message says how
 *   much; use fnn_gemm_a8w8_ws_tiled with a workspace of that size.
 * All calls on a GPU share that GPU's array: calls that overlap in time (other streams, other threads)
 * race on it and must use fnn_gemm_a8w8_ws with workspaces of their own.  The counters in the array are
 * zero at load and every call's kernel sets the ones it used back to zero before it ends; the rest keeps
 * the last call's contents and needs no clearing.  Results equal fnn_gemm_a8w8's bit for bit.
 */
int fnn_gemm_a8w8_static(void* out, const void* a, const void* b, const void* alpha_row,
                         const void* alpha_col, int64_t M, int64_t N, int64_t K, int64_t lda,
                         int64_t ldb, int64_t ldc, int out_dtype, int alpha_row_dtype,
                         int alpha_col_dtype, int tile_m, int tile_n, int kparts, void* stream);

/* fnn_gemm_a8w8_i32 through a named tile (same tiles as fnn_gemm_a8w8_tiled): lets a test check the integer
 * result of every tile bit for bit.  No counterpart in the reference API. */
int fnn_gemm_a8w8_i32_tiled(int32_t* acc, const void* a, const void* b, int64_t M, int64_t N, int64_t K,
                            int64_t lda, int64_t ldb, int64_t ldc, int tile_m, int tile_n, int waves,
                            void* stream);

/*
 * Replaces fused_moe_a8w8_forward(A, B, C, alpha_row_ptr, alpha_col_ptr, topk_weights, topk_ids,
 * sorted_token_ids, expert_ids, num_tokens_post_padded, mul_routed_weight, top_k, BM)
 * (flashnn/triton_kernels/fused_moe_a8w8.py:176-290; kernel :37-173), exported as
 * flashnn.fused_moe_a8w8_forward (flashnn/__init__.py:14).
 *
 * a: int8 [M,K] tokens (row stride lda); b: int8 [E,N,K] expert weights (stride_be between experts, ldb
 * between rows); c: fp16/bf16, addressed as [M*top_k, N] rows with row stride ldc (the reference's
 * C[M, top_k, N] with ldc = C.stride(1)).  Sorted row i (i < *num_tokens_post_padded, a multiple of
 * block_m) names the routed row t = sorted_token_ids[i]; t >= num_valid_tokens (= M*top_k) is padding.
 * Every block of block_m sorted rows belongs to the expert expert_ids[i / block_m].  For valid rows
 *   c[t, n] = (fp32(sum_k a[t / top_k, k] * b[e, n, k]) * alpha_row[t / top_k]) * alpha_col[e*stride_scale_be + n]
 * times topk_weights[t] when mul_routed_weight != 0; every product rounded to fp32, the result rounded
 * once to out_dtype (the reference always rounds to fp16, :162).  Rows of c that no valid sorted row names
 * are left untouched.  sorted_token_ids [EM], expert_ids and num_tokens_post_padded [1] are int32 device
 * arrays.  The weight-streaming kernel takes N % 16 == 0, K % 32 == 0, K >= 1024, block_m % 16 == 0,
 * EM % block_m == 0 and 16-byte aligned rows; anything else takes a slow guarded kernel.
 * Many routed rows per expert: with block_m a multiple of 128 (or of 64, from 512 routed rows on) and
 * K >= 1024 the call runs MFMA tiles over the sorted rows (tile height 64, 128 or 256 = the largest of those
 * that divides block_m) instead of streaming an expert's weights once per 64 rows; same arithmetic, same bits.
 */
int fnn_fused_moe_a8w8(void* c, const void* a, const void* b, const void* alpha_row,
                       const void* alpha_col, const void* topk_weights,
                       const int32_t* sorted_token_ids, const int32_t* expert_ids,
                       const int32_t* num_tokens_post_padded, int64_t N, int64_t K, int64_t EM,
                       int64_t num_valid_tokens, int64_t lda, int64_t stride_be, int64_t ldb,
                       int64_t ldc, int64_t stride_scale_be, int mul_routed_weight, int top_k,
                       int block_m, int out_dtype, int alpha_row_dtype, int alpha_col_dtype,
                       int topk_weights_dtype, void* stream);

/*
 * Replaces fused_moe_a16w4_forward(A, B, C, scale_b, zero_points, topk_weights, topk_ids,
 * sorted_token_ids, expert_ids, num_tokens_post_padded, mul_routed_weight, top_k, BM)
 * (flashnn/triton_kernels/fused_moe_a16w4.py:326-466; kernels :50-206 per channel, :209-323 per K block),
 * exported as flashnn.fused_moe_a16w4_forward (flashnn/__init__.py:15).
 *
 * a: fp16/bf16 [M,K] tokens; b: int8-typed [E,N,K], byte [e,j,k] holding output channel 2j in its low
 * nibble and 2j+1 in its high nibble, both two's complement (:146-147); c: same type as a, [M*top_k, 2N]
 * rows with stride ldc.  Routing arguments as for fnn_fused_moe_a8w8.  For a valid routed row t of expert e
 *   c[t, n] = sum_g scale[e, n, g] * sum_{k in block g} a[t / top_k, k] * (nibble[e, n, k] - zp[e, n, g])
 * times topk_weights[t] when mul_routed_weight != 0, accumulated in fp32 and rounded once.  group = 0:
 * one scale and zero point per channel (scale_b [E, 2N]); group = g > 0: per block of g values of K
 * (scale_b [E, 2N, K/g]).  scale[e, n, g] is read at e*stride_scale_be + n*stride_scale_n + g*stride_scale_k
 * (zero points alike; zero_points may be NULL).  zp_dtype: FNN_F16/BF16/F32 or 3 for int8.
 * The weight-streaming kernel takes group = 0 (unit channel stride, K % 32 == 0) or group = 128 (contiguous
 * [E, 2N, K/128] tables of one 16-bit type, K/128 a multiple of 8 and at most 64), floating zero points,
 * N % 16 == 0, K >= 1024, block_m % 16 == 0, EM % block_m == 0 and 16-byte aligned rows; anything else
 * takes a slow guarded kernel.  The reference multiplies the dequantised weights of a K block by their scale
 * before the dot product and rounds them to the scale type; here the block's dot product is scaled
 * afterwards, in fp32.  Many routed rows per expert: with block_m a multiple of 128, 2N % 128 == 0, K % 256 == 0
 * and either group = 0 with floating zero points or group = 128 with contiguous tables of one 16-bit type
 * (zero points in the scales' type, K <= 8192) the call runs the tiled MFMA kernel over the sorted rows (128 or
 * 256 rows x 128 channels per workgroup).
 */
int fnn_fused_moe_a16w4(void* c, const void* a, const void* b, const void* scale_b,
                        const void* zero_points, const void* topk_weights,
                        const int32_t* sorted_token_ids, const int32_t* expert_ids,
                        const int32_t* num_tokens_post_padded, int64_t N, int64_t K, int64_t EM,
                        int64_t num_valid_tokens, int64_t lda, int64_t stride_be, int64_t ldb,
                        int64_t ldc, int64_t stride_scale_be, int64_t stride_scale_n,
                        int64_t stride_scale_k, int64_t stride_zp_be, int64_t stride_zp_n,
                        int64_t stride_zp_k, int group, int mul_routed_weight, int top_k, int block_m,
                        int act_dtype, int scale_dtype, int zp_dtype, int topk_weights_dtype,
                        void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FLASHNN_HIP_H_ */
