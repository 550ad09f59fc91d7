/*
 * orbitquant_hip.h - C ABI of the MI355X (gfx950) quantized-linear forward.
 *
 * One shared library, plain pointers and sizes, no framework types.  Every
 * pointer is a DEVICE pointer unless a comment says otherwise; the library
 * borrows them for the duration of the call and keeps nothing.  Work is
 * enqueued on `stream` (a hipStream_t passed as void*; NULL = the null stream)
 * and the call returns without synchronizing, so calls may be captured into a
 * HIP graph.  Return value: OQ_OK or an oq_status error; `oq_last_error()`
 * gives the text of the last error raised on the calling thread.
 *
 * The entry points replace, for AMD GPUs, the operators the reference's native
 * package registers (paths relative to the reference checkout):
 *   native-kernels/orbitquant-packed-matmul/torch-ext/torch_binding.cpp:7-66
 *   native-kernels/orbitquant-packed-matmul/torch-ext/torch_binding.h:11-92
 * and the kernels behind them in
 *   native-kernels/orbitquant-packed-matmul/orbitquant_packed_matmul_cuda/packed_matmul.cu
 */
#ifndef ORBITQUANT_HIP_H
#define ORBITQUANT_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  OQ_OK = 0,
  OQ_ERR_INVALID = 1,     /* an argument is out of its documented range        */
  OQ_ERR_UNSUPPORTED = 2, /* valid request this build has no kernel for        */
  OQ_ERR_LAUNCH = 3       /* the HIP runtime rejected a launch / attribute set */
} oq_status;

typedef enum { OQ_F32 = 0, OQ_F16 = 1, OQ_BF16 = 2 } oq_dtype;

/* How activation codes are stored. */
typedef enum {
  OQ_CODES_U8 = 0,    /* one code per byte, [M, K]                                   */
  OQ_CODES_NIBBLE = 1 /* two codes per byte, even k in the low nibble, [M, K/2];     */
                      /* needs levels <= 16 and even K (packed_matmul.cu:648-656)    */
} oq_code_format;

/* What oq_rotate_quantize writes to `values_out`. */
typedef enum {
  OQ_VALUES_NONE = 0,
  OQ_VALUES_SCALED = 1,  /* centroid[code] * ||x||, rounded to x's dtype, [M, K]     */
                         /* (quantize_activations_cpu contract, torch_binding.h:28-37) */
  OQ_VALUES_UNIT_BF16 = 2 /* bf16(centroid[code]), [M, K]; the token norm stays in   */
                          /* norms_out and is applied by the matmul epilogue         */
} oq_values_mode;

/* Library / device probe.  Returns OQ_OK when a gfx950 device is current. */
int oq_device_ok(void);
const char *oq_last_error(void);
const char *oq_version(void);

/*
 * Fused RPBH rotate + per-token quantize.
 * Replaces quantize_activations_packed_w4 / quantize_activations_int8 /
 * quantize_activations_cpu (torch_binding.cpp:13-31,47-66; kernels
 * packed_matmul.cu:581-742; semantics src/orbitquant/functional.py:16-22):
 *
 *   s      = ||fp32(x_row)||_2                     (fixed summation order, see below)
 *   unit   = fp32(x_row) / (s + eps)               (IEEE division)
 *   y      = unit[perm] * signs                    (gather, exact)
 *   y      = blockwise FWHT(y), block `block`, butterfly distance 1,2,4,...
 *   rot    = y * inv_sqrt_block                    (one fp32 multiply)
 *   code   = #{ j : boundaries[j] < rot }          (ties to the lower code)
 *
 * Sum of squares order: the row is zero-padded to a multiple of 2048 and viewed
 * as [passes][256 lanes][8]; per (pass, lane) the eight squares are added as
 * ((s0+s1)+(s2+s3))+((s4+s5)+(s6+s7)); each lane adds its passes left to right;
 * the 256 lane sums are reduced by a balanced binary tree in lane order.  No
 * operation is contracted into an FMA.
 *
 * x            [M, K] of x_dtype, row-major, contiguous
 * perm         int32 [K], signs int8 [K] (+1/-1)
 * boundaries   fp32 [levels-1], ascending;  2 <= levels <= 256
 * centroids    fp32 [levels]; only read when values_mode != OQ_VALUES_NONE (else may be NULL)
 * block        power of two dividing K;  K <= 16384
 * rotate_plan  NULL, or the plan oq_rotate_plan_build made from these perm, signs, boundaries,
 *              levels, K, block and inv_sqrt_block: launches of more than 16 rows then take the
 *              plan-based kernel (a third of the instructions, the same results bit for bit)
 * codes_out    NULL or [M, K] u8 / [M, K/2] u8 per code_format
 * values_out   NULL or per values_mode
 * norms_out    fp32 [M]: the raw norm s (no eps); may be NULL
 */
int oq_rotate_quantize(const void *x, int x_dtype, int64_t M, int64_t K,
                       const int32_t *perm, const int8_t *signs,
                       const float *boundaries, const float *centroids, int levels,
                       int64_t block, float eps, float inv_sqrt_block, const void *rotate_plan,
                       void *codes_out, int code_format,
                       void *values_out, int values_mode,
                       float *norms_out, void *stream);

/*
 * The rotate plan: everything the rotate+quantize kernel can know about a layer before it sees
 * a token (permutation and signs merged into gather offsets, the boundaries folded with
 * inv_sqrt_block, the bucketize table), built once per layer by one small launch and kept by
 * the caller in device memory next to the layer's other constants: oq_rotate_plan_bytes(K)
 * bytes, 16-byte aligned.  No counterpart in the reference, whose kernels re-derive all of it per
 * row (packed_matmul.cu:581-657).  A plan is only valid for the arguments it was built from; a
 * call that passes a plan built for another K, block or levels writes nothing.
 */
uint64_t oq_rotate_plan_bytes(int64_t K);
int oq_rotate_plan_build(const int32_t *perm, const int8_t *signs, const float *boundaries, int levels,
                         int64_t K, int64_t block, float inv_sqrt_block, void *plan_out, void *stream);

/*
 * The weight side of a layer on the GPU: what the packed matmuls read, made from a float weight
 * matrix.  Replaces the reference's device-side weight quantization
 * (src/orbitquant/layers.py:102-125,159-222; src/orbitquant/kernels/triton_cuda.py:926-1039,2740-2935).
 * Per output row:
 *
 *   r      = ||fp32(w_row)||_2                     (the summation order of oq_rotate_quantize)
 *   rot    = blockwise FWHT(fp32(w_row)[perm] * signs) * inv_sqrt_block
 *   unit   = rot / max(r, eps)                     (IEEE division; note the order: rotate, scale, divide)
 *   idx    = #{ j : boundaries[j] < unit }
 *
 * packed_out is the flat little-endian bit stream of idx[N, K], `bits` per index
 * (ceil(N*K*bits/8) bytes; src/orbitquant/packing/bitpack.py:8-46), row_norms_out is bf16(r) [N].
 * A zero row keeps r = 0, so it dequantizes to exact zeros.
 *
 * w            [N, K] of w_dtype, row-major, 16-byte aligned;  K a multiple of 8, K <= 16384
 * rotate_plan  the plan oq_rotate_plan_build made from the layer's perm and signs with THESE
 *              boundaries, levels, K, block and inv_sqrt_block (only its gather entries are used)
 * boundaries   fp32 [levels-1] of the weight codebook;  2 <= levels <= 2^bits, 1 <= bits <= 8
 * block        power of two dividing K, 8 <= block <= 4096
 */
int oq_quantize_weight(const void *w, int w_dtype, int64_t N, int64_t K, const void *rotate_plan,
                       const float *boundaries, int levels, int64_t block, float eps, float inv_sqrt_block,
                       int bits, uint8_t *packed_out, uint16_t *row_norms_out, void *stream);

/*
 * The same, on f(x) instead of x, for an elementwise function f of a 16-bit
 * input given as a table: input_map[bits of x] = bits of f(x), 65536 entries of
 * the same dtype as x, 16-byte aligned, on the device.  The result is what
 * oq_rotate_quantize returns for the tensor f(x), bit for bit; f(x) is never
 * written to memory.  x_dtype must be OQ_F16 or OQ_BF16.  rotate_plan: as for
 * oq_rotate_quantize (bf16 rows into codes take the plan-based kernel with it).
 *
 * No counterpart in the reference's extension: there the activation between two
 * quantized linears (the GELU of an MLP, functional calls in the model code) is
 * a separate elementwise kernel that writes f(x) and the quantizer reads it
 * back; the table is how a caller hands that function to this kernel without
 * changing its results (fill it by applying the framework's own f to all
 * 65536 bit patterns).
 */
int oq_rotate_quantize_mapped(const void *x, int x_dtype, const uint16_t *input_map,
                              int64_t M, int64_t K,
                              const int32_t *perm, const int8_t *signs,
                              const float *boundaries, const float *centroids, int levels,
                              int64_t block, float eps, float inv_sqrt_block, const void *rotate_plan,
                              void *codes_out, int code_format,
                              void *values_out, int values_mode,
                              float *norms_out, void *stream);

/*
 * Sets (value != NULL) or clears one of the library's experiment switches, the OQ_* environment
 * variables that pick a launch shape or turn a kernel variant off (OQ_GEMM_TILE, OQ_GEMM_WG_SPLIT,
 * OQ_GEMV_CFG, OQ_NO_TOKEN_LINEAR, ...).  The library reads the environment once per process;
 * tests and measurements that compare variants inside one process change a switch through this
 * call.  Results stay correct under every setting; only which kernel computes them changes.
 * Not thread-safe against running calls.  No counterpart in the reference.
 * Refused (OQ_ERR_INVALID) unless the process was started with ORBITQUANT_DEBUG=1 in its
 * environment: a serving process cannot have its kernels, and so the bits of its results,
 * switched under it.
 */
int oq_debug_override(const char *name, const char *value);

/*
 * Packed-weight linear on quantized activations (the fused hot path):
 *
 *   out[m,n] = (sum_k c_a[code[m,k]] * c_w[idx[n,k]]) * s[m] * r_w[n] + bias[n]
 *
 * Replaces matmul_packed_w4a4_int8 (torch_binding.cpp:39-46; packed_matmul.cu:744-1009)
 * for every weight width, with exact (bf16-rounded) centroids instead of the
 * int8 surrogate.  M <= 64 takes the streaming small-M kernel (the weights are read and
 * decoded once, sixteen token rows per matrix instruction, up to four blocks of sixteen per
 * workgroup), larger M the MFMA tile kernel.  A token row's result does not depend on the
 * rows computed with it as long as the call stays within 64 rows.  A problem with few output
 * tiles and many K-steps (some hundred tokens on a short-and-long matrix) is shared between
 * workgroups along K when the caller provides a workspace for the fp32 partial tiles:
 *
 * workspace    NULL, or a device buffer of at least oq_packed_linear_workspace_bytes(...) bytes, 16-byte
 *              aligned, that this call may overwrite (calls on one stream are ordered and may share one).
 *              The library allocates nothing: as in the reference, whose Python wrapper owns every
 *              allocation (torch-ext/orbitquant_packed_matmul/__init__.py:130-160), kernels borrow all
 *              pointers.  NULL, or too small: the single launch.  Which kernel runs depends on the
 *              arguments alone, so a call captured into a graph computes what the eager call does, bit
 *              for bit.
 *
 * codes        activation codes in code_format (see oq_rotate_quantize)
 * token_norms  fp32 [M]
 * act_centroids fp32 [2^a_bits]
 * packed_w     flat little-endian bit stream of idx[N,K], value v at bits [v*w_bits, v*w_bits+w_bits)
 *              (src/orbitquant/packing/bitpack.py:8-46); w_bits in [1, 8]: 2, 3, 4, 6 and 8 take the
 *              tiled and streaming kernels, the other widths the shape-agnostic kernel
 * row_norms    bf16 [N] (raw uint16 bit patterns)
 * w_centroids  fp32 [2^w_bits]
 * bias         NULL or [N] of bias_dtype
 * out          [M, N] of out_dtype (OQ_BF16, OQ_F16 or OQ_F32)
 */
int oq_packed_linear(const void *codes, int code_format, const float *token_norms,
                     const float *act_centroids, int a_bits,
                     const uint8_t *packed_w, int w_bits, const uint16_t *row_norms,
                     const float *w_centroids, const void *bias, int bias_dtype,
                     int64_t M, int64_t N, int64_t K, void *out, int out_dtype,
                     void *workspace, uint64_t workspace_bytes, void *stream);

/*
 * Bytes of workspace oq_packed_linear (and _mapped, oq_quantized_linear, and each member of a group)
 * can make use of for this shape; 0 when it takes a single launch anyway.  No counterpart in the
 * reference (its wrapper sizes its own temporaries).
 */
uint64_t oq_packed_linear_workspace_bytes(int64_t M, int64_t N, int64_t K, int w_bits, int code_format, int a_bits);

/*
 * `count` packed linears on the SAME activation codes (the q, k and v projections of an attention
 * block, the gate and up projections of an MLP): out[i] = oq_packed_linear(codes, ..., packed_w[i],
 * w_bits[i], row_norms[i], w_centroids[i], bias[i], M, N[i], K), bit for bit.  The argument arrays
 * (count entries each, read during the call only) live in host memory and hold device pointers;
 * `bias` may be NULL (no matrix has one) or hold NULL entries.  For at most 32 tokens, nibble
 * codes, 2-, 3- or 4-bit weights and two to four matrices the whole group is ONE launch of the
 * streaming kernel (at decode sizes a launch is mostly fixed cost); any other group runs as
 * `count` launches.  No counterpart in the reference, whose layers each call
 * matmul_packed_* on their own (src/orbitquant/layers.py:1079-1455); it replaces `count`
 * consecutive calls of oq_packed_linear.
 */
int oq_packed_linear_group(const void *codes, int code_format, const float *token_norms,
                           const float *act_centroids, int a_bits, int count,
                           const uint8_t *const *packed_w, const int *w_bits,
                           const uint16_t *const *row_norms, const float *const *w_centroids,
                           const void *const *bias, int bias_dtype, int64_t M, const int64_t *N,
                           int64_t K, void *const *out, int out_dtype,
                           void *workspace, uint64_t workspace_bytes, void *stream);

/*
 * oq_packed_linear followed by an elementwise function of the 16-bit outputs given as a
 * table (output_map[bits of y] = bits of f(y), 65536 entries of the output dtype, 16-byte
 * aligned, on the device): out = f(linear) bit for bit, f(...) applied before the store
 * (tile kernels: in the epilogue; other kernels: by a small elementwise launch).  out_dtype
 * must be OQ_F16 or OQ_BF16.  No counterpart in the reference, like oq_rotate_quantize_mapped:
 * it is the activation that follows a linear, without its kernel.
 */
int oq_packed_linear_mapped(const void *codes, int code_format, const float *token_norms,
                            const float *act_centroids, int a_bits,
                            const uint8_t *packed_w, int w_bits, const uint16_t *row_norms,
                            const float *w_centroids, const void *bias, int bias_dtype,
                            int64_t M, int64_t N, int64_t K, void *out, int out_dtype,
                            const uint16_t *output_map, void *workspace, uint64_t workspace_bytes, void *stream);

/*
 * The whole quantized-linear forward in one call: oq_rotate_quantize (through
 * `input_map` when it is not NULL, see oq_rotate_quantize_mapped) followed by
 * oq_packed_linear, with the same results bit for bit.  It is the native form of the
 * reference layer's forward (src/orbitquant/layers.py:1079-1455: quantize_activations_*
 * then matmul_packed_*), which exists there only as Python glue between two ops.
 *
 * One token (M == 1) of a 16-bit dtype with a_bits <= 4, w_bits 2, 3 or 4, K a multiple of
 * 128 up to 8192, N up to 8192 and 16-byte aligned operands is a SINGLE launch: every workgroup
 * of the streaming kernel quantizes the token itself while its weight loads are in flight, so
 * decoding pays one launch per linear and the scratch buffers are not touched.  Callers that
 * cannot tell in advance pass scratch always; NULL scratch is an error only when it is
 * needed.  Every other shape is the two launches, with the codes
 * ([M, K/2] bytes when a_bits <= 4 and K is even, else [M, K]) and norms (fp32 [M]) passing
 * through the caller's scratch buffers (16-byte aligned).
 *
 * `rotate_plan` (NULL for none): see oq_rotate_quantize.
 *
 * `output_map` (NULL for none) is a table like `input_map`, of the OUTPUT dtype (16-bit
 * only), applied to every output value before it is stored: out = f(linear(x)) bit for bit
 * what f applied to the stored result of the plain call gives.  The tile kernels look the
 * values up in their epilogue; the small-M and shape-agnostic kernels are followed by a tiny
 * elementwise launch.  It is the cheaper place for the activation between two linears (a
 * lookup per output value in a kernel that is waiting for its stores, instead of a lookup
 * per input value in the quantizer, which has no such slack).
 */
int oq_quantized_linear(const void *x, int x_dtype, const uint16_t *input_map,
                        int64_t M, int64_t K,
                        const int32_t *perm, const int8_t *signs,
                        const float *boundaries, const float *act_centroids, int a_bits,
                        int64_t block, float eps, float inv_sqrt_block, const void *rotate_plan,
                        const uint8_t *packed_w, int w_bits, const uint16_t *row_norms,
                        const float *w_centroids, const void *bias, int bias_dtype, int64_t N,
                        void *codes_scratch, float *norms_scratch,
                        void *out, int out_dtype, const uint16_t *output_map,
                        void *workspace, uint64_t workspace_bytes, void *stream);

/*
 * oq_quantized_linear for `count` linears that read the same input (q, k and v of an attention
 * block; gate and up of an MLP): the input is quantized once into the caller's scratch buffers
 * (required; sizes as for oq_quantized_linear), then oq_packed_linear_group.  out[i] equals what
 * oq_quantized_linear gives for matrix i, bit for bit.  Arrays as in oq_packed_linear_group.
 * No counterpart in the reference (see oq_packed_linear_group).
 */
int oq_quantized_linear_group(const void *x, int x_dtype, const uint16_t *input_map,
                              int64_t M, int64_t K,
                              const int32_t *perm, const int8_t *signs, const float *boundaries,
                              const float *act_centroids, int a_bits,
                              int64_t block, float eps, float inv_sqrt_block, const void *rotate_plan,
                              int count, const uint8_t *const *packed_w, const int *w_bits,
                              const uint16_t *const *row_norms, const float *const *w_centroids,
                              const void *const *bias, int bias_dtype, const int64_t *N,
                              void *codes_scratch, float *norms_scratch,
                              void *const *out, int out_dtype,
                              void *workspace, uint64_t workspace_bytes, void *stream);

/*
 * oq_quantized_linear for callers that cannot allocate device memory or bring a workspace:
 * code running under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  No counterpart in the reference.  Same arguments as oq_quantized_linear without
 * the two scratch pointers, and the same results (except where oq_quantized_linear shares K
 * between workgroups through a buffer of the library's own, see oq_packed_linear: this call
 * never does, and the two then differ by the order of the last additions): codes and norms pass through a buffer
 * of OQ_STATIC_SCRATCH_BYTES that is part of the library's device image (every GPU the library
 * runs on holds its own copy until the process ends).  The call allocates and frees nothing.
 * Shapes whose codes ([M, K/2] bytes for a_bits <= 4 and even K, else [M, K], rounded up to
 * 256) plus norms (4 M bytes) do not fit are refused with OQ_ERR_UNSUPPORTED.  All calls on one
 * GPU share the buffer: calls that may overlap there (different streams, or graphs replayed
 * concurrently) race, and the buffer keeps the previous call's contents (every byte a call
 * reads it has written itself first).  The buffer's address on a device is looked up the
 * first time that device is current in oq_device_ok() or in this call; callers that capture
 * graphs call oq_device_ok() once beforehand.
 */
#define OQ_STATIC_SCRATCH_BYTES (8u << 20)
int oq_quantized_linear_static(const void *x, int x_dtype, const uint16_t *input_map,
                               int64_t M, int64_t K,
                               const int32_t *perm, const int8_t *signs,
                               const float *boundaries, const float *act_centroids, int a_bits,
                               int64_t block, float eps, float inv_sqrt_block, const void *rotate_plan,
                               const uint8_t *packed_w, int w_bits, const uint16_t *row_norms,
                               const float *w_centroids, const void *bias, int bias_dtype, int64_t N,
                               void *out, int out_dtype, const uint16_t *output_map, void *stream);

/*
 * Packed-weight matmul on float activations:
 *
 *   out[m,n] = (sum_k x[m,k] * c_w[idx[n,k]]) * r_w[n] + bias[n]      (out in x's dtype)
 *
 * Replaces matmul_packed_weight (torch_binding.cpp:7-12,32-38; packed_matmul.cu:1335-1713).
 * bits in [1, 8].  token_scale: NULL, or fp32 [M] multiplied into row m (lets the
 * caller pass unit-norm bf16 centroids plus token norms).
 * workspace: NULL, or oq_matmul_packed_weight_workspace_bytes(...) bytes of device memory, 16-byte aligned,
 * that the call may overwrite.  With it, bf16 activations (from two tokens on; one token on large matrices)
 * are first rewritten into the matrix core's operand order (2 * M * K bytes, rows padded to 32) and the
 * tile kernel reads that copy; without it every wavefront stages its own rows through LDS (no buffer, the
 * same sums, 10-15 % slower on large problems).  The library allocates nothing.
 */
int oq_matmul_packed_weight(const void *x, int x_dtype, const float *token_scale,
                            const uint8_t *packed_w, int bits, const uint16_t *row_norms,
                            const float *w_centroids, const void *bias, int bias_dtype,
                            int64_t M, int64_t N, int64_t K, void *out, int out_dtype,
                            void *workspace, uint64_t workspace_bytes, void *stream);

/* Bytes of workspace oq_matmul_packed_weight can make use of for this shape (0: none). */
uint64_t oq_matmul_packed_weight_workspace_bytes(int64_t M, int64_t N, int64_t K, int w_bits, int x_dtype);

/*
 * Packed INT4 group-scaled linear on bf16 activations (the AdaLN modulation linears):
 *
 *   w[n,k]   = bf16( (q[n,k] - 8) * float(scales[n, k / group_size]) )
 *   out[m,n] = bf16( sum_k x[m,k] * w[n,k] + float(bias[n]) )          (fp32 accumulation)
 *
 * Replaces matmul_packed_adaln_int4_cpu (torch_binding.cpp:47-66) and the reference's Triton
 * kernel for it (src/orbitquant/kernels/triton_cuda.py:682-819) on AMD GPUs.
 *
 * x             bf16 [M, K] (raw bit patterns), row-major
 * packed_weight 4-bit q, two per byte, low nibble first, rows padded to whole groups:
 *               [N, groups * group_size / 2] bytes with groups = ceil(K / group_size)
 *               (src/orbitquant/adaln.py:17-35)
 * scales        bf16 [N, groups]
 * bias          NULL or bf16 [N]
 * out           bf16 [M, N]
 * K a multiple of 8, group_size a multiple of 8 and a 16-byte aligned x take the streaming
 * kernel, anything else a shape-agnostic one.
 */
int oq_matmul_packed_adaln_int4(const uint16_t *x, const uint8_t *packed_weight, const uint16_t *scales,
                                const uint16_t *bias, int64_t M, int64_t N, int64_t K, int64_t group_size,
                                uint16_t *out, void *stream);

/*
 * The weight side of the AdaLN linears on the GPU: group-wise round-to-nearest INT4
 * (src/orbitquant/adaln.py:17-35 `quantize_adaln_weight_int4`; the reference runs it as torch
 * operations on whatever device holds the weight):
 *
 *   scale[n,g] = max(max_k |w[n,k]|, 1e-12) / 7            over the group's k, fp32, IEEE division
 *   q[n,k]     = clamp(round_half_even(w[n,k] / scale[n,g]), -8, 7) + 8      (padding beyond K: 8)
 *
 * w          [N, K] of w_dtype (OQ_F32 / OQ_F16 / OQ_BF16), row-major
 * packed_out [N * groups * group_size / 2] bytes, low nibble first, groups = ceil(K / group_size)
 * scales_out fp32 [N, groups] (the module stores them rounded to bf16)
 * group_size even.
 */
int oq_quantize_adaln_weight(const void *w, int w_dtype, int64_t N, int64_t K, int64_t group_size, uint8_t *packed_out,
                             float *scales_out, void *stream);

/*
 * Unpack a little-endian bit stream into one index per byte (debug / tests;
 * the GPU twin of unpack_lowbit, src/orbitquant/packing/bitpack.py:63-97).
 */
int oq_unpack_lowbit(const uint8_t *packed, int bits, int64_t count, uint8_t *out, void *stream);

/*
 * The inverse of oq_unpack_lowbit: values[i] (its low `bits` bits) into bits [i * bits, (i + 1) * bits)
 * of a little-endian stream of ceil(count * bits / 8) bytes, unused tail bits zero.
 * Replaces pack_lowbit (src/orbitquant/packing/lowbit.py) and its Triton form
 * (src/orbitquant/kernels/triton_cuda.py:878-899, 2681-2710) on AMD GPUs.  bits in [1, 8].
 */
int oq_pack_lowbit(const uint8_t *values, int bits, int64_t count, uint8_t *packed_out, void *stream);

/*
 * The dense form of a packed weight, in the rotated basis the layer multiplies in:
 *   out[n,k] = centroids[index[n,k]] * float(row_norms[n])        (one fp32 product, then rounded to out_dtype)
 * Replaces dequantize_packed_weight_with_triton (src/orbitquant/kernels/triton_cuda.py:523-547,
 * 1538-1571; fp32 out there) for the reference's `dequant_bf16` debug mode.
 * packed_weight  N * K indices of `bits` bits, one stream over the whole matrix
 * row_norms      bf16 [N];  centroids fp32 [2^bits];  out [N, K] of out_dtype.
 */
int oq_dequantize_packed_weight(const uint8_t *packed_weight, int bits, const uint16_t *row_norms, const float *centroids,
                                int64_t N, int64_t K, void *out, int out_dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* ORBITQUANT_HIP_H */
