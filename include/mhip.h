/* mhip.h — C-ABI launch shim for the gfx950 (MI355X) kernel library.
 *
 * This is the boundary a host (the reference's Swift executor, the C++ host in
 * this repository, or any FFI) binds in place of the reference's Metal kernel
 * library: one entry point per fused operator, taking a HIP stream, raw device
 * pointers, shape scalars and a small set of flags.  It mirrors the reference's
 * kernel ABI — buffers in operand order, then outputs, then scalars
 * (Sources/MetalHLOCore/Compiler/KernelTypes.swift:259-313,
 *  Sources/MetalHLOCore/Compiler/CodeGenerator.swift:5681-5879).
 *
 * All tensors are dense row-major with the last dimension contiguous.
 * Every call only enqueues work on `stream` (NULL = the default stream) and
 * returns; nothing synchronises.  Return value: MHIP_OK or an MHIP_ERR_* code;
 * mhip_last_error() then holds a message (thread-local).
 */
#ifndef MHIP_H
#define MHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element types use the numbering of MHLOElementType
 * (Sources/CMetalHLO/include/metalhlo.h:62-76). */
typedef enum {
    MHIP_F16 = 0,
    MHIP_F32 = 1,
    MHIP_F64 = 2,
    MHIP_BF16 = 3,
    MHIP_I1 = 4,
    MHIP_I8 = 5,
    MHIP_I16 = 6,
    MHIP_I32 = 7,
    MHIP_I64 = 8,
    MHIP_UI8 = 9,
    MHIP_UI16 = 10,
    MHIP_UI32 = 11,
    MHIP_UI64 = 12
} mhip_dtype;

typedef enum {
    MHIP_OK = 0,
    MHIP_ERR_INVALID_ARGUMENT = 1, /* NULL pointer, non-positive size, misaligned buffer */
    MHIP_ERR_UNSUPPORTED = 2,      /* dtype / shape outside what the kernels cover */
    MHIP_ERR_LAUNCH = 3,           /* HIP reported an error for the launch */
    MHIP_ERR_NO_DEVICE = 4
} mhip_status;

/* Activation of fused_matmul_bias_activation
 * (Sources/MetalHLOCore/Compiler/IntegrationTypes.swift:328-355). */
typedef enum {
    MHIP_ACT_NONE = 0,
    MHIP_ACT_RELU = 1,
    MHIP_ACT_GELU = 2, /* tanh approximation, CustomCallHandlers.swift:540-558 */
    MHIP_ACT_SILU = 3,
    MHIP_ACT_TANH = 4,
    MHIP_ACT_SIGMOID = 5,
    MHIP_ACT_GELU_ERF = 6 /* 0.5 x (1 + erf(x / sqrt 2)): what "gelu_exact" names (CustomCallHandlers.swift:893-894;
                            the reference falls back to the tanh form there, :540-558, this build does not) */
} mhip_activation;

/* Library / device ------------------------------------------------------- */

/* Version string, static storage (cf. mhlo_version, metalhlo.h:23). */
const char* mhip_version(void);

/* Last error message of the calling thread, "" if none
 * (cf. mhlo_get_last_error, metalhlo.h:53). */
const char* mhip_last_error(void);

/* Number of visible HIP devices; 0 when there is none. */
int mhip_device_count(void);

/* Device facts used by launch heuristics and reports: compute units, LDS bytes
 * per workgroup, gcn arch name (written into `arch`, NUL-terminated). Replaces
 * MTLDevice queries in Metal/Kernels/KernelRegistry.swift:122-165. */
int mhip_device_info(int device, int* out_cus, int* out_lds_bytes, char* arch, size_t arch_len);

/* Row operators (HBM-bound) ---------------------------------------------- */

/* y = softmax(x) over the last axis of x[rows, cols].
 * Replaces SoftmaxKernel (Metal/Kernels/SoftmaxKernel.swift:16-215) and
 * generateSoftmaxSource (Compiler/CodeGenerator.swift:4690-4794).
 * dtype: F32, F16, BF16 (16-bit types compute in fp32, one final rounding). */
int mhip_softmax(void* stream, const void* x, void* y, int64_t rows, int64_t cols, int dtype);

/* Softmax over a middle axis: x viewed as [outer, axis_len, inner], inner > 1.
 * (Compiler/CodeGenerator.swift:4690-4697 general-axis variant.) */
int mhip_softmax_strided(void* stream, const void* x, void* y, int64_t outer, int64_t axis_len,
                         int64_t inner, int dtype);

/* y = (x - mean) * rsqrt(var + eps) * gamma + beta over the last axis.
 * gamma / beta may be NULL (layer_norm_no_affine_kernel).
 * Replaces LayerNormKernel (Metal/Kernels/LayerNormKernel.swift:34-408);
 * operand order [x, gamma, beta] of FusedLayerNormHandler
 * (Compiler/CustomCallHandlers.swift:285-346). Variance is two-pass. */
int mhip_layer_norm(void* stream, const void* x, const void* gamma, const void* beta, void* y,
                    int64_t rows, int64_t cols, float eps, int dtype);

/* y = x * rsqrt(mean(x^2) + eps) * gamma; gamma may be NULL.
 * Replaces RMSNormKernel (Metal/Kernels/LayerNormKernel.swift:420-733). */
int mhip_rms_norm(void* stream, const void* x, const void* gamma, void* y, int64_t rows,
                  int64_t cols, float eps, int dtype);

/* y = gelu_tanh(x + bias[col]); bias may be NULL (plain fused_gelu).
 * Replaces GELUKernel (Metal/Kernels/GELUKernel.swift:15-123) and the epilogue
 * of generateMatMulBiasActSource (Compiler/CodeGenerator.swift:4797-4850). */
int mhip_bias_gelu(void* stream, const void* x, const void* bias, void* y, int64_t rows,
                   int64_t cols, int dtype);
/* The same with the exact form 0.5 v (1 + erf(v / sqrt 2)), v = x + bias: what a decomposed
 * erf GELU (jax.nn.gelu(approximate=False)) is rewritten to.  The reference has no kernel for it
 * (Metal/Kernels/GELUKernel.swift:15-123 is the tanh form only). */
int mhip_bias_gelu_erf(void* stream, const void* x, const void* bias, void* y, int64_t rows,
                       int64_t cols, int dtype);

/* dot_general ------------------------------------------------------------ */

/* C[b] = act(op(A[b]) . op(B[b]) + bias[col]) for b in [0, batch).
 * op(A) is [M,K] (stored [K,M] when trans_a), op(B) is [K,N] (stored [N,K]
 * when trans_b); strides are in elements between consecutive batch matrices
 * (0 broadcasts an operand).  bias (length N, same dtype) may be NULL.
 * fp32 accumulate, one rounding at the store.  dtype: BF16, F16, F32; also F64 (f64
 * accumulate) and I32 / I64 (wrap-around), those three without activation.
 * Replaces the kernel_matmul family and kernel_matmul_bias_act
 * (Compiler/CodeGenerator.swift:3155-4068, 4797-4850); M/K/N/batch are what
 * dotGeneralDims (:5939-5970) derives. */
int mhip_gemm(void* stream, const void* a, const void* b, const void* bias, void* c, int64_t M,
              int64_t N, int64_t K, int64_t batch, int64_t stride_a, int64_t stride_b,
              int64_t stride_c, int trans_a, int trans_b, int activation, int dtype);

/* The same with a residual: C[b] = act(op(A[b]) . op(B[b]) + bias[col]) + R[b], R laid out
 * like C (same batch stride; R may be C itself).  The stored value is rounded to the element
 * type before R is added and the sum is rounded again, i.e. bit for bit what mhip_gemm
 * followed by mhip_add produces, without the extra pass over C.  Serves the
 * `x + proj(...)` pairs of a transformer block, which the reference runs as dot_general
 * followed by a separate add kernel (Compiler/CodeGenerator.swift:921-1100 binary ops). */
int mhip_gemm_residual(void* stream, const void* a, const void* b, const void* bias,
                       const void* residual, void* c, int64_t M, int64_t N, int64_t K,
                       int64_t batch, int64_t stride_a, int64_t stride_b, int64_t stride_c,
                       int trans_a, int trans_b, int activation, int dtype);

/* Attention -------------------------------------------------------------- */

/* O = softmax(scale * Q K^T + mask, causal) V.
 * Q,O [B,H,Sq,D]; K,V [B,H,Skv,D]; mask NULL or additive [B,H,Sq,Skv] with
 * batch/head strides `mask_stride_b`, `mask_stride_h` in elements (0 = broadcast).
 * Causal rule: key position > query position is masked; a row with no
 * unmasked key yields zeros.  fp32 softmax state and accumulation.
 * Replaces FlashAttentionTiledKernel (Metal/Kernels/FlashAttentionKernel.swift:462-671)
 * launched from MetalExecutor.executeFlashAttentionDirect
 * (Runtime/MetalExecutor.swift:502-564). dtype: BF16, F16, F32. D in {64, 128}
 * for the MFMA path; other D up to 256 take a scalar path. */
int mhip_flash_attention(void* stream, const void* q, const void* k, const void* v,
                         const void* mask, void* o, int64_t B, int64_t H, int64_t Sq, int64_t Skv,
                         int64_t D, float scale, int is_causal, int64_t mask_stride_b,
                         int64_t mask_stride_h, int dtype);

/* The same operator on tensors that are views: `strides` holds twelve element strides,
 * {batch, head, row} for q, k, v, o in that order (NULL = packed, as above); the head
 * dimension itself is contiguous.  This lets attention read Q, K, V straight out of a
 * fused QKV projection [B,S,3,H,D] and write O as [B,S,H,D], in place of the
 * transpose / reshape / slice operations the reference materialises around its attention
 * call (it has no strided variant: MetalExecutor.swift:502-564 binds packed buffers).
 * Strided layouts need bf16 / f16, D in {64, 128}, 16-byte aligned pointers and strides
 * that are multiples of 8 elements; anything else returns 2 (unsupported). */
int mhip_flash_attention_strided(void* stream, const void* q, const void* k, const void* v,
                                 const void* mask, void* o, int64_t B, int64_t H, int64_t Sq,
                                 int64_t Skv, int64_t D, float scale, int is_causal,
                                 int64_t mask_stride_b, int64_t mask_stride_h, int dtype,
                                 const int64_t* strides);

/* Glue operators (index / data movement; integer results are bit-exact) ---- */

/* out[i, :] = table[clamp(idx[i], 0, n_rows-1), :], rows of `row_elems` elements.
 * StableHLO gather with whole-row slices; the clamp is the specification's
 * ([0, dim - slice_size]), not the reference's (Compiler/CodeGenerator.swift:1252-1254).
 * Replaces the gather kernels of Compiler/CodeGenerator.swift:1133-1397.
 * table_dtype: any 1/2/4/8-byte type; idx_dtype: I32 or I64. */
int mhip_gather_rows(void* stream, const void* table, const void* indices, void* out,
                     int64_t n_idx, int64_t n_rows, int64_t row_elems, int table_dtype,
                     int idx_dtype);

/* General stablehlo.gather from a descriptor the caller derives from the dimension
 * numbers: for the result element with indices i_0 .. i_{rank-1},
 *   out[i] = operand[sum_d i_d * out_operand_strides[d]
 *                    + sum_c clamp(indices[sum_d i_d * out_index_strides[d] + c * component_stride],
 *                                  0, component_max[c]) * component_operand_strides[c]]
 * (offset and batching dims carry an operand stride, batch dims an index stride; component c is
 * the start index along operand dim start_index_map[c], clamped to dim - slice_size).  rank and
 * n_components <= 8; elem_size in {1,2,4,8}; idx_dtype I32 or I64.
 * Replaces the gather kernels of Compiler/CodeGenerator.swift:1133-1397 in their general form. */
int mhip_gather(void* stream, const void* operand, const void* indices, void* out, int rank,
                const int64_t* out_shape, const int64_t* out_operand_strides,
                const int64_t* out_index_strides, int n_components, int64_t component_stride,
                const int64_t* component_operand_strides, const int64_t* component_max, int elem_size,
                int idx_dtype);

/* dst = src, `bytes` bytes, device to device, as one streaming kernel (reshape /
 * copy; also the calibration kernel for the HBM traffic counters).
 * Replaces the copy kernels of Compiler/CodeGenerator.swift:851-921. */
int mhip_copy(void* stream, const void* src, void* dst, int64_t bytes);

/* out[b, s, :] = convert(wte[ids[b, s], :] + wpe[s, :]) — token + position
 * embedding in one pass (gather :1133-1397, add :921, convert :1012-1078 of
 * Compiler/CodeGenerator.swift).  ids are I32 [B,S]; params F32 or the output
 * type; the sum is formed in fp32 and rounded once (RNE). */
int mhip_embed_tokens(void* stream, const void* ids, const void* wte, const void* wpe, void* out,
                      int64_t B, int64_t S, int64_t d_model, int64_t vocab, int param_dtype,
                      int out_dtype);

/* y = a + b elementwise over n elements (Compiler/CodeGenerator.swift:921).
 * F32/F16/BF16 add in fp32 and round once; I32/I64 wrap. */
int mhip_add(void* stream, const void* a, const void* b, void* y, int64_t n, int dtype);

/* y = convert(x), n elements (Compiler/CodeGenerator.swift:1012-1078).
 * Any pair of the element types; float narrowing is round-to-nearest-even, float -> int
 * truncates toward zero, int -> int keeps the low bits, anything -> I1 is x != 0. */
int mhip_convert(void* stream, const void* x, void* y, int64_t n, int src_dtype, int dst_dtype);

/* ys[i] = convert(xs[i]), ns[i] elements each, for `count` tensors in as few launches as the
 * table allows (96 tensors per launch): the same conversion (CodeGenerator.swift:1012-1078,
 * round to nearest even) as mhip_convert, for the many small tensors of a model's parameters.
 * F32 -> BF16 / F16 only; anything else returns 2 and the caller converts one by one. */
int mhip_convert_batch(void* stream, int count, const void* const* xs, void* const* ys,
                       const int64_t* ns, int src_dtype, int dst_dtype);

/* [d0,d1,d2,d3] -> [d0,d2,d1,d3] (head split / merge;
 * Compiler/CodeGenerator.swift:2840-3056). Any 2/4-byte type. */
int mhip_transpose_0213(void* stream, const void* x, void* y, int64_t d0, int64_t d1, int64_t d2,
                        int64_t d3, int dtype);

/* qkv [B,S,3*H*D] -> q,k,v each [B,H,S,D] (slice + reshape + transpose fused). */
int mhip_split_qkv_heads(void* stream, const void* qkv, void* q, void* k, void* v, int64_t B,
                         int64_t S, int64_t H, int64_t D, int dtype);

/* y[o, i, j] = i for a tensor viewed as [outer, n, inner]
 * (stablehlo.iota, Compiler/CodeGenerator.swift:1977). Integer and float types. */
int mhip_iota(void* stream, void* y, int64_t outer, int64_t n, int64_t inner, int dtype);

/* Last-axis argmax of x[rows, cols]: lowest index among equal maxima, a NaN
 * wins over any number (JAX's tie-break; the reference has no native
 * arg-reduction, python/README.md:122).  out_val may be NULL.
 * idx_dtype: I32 or I64. */
int mhip_argmax(void* stream, const void* x, void* out_idx, void* out_val, int64_t rows,
                int64_t cols, int dtype, int idx_dtype);

/* Rotary position embedding (FusedRoPEHandler, Compiler/CustomCallHandlers.swift:720-846):
 * x and y are [rows, D] with rows = (leading axes) x S; the row's position is row % S.  With
 * x = [x1 | x2] (halves of D / 2 elements): y = [x1 cos - x2 sin | x1 sin + x2 cos].
 * freqs_are_angles = 0: freqs is [S, D], cos in the first half of a row and sin in the second
 * (:783-808); 1: freqs is [S, D / 2] angles and cos / sin are computed (:809-812).  freqs has the
 * element type of x.  F32 / F16 / BF16, fp32 arithmetic, one rounding. */
int mhip_rope(void* stream, const void* x, const void* freqs, void* y, int64_t rows, int64_t S,
              int64_t D, int freqs_are_angles, int dtype);

/* Batch normalisation with given statistics (FusedBatchNormHandler, Compiler/CustomCallHandlers.swift:414-452;
 * the operands the fusion pass hands it, Compiler/PassManager.swift:1006-1080): x and y are
 * [rows, channels] (channels = the last axis), gamma / beta / mean / variance [channels] of x's
 * element type;  y = (x - mean) / sqrt(variance + eps) * gamma + beta.  F32 / F16 / BF16, fp32
 * arithmetic, one rounding. */
int mhip_batch_norm(void* stream, const void* x, const void* gamma, const void* beta, const void* mean,
                    const void* variance, void* y, int64_t rows, int64_t channels, float eps, int dtype);

/* Attention of one query row over a few key / value rows (FusedDepthAttentionHandler,
 * Compiler/CustomCallHandlers.swift:1084-1140; the reference's own kernel for it,
 * Metal/Kernels/DepthAttentionKernel.swift:17-20): q and out [rows, hidden], k and v
 * [rows, depth, hidden];  out = softmax(q k^T scale) v per row.  depth 1 .. 64 (the reference's
 * kernel reads at most 32 rows and ignores the rest; more than 64 is refused here).
 * F32 / F16 / BF16, fp32 arithmetic, one rounding. */
int mhip_depth_attention(void* stream, const void* q, const void* k, const void* v, void* out,
                         int64_t rows, int64_t depth, int64_t hidden, float scale, int dtype);

/* A chain of elementwise operations in one launch (FusedElementwiseHandler,
 * CustomCallHandlers.swift:927-1079): the running value starts as inputs[0]; ops[i] is either a
 * mhip_unary_op code, applied to the running value, or MHIP_CHAIN_BINARY + a mhip_binary_op code,
 * which combines the running value (left) with the next input (right).  The chain must consume
 * exactly n_inputs inputs.  input_elements[k] is n, or 1 for an input used at every position.
 * F32 / F16 / BF16; the whole chain is computed in fp32 and rounded once at the store (the
 * reference's graph rounds after every operation). */
#define MHIP_CHAIN_MAX_INPUTS 8
#define MHIP_CHAIN_MAX_OPS 16
#define MHIP_CHAIN_BINARY 100
int mhip_elementwise_chain(void* stream, int n_inputs, const void* const* inputs,
                           const int64_t* input_elements, int n_ops, const int* ops, void* y,
                           int64_t n, int dtype);

/* Unfused StableHLO glue for a host executor ------------------------------- */

typedef enum { MHIP_UN_EXP = 0, MHIP_UN_TANH, MHIP_UN_RSQRT, MHIP_UN_SQRT, MHIP_UN_NEG,
               MHIP_UN_LOGISTIC, MHIP_UN_ABS, MHIP_UN_LOG, MHIP_UN_ERF, MHIP_UN_SIN, MHIP_UN_COS,
               MHIP_UN_FLOOR, MHIP_UN_CEIL } mhip_unary_op;
typedef enum { MHIP_BIN_ADD = 0, MHIP_BIN_SUB, MHIP_BIN_MUL, MHIP_BIN_DIV, MHIP_BIN_MAX,
               MHIP_BIN_MIN, MHIP_BIN_POW } mhip_binary_op;
typedef enum { MHIP_CMP_EQ = 0, MHIP_CMP_NE, MHIP_CMP_LT, MHIP_CMP_LE, MHIP_CMP_GT,
               MHIP_CMP_GE } mhip_compare_dir;
typedef enum { MHIP_RED_SUM = 0, MHIP_RED_MAX, MHIP_RED_MIN, MHIP_RED_PROD } mhip_reduce_op;

/* y = op(x) elementwise (unary kernels, Compiler/CodeGenerator.swift:851-920).
 * F32/F16/BF16 (fp32 math, one rounding) and F64; NEG and ABS also on every integer
 * type (negate wraps, also for the unsigned types). */
int mhip_unary(void* stream, int op, const void* x, void* y, int64_t n, int dtype);

/* y = a op b elementwise, equal shapes (binary kernels, CodeGenerator.swift:921-1010).
 * Floats: fp32 math (F64: f64), one rounding, max/min propagate NaN; integers wrap, POW
 * with a negative exponent gives 1 / x^|e| truncated (1, +-1 or 0); I1: ADD and MAX are
 * OR, MUL and MIN are AND, no DIV / POW. */
int mhip_binary(void* stream, int op, const void* a, const void* b, void* y, int64_t n, int dtype);

/* y[i] = (a[i] <dir> b[i]) as one byte 0/1 (stablehlo.compare, CodeGenerator.swift:1101). */
int mhip_compare(void* stream, int direction, const void* a, const void* b, void* y, int64_t n,
                 int dtype);

/* y[i] = pred[i] ? a[i] : b[i]; pred is bytes, or one byte when scalar_pred
 * (stablehlo.select, CodeGenerator.swift:2008). elem_size in {1,2,4,8}. */
int mhip_select(void* stream, const void* pred, const void* a, const void* b, void* y, int64_t n,
                int elem_size, int scalar_pred);

/* y[o] = x[in_offset + sum_d idx_d(o) * in_strides[d]] over a dense row-major
 * output of `out_shape` (rank <= 8; stride 0 broadcasts).  One kernel for
 * broadcast_in_dim (:3057), transpose (:2840-3056) and slice of
 * Compiler/CodeGenerator.swift. */
int mhip_strided_copy(void* stream, const void* x, void* y, int rank, const int64_t* out_shape,
                      const int64_t* in_strides, int64_t in_offset, int elem_size);

/* y[o, i] = reduce_l x[o, l, i] starting from `init`, in index order
 * (stablehlo.reduce with add / maximum / minimum / multiply bodies,
 * Parser/Parser.swift:657-730). F32/F16/BF16/I32/I64. */
int mhip_reduce(void* stream, int op, const void* x, void* y, int64_t outer, int64_t len,
                int64_t inner, double init, int dtype);

/* y[i] = the low elem_size bytes of `pattern`, n elements (splat constants). */
int mhip_fill(void* stream, void* y, int64_t n, uint64_t pattern, int elem_size);

/* Autotuner -----------------------------------------------------------------
 * The role of the reference's AutoTuner (Tuning/AutoTuner.swift:12-103,301-458: a search space,
 * a validity filter, timed candidates) and TuningDatabase (Tuning/TuningDatabase.swift:15-160:
 * results persisted per device).  Each pass times every launch form the library has for the
 * problem (forms the shape, the 160 KB of LDS or the register file rule out are skipped) with
 * `iters` real launches on `stream`, stores the fastest in the process-wide table the entry
 * point consults before its heuristic, and reports it.  Passes overwrite their output tensor
 * and synchronise with the stream. */

/* GEMM kernel variants (128x128 tiles / 4 waves, 256x256 / 8 waves, the four-wave LDS-ring kernel
 * on 256x256 and on 256x128 tiles, the latter also as persistent workgroups, and wide tiles plus a
 * band of narrow ones): variant code 128 | 256 | 2560 | 2561 | 2562 | 2563, and the other members of the
 * generated ring-kernel family (tile width 384 / 256 / 128 x ring depth 4 / 5 / 6, those that fit 160 KB of
 * LDS and the register file): 2564 = 256x128 with six stages, 2565 = 256x128 with four, 2566 = 256x256
 * with four, 2567 = 256x384 with four (a third of its accumulators in ordinary registers; no
 * activation, relu or tanh-GELU), 2568 = 256x128 with three, in 256 registers a wave, two workgroups
 * per compute unit, 2569 = 128x192 with six (for problems with so few columns that 256-row tiles
 * leave compute units idle), 2570 = 256x288 with four (four waves one above the other; the same
 * activations as 2567);
 * microseconds per launch. */
int mhip_gemm_autotune(void* stream, const void* a, const void* b, const void* bias, void* c,
                       int64_t M, int64_t N, int64_t K, int64_t batch, int64_t stride_a,
                       int64_t stride_b, int64_t stride_c, int trans_a, int trans_b, int activation,
                       int dtype, int iters, int* out_variant, float* out_us);

/* The same search as a GEMM inside a model meets its operands: before every timed launch `flush`
 * (device memory the caller lends, at least 64 MB) is overwritten -- 64 to 128 MB empty the L2s and
 * leave most of the memory-side cache, the state of weights written a millisecond earlier; 512 MB and
 * more empty both -- and A is rewritten in place, as the kernel in front of the GEMM would have left
 * it.  Each launch is timed on its own, the median of `iters` decides and is recorded under the
 * same key as mhip_gemm_autotune (the later pass wins). */
int mhip_gemm_autotune_in_model(void* stream, const void* a, const void* b, const void* bias, void* c,
                                int64_t M, int64_t N, int64_t K, int64_t batch, int64_t stride_a,
                                int64_t stride_b, int64_t stride_c, int trans_a, int trans_b, int activation,
                                int dtype, int iters, void* flush, int64_t flush_bytes, int* out_variant,
                                float* out_us);

/* Records `variant` for a GEMM problem (0 removes the entry): for searches that time more than one
 * kernel, such as `python -m metalhlo_amd.tune`, which times a whole GPT-2 forward pass per candidate. */
int mhip_tuning_set_gemm(int64_t M, int64_t N, int64_t K, int64_t batch, int trans_a, int trans_b, int dtype,
                         int variant, float us);

/* The kernel variant (codes above; 0 = none of them: fp32, integer, f64 or unaligned operands) that
 * the calling thread's most recent mhip_gemm / mhip_gemm_residual call launched.  The tuner's
 * effect and the heuristic's choice can be observed with it. */
int mhip_gemm_last_variant(void);

/* Row operators (op 0 softmax, 1 LayerNorm, 2 RMSNorm; arguments as for the operator itself).
 * Searched: one wave per row with the parameters in LDS on a persistent grid (resident workgroups
 * per CU 0 = occupancy query, 2, 4, 6, 8) or a row split over the waves of a workgroup (one or two
 * rows per wave group; grid in address order, or persistent with 0 / 8 / 16 workgroups per CU).
 * out_choice[4] = {kind 1 | 2, rows per wave group, ordered 0 | 1, workgroups per CU}. */
int mhip_row_autotune(void* stream, int op, const void* x, const void* gamma, const void* beta, void* y,
                      int64_t rows, int64_t cols, float eps, int dtype, int iters, int* out_choice,
                      float* out_us);

/* Attention kernels for packed [B,H,S,D] operands without a mask: 1 = 128 query rows per workgroup,
 * 2 = the 256-row pipelined kernel (head size 128, Sq >= 256), 3 = the same with causal tiles
 * paired (causal only).  (AutoTuner.swift:629-723 chooses an attention block size likewise.) */
int mhip_attention_autotune(void* stream, const void* q, const void* k, const void* v, void* o, int64_t B,
                            int64_t H, int64_t Sq, int64_t Skv, int64_t D, float scale, int is_causal,
                            int dtype, int iters, int* out_variant, float* out_us);

/* The tuning table as text, one "<operator> <device> <problem> = <choice> @ <microseconds>" line per
 * entry (Tuning/TuningDatabase.swift:109-150); <device> is the architecture name and the number
 * of compute units ("gfx950/256", TuningDatabase.swift:15-60 keys by device too), and only
 * entries of the current device are used.  Loading merges into the table.  At first use the
 * library loads the table that ships with it for the device in use (../tuning/<arch>_<CUs>.txt beside
 * the shared object, written by `python -m metalhlo_amd.tune`) and then the file the environment
 * variable MHIP_TUNING_DB names; MHIP_TUNING_DB=none loads neither, mhip_tuning_clear empties the table. */
int mhip_tuning_save(const char* path);
int mhip_tuning_load(const char* path);
void mhip_tuning_clear(void);
int mhip_tuning_count(void);
/* The current device's key as it appears in the table (library-owned string). */
const char* mhip_tuning_device(void);

#ifdef __cplusplus
}
#endif
#endif /* MHIP_H */
