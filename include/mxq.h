/* C ABI of libmxq_gfx950.so -- MI355X (gfx950) kernels for microxcaling's MX / bfloat quantization.
 *
 * The library replaces the native extension the reference builds at import time
 * (mx/custom_extensions.py:11-19 -> mx/cpp/funcs.cpp:234-242).  Each entry point below names the
 * reference function it stands in for.  Differences from the reference's pybind surface, all of
 * which keep torch types out of the signatures:
 *   - tensors are raw device pointers plus a dtype code; shapes arrive collapsed to
 *     (pre, axis, post) as 64-bit counts, the way mx/cpp/mx.cu:29-46 collapses them;
 *   - the caller allocates the output (the reference returns empty_like(input));
 *   - every launch goes to the HIP stream the caller passes (the reference uses the legacy
 *     default stream, mx/cpp/mx.cu:57);
 *   - failures return a non-zero status and leave a message for mxq_last_error(); the reference
 *     prints and calls exit() (mx/cpp/common.cuh:247-255).
 * Entry points never allocate and never synchronise.  Results never depend on earlier calls; the only
 * state the library keeps is set-up done once per device under a lock (the dynamic-LDS limit of the
 * large-tile GEMM kernel with that device's CU count, and the address of the scratch array of
 * mxq_reduce_outer_static), so calls may come from several host threads.
 *
 * Numerics: results are bit-identical to the reference's pure-PyTorch CPU path
 * (custom_cuda=False) for fp32, bf16 and fp16 tensors, including its floor(log2(x)) rounding just
 * below powers of two and, for the 16-bit dtypes, the rounding to the tensor dtype after every op
 * (fp16: 2**shared_exp overflows from 2^16 and underflows below 2^-24, which turns such blocks --
 * all-zero blocks at scale_bits 8 among them -- into NaN, as it does there; a clamp bound beyond the
 * fp16 range is MXQ_ERR_ARGUMENT, where the reference's torch.clamp raises).
 * MXQ_FLAG_EXACT_EXPONENT switches to bit-field exponents, which is what the reference's own CUDA
 * kernels compute (mx/cpp/common.cuh:146-154); fp16 tensors are then widened to fp32, quantized and
 * rounded back to fp16 once, as those kernels do (mx/cpp/mx.cuh:72,88).  The packing entry points
 * take fp16 tensors under that flag only.
 */
#ifndef MXQ_H
#define MXQ_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* dtype codes */
#define MXQ_DTYPE_F32 0
#define MXQ_DTYPE_F16 1
#define MXQ_DTYPE_BF16 2

/* rounding modes = int(RoundingMode), mx/formats.py:12-19 */
#define MXQ_ROUND_NEAREST 0 /* half away from zero */
#define MXQ_ROUND_FLOOR 1   /* toward zero */
#define MXQ_ROUND_EVEN 2    /* half to even */

/* flags */
#define MXQ_FLAG_EXACT_EXPONENT 1 /* bit-field exponents instead of torch's floor(log2(x)) */
#define MXQ_FLAG_PACK_NIBBLES 4   /* mxq_pack_mx / _t, fp4 (e2m1) only: 4-bit codes, two per byte */
#define MXQ_FLAG_PACK_SIXBIT 8    /* mxq_pack_mx / _t, fp6 (e2m3, e3m2) only: 6-bit codes, four in three bytes */
#define MXQ_FLAG_PRE_BFLOAT16 32   /* mxq_pack_mx, bf16 tensors only: every element first goes through the
                                     elementwise quantizer to bfloat16 with round-half-away (bits 9, exp_bits 8,
                                     subnormals kept) -- what the layers apply to an operand before its MX
                                     quantization (mx/bmm.py:27-32, mx/matmul.py:45-50) -- in the same pass */
#define MXQ_FLAG_GENERAL_FORM 16  /* softmax / norm / activation kernels: no shortcut for values in the plain
                                   * range of the bfloat16 quantizer (same results, slower; for tests) */

/* kinds of packed element codes */
#define MXQ_CODES_E4M3 0 /* one OCP e4m3 byte per element */
#define MXQ_CODES_E5M2 1 /* one OCP e5m2 byte per element */
#define MXQ_CODES_E2M3 2 /* OCP e2m3, 6 bits per element: element j of a row in bits 6 j .. 6 j + 5 of the row */
#define MXQ_CODES_E3M2 3 /* OCP e3m2, 6 bits per element, same packing */
#define MXQ_CODES_E2M1 4 /* one OCP e2m1 nibble per element, the lower K index in the low nibble */

/* status codes */
#define MXQ_OK 0
#define MXQ_ERR_ARGUMENT 1 /* bad dtype / sizes / parameters; nothing was launched */
#define MXQ_ERR_LAUNCH 2   /* hipGetLastError() reported a failed launch */

/* Message for the last non-zero status returned on the calling thread. */
const char* mxq_last_error(void);

/* Library version (major * 100 + minor). */
int mxq_version(void);

/* Hex sha256 of the source files this library was compiled from (include/mxq.h and every .h, .hip
 * and .cpp under microxcaling_amd/csrc, as microxcaling_amd/build_ext.py computes it), or "unknown"
 * for a build made another way.  No counterpart in the reference: it lets a caller, and the tests,
 * tell a stale library from the one that belongs to the sources at hand. */
const char* mxq_build_digest(void);

/* quantize_mx_by_tile_func_cuda (mx/cpp/funcs.cpp:177-197, mx/cpp/mx.cu:116-287).
 * MX-quantize `in`, shape (pre, axis_size, post) contiguous, sharing one exponent per
 * `tile_size` consecutive elements of the middle axis (a shorter last tile is allowed;
 * tile_size <= 0 means the whole axis).  `out` has the same shape and dtype. */
int mxq_quantize_mx_by_tile(const void* in, void* out, int dtype, int64_t pre, int64_t axis_size,
                            int64_t post, int scale_bits, int elem_ebits, int elem_mbits,
                            float elem_max_norm, int64_t tile_size, int flush_fp32_subnorms,
                            int rmode, int flags, void* hip_stream);

/* _quantize_mx with one exponent shared over the blocks of two or three axes at once, e.g. tiles of
 * 32 x 32 elements (mx/mx_ops.py:226-298 with len(axes) > 1, blocks built by _reshape_to_blocks,
 * mx/mx_ops.py:95-154).  The reference serves this case on its pure-PyTorch path only, its extension
 * takes a single axis (mx/mx_ops.py:240-246).  The contiguous tensor is described by
 * extents[0 .. 2 * n_axes]: outer_0, shared_0, outer_1, shared_1, ..., outer_n, where outer_i is the
 * product of the axes between two shared ones (1 if there is none); n_axes in 1..3.  A tile takes
 * tile_size consecutive positions of every shared axis (shorter at the end of an axis;
 * tile_size <= 0: the whole axis). */
int mxq_quantize_mx_axes(const void* in, void* out, int dtype, int n_axes, const int64_t* extents,
                         int scale_bits, int elem_ebits, int elem_mbits, float elem_max_norm,
                         int64_t tile_size, int flush_fp32_subnorms, int rmode, int flags,
                         void* hip_stream);

/* round='dither' (_round_mantissa, mx/elemwise_ops.py:57-59): the scaled value is rounded as
 * floor(|s| + noise[i]) with noise in [0, 1), one value per element in the tensor's dtype, drawn by
 * the caller (the reference draws it with torch.rand_like and serves this mode on its pure-PyTorch
 * path only, mx/mx_ops.py:196-197).  Otherwise as mxq_quantize_mx_by_tile / mxq_quantize_elemwise.
 * Given the same noise the result is that of the pure path, bit for bit. */
int mxq_quantize_mx_dither_by_tile(const void* in, const void* noise, void* out, int dtype, int64_t pre,
                                   int64_t axis_size, int64_t post, int scale_bits, int elem_ebits,
                                   int elem_mbits, float elem_max_norm, int64_t tile_size,
                                   int flush_fp32_subnorms, int flags, void* hip_stream);
int mxq_quantize_elemwise_dither(const void* in, const void* noise, void* out, int dtype, int64_t n, int bits,
                                 int exp_bits, float max_norm, int saturate_normals, int allow_denorm,
                                 int flags, void* hip_stream);

/* quantize_mx_func_cuda (mx/cpp/funcs.cpp:154-175, mx/cpp/mx.cu:12-110).
 * As above, but the shared exponent of element (i, k, j) comes from max_values[i * post + j]
 * (the keepdim abs-max over the middle axis, same dtype as `in`). */
int mxq_quantize_mx_given_max(const void* in, void* out, const void* max_values, int dtype,
                              int64_t pre, int64_t axis_size, int64_t post, int scale_bits,
                              int elem_ebits, int elem_mbits, float elem_max_norm,
                              int flush_fp32_subnorms, int rmode, int flags, void* hip_stream);

/* quantize_elemwise_func_cuda (mx/cpp/funcs.cpp:199-217, mx/cpp/elemwise.cu:12-94).
 * Round each of the n elements to a (bits, exp_bits, max_norm) format. */
int mxq_quantize_elemwise(const void* in, void* out, int dtype, int64_t n, int bits, int exp_bits,
                          float max_norm, int rmode, int saturate_normals, int allow_denorm,
                          int flags, void* hip_stream);

/* reduce_sum_inner_dim / reduce_max_inner_dim (mx/cpp/funcs.cpp:219-231, mx/cpp/reduce.cu:15-89).
 * fp32 (rows, inner) -> fp32 (rows).  Unlike the reference there is no restriction on `inner`,
 * the sum order is fixed (no atomics), and max propagates NaN like torch.max. */
int mxq_reduce_sum_inner(const float* in, float* out, int64_t rows, int64_t inner,
                         void* hip_stream);
int mxq_reduce_max_inner(const float* in, float* out, int64_t rows, int64_t inner,
                         void* hip_stream);

/* Reductions over the outermost axis: fp32 (outer, inner) -> fp32 (inner).  No counterpart in the
 * reference's extension (its callers use torch.sum / torch.max for other axes).  `workspace` must
 * hold mxq_reduce_outer_workspace_bytes(outer, inner) bytes of device memory. */
int64_t mxq_reduce_outer_workspace_bytes(int64_t outer, int64_t inner);
int mxq_reduce_sum_outer(const float* in, float* out, void* workspace, int64_t outer,
                         int64_t inner, void* hip_stream);
int mxq_reduce_max_outer(const float* in, float* out, void* workspace, int64_t outer,
                         int64_t inner, void* hip_stream);

/* The outer-axis reduction for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 * Same kernels, same launch geometry and therefore the same bits as mxq_reduce_sum_outer (op 0) /
 * mxq_reduce_max_outer (op 1), but the partial results live in a 16 MiB device array that is part of
 * the library (every GPU the library runs on holds it until the process ends) instead of a
 * caller-provided workspace.  Shapes for which mxq_reduce_outer_workspace_bytes(outer, inner) exceeds
 * MXQ_REDUCE_OUTER_STATIC_BYTES are refused with MXQ_ERR_ARGUMENT ([16384, 8192] needs exactly that
 * much).  Calls on one GPU share the array: two that overlap in time (different streams or host
 * threads) race; calls on one stream are ordered and safe.  Nothing needs clearing between calls
 * (every partial that is read has been written by the same call). */
#define MXQ_REDUCE_OUTER_STATIC_BYTES (16 << 20)
int mxq_reduce_outer_static(const float* in, float* out, int op, int64_t outer, int64_t inner,
                            void* hip_stream);

/* SoftmaxFunction.forward (mx/softmax.py:20-54) over the last axis of a contiguous (rows, n) fp32
 * or bf16 tensor, as one kernel: quantize, row maximum, subtract, exponential, row sum, divide, with
 * the elementwise quantization of mx/vector_ops.py:38-130 (format bits / exp_bits / max_norm,
 * overflow to Inf as in _quantize_bfloat / _quantize_fp) after every step.  bits == 0 means "no
 * format": the steps are only rounded to the tensor dtype (what quantize_elemwise_op does without
 * bfloat / fp, and for bfloat16 with round-half-even on a bf16 tensor).
 * exp_mode 0: exp(x); 1: 2^x (mx_specs['softmax_exp2']); 2: 2^Q(x * 1.4453125) (['vec_use_exp2']).
 * use_recip: e * Q(1 / sum) instead of e / sum (['vec_use_recip']).
 * n must be a multiple of 16 bytes worth of elements and at most 16384.  The reference has no native
 * counterpart (it runs ten tensor ops); results agree with that chain up to the last-bit
 * differences of exp and of the summation order. */
int mxq_softmax_lastdim(const void* in, void* out, int dtype, int64_t rows, int64_t n, int bits,
                        int exp_bits, float max_norm, int rmode, int allow_denorm, int exp_mode,
                        int use_recip, int flags, void* hip_stream);

/* LayerNormFunction.forward / RMSNormFunction.forward (mx/layernorm.py:17-45, 100-131, over
 * mx/norm_utils.py:25-114) for the last axis of a contiguous (rows, n) fp32 or bf16 tensor, as one
 * kernel, with the elementwise quantizer (bits / exp_bits / max_norm as in mxq_softmax_lastdim,
 * bits == 0: none) after every step.  weight, bias: n values of the tensor dtype, already quantized.
 * out: (rows, n).  x_norm (may be NULL): (rows, n), the normalized input the layer saves for its
 * backward pass.  row_stat: rows values, var + eps (LayerNorm) or 1 / rms (RMSNorm), also saved.
 * n: multiple of 16 bytes worth of elements, at most 16384.  Agrees with the reference's chain of
 * tensor ops up to the order of the two row sums. */
int mxq_norm_lastdim(const void* in, const void* weight, const void* bias, void* out, void* x_norm,
                     void* row_stat, int dtype, int64_t rows, int64_t n, float eps, int rms_norm,
                     int bits, int exp_bits, float max_norm, int rmode, int allow_denorm, int flags,
                     void* hip_stream);

/* vec_add / vec_sub / vec_mul / vec_div / vec_recip (mx/vector_ops.py:38-75): `a op b` on contiguous
 * fp32 or bf16 tensors of n elements, rounded to the tensor dtype, then the elementwise quantizer
 * (as in mxq_quantize_elemwise; bits == 0: none) -- one pass instead of two.  op: 0 add, 1 sub,
 * 2 mul, 3 div.  mode 0: b is a tensor; 1: a op scalar; 2: scalar op a (b is ignored in modes 1, 2).
 * Bit-identical to the tensor op followed by quantize_elemwise_op. */
int mxq_binary_elemwise(const void* a, const void* b, float scalar, int mode, void* out, int dtype,
                        int64_t n, int op, int bits, int exp_bits, float max_norm, int rmode,
                        int allow_denorm, int flags, void* hip_stream);

/* The gradient with respect to the input of the same two layers (LayerNormFunction.backward via
 * _norm_backward_LN, mx/norm_utils.py:188-258; RMSNormFunction.backward, mx/layernorm.py:150-168)
 * from what mxq_norm_lastdim wrote: x_norm and row_stat.  weight: the n values the layer saved.
 * The gradients of weight and bias are column sums and stay separate steps.  Agrees with the
 * reference's chain up to the order of the row sums. */
int mxq_norm_backward_lastdim(const void* grad_out, const void* weight, const void* x_norm,
                              const void* row_stat, void* grad_in, int dtype, int64_t rows, int64_t n,
                              int rms_norm, int bits, int exp_bits, float max_norm, int rmode,
                              int allow_denorm, int flags, void* hip_stream);

/* The gradients of the weight and the bias of the same two layers (LayerNormFunction.backward,
 * mx/layernorm.py:51-59; RMSNormFunction.backward, mx/layernorm.py:148-156):
 *   grad_bias = Q(sum over rows of g),  grad_weight = Q(sum over rows of Q(g * x_norm))
 * for contiguous [rows, n] fp32 or bf16 tensors x_norm and g = Q(grad_out) (quantized on the way in,
 * like mxq_norm_backward_lastdim does: the caller need not run that pass), Q the elementwise
 * quantizer as in mxq_quantize_elemwise (bits == 0: none).  Sums are accumulated in fp32
 * in a fixed order and rounded to the tensor dtype once, like torch.sum; agrees with the reference's
 * steps up to that order.  grad_weight, grad_bias: n elements of the tensor dtype.  n must be a
 * multiple of 16 bytes of elements.  workspace: mxq_norm_param_grads_workspace_bytes(dtype, rows, n)
 * bytes of device memory, 16-byte aligned.  Two launches; g and x_norm are read once. */
int64_t mxq_norm_param_grads_workspace_bytes(int dtype, int64_t rows, int64_t n);
int mxq_norm_param_grads(const void* grad_out, const void* x_norm, void* grad_weight, void* grad_bias,
                         void* workspace, int64_t workspace_bytes, int dtype, int64_t rows, int64_t n,
                         int bits, int exp_bits, float max_norm, int rmode, int allow_denorm, int flags,
                         void* hip_stream);

/* The forward passes of SigmoidFunction, TanhFunction, SiLUFunction and GELUFunction
 * (mx/activations.py:237-297, 418-557) on a contiguous fp32 or bf16 tensor of n elements, as one
 * kernel, with the elementwise quantizer (bits / exp_bits / max_norm as in mxq_softmax_lastdim,
 * bits == 0: none) after every step of the reference's chain of vec_* ops.
 * act: MXQ_ACT_*.  exp_mode 0: exp(x); 2: 2^Q(x * 1.4453125) (mx_specs['vec_use_exp2']).
 * out: the result.  aux (may be NULL): the logistic factor that silu (sigmoid(x)) and gelu (phi) save
 * for their backward passes.  q_in (may be NULL): the quantized input, which gelu saves.
 * Agrees with the reference's chain up to the last-bit differences of exp and tanh. */
#define MXQ_ACT_SIGMOID 0
#define MXQ_ACT_TANH 1
#define MXQ_ACT_SILU 2
#define MXQ_ACT_GELU_FIRST_ORDER 3 /* x * sigmoid(1.702 x) */
#define MXQ_ACT_GELU 4             /* x * sigmoid(1.5958 (x + 0.044715 x^3)) */
int mxq_activation_forward(const void* in, void* out, void* aux, void* q_in, int dtype, int64_t n,
                           int act, int bits, int exp_bits, float max_norm, int rmode,
                           int allow_denorm, int exp_mode, int flags, void* hip_stream);

/* The backward passes of the same four layers (mx/activations.py:251-267, 284-297, 437-455,
 * 500-557) from what their forward passes saved: `saved` = the output (sigmoid, tanh, silu) or the
 * (quantized) input (gelu); `aux` = sigmoid(x) (silu) or phi (gelu), NULL otherwise.  Exact
 * arithmetic and the quantizer only: bit-identical to the reference's chain of vec_* ops. */
int mxq_activation_backward(const void* grad_out, const void* saved, const void* aux, void* grad_in,
                            int dtype, int64_t n, int act, int bits, int exp_bits, float max_norm,
                            int rmode, int allow_denorm, int flags, void* hip_stream);

/* SoftmaxFunction.backward (mx/softmax.py:56-88) over the last axis of contiguous (rows, n) tensors:
 * y is the saved output.  scale_ln2: the extra multiplication by ln 2 of mx_specs['softmax_exp2'].
 * Same limits as mxq_softmax_lastdim; agrees with the reference's chain up to the order of the
 * row sum. */
int mxq_softmax_backward_lastdim(const void* grad_out, const void* y, void* grad_in, int dtype,
                                 int64_t rows, int64_t n, int bits, int exp_bits, float max_norm,
                                 int rmode, int allow_denorm, int scale_ln2, int flags, void* hip_stream);

/* ---- packed MX tensors and the fused GEMM (no counterpart in the reference, which only ever
 * fake-quantizes and then calls a dense GEMM: mx/linear.py:62-86, mx/bmm.py:40-59) ---------------
 * Packed form of a (rows, K) tensor quantized along K in blocks of 32:
 *   codes  uint8 (rows, K)     OCP e4m3 for fp8_e4m3 / fp6_e3m2 / fp6_e2m3 / fp4_e2m1 elements (e4m3
 *                              holds all their values exactly), OCP e5m2 for fp8_e5m2 elements;
 *          or uint8 (rows, K/2) OCP e2m1 nibbles for fp4_e2m1 with MXQ_FLAG_PACK_NIBBLES
 *          or uint8 (rows, 3K/4) OCP 6-bit codes for fp6_e2m3 / fp6_e3m2 with MXQ_FLAG_PACK_SIXBIT
 *   scales uint8 (rows, K/32)  E8M0 (shared exponent + 127; 255 = the block is NaN)
 * value = code * 2^(scale - 127), identical to what mxq_quantize_mx_by_tile returns. */
int mxq_pack_mx(const void* in, void* codes, void* scales, int dtype, int64_t rows, int64_t K,
                int scale_bits, int elem_ebits, int elem_mbits, float elem_max_norm,
                int flush_fp32_subnorms, int rmode, int flags, void* hip_stream);
int mxq_unpack_mx(const void* codes, const void* scales, int code_kind, void* out, int dtype,
                  int64_t rows, int64_t K, void* hip_stream);
/* Quantize along the second-to-last axis and transpose while packing: in (batch, R, C) contiguous,
 * blocks of 32 along R; codes (batch, C, R), scales (batch, C, R / 32) -- the K-major operand of
 * mxq_gemm_mx_nt when the contraction runs over R, as in the gradient GEMMs of the layers
 * (mx/linear.py:124-173: input and grad_output along axis -2, the weight along axis 0).
 * unpack(codes, scales) is the transpose of mxq_quantize_mx_by_tile(in, axis = R). */
int mxq_pack_mx_t(const void* in, void* codes, void* scales, int dtype, int64_t batch, int64_t R,
                  int64_t C, int scale_bits, int elem_ebits, int elem_mbits, float elem_max_norm,
                  int flush_fp32_subnorms, int rmode, int flags, void* hip_stream);
/* C[b] (M, N) = A[b] (M, K) x B[b] (N, K)^T for b < batch, all tensors contiguous, fp32
 * accumulation on the scaled MFMA units; c_dtype is a MXQ_DTYPE_* code.  a_kind, b_kind:
 * MXQ_CODES_* of the operands; e4m3 and e5m2 bytes mix freely (K % 128 == 0), e2m1 nibbles need both
 * operands in that form (K % 256 == 0) and run at the 4-bit MFMA rate.  6-bit codes (e2m3, e3m2)
 * are a storage form only: the call rejects them, fp6 operands come as byte codes.
 * bias (optional, may be NULL): N values of dtype c_dtype; then C = round(round(A x B^T) + bias),
 * both roundings to c_dtype, which is what "matmul, then add the bias" gives as tensor ops.
 * epilogue_quant = 1 (bf16 C only): additionally apply the elementwise quantization of the layers
 * with mx_specs['bfloat'] = 16 and round-half-away (quantize_elemwise_op, mx/linear.py:88-96,
 * mx/bmm.py:55-57) to the rounded product and again to the rounded sum with the bias.
 * workspace (may be NULL): mxq_gemm_workspace_bytes(...) bytes of device memory, 16-byte aligned.
 * Products with few output tiles (decode shapes: M <= 128) split K over several workgroups per
 * tile and add the fp32 partial tiles up in a second launch, in a fixed order; without a workspace
 * they run unsplit (same result up to the order of the additions, several times slower). */
int mxq_gemm_mx_nt(const void* a_codes, const void* a_scales, int a_kind, const void* b_codes,
                   const void* b_scales, int b_kind, const void* bias, void* c, int c_dtype,
                   int64_t batch, int64_t M, int64_t N, int64_t K, int epilogue_quant,
                   void* workspace, int64_t workspace_bytes, void* hip_stream);
/* Attention scores in one launch (no counterpart in the reference, which runs mx.bmm and mx.softmax
 * as separate tensor passes: mx/bmm.py:40-59, mx/softmax.py:26-48):
 *   out[b] = softmax over the last axis of Q(A[b] x B[b]^T),  bf16 (batch, M, N)
 * for packed operands with 8-bit codes (MXQ_CODES_E4M3 / _E5M2) and K = 128 (head_dim 128), N a multiple
 * of 32 up to 2048, with the elementwise quantizer of mx_specs['bfloat'] = 16 and round-half-away
 * after the product and after every softmax step (exp2 = 1: 2^x as with softmax_exp2).  The logits
 * stay in registers.  Results agree with mxq_gemm_mx_nt(epilogue_quant = 1) + mxq_softmax_lastdim
 * within those kernels' own tolerance against the CPU chain (one step of the bfloat16 grid on a few
 * percent of the elements: the exponential is the hardware's -- about 1 ulp for 2^x; for e^x the rounded
 * product x * log2(e) in front of it adds up to 2.6e-6 of the value at x = -85 -- and the row sum has its
 * own order).
 * flags: MXQ_FLAG_GENERAL_FORM. */
int mxq_bmm_softmax_mx_nt(const void* a_codes, const void* a_scales, int a_kind, const void* b_codes,
                          const void* b_scales, int b_kind, void* out, int64_t batch, int64_t M, int64_t N,
                          int64_t K, int exp2, int flags, void* hip_stream);

/* 0 when the product would not be split. */
int64_t mxq_gemm_workspace_bytes(int64_t batch, int64_t M, int64_t N, int64_t K, int a_kind);
/* Which kernel mxq_gemm_mx_nt launches for a shape (no counterpart in the reference; for tests and
 * benchmarks that must know what they measured), or -1 for a shape it refuses:
 * persistent workgroups on 256 x 256 tiles; 128 x 128 tiles; the same with K split over several
 * workgroups per tile (needs the workspace, else unsplit); 128 x 128 tiles whose K is a single step. */
#define MXQ_GEMM_PLAN_SMALL_TILES 0
#define MXQ_GEMM_PLAN_SPLIT_K 1
#define MXQ_GEMM_PLAN_LARGE_TILES 2
#define MXQ_GEMM_PLAN_ONE_STEP 3
int mxq_gemm_plan(int64_t batch, int64_t M, int64_t N, int64_t K, int a_kind);

/* ---- libmxq_host.so: the same arithmetic compiled for the host ----------------------------------
 * quantize_mx_func_cpp (mx/cpp/funcs.cpp:23-98) and quantize_elemwise_func_cpp
 * (mx/cpp/funcs.cpp:117-149) take CPU tensors; these are their stand-ins.  Pointers are host
 * pointers and a call returns when the work is done.  A call with more than about 128 K elements is
 * spread over up to 16 threads of its own (blocks are independent and each is computed by exactly one
 * thread, so the result does not depend on their number); MXQ_HOST_THREADS in the environment (read once
 * per process) sets another upper limit, 1 keeps everything on the calling thread.  The by-tile variant has no
 * CPU counterpart in the reference; it mirrors mxq_quantize_mx_by_tile so the kernel arithmetic
 * can be checked on a machine without a GPU.  mxq_host_quantize_mx_axes mirrors mxq_quantize_mx_axes. */
#define MXQ_HOST_FLAG_ROUND_EVERY_OP 2 /* bf16: round to bf16 after every op, no shortcuts */
#define MXQ_HOST_FLAG_CLOSED_FORM 4    /* elementwise, bf16 tensor -> bfloat16, nearest: the closed
                                          form the fused softmax kernel uses (else: an error) */
#define MXQ_HOST_FLAG_CLOSED_FORM_NONNEG 8 /* with CLOSED_FORM: its variant for +0 <= x < 2^127,
                                              +Inf and NaN (other inputs: unspecified) */

const char* mxq_host_last_error(void);
const char* mxq_host_build_digest(void); /* as mxq_build_digest, for libmxq_host.so */
int mxq_host_quantize_mx_given_max(const void* in, void* out, const void* max_values, int dtype,
                                   int64_t pre, int64_t axis_size, int64_t post, int scale_bits,
                                   int elem_ebits, int elem_mbits, float elem_max_norm,
                                   int flush_fp32_subnorms, int rmode, int flags);
int mxq_host_quantize_mx_by_tile(const void* in, void* out, int dtype, int64_t pre,
                                 int64_t axis_size, int64_t post, int scale_bits, int elem_ebits,
                                 int elem_mbits, float elem_max_norm, int64_t tile_size,
                                 int flush_fp32_subnorms, int rmode, int flags);
int mxq_host_quantize_mx_axes(const void* in, void* out, int dtype, int n_axes, const int64_t* extents,
                              int scale_bits, int elem_ebits, int elem_mbits, float elem_max_norm,
                              int64_t tile_size, int flush_fp32_subnorms, int rmode, int flags);
int mxq_host_quantize_mx_dither_by_tile(const void* in, const void* noise, void* out, int dtype, int64_t pre,
                                        int64_t axis_size, int64_t post, int scale_bits, int elem_ebits,
                                        int elem_mbits, float elem_max_norm, int64_t tile_size,
                                        int flush_fp32_subnorms, int flags);
int mxq_host_quantize_elemwise_dither(const void* in, const void* noise, void* out, int dtype, int64_t n,
                                      int bits, int exp_bits, float max_norm, int saturate_normals,
                                      int allow_denorm, int flags);
int mxq_host_quantize_elemwise(const void* in, void* out, int dtype, int64_t n, int bits,
                               int exp_bits, float max_norm, int rmode, int saturate_normals,
                               int allow_denorm, int flags);

#ifdef __cplusplus
}
#endif
#endif /* MXQ_H */
