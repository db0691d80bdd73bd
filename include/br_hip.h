/*
 * br_hip.h -- C ABI of libbr_hip.so, the MI355X (gfx950) kernel library
 * behind BlackRiver's tensor operator API.
 *
 * One entry point per kernel family.  Every function takes raw device
 * pointers, explicit sizes and the HIP stream to launch on (a hipStream_t
 * passed as void*; NULL is the default stream) and returns 0 on success, a
 * positive hipError_t value when the HIP runtime failed, or a negative
 * BR_ERR_* value when the arguments are rejected before any launch.  Nothing
 * here allocates device memory except br_hip_malloc / br_hip_host_malloc;
 * kernels that need scratch take a caller-provided workspace (one entry,
 * br_hip_layernorm_bwd_static, uses a buffer built into the library instead).
 *
 * Tensors are dense row-major.  "dtype" arguments use the numbering of the
 * reference's br::DataType (blackriver/tensortype.hpp:16-21).
 *
 * Each declaration cites the reference interface it stands in for (paths
 * relative to the reference tree).
 */
#ifndef BR_HIP_H_
#define BR_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* br_stream_t; /* hipStream_t */
typedef void* br_event_t;  /* hipEvent_t  */

enum {
    BR_F32 = 0,
    BR_BF16 = 1,
    BR_F16 = 2,
    BR_I32 = 3
};

enum {
    BR_OK = 0,
    BR_ERR_TODO = -1,     /* combination not implemented  (OP_TODO_ERROR)   */
    BR_ERR_INPUT = -2,    /* bad input argument           (OP_INPUT_ERROR)  */
    BR_ERR_OUTPUT = -3,   /* bad output argument          (OP_OUTPUT_ERROR) */
    BR_ERR_ATTR = -4,     /* bad scalar attribute / size  (OP_ATTR_ERROR)   */
    BR_ERR_SCRATCH = -5   /* problem needs more scratch than the library's
                             built-in buffer holds (allocation-free entries) */
};

/* ---- runtime plumbing -------------------------------------------------- */
/* Stand in for the CUDA runtime calls of blackriver/context.cpp:18-43
 * (cudaSetDevice, cudaStreamCreate, cudaMalloc of the workspace) and of
 * blackriver/cuda_tensor.hpp:11-20 (cudaMalloc / cudaFree per tensor). */
int br_hip_device_count(int* count);
int br_hip_set_device(int device);
const char* br_hip_error_string(int code);
int br_hip_malloc(void** ptr, size_t bytes);
int br_hip_free(void* ptr);
int br_hip_host_malloc(void** ptr, size_t bytes); /* pinned host memory */
int br_hip_host_free(void* ptr);
int br_hip_stream_create(br_stream_t* stream);
int br_hip_stream_destroy(br_stream_t stream);
int br_hip_stream_sync(br_stream_t stream); /* nn.cpp:16-22 (op.sync) */
int br_hip_event_create(br_event_t* event);
int br_hip_event_destroy(br_event_t event);
int br_hip_event_record(br_event_t event, br_stream_t stream);
int br_hip_event_sync(br_event_t event);
int br_hip_event_elapsed_ms(br_event_t start, br_event_t stop, float* ms);

/* cudaMemcpyAsync in cuda_tensor.cpp:135,139 and cpu_tensor.cpp:31, and
 * cudaMemset in cuda_tensor.cpp:104.  Asynchronous on `stream`. */
int br_hip_memcpy_h2d(void* dst, const void* src, size_t bytes, br_stream_t stream);
int br_hip_memcpy_d2h(void* dst, const void* src, size_t bytes, br_stream_t stream);
int br_hip_memcpy_d2d(void* dst, const void* src, size_t bytes, br_stream_t stream);
int br_hip_memset(void* dst, int byte_value, size_t bytes, br_stream_t stream);

/* ---- elementwise ------------------------------------------------------- */
/* cudnnSetTensor in cuda_tensor.cpp:111-125 (op_fill). */
int br_hip_fill(void* dst, int dtype, float value, int64_t n, br_stream_t stream);
/* Synthetic initialisation: dst[i] = mean + std * z(seed, i), z standard normal
 * from a counter-based generator (SplitMix64 + Box-Muller), dtype BR_F32 /
 * BR_F16 / BR_BF16.  No counterpart in the reference, which only ever reads
 * weights from files (io_load, cuda_tensor.cpp:52-72); benchmarks and tests of
 * whole models use it where those files do not exist. */
int br_hip_normal(void* dst, int dtype, float mean, float std, uint64_t seed, int64_t n,
                  br_stream_t stream);

/* Storage conversion between BR_F32, BR_F16 and BR_BF16 (no counterpart in
 * the reference, whose only implemented dtype is fp32). */
int br_hip_cast(const void* src, int src_dtype, void* dst, int dst_dtype, int64_t n,
                br_stream_t stream);

/* cudnnOpTensor(ADD) in cuda_tensor.cpp:206-232 (op_add): c = a + b where b
 * is broadcast along every dimension in which b_shape is 1.  Shapes are
 * rank 4 (lower ranks mapped as cuda_tensor.hpp:39-49).  c may alias a. */
int br_hip_add_bcast(const void* a, const void* b, void* c, int dtype,
                     const int64_t a_shape[4], const int64_t b_shape[4], br_stream_t stream);

/* kernels::gelu_forward / gelu_backward, kernels/gelu.cu:46-59,72-85
 * (declared kernels/kernels.h:518-519), called at cuda_tensor.cpp:400-412,814-828.
 * dtype is the storage type of x / y / dy / dx (BR_F32 or BR_F16); math is
 * fp32.  dx may alias x. */
int br_hip_gelu_fwd(const void* x, void* y, int dtype, int64_t n, br_stream_t stream);
/* The same forward with fp32 x and a 16-bit y (BR_F16 or BR_BF16; n % 8 == 0,
 * 16-byte aligned): for an activation that only feeds a 16-bit product, which
 * would round an fp32 y the same way. */
int br_hip_gelu_fwd_f32_to_16(const float* x, void* y, int y_dtype, int64_t n, br_stream_t stream);
int br_hip_gelu_bwd(const void* dy, const void* x, void* dx, int dtype, int64_t n,
                    br_stream_t stream);

/* y = gelu(x + bias[col]): the cudnnAddTensor bias pass of
 * cuda_tensor.cpp:180-190 fused with kernels::gelu_forward.  bias is fp32. */
int br_hip_bias_gelu_fwd(const void* x, const float* bias, void* y, int dtype, int64_t rows,
                         int64_t cols, br_stream_t stream);
/* dx = dy * gelu'(x + bias) (bias may be NULL: x already holds it); when
 * dbias != NULL also dbias[col] = dbias_scale * sum_rows dx (the
 * cudnnReduceTensor of cuda_tensor.cpp:738-760; the sum is over dx as stored).
 * workspace must hold br_hip_bias_gelu_bwd_workspace(rows, cols) bytes when
 * dbias != NULL. */
size_t br_hip_bias_gelu_bwd_workspace(int64_t rows, int64_t cols);
int br_hip_bias_gelu_bwd(const void* dy, const void* x, const float* bias, void* dx,
                         float* dbias, int dtype, int64_t rows, int64_t cols, float dbias_scale,
                         void* workspace, size_t workspace_bytes, br_stream_t stream);

/* kernels::launch_transform_0213<float>, kernels/transform_kernels.cu:56-65
 * (declared kernels/kernels.h:35), called at cuda_tensor.cpp:257-275: [s0,s1,s2,s3] -> [s0,s2,s1,s3].
 * elem_bytes is 2 or 4. */
int br_hip_transpose_0213(const void* x, void* y, int elem_bytes, int64_t s0, int64_t s1,
                          int64_t s2, int64_t s3, br_stream_t stream);

/* cudnnReduceTensor(ADD) of cuda_tensor.cpp:738-760: out[c] = sum_r x[r,c]
 * (x fp32, fp16 or bf16, out fp32), times out_scale (1 for the plain sum; a
 * backward pass that carries its activation gradients lifted by a power of two
 * S passes 1/S here to get the bias gradient at its true scale).
 * workspace: br_hip_colsum_workspace bytes. */
size_t br_hip_colsum_workspace(int64_t rows, int64_t cols);
int br_hip_colsum(const void* x, int dtype, float* out, int64_t rows, int64_t cols, float out_scale,
                  void* workspace, size_t workspace_bytes, br_stream_t stream);
/* The same column sums of an fp32 x together with a 16-bit copy of x (x16,
 * BR_F16 or BR_BF16, dense [rows, cols]) in one pass: op_linear_backward
 * (cuda_tensor.cpp:730-812) needs the sums as the bias gradient and, with a
 * 16-bit MFMA type, the copy as the operand of its two products.  cols % 4 == 0,
 * x 16-byte aligned; workspace as for br_hip_colsum. */
int br_hip_colsum_cast(const float* x, float* out, void* x16, int x16_dtype, int64_t rows, int64_t cols,
                       float out_scale, void* workspace, size_t workspace_bytes, br_stream_t stream);

/* br_hip_gelu_bwd (fp32) and br_hip_colsum_cast in one pass: dx = dy * gelu'(x)
 * is written as fp32 (dx may be x's or dy's own buffer), as a 16-bit copy dx16
 * and column-summed into out -- `op.gelu_backward` followed by the head of the
 * `op.linear_backward` below it (bloomz-7b/train.words:200-202; gelu.cu:61-85,
 * cuda_tensor.cpp:730-760).  All three results are bit for bit those of the two
 * separate entries.  BR_ERR_TODO unless cols % 4 == 0 and 16-byte aligned
 * operands; workspace as for br_hip_colsum. */
int br_hip_gelu_bwd_colsum_cast(const float* dy, const float* x, float* dx, float* out, void* dx16,
                                int dx16_dtype, int64_t rows, int64_t cols, float out_scale, void* workspace,
                                size_t workspace_bytes, br_stream_t stream);

/* ---- LayerNorm --------------------------------------------------------- */
/* kernels::launch_layer_norm_float, kernels/normalize_kernels.cu:87-102
 * (declared kernels/kernels.h:24), called at cuda_tensor.cpp:236-255.  var receives sigma^2 + eps; mean and
 * var may be NULL. */
int br_hip_layernorm_fwd(const float* x, const float* gamma, const float* beta, float* y,
                         float* mean, float* var, int64_t rows, int64_t cols, float eps,
                         br_stream_t stream);

/* The same forward, which also writes y rounded to nearest as fp16 / bf16
 * (y16_dtype = BR_F16 / BR_BF16) into y16: the `op.layernorm` + `op.copy`
 * pair of a script whose next consumer is a 16-bit matrix product
 * (cuda_tensor.cpp:236-255 followed by op_copy, :128-144), in one pass over x.  y16 holds
 * exactly what a cast of y would.  BR_ERR_TODO when the shape or alignment
 * needs the general kernel: the caller then runs the two steps separately. */
int br_hip_layernorm_fwd_copy16(const float* x, const float* gamma, const float* beta, float* y,
                                void* y16, int y16_dtype, float* mean, float* var, int64_t rows,
                                int64_t cols, float eps, br_stream_t stream);

/* kernels::launch_ln_bw_float, kernels/normalize_kernels.cu:361-383
 * (declared kernels/kernels.h:28) with means == nullptr, called at cuda_tensor.cpp:699-727.  y is the forward
 * OUTPUT, var what the forward stored; dgamma / dbeta are overwritten with
 * the sums times param_scale (1, or 1/S when dy carries a power-of-two lift S
 * that dx keeps and the parameter gradients must not). */
size_t br_hip_layernorm_bwd_workspace(int64_t rows, int64_t cols);
int br_hip_layernorm_bwd(const float* dy, const float* y, const float* gamma,
                         const float* beta, const float* var, float* dgamma, float* dbeta,
                         float* dx, int64_t rows, int64_t cols, float eps, float param_scale,
                         void* workspace, size_t workspace_bytes, br_stream_t stream);

/* br_hip_layernorm_bwd without the workspace argument, for callers that cannot
 * allocate device memory or hand a workspace in: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart
 * in the reference.  The partial sums go to a buffer built into the library
 * (br_hip_layernorm_bwd_static_limit() bytes, 16 MiB, held once per GPU for the
 * life of the process); the call makes no hipMalloc / hipFree and uses the
 * same kernels as br_hip_layernorm_bwd, so results are identical bit for bit.
 * Returns BR_ERR_SCRATCH when br_hip_layernorm_bwd_workspace(rows, cols)
 * exceeds the limit (e.g. cols > 8192 at 512 or more rows).  All calls on one
 * GPU share the buffer: calls that overlap in time on one GPU (two streams)
 * race; calls on one stream, or ordered by events, are safe. */
size_t br_hip_layernorm_bwd_static_limit(void);
int br_hip_layernorm_bwd_static(const float* dy, const float* y, const float* gamma,
                                const float* beta, const float* var, float* dgamma, float* dbeta,
                                float* dx, int64_t rows, int64_t cols, float eps, float param_scale,
                                br_stream_t stream);

/* The same backward with a residual gradient added to the input gradient:
 * dx = layernorm_backward(...) + residual, the `op.layernorm_backward` +
 * `op.add` pair of train.words:207-208 and :240-243 (cuda_tensor.cpp:699-727
 * followed by :206-232) in one pass.  dx is rounded to fp32 before the add, so
 * the result equals the two operators' bit for bit; dx may be the residual's
 * or dy's own buffer (a row is read completely before it is written).  BR_ERR_TODO when the shape needs the general kernels. */
int br_hip_layernorm_bwd_residual(const float* dy, const float* y, const float* gamma,
                                  const float* beta, const float* var, const float* residual,
                                  float* dgamma, float* dbeta, float* dx, int64_t rows,
                                  int64_t cols, float eps, float param_scale, void* workspace,
                                  size_t workspace_bytes, br_stream_t stream);

/* The same followed by what the `op.linear_backward` of the layer below does to
 * dx first (cuda_tensor.cpp:738-760: its bias gradient, the column sums of dx;
 * and, for 16-bit products, the 16-bit image of dx both of its products read):
 * dx16 = dx rounded to dx16_dtype (BR_F16 / BR_BF16), dx_sum[c] = param_scale *
 * sum over rows of dx[r, c], the sums in a fixed order.  dx16 and dx are what
 * br_hip_colsum_cast would make of dx; the sums agree with its to rounding (a
 * different but equally fixed summation order).  Workspace:
 * br_hip_layernorm_bwd_sums_workspace.  BR_ERR_TODO for rows wider than 4096
 * columns, unaligned dgamma / dbeta / dx_sum / dx16 and whatever
 * br_hip_layernorm_bwd_residual declines: callers then run the two steps. */
size_t br_hip_layernorm_bwd_sums_workspace(int64_t rows, int64_t cols);
int br_hip_layernorm_bwd_residual_sums(const float* dy, const float* y, const float* gamma,
                                       const float* beta, const float* var, const float* residual,
                                       float* dgamma, float* dbeta, float* dx, void* dx16,
                                       int dx16_dtype, float* dx_sum, int64_t rows, int64_t cols,
                                       float eps, float param_scale, void* workspace,
                                       size_t workspace_bytes, br_stream_t stream);

/* ---- softmax family ---------------------------------------------------- */
/* cudnnSoftmaxForward(ACCURATE, INSTANCE) at cuda_tensor.cpp:332-356 and
 * cudnnSoftmaxBackward at :890-918.  y may alias x; dx may alias dy. */
int br_hip_softmax_fwd(const float* x, float* y, int64_t rows, int64_t cols,
                       br_stream_t stream);
int br_hip_softmax_bwd(const float* dy, const float* y, float* dx, int64_t rows, int64_t cols,
                       br_stream_t stream);

/* cudnnSoftmaxBackward at cuda_tensor.cpp:890-918 with the gradient stored
 * only as fp16 / bf16 (round to nearest of the fp32 value br_hip_softmax_bwd
 * stores), for a consumer that is a 16-bit matrix product
 * (op_qk_backward, cuda_tensor.cpp:1006).  dx16 must not alias the inputs.
 * BR_ERR_TODO when the rows do not fit the one-wave-per-row kernel. */
int br_hip_softmax_bwd_to16(const float* dy, const float* y, void* dx16, int dx16_dtype,
                            int64_t rows, int64_t cols, br_stream_t stream);

/* The three-word sequence of bloomz-7b/train.words:158-162 in one pass:
 * p = softmax((s + alibi[h,:]) + xmask[b,q,:]) over the last dimension of
 * s[batch, heads, tq, tk], with alibi[heads, tk] and xmask[batch, tq, tk]
 * (either may be NULL).  Same operation order as the separate ops, so the
 * result is bit-identical to them.  p may alias s. */
int br_hip_alibi_masked_softmax_fwd(const float* s, const float* alibi, const float* xmask,
                                    float* p, int64_t batch, int64_t heads, int64_t tq,
                                    int64_t tk, br_stream_t stream);

/* br_hip_alibi_masked_softmax_fwd, which also writes p rounded to nearest as
 * fp16 / bf16 into p16 (what a cast of p would hold), so that the attention
 * product can read the 16-bit probabilities while the backward keeps the fp32
 * ones.  BR_ERR_TODO when the rows do not fit the one-wave-per-row kernel. */
int br_hip_alibi_masked_softmax_fwd_copy16(const float* s, const float* alibi,
                                           const float* xmask, float* p, void* p16,
                                           int p16_dtype, int64_t batch, int64_t heads,
                                           int64_t tq, int64_t tk, br_stream_t stream);

/* The same, with the ALiBi bias and the causal / padding mask of
 * blackriver/train_bloom.cpp:58-90 computed in the kernel from the device
 * arrays slopes[heads] (fp64, as br_hip_alibi_slopes returns them) and
 * valid[batch] (= number of leading non-zero mask entries per sequence)
 * instead of being read from tables; bit-identical to the table form. */
int br_hip_alibi_causal_softmax_fwd(const float* s, const double* slopes, const int32_t* valid,
                                    float* p, int64_t batch, int64_t heads, int64_t tq,
                                    int64_t tk, br_stream_t stream);

/* cudnnSoftmaxForward(LOG) + kernels::nllloss_forward
 * (kernels/nll_loss.cu:45-58, declared kernels/kernels.h:520) of cuda_tensor.cpp:535-553,640-652, one pass
 * over logits[rows, vocab]:
 *   lse[r]        = logsumexp(logits[r,:])
 *   row_logp[r]   = keep[r] && 0 <= target[r] < vocab ?
 *                   logits[r,target[r]] - lse[r] : 0
 *   result[0]     = sum_r row_logp[r] / count   (+mean log-prob, the
 *                   reference's sign convention, cuda_tensor.cpp:691)
 *   result[1]     = count = #{r : keep[r] != 0}
 * lse, row_logp: device fp32 [rows]; result: device fp32 [2]. */
int br_hip_logsoftmax_nll_fwd(const float* logits, const int32_t* target, const int32_t* keep,
                              float* lse, float* row_logp, float* result, int64_t rows,
                              int64_t vocab, br_stream_t stream);

/* cudnnSoftmaxBackward(LOG) of cuda_tensor.cpp:656-668 applied to the seed
 * written by nll_loss.cu:33:
 *   dlogits[r,c] = keep[r] ? (exp(logits[r,c]-lse[r]) - [c==target[r]])*scale : 0
 * dlogits_dtype is BR_F32, BR_F16 or BR_BF16; dlogits may alias logits when
 * fp32.  A 16-bit dlogits that feeds matrix products should be written with a
 * scale that keeps small probabilities representable (fp16 flushes below
 * 3e-8): pass a power of two here and fold 1/count and its inverse into the
 * products' alpha. */
int br_hip_logsoftmax_nll_bwd(const float* logits, const int32_t* target, const int32_t* keep,
                              const float* lse, void* dlogits, int dlogits_dtype, float scale,
                              int64_t rows, int64_t vocab, br_stream_t stream);

/* ---- GEMM -------------------------------------------------------------- */
enum {
    BR_GEMM_F16 = 0,  /* operands rounded to fp16, v_mfma_f32_32x32x16_f16  */
    BR_GEMM_BF16 = 1, /* operands rounded to bf16, v_mfma_f32_32x32x16_bf16 */
    BR_GEMM_F32 = 2   /* fp32 operands, v_mfma_f32_32x32x2_f32              */
};

/* kernels::LtSgemm, kernels/LtSgemm.cu:55-126 (declared kernels/kernels.h:528-543),
 * and the per-head loops around it at cuda_tensor.cpp:294-308,380-394 etc.
 * Row-major, strided-batched, fp32 accumulation:
 *
 *   C[b][i,j] = alpha * sum_p opA[b][i,p] * opB[b][p,j]
 *               + (accumulate ? C[b][i,j] : 0) + (bias ? bias[j] : 0)
 *
 *   trans_a == 0: A[b] is [m,k] with row stride lda;  1: A[b] is [k,m].
 *   trans_b == 0: B[b] is [k,n] with row stride ldb;  1: B[b] is [n,k].
 *
 * a_dtype / b_dtype / c_dtype are BR_F32, BR_F16 or BR_BF16 storage types;
 * `compute` picks the MFMA type operands are converted to on load.  stride_*
 * are element strides between batch entries.  bias is fp32 [n] or NULL. */
int br_hip_gemm(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, float alpha,
                const void* a, int a_dtype, int64_t lda, int64_t stride_a,
                const void* b, int b_dtype, int64_t ldb, int64_t stride_b,
                int accumulate, void* c, int c_dtype, int64_t ldc, int64_t stride_c,
                const float* bias, int64_t batch, int compute, br_stream_t stream);

/* The same product for callers that can lend scratch memory.  fp32 operands
 * are first converted to the 16-bit compute type into `workspace` (dense
 * copies, one pass each), so that the product runs on the direct-to-LDS
 * kernel that needs both operands in the MFMA type.  Replaces the same
 * kernels::LtSgemm call (LtSgemm.cu:55-126); `workspace` plays the part of
 * the scratch the reference hands to cublasLtMatmul (context.cpp:31).  An
 * unbatched product with too few output tiles for the 256 CUs and a long K is
 * split along K into fp32 partials in the same workspace and summed in a fixed
 * order (deterministic).  Falls back to br_hip_gemm when `compute`
 * is BR_GEMM_F32, no operand is fp32, the shape is not 16-byte friendly
 * (k % 32, operand row lengths % 8) or the workspace is smaller than
 * br_hip_gemm_staged_workspace() bytes.  Results equal br_hip_gemm's for the
 * same `compute` up to the order of the fp32 summation (same rounding of the
 * operands). */
size_t br_hip_gemm_staged_workspace(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k,
                                    int a_dtype, int b_dtype, int64_t batch);
int br_hip_gemm_staged(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, float alpha,
                       const void* a, int a_dtype, int64_t lda, int64_t stride_a,
                       const void* b, int b_dtype, int64_t ldb, int64_t stride_b,
                       int accumulate, void* c, int c_dtype, int64_t ldc, int64_t stride_c,
                       const float* bias, int64_t batch, int compute,
                       void* workspace, size_t workspace_bytes, br_stream_t stream);

/* op_linear followed by op_gelu (cuda_tensor.cpp:146-193 and :400-412; the pair
 * of bloomz-7b/train.words:188-189) in one product whose epilogue writes both
 * tensors the backward pass needs, in the products' own 16-bit type:
 *   u[r, o] = sum_i x[r, i] * w[o, i] + bias[o]      y[r, o] = gelu(u[r, o])
 * x [rows, in], w [out, in], u and y [rows, out] are dense, all of `dtype`
 * (BR_F16 or BR_BF16); bias fp32 (may be NULL).  The activation is evaluated on
 * the fp32 sum, before u is rounded.  BR_ERR_TODO when the shape or alignment
 * rules out the direct-to-LDS kernel (in % 32, 16-byte aligned rows): the
 * caller then runs the two operators. */
int br_hip_linear_gelu(const void* x, const void* w, const float* bias, void* u, void* y, int dtype,
                       int64_t rows, int64_t out, int64_t in, br_stream_t stream);

/* op_linear followed by op_add of a residual (cuda_tensor.cpp:146-193 and
 * :206-232; the pair of bloomz-7b/train.words:172-173 and :191-192) in one
 * product whose epilogue adds the residual:
 *   y[r, o] = sum_i x[r, i] * w[o, i] + bias[o] + res[r, o]
 * x [rows, in], w [out, in] (each fp32 or the 16-bit type of `compute`), res and
 * y [rows, out] of y_dtype, dense; res may be y itself.  The sum is formed as
 * the two operators form it (product + bias rounded to fp32, then the residual
 * added), so the result has the bits of the pair.  workspace as for
 * br_hip_gemm_staged (br_hip_gemm_staged_workspace(0, 1, rows, out, in, ...)). */
int br_hip_linear_residual(const void* x, int x_dtype, const void* w, int w_dtype, const float* bias,
                           const void* res, void* y, int y_dtype, int64_t rows, int64_t out, int64_t in,
                           int compute, void* workspace, size_t workspace_bytes, br_stream_t stream);

/* ---- fused attention --------------------------------------------------- */
/* The operator chain of bloomz-7b/train.words:154-166 in one kernel:
 *   o = softmax((q . k^T) / sqrt(head_dim) + alibi[h, key] + mask) . v
 * replacing op_qk (cuda_tensor.cpp:277-330), two op_add (:206-232), op_softmax
 * (:332-356) and op_attn (:358-398) and the [batch, heads, tokens, tokens]
 * tensors between them.  mask(b, query, key) = 0 where key <= query and
 * key < valid[b], else -FLT_MAX: the table of train_bloom.cpp:73-90 for a batch
 * whose sequences are padded on the right (valid = number of real tokens; a
 * sequence with valid == 0 gets uniform probabilities, as the chain gives).
 * q, k, v, o: fp16 / bf16 (dtype); element (b, t, h, d) of q, k, v at
 * b * batch_stride + t * row_stride + h * head_stride + d, of o at
 * b * o_batch_stride + t * o_row_stride + h * head_stride + d.  So
 * [B, T, heads, 128] (the projections' own output), [B, heads, T, 128] and a
 * packed [B, T, 3, heads, 128] projection (q, k, v pointing at its thirds,
 * row_stride = 3 * heads * 128) all work without a transpose.
 * alibi: fp32 [heads, tokens] (br_hip_alibi_table); valid: device int32 [batch].
 * lse[batch, heads, tokens] receives log sum exp of each score row, which the
 * backward needs.  Probabilities are rounded to `dtype` before the product
 * with v.  BR_ERR_TODO unless head_dim == 128, strides % 8 == 0, token
 * strides below 2^24 elements and 16-byte aligned bases: callers then run
 * the unfused chain. */
int br_hip_flash_attn_fwd(const void* q, const void* k, const void* v, int dtype, const float* alibi,
                          const int32_t* valid, void* o, float* lse, int64_t batch, int64_t heads,
                          int64_t tokens, int64_t head_dim, int64_t row_stride, int64_t head_stride,
                          int64_t batch_stride, int64_t o_row_stride, int64_t o_batch_stride,
                          br_stream_t stream);

/* Backward of br_hip_flash_attn_fwd: the chain op_attn_backward
 * (cuda_tensor.cpp:830-888), op_softmax_backward (:890-918) and op_qk_backward
 * (:1004-1063) of train.words:217-226 without the [batch, heads, tokens, tokens]
 * tensors: probabilities are recomputed from q, k and lse.  o is the forward's
 * output, d_o its gradient (both `dtype`, o's strides); dq, dk, dv are of
 * grad_dtype (BR_F32, or `dtype`: the gradients rounded once, as the products
 * of the projection's backward would round them) with the element strides of
 * q, k, v.  delta: fp32 scratch of
 * batch * heads * tokens entries (receives rowsum(d_o * o)).  Deterministic: one
 * pass accumulates dq per query block (and forms delta on the way), a second one
 * dk / dv per key block.  dq, dk and dv must not be q, k, v, o or d_o themselves
 * (BR_ERR_OUTPUT): the second pass still reads all five.
 * Same shape limits as the forward (BR_ERR_TODO otherwise). */
int br_hip_flash_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o,
                          int dtype, const float* alibi, const int32_t* valid, const float* lse,
                          float* delta, void* dq, void* dk, void* dv, int grad_dtype, int64_t batch,
                          int64_t heads, int64_t tokens, int64_t head_dim, int64_t row_stride, int64_t head_stride,
                          int64_t batch_stride, int64_t o_row_stride, int64_t o_batch_stride,
                          br_stream_t stream);

/* ---- optimizer ---------------------------------------------------------- */
/* One AdamW step (decoupled weight decay) over n parameters, all arithmetic in
 * fp32:  p *= 1 - lr*wd;  m += (g - m)(1 - beta1);  v = beta2 v + (1 - beta2) g^2;
 * p -= lr / (1 - beta1^step) * m / (sqrt(v) / sqrt(1 - beta2^step) + eps).
 * param_dtype BR_F32: master must be NULL, the parameter is updated in place.
 * BR_F16 / BR_BF16: with an fp32 `master` copy the master is updated and param
 * receives its rounding; without one the 16-bit value itself is the state.
 * step counts from 1.  The reference has no optimizer (its training loop stops
 * at the gradients, bloomz-7b/train.words:320-366); this is what a training
 * run needs after them. */
int br_hip_adamw(void* param, int param_dtype, float* master, const float* grad, float* m, float* v,
                 int64_t n, float lr, float beta1, float beta2, float eps, float weight_decay,
                 int64_t step, br_stream_t stream);

/* ---- data preparation (bit-exact integer / gather work) ---------------- */
/* The embedding row gather of blackriver/train_bloom.cpp:50-56. */
int br_hip_embedding_gather(const void* table, const int32_t* ids, void* out, int elem_bytes,
                            int64_t n, int64_t hidden, int64_t vocab, br_stream_t stream);
/* Backward of that gather: grad[ids[i], :] += dx_scale * dx[i, :] for i = 0 .. n-1 in
 * ascending i (fp32; repeated ids are summed in position order, so the result
 * is deterministic); ids outside [0, vocab) are skipped.  The reference has no
 * embedding gradient (its table is frozen, train.words:264-268 only gathers);
 * with the LM head tied to the table this completes the table's gradient. */
int br_hip_embedding_scatter_add(const float* dx, const int32_t* ids, float* grad, int64_t n,
                                 int64_t hidden, int64_t vocab, float dx_scale, br_stream_t stream);
/* The ALiBi table of train_bloom.cpp:58-71: alibi[h,k] = (float)(k*slope_h),
 * slope_h = (2^(-2^(3-log2 heads)))^(h+1) evaluated in fp64 on the host. */
int br_hip_alibi_table(float* alibi, int64_t heads, int64_t tokens, br_stream_t stream);
/* The additive mask of train_bloom.cpp:73-90: xmask[b,q,k] = 0 when k <= q
 * and mask[b,0..k] are all non-zero, else -FLT_MAX.  mask is device int32. */
int br_hip_xmask_table(const int32_t* mask, float* xmask, int64_t batch, int64_t tokens,
                       br_stream_t stream);
/* Host helper: the fp64 ALiBi slopes of train_bloom.cpp:60-66. */
int br_hip_alibi_slopes(double* slopes_host, int64_t heads);

#ifdef __cplusplus
}
#endif
#endif
