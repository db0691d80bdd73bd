/*
 * br_oracle.h -- CPU restatement of BlackRiver's CUDA-path operator semantics.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the parity checker and the timed
 * CPU baseline.  Nothing in the shipped path (the HIP kernel library, the
 * host runtime, the word bindings) may include, link or call it; only the
 * test-suite, the smoke check and the benchmark's CPU-baseline leg do.
 *
 * Conventions: tensors are dense row-major fp32 (int32 for ids / masks);
 * every reduction is accumulated in fp64 and rounded to fp32 once, so the
 * result is independent of the GPU's reduction order.  Each function cites
 * the reference source it restates (paths relative to the reference tree).
 *
 * Pinning status (what independent evidence each function is checked against
 * lives in tests/test_oracle_*.py):
 *   layernorm fwd/bwd      closed form, finite differences, row invariants
 *   gelu fwd/bwd           closed form, central differences, odd symmetry
 *   linear / batched GEMMs naive fp64 einsum, finite differences
 *   softmax family         row sums, shift invariance, finite differences
 *   loss head              reference fixtures (ids/mask) brute force, FD
 *   fetch_data pieces      reference fixtures, closed-form ALiBi slopes
 *   embedding scatter-add  (not in the reference) np.add.at, one-hot product,
 *                          torch autograd of the tied table
 *   AdamW (oracle/__init__.py, numpy; not in the reference)
 *                          torch.optim.AdamW over five steps
 * The arithmetic of cuDNN / cuBLASLt / OpenBLAS that the reference calls is
 * not vendored there and no version is pinned; those calls are restated from
 * their published definitions (softmax, broadcast add, column sum, SGEMM).
 */
#ifndef BR_ORACLE_H_
#define BR_ORACLE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* blackriver/kernels/normalize_kernels.cu:40-85 (ker_layer_norm), called from
 * blackriver/cuda_tensor.cpp:236-255.  var_out holds sigma^2 + eps. */
void orc_layernorm_fwd(const float* x, const float* gamma, const float* beta,
                       float* y, float* mean_out, float* var_out,
                       int64_t rows, int64_t cols, float eps);

/* normalize_kernels.cu:14-17,134-221,253-340 with means == nullptr, called
 * from cuda_tensor.cpp:699-727.  var_in is what the forward stored. */
void orc_layernorm_bwd(const float* dy, const float* y, const float* gamma,
                       const float* beta, const float* var_in,
                       float* dgamma, float* dbeta, float* dx,
                       int64_t rows, int64_t cols, float eps);

/* blackriver/kernels/gelu.cu:37-44 */
void orc_gelu_fwd(const float* x, float* y, int64_t n);
/* blackriver/kernels/gelu.cu:61-70 (fp64 arithmetic, tanh rounded to fp32) */
void orc_gelu_bwd(const float* dy, const float* x, float* dx, int64_t n);

/* Extension used by the bias-GELU kernels: y = gelu(x + bias[col]); the
 * backward also returns dbias[col] = sum_rows dx when dbias != NULL. */
void orc_bias_gelu_fwd(const float* x, const float* bias, float* y,
                       int64_t rows, int64_t cols);
void orc_bias_gelu_bwd(const float* dy, const float* x, const float* bias,
                       float* dx, float* dbias, int64_t rows, int64_t cols);

/* cuda_tensor.cpp:146-193: y[n,o] = sum_k x[n,k] w[o,k] + b[o] */
void orc_linear_fwd(const float* x, const float* w, const float* b, float* y,
                    int64_t n, int64_t in, int64_t out);
/* cuda_tensor.cpp:730-812: db, dW, dx (in that order; dx may alias x) */
void orc_linear_bwd(const float* dy, const float* x, const float* w,
                    float* dx, float* dw, float* db,
                    int64_t n, int64_t in, int64_t out);

/* blackriver/kernels/transform_kernels.cu:40-54 */
void orc_transpose_0213(const float* x, float* y, int64_t s0, int64_t s1,
                        int64_t s2, int64_t s3);

/* cuda_tensor.cpp:206-232 (cudnnOpTensor ADD): c = a + b, b broadcast over
 * every dimension where its extent is 1.  Shapes are rank-4 (lower ranks are
 * mapped as cuda_tensor.hpp:26-52 does).  c may alias a. */
void orc_add_bcast(const float* a, const int64_t* ashape, const float* b,
                   const int64_t* bshape, float* c);

/* cuda_tensor.cpp:277-330 */
void orc_qk(const float* q, const float* k, float* s, int64_t bh, int64_t t,
            int64_t hd);
/* cuda_tensor.cpp:332-356 (cudnnSoftmaxForward ACCURATE); out may alias x */
void orc_softmax_fwd(const float* x, float* y, int64_t rows, int64_t cols);
/* cuda_tensor.cpp:890-918 (cudnnSoftmaxBackward ACCURATE) */
void orc_softmax_bwd(const float* dy, const float* y, float* dx, int64_t rows,
                     int64_t cols);
/* cuda_tensor.cpp:358-398 */
void orc_attn(const float* p, const float* v, float* o, int64_t bh, int64_t t,
              int64_t hd);
/* cuda_tensor.cpp:830-888 */
void orc_attn_bwd(const float* d_o, const float* p, const float* v, float* dp,
                  float* dv, int64_t bh, int64_t t, int64_t hd);
/* cuda_tensor.cpp:920-1002; ds may alias p */
void orc_softmax_attn_bwd(const float* d_o, const float* p, const float* v,
                          float* ds, float* dv, int64_t bh, int64_t t,
                          int64_t hd);
/* cuda_tensor.cpp:1004-1063 */
void orc_qk_bwd(const float* ds, const float* q, const float* k, float* dq,
                float* dk, int64_t bh, int64_t t, int64_t hd);

/* cuda_tensor.cpp:414-462 */
void orc_last_logits(const float* x, const int32_t* mask, const float* lm_head,
                     float* out, int64_t batch, int64_t tokens, int64_t hidden,
                     int64_t vocab);

/* Integer half of cuda_tensor.cpp:464-697: labels[b,t] = ids[b,t+1] where
 * mask[b,t] and mask[b,t+1] are both non-zero and t < T-1, else -100
 * (:617-624).  Returns the loss-token count (:555-568). */
int64_t orc_loss_labels(const int32_t* ids, const int32_t* mask, int64_t batch,
                        int64_t tokens, int32_t* labels);
/* Group walk of cuda_tensor.cpp:596-616: writes (batch, begin_t, size) triples
 * for every non-empty group after trailing masked positions are trimmed.
 * Returns the number of groups (at most max_groups are written). */
int64_t orc_loss_groups(const int32_t* mask, int64_t batch, int64_t tokens,
                        int64_t group_max, int64_t* triples,
                        int64_t max_groups);
/* Float half of cuda_tensor.cpp:464-697 and kernels/nll_loss.cu:10-43.
 * Returns +mean log-prob of the labels; x_g is overwritten, lm_head_g is
 * accumulated into.  dlogits_out (optional, [batch*tokens, vocab]) receives
 * (softmax - onehot)/count on loss rows, 0 elsewhere. */
float orc_loss_backward(const float* x, const int32_t* ids,
                        const int32_t* mask, const float* lm_head, float* x_g,
                        float* lm_head_g, float* dlogits_out, int64_t batch,
                        int64_t tokens, int64_t hidden, int64_t vocab);

/* Kernel-level view of the same head (rows of logits given directly):
 * lse[r] = logsumexp(logits[r,:]); returns sum_r keep[r]*(logits[r,target[r]]
 * - lse[r]) / count with count = #{keep != 0}; dlogits (optional) =
 * keep*(softmax - onehot)/count. */
float orc_logsoftmax_nll(const float* logits, const int32_t* target,
                         const int32_t* keep, float* lse, float* dlogits,
                         int64_t rows, int64_t vocab);

/* blackriver/train_bloom.cpp:50-56 */
void orc_embedding_gather(const float* vocab, const int32_t* ids, float* out,
                          int64_t n, int64_t hidden);
/* Backward of the gather: grad[ids[i],:] += dx[i,:], i ascending.  Not in the
 * reference (frozen table); pinned by autograd of the tied table in
 * tests/test_oracle_model.py and by brute force in tests/test_oracle_ops.py. */
void orc_embedding_scatter_add(float* grad, const float* dx, const int32_t* ids,
                               int64_t n, int64_t hidden, int64_t vocab);
/* train_bloom.cpp:58-71 */
void orc_alibi(float* alibi, int64_t heads, int64_t tokens);
/* train_bloom.cpp:73-90 */
void orc_xmask(const int32_t* mask, float* xmask, int64_t batch,
               int64_t tokens);

/* fp16 <-> fp32 helpers (IEEE binary16, round-to-nearest-even) so that the
 * fp16-storage kernels can be checked without a GPU. */
void orc_f32_to_f16(const float* x, uint16_t* y, int64_t n);
void orc_f16_to_f32(const uint16_t* x, float* y, int64_t n);

/* Thread count the library will use (OpenMP). */
int orc_threads(void);

#ifdef __cplusplus
}
#endif
#endif
