/*
 * br_host.h -- C embedding API of libblackriver.so, the C++ host runtime
 * (operator API, tensors, word machine) that sits above the br_hip kernel ABI.
 *
 * It lets a driver, a test or a benchmark written in any language boot the
 * runtime, run word scripts and move tensor contents in and out.  It is the
 * programmatic equivalent of what the reference's driver does in C++
 * (blackriver/train_bloom.cpp:123-199: build an Enviroment, load the nn
 * words, execute init.words / train.words, run user words).
 *
 * Errors: the host runtime is fail-fast (a panic aborts the process) unless
 * it is entered through this API, in which case the panic is caught, the
 * call returns -1 and br_host_last_error() returns the message.  After a
 * panic the environment's stack may hold leftovers; br_env_stack_clear()
 * resets it.
 */
#ifndef BR_HOST_H_
#define BR_HOST_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct br_env br_env_t;

/* Boots MemoryContext (host arena of host_arena_bytes), CollectiveContext
 * (single process) and, when device >= 0, ComputingContext on that GPU --
 * the sequence of train_bloom.cpp:201-232.  device < 0 boots a host-only
 * runtime in which creating a "cuda" tensor panics. */
int br_host_boot(int device, size_t host_arena_bytes);
int br_host_shutdown(void);
const char* br_host_last_error(void);
/* Device stream every operator launches on (hipStream_t), NULL before boot. */
void* br_host_stream(void);
int br_host_sync(void);
/* BR_GEMM_F16 / BR_GEMM_BF16 / BR_GEMM_F32 for products of fp32-stored operands. */
int br_host_set_fp32_gemm_compute(int compute);
/* op.loss_backward prints "#################  <count> <loss>" on stdout as the
 * reference does (cuda_tensor.cpp:692); 0 turns that off for drivers that own
 * stdout. */
int br_host_set_echo_loss(int on);

/* An Enviroment with `hashes` namespaces and the io.* / op.* words loaded
 * (train_bloom.cpp:125-126). */
br_env_t* br_env_create(int hashes);
void br_env_destroy(br_env_t* env);

/* Enviroment::execute: compile, link and run `text` once. */
int br_env_execute(br_env_t* env, const char* text);
/* Enviroment::build / run: compile and link once, run many times.  Programs
 * are owned by the environment and identified by the returned index. */
int br_env_build(br_env_t* env, const char* text, int* program);
int br_env_run(br_env_t* env, int program);

/* Compile and link `text` without running it and write the flat program,
 * one step per line ("N:<number>", "S:<string>", "B:<builtin>",
 * "W:<native word>"), into out.  Returns -2 when out_bytes is too small. */
int br_env_disassemble(br_env_t* env, const char* text, char* out, size_t out_bytes);
/* The same listing after the fusion pass that build / execute apply to a linked
 * program ("-:<word>" marks a word whose work moved into the fused word that
 * follows it). */
int br_env_disassemble_fused(br_env_t* env, const char* text, char* out, size_t out_bytes);

int br_env_change_hash(br_env_t* env, int hash);
int br_env_current_hash(br_env_t* env);
int br_env_set_number(br_env_t* env, const char* name, double value);
int br_env_set_string(br_env_t* env, const char* name, const char* value);
int br_env_get_number(br_env_t* env, const char* name, double* value);
int br_env_has(br_env_t* env, const char* name);

int br_env_stack_size(br_env_t* env);
int br_env_stack_clear(br_env_t* env);
int br_env_stack_pop_number(br_env_t* env, double* value);

/* Tensor stored under `name` in the current hash.  dtype uses the BR_F32 /
 * BR_BF16 / BR_F16 / BR_I32 numbering; shape receives at most 8 extents. */
int br_env_tensor_info(br_env_t* env, const char* name, int* dtype, int* on_device, int* rank,
                       int64_t shape[8], void** data);
/* fp32 host buffer <-> tensor contents (converted when the tensor is stored
 * in 16 bits; int32 tensors use the _i32 pair).  Synchronous. */
int br_env_tensor_write(br_env_t* env, const char* name, const float* src, int64_t n);
int br_env_tensor_read(br_env_t* env, const char* name, float* dst, int64_t n);
int br_env_tensor_write_i32(br_env_t* env, const char* name, const int32_t* src, int64_t n);
int br_env_tensor_read_i32(br_env_t* env, const char* name, int32_t* dst, int64_t n);

/* Whole-model training on one GPU: the main loop of blackriver/train_bloom.cpp:123-199
 * (create the tensors, then per step: fetch_data + run the training words)
 * without MPI ranks and host weight streaming.  `env` needs layers + 1 hashes
 * and must already have executed bloom.words and bloom_model.words.  Block i
 * lives in hash i (weights, fp32 gradients, its own activation arena), the
 * embedding / final LayerNorm / LM head in hash 0.
 *   create: allocates everything and compiles the step program
 *   init:   N(0, std) matrices, unit LayerNorm scales, zero biases
 *   step:   ids / mask are [batch, tokens] int32 host arrays; *loss receives
 *           what op.loss_backward returns (mean log-probability of the labels) */
int br_bloom_model_create(br_env_t* env, int layers, int64_t batch, int64_t tokens, int64_t hidden,
                          int64_t heads, int64_t vocab, float eps, const char* weight_dtype,
                          const char* gemm_precision);
/* Before br_bloom_model_create: whether attention runs as one fused kernel per
 * direction (default; applies with 16-bit weights multiplied in their own
 * type and head size 128) or as the reference's operator
 * chain through [batch, heads, tokens, tokens] tensors. */
int br_bloom_model_set_fused_attention(br_env_t* env, int on);
int br_bloom_model_init(br_env_t* env, uint64_t seed, float std);
int br_bloom_model_step(br_env_t* env, const int32_t* ids, const int32_t* mask, float* loss);
/* The power of two S that the last step's backward pass carried on its
 * activation gradients (chosen by the loss head when products run in 16 bit so
 * that small gradients stay clear of fp16's subnormal range; 1 with fp32
 * products).  Parameter gradients are at their true scale; activation-gradient
 * buffers left behind (e.g. `xc`, the embedding rows' gradient) hold S times
 * the true values. */
int br_bloom_model_grad_lift(br_env_t* env, float* lift);
/* AdamW over every parameter of the model (the reference's loop ends at the
 * gradients, bloomz-7b/train.words:320-366).  optimizer_create allocates the
 * moments and, for 16-bit matrices, fp32 master copies initialised from the
 * matrices as they are at that moment; optimizer_step applies one update from
 * the gradients the last br_bloom_model_step left. */
int br_bloom_model_optimizer_create(br_env_t* env, float lr, float beta1, float beta2, float eps,
                                    float weight_decay);
int br_bloom_model_optimizer_step(br_env_t* env);

/* The host-side batch preparation of BloomInput::fetch_data
 * (train_bloom.cpp:41-93) on caller-provided host buffers:
 *   xinput[i,:] = vocab[ids[i],:]             (when vocab != NULL)
 *   alibi[h,k]  = (float)(k * slope_h)        (when alibi != NULL)
 *   xmask[b,q,k] = 0 if k <= q and mask[b,0..k] all non-zero else -FLT_MAX
 */
int br_bloom_fetch_data(const int32_t* ids, const int32_t* mask, int64_t batch, int64_t tokens,
                        const float* vocab, int64_t hidden, int64_t heads, float* xinput, float* alibi,
                        float* xmask);

#ifdef __cplusplus
}
#endif
#endif
