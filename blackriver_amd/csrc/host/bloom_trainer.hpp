// Whole-model training driver for one GPU: the counterpart of the main loop
// of blackriver/train_bloom.cpp:123-199 without MPI ranks, host weight
// streaming or per-layer recomputation.  Every decoder block lives in its own
// hash (weights, fp32 gradients and a private activation arena), the model
// level (embedding, final LayerNorm, LM head) in hash 0; the driver writes the
// per-block lines of the setup and step programs because the word language
// has no loops (the reference unrolls its layers by hand the same way,
// bloomz-7b/train.words:274-298).
#pragma once

#include <cstdint>
#include <memory>
#include <string>

#include "vm.hpp"

namespace br {

struct BloomModelConfig {
    int layers = 1;
    int64_t batch = 1, tokens = 512;
    int64_t hidden = 4096, heads = 32, vocab = 250880;
    float eps = 1e-5f;
    std::string weight_dtype = "f16";     // "float", "f16" or "bf16": storage of the weight matrices
    std::string gemm_precision = "f16";   // MFMA type for products of fp32-stored operands
    // one fused attention kernel per direction instead of the operator chain
    // through [B, heads, T, T] tensors; used when the shape allows (see flash())
    bool fused_attention = true;
};

class BloomTrainer {
public:
    // `env` must have been created with at least cfg.layers + 1 hashes and must
    // already hold the block-level and model-level word definitions.
    BloomTrainer(Enviroment& env, const BloomModelConfig& cfg);

    // Creates every tensor and compiles the step program.
    void create();
    // N(0, std) matrices, unit LayerNorm scales, zero biases; block i uses seed + i.
    void init_synthetic(uint64_t seed, float std);
    // One step: ids / mask are [batch, tokens] int32 on the host.  Returns the
    // mean log-probability of the labels (the sign convention of op.loss_backward).
    float step(const int32_t* ids, const int32_t* mask);
    // The power of two the last step's backward pass carried on its activation
    // gradients (what is left in the blocks' and hash 0's gradient buffers, e.g.
    // the embedding rows' gradient `xc`, is that many times the true gradient;
    // parameter gradients are at their true scale).  1 with fp32 products.
    float grad_lift() const { return grad_lift_; }

    // AdamW state for every parameter (moments; fp32 master copies of 16-bit
    // matrices, initialised from the matrices as they are now: call after the
    // weights have their starting values).
    void create_optimizer(float lr, float beta1, float beta2, float eps, float weight_decay);
    // One AdamW step over every parameter from the gradients of the last step().
    void optimizer_step();
    int64_t optimizer_steps() const { return adam_step_; }

    const BloomModelConfig& config() const { return cfg_; }
    // floats of a block's arena / of hash 0's arena (which ends in the logits rows)
    int64_t block_arena_floats() const;
    int64_t model_arena_floats() const;
    bool mixed() const;
    // fused attention is on and applies: 16-bit operand buffers, head size 128
    bool flash() const;
    std::string setup_script() const;
    std::string step_script() const;

private:
    Enviroment& env_;
    BloomModelConfig cfg_;
    std::unique_ptr<DaG> step_;
    bool masters() const { return cfg_.weight_dtype != "float"; }
    bool has_optimizer_ = false;
    int64_t adam_step_ = 0;
    float grad_lift_ = 1.0f;
};

}  // namespace br
