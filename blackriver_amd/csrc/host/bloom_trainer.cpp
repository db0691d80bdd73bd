#include "bloom_trainer.hpp"

#include <cmath>
#include <cstring>
#include <sstream>
#include <vector>

#include "br_hip.h"
#include "common.hpp"
#include "runtime.hpp"
#include "tensor.hpp"

namespace br {

BloomTrainer::BloomTrainer(Enviroment& env, const BloomModelConfig& cfg) : env_(env), cfg_(cfg) {
    br_assert(cfg.layers >= 1, "a model needs at least one block");
    br_assert(cfg.hidden % cfg.heads == 0, "hidden size must divide among the heads");
    br_assert(cfg.batch >= 1 && cfg.tokens >= 2, "batch >= 1 and tokens >= 2");
    br_assert((size_t)cfg.layers + 1 <= env.hashes_num(), "the environment has too few hashes for the layers");
}

// The carve-up of create_dynamic_here (bloom.words): ten [B,T,H] buffers, two
// [B,T,4H], alibi, three [H] statistics vectors, xmask and the probabilities.
int64_t BloomTrainer::block_arena_floats() const {
    const int64_t bth = cfg_.batch * cfg_.tokens * cfg_.hidden;
    return 10 * bth + 2 * 4 * bth + cfg_.heads * cfg_.tokens + 3 * cfg_.hidden +
           cfg_.batch * cfg_.tokens * cfg_.tokens + cfg_.batch * cfg_.heads * cfg_.tokens * cfg_.tokens;
}

// 16-bit weights multiplied in their own type: product-only activations can
// live in 16-bit operand buffers (same bits out, fewer conversions).
bool BloomTrainer::mixed() const {
    return cfg_.weight_dtype == cfg_.gemm_precision && (cfg_.weight_dtype == "f16" || cfg_.weight_dtype == "bf16");
}

bool BloomTrainer::flash() const {
    return cfg_.fused_attention && mixed() && cfg_.hidden / cfg_.heads == 128;
}

int64_t BloomTrainer::model_arena_floats() const {
    // plus one logits row per position: the loss head then needs a single group
    return block_arena_floats() + cfg_.batch * cfg_.tokens * cfg_.vocab;
}

std::string BloomTrainer::setup_script() const {
    std::ostringstream s;
    s.precision(9);
    auto dims = [&]() {
        s << cfg_.hidden << " " << cfg_.heads << " " << cfg_.vocab << " " << cfg_.eps << " model_dims\n";
        s << "'cuda' $DEVICE !  '" << cfg_.weight_dtype << "' $WDTYPE !\n";
    };
    s << "0 #\n";
    dims();
    s << "'" << cfg_.gemm_precision << "' op.gemm_precision\n";
    s << "create_model_weight create_model_grad\n";
    s << model_arena_floats() << " create_var\n";
    s << cfg_.batch << " " << cfg_.tokens << " create_model_dynamic\n";
    for (int i = 1; i <= cfg_.layers; i++) {
        s << i << " #\n";
        dims();
        s << "create_layer_weight create_layer_grad\n";
        // the block's view of logits rows is never used; one row keeps the view well-formed
        s << block_arena_floats() + cfg_.vocab << " create_var\n";
        s << cfg_.batch << " " << cfg_.tokens << " create_dynamic_here\n";
        if (mixed()) s << "create_operand_buffers\n";
        if (flash()) s << "create_flash_buffers\n";
        s << "0 #  " << i << " share_batch_tensors\n";
    }
    // Activations pass between neighbouring blocks by name, not by copy: block i reads as its xinput the very tensor
    // block i-1 leaves its output in, and as its yout_g the one block i+1 leaves its input gradient in.  Both are
    // written again by their owner only after the reader is done with them (a block's backward pass reuses its xa
    // for the gradient once every later block has finished, forward and backward).
    for (int i = 2; i <= cfg_.layers; i++) s << i - 1 << " # 'xa' @  " << i << " # 'xinput' !\n";
    for (int i = 1; i < cfg_.layers; i++) s << i + 1 << " # 'xa' @  " << i << " # 'yout_g' !\n";
    s << "0 #\n";
    return s.str();
}

std::string BloomTrainer::step_script() const {
    std::ostringstream s;
    const int n = cfg_.layers;
    const char* forward = flash() ? "layer_forward_flash" : mixed() ? "layer_forward_mixed" : "layer_forward";
    const char* backward = flash() ? "layer_backward_flash" : mixed() ? "layer_backward_mixed" : "layer_backward_core";
    s << "0 # model_input\n";
    s << "1 # 'xinput' @  0 # 'xinput' @  op.copy   1 # " << forward << "\n";
    for (int i = 2; i <= n; i++) s << i << " # " << forward << "\n";  // xinput is block i-1's xa
    s << "0 # 'xa' @  " << n << " # 'xa' @  op.copy   0 # model_head\n";
    s << n << " # 'yout_g' @  0 # 'xc' @  op.copy   " << n << " # " << backward << "\n";
    for (int i = n - 1; i >= 1; i--) s << i << " # " << backward << "\n";  // yout_g is block i+1's xa
    s << "0 # 'xb' @  1 # 'xa' @  op.copy   0 # model_input_backward\n";
    s << "op.sync\n";
    return s.str();
}

void BloomTrainer::create() {
    env_.execute(setup_script());
    step_.reset(env_.build(step_script()));
}

void BloomTrainer::init_synthetic(uint64_t seed, float std) {
    std::ostringstream s;
    s.precision(9);
    auto matrix = [&](const char* name, uint64_t sd) {
        s << "'" << name << "' @ 0 " << std << " " << sd << " bloom.normal\n";
    };
    s << "0 #\n";
    matrix("word_embeddings.weight", seed * 1000003ull);
    s << "'word_embeddings_layernorm.weight' @ 1 op.fill  'word_embeddings_layernorm.bias' @ op.zero\n";
    s << "'ln_f.weight' @ 1 op.fill  'ln_f.bias' @ op.zero\n";
    for (int i = 1; i <= cfg_.layers; i++) {
        const uint64_t base = (seed + (uint64_t)i) * 1000003ull;
        s << i << " #\n";
        matrix("query_key_value.weight", base + 1);
        matrix("dense.weight", base + 2);
        matrix("dense_h_to_4h.weight", base + 3);
        matrix("dense_4h_to_h.weight", base + 4);
        s << "'input_layernorm.weight' @ 1 op.fill  'input_layernorm.bias' @ op.zero\n";
        s << "'post_attention_layernorm.weight' @ 1 op.fill  'post_attention_layernorm.bias' @ op.zero\n";
        s << "'query_key_value.bias' @ op.zero  'dense.bias' @ op.zero\n";
        s << "'dense_h_to_4h.bias' @ op.zero  'dense_4h_to_h.bias' @ op.zero\n";
    }
    s << "0 # op.sync\n";
    env_.execute(s.str());
}

void BloomTrainer::create_optimizer(float lr, float beta1, float beta2, float eps, float weight_decay) {
    br_assert(step_ != nullptr, "BloomTrainer::create has not run");
    br_assert(!has_optimizer_, "the optimizer state exists already");
    std::ostringstream s;
    s.precision(9);
    for (int i = 0; i <= cfg_.layers; i++) {
        s << i << " #  " << lr << " " << beta1 << " " << beta2 << " " << eps << " " << weight_decay << " adamw_hyper\n";
        s << (i == 0 ? "create_model_adamw" : "create_layer_adamw");
        if (masters()) s << (i == 0 ? " create_model_masters" : " create_layer_masters");
        s << "\n";
    }
    s << "0 # op.sync\n";
    env_.execute(s.str());
    has_optimizer_ = true;
    adam_step_ = 0;
}

void BloomTrainer::optimizer_step() {
    br_assert(has_optimizer_, "BloomTrainer::create_optimizer has not run");
    adam_step_++;
    // the step count changes every call, so the (short) program is compiled per call
    std::ostringstream s;
    const char* sfx = masters() ? "16" : "";
    s << "0 #  " << adam_step_ << " $adam_step !  model_adamw" << sfx << "\n";
    for (int i = 1; i <= cfg_.layers; i++)
        s << i << " #  " << adam_step_ << " $adam_step !  layer_adamw" << sfx << "\n";
    s << "0 # op.sync\n";
    env_.execute(s.str());
}

float BloomTrainer::step(const int32_t* ids, const int32_t* mask) {
    br_assert(step_ != nullptr, "BloomTrainer::create has not run");
    env_.change(0);
    const size_t n = (size_t)(cfg_.batch * cfg_.tokens);
    tensor_t t_ids = env_.hash().find_tensor("ids_");
    tensor_t t_mask = env_.hash().find_tensor("mask_");
    memcpy(t_ids->data(), ids, n * sizeof(int32_t));
    memcpy(t_mask->data(), mask, n * sizeof(int32_t));
    // 16-bit products: the loss head picks a gradient lift for this step's
    // backward pass; the setting is this step's only (the context is global)
    ComputingContext::grad_lift_auto = cfg_.gemm_precision != "f32" && cfg_.gemm_precision != "float";
    ComputingContext::grad_lift = 1.0f;
    env_.run(step_.get());
    grad_lift_ = ComputingContext::grad_lift;
    ComputingContext::grad_lift_auto = false;
    ComputingContext::grad_lift = 1.0f;
    // Overflow guard.  A lifted 16-bit activation gradient saturates to inf once a per-token gradient exceeds
    // 65504 / lift, and every gradient further down the backward chain inherits it.  The embedding LayerNorm sits at
    // the bottom of that chain: its weight gradient (hidden floats) and the loss being finite means no activation
    // gradient of this step overflowed.
    const float loss = ComputingContext::last_loss;
    tensor_t probe = env_.hash().find_tensor("word_embeddings_layernorm.weight_g");
    std::vector<float> g((size_t)cfg_.hidden);
    br_assert(probe->items() == g.size(), "embedding LayerNorm gradient has an unexpected size");
    if (br_hip_memcpy_d2h(g.data(), probe->data(), g.size() * sizeof(float), ComputingContext::stream) != 0)
        br_panic("BloomTrainer::step: reading back the embedding LayerNorm gradient failed");
    ComputingContext::sync();
    bool finite = std::isfinite(loss);
    for (float v : g) finite = finite && std::isfinite(v);
    if (!finite) {
        std::ostringstream why;
        why << "BloomTrainer::step: non-finite loss or gradient (loss " << loss << ", gradient lift " << grad_lift_
            << "); with 16-bit products lower the lift by a power of two with `<S> op.grad_lift`, or run the products "
               "in bf16 / fp32";
        br_panic(why.str().c_str());
    }
    return loss;
}

}  // namespace br
