#include "bloom_input.hpp"

#include <cfloat>
#include <cmath>
#include <cstring>
#include <vector>

#include "br_hip.h"
#include "runtime.hpp"
#include "tensor.hpp"

namespace br {

void BloomInput::gather_embeddings(const float* vocab, int64_t hidden, const int32_t* ids, int64_t n,
                                   float* xinput) {
    for (int64_t i = 0; i < n; i++)
        memcpy(xinput + i * hidden, vocab + (int64_t)ids[i] * hidden, (size_t)hidden * sizeof(float));
}

void BloomInput::build_alibi(int64_t heads, int64_t tokens, float* alibi) {
    std::vector<double> slopes((size_t)heads);
    br_hip_alibi_slopes(slopes.data(), heads);  // pure host arithmetic
    for (int64_t h = 0; h < heads; h++)
        for (int64_t k = 0; k < tokens; k++) alibi[h * tokens + k] = (float)((double)k * 1.0 * slopes[(size_t)h]);
}

void BloomInput::build_xmask(const int32_t* mask, int64_t batch, int64_t tokens, float* xmask) {
    for (int64_t b = 0; b < batch; b++) {
        const int32_t* m = mask + b * tokens;
        // number of leading real tokens: keys at or beyond it are closed for every query
        int64_t open = 0;
        while (open < tokens && m[open] != 0) open++;
        float* plane = xmask + b * tokens * tokens;
        for (int64_t q = 0; q < tokens; q++) {
            const int64_t lim = q + 1 < open ? q + 1 : open;
            float* row = plane + q * tokens;
            for (int64_t k = 0; k < lim; k++) row[k] = 0.0f;
            for (int64_t k = lim; k < tokens; k++) row[k] = -FLT_MAX;
        }
    }
}

namespace {

struct Embed : public NativeWord {
    void run(Stack& stack) override {
        tensor_t out = stack.pop_tensor();
        tensor_t table = stack.pop_tensor();
        tensor_t ids = stack.pop_tensor();
        br_assert(ids->is_cpu() && ids->dtype() == DataType::Int, "bloom.embed: ids must be a cpu int tensor");
        br_assert(table->is_cuda() && out->is_cuda() && table->dtype() == out->dtype(),
                  "bloom.embed: table and out must be device tensors of one type");
        const int64_t hidden = (int64_t)table->shape().vec().back();
        const int64_t vocab = (int64_t)table->items() / hidden;
        const int64_t n = (int64_t)out->items() / hidden;
        br_assert((int64_t)ids->items() >= n, "bloom.embed: not enough ids");
        int32_t* d_ids = static_cast<int32_t*>(ComputingContext::scratch((size_t)n * sizeof(int32_t)));
        BR_HIP_CHECK(br_hip_memcpy_h2d(d_ids, ids->data(), (size_t)n * sizeof(int32_t), ComputingContext::stream));
        BR_HIP_CHECK(br_hip_embedding_gather(table->data(), d_ids, out->data(), (int)DataType_size(table->dtype()), n,
                                             hidden, vocab, ComputingContext::stream));
    }
    NWORD_CREATOR_DEFINE_LR(Embed)
};

// ( ids dx grad -- )  grad[ids[i], :] += dx[i, :]: the gather's backward
// (dx carries the gradient lift of the backward pass, the table's gradient does not)
struct EmbedBackward : public NativeWord {
    void run(Stack& stack) override {
        tensor_t grad = stack.pop_tensor();
        tensor_t dx = stack.pop_tensor();
        tensor_t ids = stack.pop_tensor();
        br_assert(ids->is_cpu() && ids->dtype() == DataType::Int, "bloom.embed_backward: ids must be a cpu int tensor");
        br_assert(grad->is_cuda() && dx->is_cuda() && grad->dtype() == DataType::Float &&
                      dx->dtype() == DataType::Float,
                  "bloom.embed_backward: dx and grad must be device fp32 tensors");
        const int64_t hidden = (int64_t)grad->shape().vec().back();
        const int64_t vocab = (int64_t)grad->items() / hidden;
        br_assert((int64_t)dx->shape().vec().back() == hidden, "bloom.embed_backward: row lengths differ");
        const int64_t n = (int64_t)dx->items() / hidden;
        br_assert((int64_t)ids->items() >= n, "bloom.embed_backward: not enough ids");
        int32_t* d_ids = static_cast<int32_t*>(ComputingContext::scratch((size_t)n * sizeof(int32_t)));
        BR_HIP_CHECK(br_hip_memcpy_h2d(d_ids, ids->data(), (size_t)n * sizeof(int32_t), ComputingContext::stream));
        BR_HIP_CHECK(br_hip_embedding_scatter_add(static_cast<const float*>(dx->data()), d_ids,
                                                  static_cast<float*>(grad->data()), n, hidden, vocab,
                                                  1.0f / ComputingContext::grad_lift, ComputingContext::stream));
    }
    NWORD_CREATOR_DEFINE_LR(EmbedBackward)
};

struct Alibi : public NativeWord {
    void run(Stack& stack) override {
        tensor_t alibi = stack.pop_tensor();
        br_assert(alibi->is_cuda() && alibi->dtype() == DataType::Float && alibi->shape().dim() == 4,
                  "bloom.alibi: expects a device fp32 tensor [1, heads, 1, tokens]");
        BR_HIP_CHECK(br_hip_alibi_table(static_cast<float*>(alibi->data()), (int64_t)alibi->shape()[1],
                                        (int64_t)alibi->shape()[3], ComputingContext::stream));
    }
    NWORD_CREATOR_DEFINE_LR(Alibi)
};

struct XMask : public NativeWord {
    void run(Stack& stack) override {
        tensor_t xmask = stack.pop_tensor();
        tensor_t mask = stack.pop_tensor();
        br_assert(mask->is_cpu() && mask->dtype() == DataType::Int, "bloom.xmask: mask must be a cpu int tensor");
        br_assert(xmask->is_cuda() && xmask->dtype() == DataType::Float && xmask->shape().dim() == 4,
                  "bloom.xmask: expects a device fp32 tensor [batch, 1, tokens, tokens]");
        const int64_t batch = (int64_t)xmask->shape()[0], tokens = (int64_t)xmask->shape()[3];
        br_assert((int64_t)mask->items() >= batch * tokens, "bloom.xmask: mask too small");
        int32_t* d_mask = static_cast<int32_t*>(ComputingContext::scratch((size_t)(batch * tokens) * sizeof(int32_t)));
        BR_HIP_CHECK(br_hip_memcpy_h2d(d_mask, mask->data(), (size_t)(batch * tokens) * sizeof(int32_t),
                                       ComputingContext::stream));
        BR_HIP_CHECK(br_hip_xmask_table(d_mask, static_cast<float*>(xmask->data()), batch, tokens,
                                        ComputingContext::stream));
    }
    NWORD_CREATOR_DEFINE_LR(XMask)
};

// ( mask valid -- )  valid[b] = number of leading non-zero entries of mask[b, :]
// (for a batch padded on the right: the sequence length), as int32 values in
// the storage of a 4-byte-element device tensor; the fused attention words
// derive the causal / padding mask from it instead of reading the mask table.
struct Valid : public NativeWord {
    void run(Stack& stack) override {
        tensor_t valid = stack.pop_tensor();
        tensor_t mask = stack.pop_tensor();
        br_assert(mask->is_cpu() && mask->dtype() == DataType::Int && mask->shape().dim() == 2,
                  "bloom.valid: mask must be a [batch, tokens] cpu int tensor");
        const int64_t batch = (int64_t)mask->shape()[0], tokens = (int64_t)mask->shape()[1];
        br_assert(valid->is_cuda() && valid->dtype() == DataType::Float && (int64_t)valid->items() >= batch,
                  "bloom.valid: expects a device fp32-typed tensor of at least batch entries");
        std::vector<int32_t> count((size_t)batch);
        const int32_t* m = static_cast<const int32_t*>(mask->data());
        for (int64_t b = 0; b < batch; b++) {
            int64_t n = 0;
            while (n < tokens && m[b * tokens + n] != 0) n++;
            count[(size_t)b] = (int32_t)n;
        }
        BR_HIP_CHECK(br_hip_memcpy_h2d(valid->data(), count.data(), (size_t)batch * sizeof(int32_t),
                                       ComputingContext::stream));
        ComputingContext::sync();  // `count` leaves scope; once per batch
    }
    NWORD_CREATOR_DEFINE_LR(Valid)
};

// ( tensor mean std seed -- )  synthetic initialisation of a device tensor
struct Normal : public NativeWord {
    void run(Stack& stack) override {
        const double seed = stack.pop_number();
        const double std = stack.pop_number();
        const double mean = stack.pop_number();
        tensor_t t = stack.pop_tensor();
        br_assert(t->is_cuda() && t->dtype() != DataType::Int, "bloom.normal: expects a device float tensor");
        BR_HIP_CHECK(br_hip_normal(t->data(), (int)t->dtype(), (float)mean, (float)std, (uint64_t)seed,
                                   (int64_t)t->items(), ComputingContext::stream));
    }
    NWORD_CREATOR_DEFINE_LR(Normal)
};

// ( -- loss )  what the most recent op.loss_backward returned
struct LastLoss : public NativeWord {
    void run(Stack& stack) override { stack.push_number((double)ComputingContext::last_loss); }
    NWORD_CREATOR_DEFINE_LR(LastLoss)
};

// ( -- S )  the gradient lift the current backward pass carries (1 = none)
struct GradLiftValue : public NativeWord {
    void run(Stack& stack) override { stack.push_number((double)ComputingContext::grad_lift); }
    NWORD_CREATOR_DEFINE_LR(GradLiftValue)
};

}  // namespace

void load_bloom_words(Enviroment& env) {
    env.insert_native_word("bloom.normal", Normal::creator);
    env.insert_native_word("bloom.last_loss", LastLoss::creator);
    env.insert_native_word("bloom.grad_lift", GradLiftValue::creator);
    env.insert_native_word("bloom.embed", Embed::creator);
    env.insert_native_word("bloom.embed_backward", EmbedBackward::creator);
    env.insert_native_word("bloom.alibi", Alibi::creator);
    env.insert_native_word("bloom.xmask", XMask::creator);
    env.insert_native_word("bloom.valid", Valid::creator);
}

}  // namespace br
