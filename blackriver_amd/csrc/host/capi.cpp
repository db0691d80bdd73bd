// C embedding API (include/br_host.h): boots the runtime, runs word scripts
// and moves tensor contents, turning panics into error returns.
#include "br_host.h"

#include <cstring>
#include <memory>

#include "bloom_input.hpp"
#include "bloom_trainer.hpp"
#include "br_hip.h"
#include "runtime.hpp"
#include "tensor.hpp"
#include "vm.hpp"
#include "words.hpp"

using namespace br;

struct br_env {
    std::unique_ptr<Enviroment> env;
    std::vector<std::unique_ptr<DaG>> programs;
    std::unique_ptr<BloomTrainer> trainer;
    bool fused_attention = true;
};

namespace {

std::string g_last_error;

void throwing_hook(const std::string& message) { throw Panic(message); }

// Runs `f` with panics converted to exceptions; -1 and a message on failure.
template <typename F>
int guarded(F&& f) {
    set_panic_hook(throwing_hook);
    try {
        f();
        set_panic_hook(nullptr);
        return 0;
    } catch (const std::exception& e) {
        g_last_error = e.what();
    } catch (...) {
        g_last_error = "unknown C++ exception";
    }
    set_panic_hook(nullptr);
    return -1;
}

tensor_t find_tensor(br_env_t* e, const char* name) {
    Hash::Item item = e->env->hash().find(name);
    if (item.index() != 2) br_panic("value is not a tensor");
    return std::get<2>(item);
}

}  // namespace

extern "C" {

const char* br_host_last_error(void) { return g_last_error.c_str(); }

int br_host_boot(int device, size_t host_arena_bytes) {
    return guarded([&]() {
        CollectiveContext::boot(0, nullptr, 1);
        MemoryContext::boot(host_arena_bytes);
        if (device >= 0) ComputingContext::boot(device);
    });
}

int br_host_shutdown(void) {
    return guarded([&]() {
        ComputingContext::shutdown();
        MemoryContext::shutdown();
        CollectiveContext::shutdown();
    });
}

void* br_host_stream(void) { return ComputingContext::stream; }

int br_host_sync(void) {
    return guarded([&]() { ComputingContext::sync(); });
}

int br_host_set_fp32_gemm_compute(int compute) {
    if (compute != BR_GEMM_F16 && compute != BR_GEMM_BF16 && compute != BR_GEMM_F32) return -1;
    ComputingContext::fp32_gemm_compute = compute;
    return 0;
}

int br_host_set_echo_loss(int on) {
    ComputingContext::echo_loss = on != 0;
    return 0;
}

br_env_t* br_env_create(int hashes) {
    br_env_t* e = new br_env();
    if (guarded([&]() {
            e->env.reset(new Enviroment(hashes));
            load_nn_words(*e->env);
            load_bloom_words(*e->env);
        }) != 0) {
        delete e;
        return nullptr;
    }
    return e;
}

void br_env_destroy(br_env_t* e) {
    if (!e) return;
    guarded([&]() {
        e->trainer.reset();
        e->programs.clear();
        e->env.reset();
    });
    delete e;
}

int br_env_execute(br_env_t* e, const char* text) {
    return guarded([&]() { e->env->execute(text); });
}

int br_env_build(br_env_t* e, const char* text, int* program) {
    return guarded([&]() {
        e->programs.emplace_back(e->env->build(text));
        if (program) *program = (int)e->programs.size() - 1;
    });
}

int br_env_run(br_env_t* e, int program) {
    return guarded([&]() {
        br_assert(program >= 0 && (size_t)program < e->programs.size(), "no such program");
        e->env->run(e->programs[(size_t)program].get());
    });
}

namespace {
int disassemble_into(br_env_t* e, const char* text, bool fused, char* out, size_t out_bytes);
}

int br_env_disassemble(br_env_t* e, const char* text, char* out, size_t out_bytes) {
    return disassemble_into(e, text, false, out, out_bytes);
}

int br_env_disassemble_fused(br_env_t* e, const char* text, char* out, size_t out_bytes) {
    return disassemble_into(e, text, true, out, out_bytes);
}

namespace {
int disassemble_into(br_env_t* e, const char* text, bool fused, char* out, size_t out_bytes) {
    std::string joined;
    const int rc = guarded([&]() {
        for (const std::string& s : e->env->disassemble(text, fused)) {
            joined += s;
            joined += '\n';
        }
    });
    if (rc != 0) return rc;
    if (joined.size() + 1 > out_bytes) return -2;
    memcpy(out, joined.c_str(), joined.size() + 1);
    return 0;
}
}  // namespace

int br_env_change_hash(br_env_t* e, int hash) {
    return guarded([&]() { e->env->change((size_t)hash); });
}

int br_env_current_hash(br_env_t* e) { return (int)e->env->hashes_current(); }

int br_env_set_number(br_env_t* e, const char* name, double value) {
    return guarded([&]() { e->env->hash().set(name, value); });
}

int br_env_set_string(br_env_t* e, const char* name, const char* value) {
    return guarded([&]() { e->env->hash().set(name, std::string(value)); });
}

int br_env_get_number(br_env_t* e, const char* name, double* value) {
    return guarded([&]() {
        Hash::Item item = e->env->hash().find(name);
        if (item.index() != 0) br_panic("value is not a number");
        *value = std::get<0>(item);
    });
}

int br_env_has(br_env_t* e, const char* name) { return e->env->hash().has(name) ? 1 : 0; }

int br_env_stack_size(br_env_t* e) { return (int)e->env->stack().size(); }

int br_env_stack_clear(br_env_t* e) {
    e->env->stack().clear();
    return 0;
}

int br_env_stack_pop_number(br_env_t* e, double* value) {
    return guarded([&]() { *value = e->env->stack().pop_number(); });
}

int br_env_tensor_info(br_env_t* e, const char* name, int* dtype, int* on_device, int* rank, int64_t shape[8],
                       void** data) {
    return guarded([&]() {
        tensor_t t = find_tensor(e, name);
        if (dtype) *dtype = (int)t->dtype();
        if (on_device) *on_device = t->is_cuda() ? 1 : 0;
        if (rank) *rank = (int)t->shape().dim();
        if (shape)
            for (size_t i = 0; i < t->shape().dim() && i < 8; i++) shape[i] = (int64_t)t->shape()[(int)i];
        if (data) *data = t->data();
    });
}

int br_env_tensor_write(br_env_t* e, const char* name, const float* src, int64_t n) {
    return guarded([&]() {
        tensor_t t = find_tensor(e, name);
        br_assert((int64_t)t->items() == n, "tensor_write: element count differs");
        br_assert(t->dtype() != DataType::Int, "tensor_write: use the _i32 variant");
        const size_t bytes = (size_t)n * sizeof(float);
        if (t->is_cpu()) {
            memcpy(t->data(), src, bytes);
            return;
        }
        if (t->dtype() == DataType::Float) {
            BR_HIP_CHECK(br_hip_memcpy_h2d(t->data(), src, bytes, ComputingContext::stream));
        } else {
            void* stage = ComputingContext::scratch(bytes);
            BR_HIP_CHECK(br_hip_memcpy_h2d(stage, src, bytes, ComputingContext::stream));
            BR_HIP_CHECK(br_hip_cast(stage, BR_F32, t->data(), (int)t->dtype(), n, ComputingContext::stream));
        }
        ComputingContext::sync();
    });
}

int br_env_tensor_read(br_env_t* e, const char* name, float* dst, int64_t n) {
    return guarded([&]() {
        tensor_t t = find_tensor(e, name);
        br_assert((int64_t)t->items() == n, "tensor_read: element count differs");
        br_assert(t->dtype() != DataType::Int, "tensor_read: use the _i32 variant");
        const size_t bytes = (size_t)n * sizeof(float);
        if (t->is_cpu()) {
            memcpy(dst, t->data(), bytes);
            return;
        }
        if (t->dtype() == DataType::Float) {
            BR_HIP_CHECK(br_hip_memcpy_d2h(dst, t->data(), bytes, ComputingContext::stream));
        } else {
            void* stage = ComputingContext::scratch(bytes);
            BR_HIP_CHECK(br_hip_cast(t->data(), (int)t->dtype(), stage, BR_F32, n, ComputingContext::stream));
            BR_HIP_CHECK(br_hip_memcpy_d2h(dst, stage, bytes, ComputingContext::stream));
        }
        ComputingContext::sync();
    });
}

int br_env_tensor_write_i32(br_env_t* e, const char* name, const int32_t* src, int64_t n) {
    return guarded([&]() {
        tensor_t t = find_tensor(e, name);
        br_assert(t->is_cpu() && t->dtype() == DataType::Int, "tensor_write_i32: not a cpu int tensor");
        br_assert((int64_t)t->items() >= n, "tensor_write_i32: too many elements");
        memcpy(t->data(), src, (size_t)n * sizeof(int32_t));
    });
}

int br_env_tensor_read_i32(br_env_t* e, const char* name, int32_t* dst, int64_t n) {
    return guarded([&]() {
        tensor_t t = find_tensor(e, name);
        br_assert(t->is_cpu() && t->dtype() == DataType::Int, "tensor_read_i32: not a cpu int tensor");
        br_assert((int64_t)t->items() >= n, "tensor_read_i32: too many elements");
        memcpy(dst, t->data(), (size_t)n * sizeof(int32_t));
    });
}

int br_bloom_model_create(br_env_t* e, int layers, int64_t batch, int64_t tokens, int64_t hidden, int64_t heads,
                          int64_t vocab, float eps, const char* weight_dtype, const char* gemm_precision) {
    return guarded([&]() {
        BloomModelConfig cfg;
        cfg.layers = layers;
        cfg.batch = batch;
        cfg.tokens = tokens;
        cfg.hidden = hidden;
        cfg.heads = heads;
        cfg.vocab = vocab;
        cfg.eps = eps;
        cfg.weight_dtype = weight_dtype ? weight_dtype : "f16";
        cfg.gemm_precision = gemm_precision ? gemm_precision : "f16";
        cfg.fused_attention = e->fused_attention;
        e->trainer.reset(new BloomTrainer(*e->env, cfg));
        e->trainer->create();
    });
}

int br_bloom_model_set_fused_attention(br_env_t* e, int on) {
    return guarded([&]() { e->fused_attention = on != 0; });
}

int br_bloom_model_init(br_env_t* e, uint64_t seed, float std) {
    return guarded([&]() {
        br_assert(e->trainer != nullptr, "br_bloom_model_create has not run");
        e->trainer->init_synthetic(seed, std);
    });
}

int br_bloom_model_step(br_env_t* e, const int32_t* ids, const int32_t* mask, float* loss) {
    return guarded([&]() {
        br_assert(e->trainer != nullptr, "br_bloom_model_create has not run");
        const float l = e->trainer->step(ids, mask);
        if (loss) *loss = l;
    });
}

int br_bloom_model_grad_lift(br_env_t* e, float* lift) {
    return guarded([&]() {
        br_assert(e->trainer != nullptr, "br_bloom_model_create has not run");
        br_assert(lift != nullptr, "br_bloom_model_grad_lift: null output");
        *lift = e->trainer->grad_lift();
    });
}

int br_bloom_model_optimizer_create(br_env_t* e, float lr, float beta1, float beta2, float eps, float weight_decay) {
    return guarded([&]() {
        br_assert(e->trainer != nullptr, "br_bloom_model_create has not run");
        e->trainer->create_optimizer(lr, beta1, beta2, eps, weight_decay);
    });
}

int br_bloom_model_optimizer_step(br_env_t* e) {
    return guarded([&]() {
        br_assert(e->trainer != nullptr, "br_bloom_model_create has not run");
        e->trainer->optimizer_step();
    });
}

int br_bloom_fetch_data(const int32_t* ids, const int32_t* mask, int64_t batch, int64_t tokens, const float* vocab,
                        int64_t hidden, int64_t heads, float* xinput, float* alibi, float* xmask) {
    return guarded([&]() {
        if (vocab && xinput) BloomInput::gather_embeddings(vocab, hidden, ids, batch * tokens, xinput);
        if (alibi) BloomInput::build_alibi(heads, tokens, alibi);
        if (xmask) BloomInput::build_xmask(mask, batch, tokens, xmask);
    });
}

}  // extern "C"
