#include "hip_tensor.hpp"

#include <cmath>
#include <cstring>

#include "br_hip.h"
#include "host_tensor.hpp"

namespace br {

void* hip_tensor_alloc(size_t bytes) {
    br_assert(ComputingContext::booted(), "device tensors need ComputingContext::boot() first");
    void* p = nullptr;
    BR_HIP_CHECK(br_hip_malloc(&p, bytes));
    return p;
}

void hip_tensor_free(void* p) {
    // kernels that still use the block may be in flight on the stream
    if (ComputingContext::booted()) ComputingContext::sync();
    BR_HIP_CHECK(br_hip_free(p));
}

namespace {

br_stream_t stream() { return ComputingContext::stream; }

// Negative codes are argument rejections and map one to one onto
// ComputingReturn; positive codes are HIP runtime failures and are fatal.
ComputingReturn done(int code, const char* what) {
    if (code > 0) hip_check_at(what, code, __FILE__, __LINE__);
    return static_cast<ComputingReturn>(code);
}
#define BR_OP(call)                                       \
    do {                                                  \
        ComputingReturn r_ = done((call), #call);         \
        if (r_ != OP_OK) return r_;                       \
    } while (0)

int code(const tensor_t& t) { return static_cast<int>(t->dtype()); }
bool dev(const tensor_t& t) { return t->is_cuda(); }
bool dev_f32(const tensor_t& t) { return t->is_cuda() && t->dtype() == DataType::Float; }

// MFMA element type for a product: a 16-bit operand decides; products of
// fp32-only operands follow the context's policy.
int pick_compute(std::initializer_list<tensor_t> ops) {
    bool f16 = false, bf16 = false;
    for (const auto& t : ops) {
        f16 = f16 || t->dtype() == DataType::F16;
        bf16 = bf16 || t->dtype() == DataType::BF16;
    }
    if (bf16) return BR_GEMM_BF16;
    if (f16) return BR_GEMM_F16;
    return ComputingContext::fp32_gemm_compute;
}

// Small regions at the tail of the 128 MiB workspace, clear of what the
// reduction kernels use at its head.
constexpr size_t kTailBytes = 8u << 20;
char* tail() { return static_cast<char*>(ComputingContext::workspace) + ComputingContext::workspace_size - kTailBytes; }
size_t head_bytes() { return ComputingContext::workspace_size - kTailBytes; }

// Every matrix product of the backend.  With a 16-bit MFMA type the product
// goes through br_hip_gemm_staged: fp32 operands are staged as 16-bit copies
// first, which lets the product run on the direct-to-LDS kernel, and products
// with few output tiles are split along K; fp32 compute goes straight through.
int product(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, float alpha, const void* a, int a_dtype,
            int64_t lda, int64_t stride_a, const void* b, int b_dtype, int64_t ldb, int64_t stride_b, int accumulate,
            void* c, int c_dtype, int64_t ldc, int64_t stride_c, const float* bias, int64_t batch, int compute) {
    void* stream = ComputingContext::stream;
    if (compute == BR_GEMM_F32)
        return br_hip_gemm(trans_a, trans_b, m, n, k, alpha, a, a_dtype, lda, stride_a, b, b_dtype, ldb, stride_b,
                           accumulate, c, c_dtype, ldc, stride_c, bias, batch, compute, stream);
    const size_t need = br_hip_gemm_staged_workspace(trans_a, trans_b, m, n, k, a_dtype, b_dtype, batch);
    void* ws = ComputingContext::gemm_staging(0, need);
    return br_hip_gemm_staged(trans_a, trans_b, m, n, k, alpha, a, a_dtype, lda, stride_a, b, b_dtype, ldb, stride_b,
                              accumulate, c, c_dtype, ldc, stride_c, bias, batch, compute, ws, need, stream);
}

// An operand that several products of one operator read: with a 16-bit MFMA
// type an fp32 operand is converted once here (same rounding as the staged
// GEMM entry point applies), otherwise it is passed through.
struct Operand {
    const void* ptr;
    int dtype;
};
// Factor that takes the backward pass's gradient lift out of a parameter gradient.
float unlift() { return 1.0f / ComputingContext::grad_lift; }

Operand shared_operand(const void* p, int dtype, int64_t items, int compute) {
    if (dtype != BR_F32 || compute == BR_GEMM_F32 || items % 8 != 0) return {p, dtype};
    const int native = compute == BR_GEMM_F16 ? BR_F16 : BR_BF16;
    void* dst = ComputingContext::gemm_staging(1, (size_t)items * 2);
    BR_HIP_CHECK(br_hip_cast(p, BR_F32, dst, native, items, ComputingContext::stream));
    return {dst, native};
}

// The two products of a linear layer's backward once the gradient dy[n,out] is
// available in the products' type: weight_g[out,in] = dy^T . x, then
// x_g[n,in] = dy . W (in that order: x_g may overwrite x).
int linear_backward_products(const Operand& dy, const tensor_t& x, const tensor_t& weight, const tensor_t& x_g,
                             const tensor_t& weight_g, int64_t n, int64_t in, int64_t out, int compute) {
    int rc = product(1, 0, out, in, n, unlift(), dy.ptr, dy.dtype, out, 0, x->data(), code(x), in, 0, 0, weight_g->data(),
                     code(weight_g), in, 0, nullptr, 1, compute);
    if (rc != BR_OK) return rc;
    return product(0, 0, n, in, out, 1.0f, dy.ptr, dy.dtype, out, 0, weight->data(), code(weight), in, 0, 0,
                   x_g->data(), code(x_g), in, 0, nullptr, 1, compute);
}

// fp32 device pointer to a bias vector, converting 16-bit storage on the fly
// into workspace tail slot `slot` (each slot 1 MiB).
const float* bias_f32(const tensor_t& b, int slot) {
    if (b->dtype() == DataType::Float) return static_cast<const float*>(b->data());
    br_assert(b->items() * sizeof(float) <= (1u << 20), "bias vector too long for the conversion slot");
    float* dst = reinterpret_cast<float*>(tail() + (size_t)slot * (1u << 20));
    BR_HIP_CHECK(br_hip_cast(b->data(), code(b), dst, BR_F32, (int64_t)b->items(), stream()));
    return dst;
}

void shape4(const ShapeType& s, int64_t out[4]) {
    // rank <= 4 to rank 4 the way the reference describes tensors to cuDNN
    // (blackriver/cuda_tensor.hpp:39-49)
    const auto& v = s.vec();
    switch (v.size()) {
        case 4: out[0] = v[0]; out[1] = v[1]; out[2] = v[2]; out[3] = v[3]; break;
        case 3: out[0] = v[0]; out[1] = v[1]; out[2] = 1; out[3] = v[2]; break;
        case 2: out[0] = v[0]; out[1] = v[1]; out[2] = 1; out[3] = 1; break;
        case 1: out[0] = 1; out[1] = v[0]; out[2] = 1; out[3] = 1; break;
        default: br_panic("can't convert shape to rank 4");
    }
}

template <typename T>
void print_ends(const std::vector<T>& first, const std::vector<T>& last) {
    std::cout << "--------------------------" << std::endl;
    std::cout << "First " << first.size() << " : ";
    for (auto v : first) std::cout << v << " ";
    std::cout << std::endl;
    std::cout << "Last " << last.size() << " : ";
    for (auto v : last) std::cout << v << " ";
    std::cout << std::endl;
}

}  // namespace

// ------------------------------------------------------------------- io
template <DataType DT>
ComputingReturn HIPTensor<DT>::io_dump(tensor_t self) {
    const size_t n = std::min(self->shape().vec().back(), (size_t)8);
    const size_t items = self->items();
    // convert the two ends to fp32 on the device when stored in 16 bits
    float* stage = reinterpret_cast<float*>(tail());
    const size_t es = DataType_size(DT);
    const char* base = static_cast<const char*>(mem_);
    BR_OP(br_hip_cast(base, (int)DT, stage, BR_F32, (int64_t)n, stream()));
    BR_OP(br_hip_cast(base + (items - n) * es, (int)DT, stage + 8, BR_F32, (int64_t)n, stream()));
    std::vector<float> first(n), last(n);
    BR_OP(br_hip_memcpy_d2h(first.data(), stage, n * sizeof(float), stream()));
    BR_OP(br_hip_memcpy_d2h(last.data(), stage + 8, n * sizeof(float), stream()));
    ComputingContext::sync();
    print_ends(first, last);
    return OP_OK;
}

// Files hold raw fp32; 16-bit tensors are converted on the device.
template <DataType DT>
ComputingReturn HIPTensor<DT>::io_load(tensor_t self, const char* fileName) {
    std::vector<float> src;
    read_data(fileName, src);
    br_assert(src.size() == self->items(), "loaded data must has same size");
    const size_t bytes = src.size() * sizeof(float);
    if (DT == DataType::Float) {
        BR_OP(br_hip_memcpy_h2d(mem_, src.data(), bytes, stream()));
    } else {
        void* stage = ComputingContext::scratch(bytes);
        BR_OP(br_hip_memcpy_h2d(stage, src.data(), bytes, stream()));
        BR_OP(br_hip_cast(stage, BR_F32, mem_, (int)DT, (int64_t)src.size(), stream()));
    }
    ComputingContext::sync();  // `src` goes away when this returns
    return OP_OK;
}

template <DataType DT>
ComputingReturn HIPTensor<DT>::io_save(tensor_t self, const char* fileName) {
    const size_t n = self->items();
    std::vector<float> dst(n);
    if (DT == DataType::Float) {
        BR_OP(br_hip_memcpy_d2h(dst.data(), mem_, n * sizeof(float), stream()));
    } else {
        void* stage = ComputingContext::scratch(n * sizeof(float));
        BR_OP(br_hip_cast(mem_, (int)DT, stage, BR_F32, (int64_t)n, stream()));
        BR_OP(br_hip_memcpy_d2h(dst.data(), stage, n * sizeof(float), stream()));
    }
    ComputingContext::sync();
    std::ofstream out(fileName, std::ios::binary | std::ios::trunc);
    if (!out) return OP_OUTPUT_ERROR;
    out.write(reinterpret_cast<const char*>(dst.data()), n * sizeof(float));
    return out.good() ? OP_OK : OP_OUTPUT_ERROR;
}

// Point-to-point activation hand-off between pipeline stages.  All stages
// live in this process, so the payload goes through the in-process mailbox.
template <DataType DT>
ComputingReturn HIPTensor<DT>::io_nccl_send(tensor_t self, int dst) {
    const size_t bytes = self->items() * DataType_size(DT);
    std::vector<unsigned char> buf(bytes);
    BR_OP(br_hip_memcpy_d2h(buf.data(), mem_, bytes, stream()));
    ComputingContext::sync();
    CollectiveContext::post(CollectiveContext::nccl_rank, dst, buf.data(), bytes);
    return OP_OK;
}

template <DataType DT>
ComputingReturn HIPTensor<DT>::io_nccl_recv(tensor_t self, int src) {
    const size_t bytes = self->items() * DataType_size(DT);
    std::vector<unsigned char> buf(bytes);
    if (!CollectiveContext::take(src, CollectiveContext::nccl_rank, buf.data(), bytes)) return OP_INPUT_ERROR;
    BR_OP(br_hip_memcpy_h2d(mem_, buf.data(), bytes, stream()));
    ComputingContext::sync();
    return OP_OK;
}

// ------------------------------------------------------------- plumbing
template <DataType DT>
ComputingReturn HIPTensor<DT>::op_zero(tensor_t self) {
    // a fill kernel rather than a memset node, so callers may graph-capture it
    BR_OP(br_hip_fill(mem_, (int)DT, 0.0f, (int64_t)self->items(), stream()));
    return OP_OK;
}

template <DataType DT>
ComputingReturn HIPTensor<DT>::op_fill(tensor_t self, float value) {
    BR_OP(br_hip_fill(mem_, (int)DT, value, (int64_t)self->items(), stream()));
    return OP_OK;
}

template <DataType DT>
ComputingReturn HIPTensor<DT>::op_copy(tensor_t self, tensor_t src) {
    const size_t n = self->items();
    if (src->is_cpu()) {
        if (src->dtype() != DataType::Float) return OP_INPUT_ERROR;
        if (DT == DataType::Float) {
            BR_OP(br_hip_memcpy_h2d(mem_, src->data(), n * sizeof(float), stream()));
        } else {
            void* stage = ComputingContext::scratch(n * sizeof(float));
            BR_OP(br_hip_memcpy_h2d(stage, src->data(), n * sizeof(float), stream()));
            BR_OP(br_hip_cast(stage, BR_F32, mem_, (int)DT, (int64_t)n, stream()));
        }
        return OP_OK;
    }
    if (src->dtype() == DT) {
        BR_OP(br_hip_memcpy_d2d(mem_, src->data(), n * DataType_size(DT), stream()));
    } else {
        // storage conversion, e.g. fp32 master weights into fp16 compute copies
        BR_OP(br_hip_cast(src->data(), code(src), mem_, (int)DT, (int64_t)n, stream()));
    }
    return OP_OK;
}

template <DataType DT>
TransformerComputing::view_result_t HIPTensor<DT>::op_view(tensor_t self, size_t offset,
                                                           const std::vector<size_t>& newShape) {
    void* p = static_cast<char*>(mem_) + offset * DataType_size(DT);
    return std::make_shared<TensorType>(new HIPTensor<DT>(p), ShapeType(newShape));
}

// -------------------------------------------------------------- forward
template <DataType DT>
ComputingReturn HIPTensor<DT>::op_add(tensor_t self, tensor_t b, tensor_t c) {
    if (DT == DataType::BF16) return OP_TODO_ERROR;
    if (!dev(b) || b->dtype() != DT) return OP_INPUT_ERROR;
    if (!dev(c) || c->dtype() != DT || c->items() != self->items()) return OP_OUTPUT_ERROR;
    int64_t as[4], bs[4];
    shape4(self->shape(), as);
    shape4(b->shape(), bs);
    BR_OP(br_hip_add_bcast(mem_, b->data(), c->data(), (int)DT, as, bs, stream()));
    return OP_OK;
}

template <DataType DT>
ComputingReturn HIPTensor<DT>::op_linear(tensor_t self, tensor_t w, tensor_t bias, tensor_t y) {
    if (!dev(w) || !dev(bias)) return OP_INPUT_ERROR;
    if (!dev(y)) return OP_OUTPUT_ERROR;
    const int64_t n = (int64_t)(self->shape()[0] * self->shape()[1]);
    const int64_t in = (int64_t)self->shape()[2];
    const int64_t out = (int64_t)w->shape()[0];
    if ((int64_t)w->shape()[1] != in || (int64_t)bias->items() != out) return OP_INPUT_ERROR;
    if ((int64_t)y->items() != n * out) return OP_OUTPUT_ERROR;
    // y[n,out] = x[n,in] . w[out,in]^T + bias, the bias added in the GEMM epilogue
    BR_OP(product(0, 1, n, out, in, 1.0f, mem_, (int)DT, in, 0, w->data(), code(w), in, 0, 0, y->data(), code(y),
                      out, 0, bias_f32(bias, 0), 1, pick_compute({self, w, y})));
    return OP_OK;
}

template <DataType DT>
ComputingReturn HIPTensor<DT>::op_layernorm(tensor_t self, tensor_t mean, tensor_t var, tensor_t scale, tensor_t bias,
                                            tensor_t y, float eps) {
    if (DT != DataType::Float) return OP_TODO_ERROR;
    if (!dev_f32(scale) || !dev_f32(bias)) return OP_INPUT_ERROR;
    if (!dev_f32(y) || !dev_f32(mean) || !dev_f32(var)) return OP_OUTPUT_ERROR;
    const int64_t rows = (int64_t)(self->shape()[0] * self->shape()[1]);
    const int64_t cols = (int64_t)self->shape()[2];
    // mean / var may be larger scratch tensors; only the first `rows` entries are written
    if ((int64_t)mean->items() < rows || (int64_t)var->items() < rows) return OP_OUTPUT_ERROR;
    if ((int64_t)scale->items() != cols || (int64_t)bias->items() != cols) return OP_INPUT_ERROR;
    BR_OP(br_hip_layernorm_fwd(static_cast<const float*>(mem_), static_cast<const float*>(scale->data()),
                               static_cast<const float*>(bias->data()), static_cast<float*>(y->data()),
                               static_cast<float*>(mean->data()), static_cast<float*>(var->data()), rows, cols, eps,
                               stream()));
    return OP_OK;
}

template <DataType DT>
ComputingReturn HIPTensor<DT>::op_transpos_0213(tensor_t self, tensor_t y) {
    if (self->shape().dim() != 4) return OP_INPUT_ERROR;
    if (!dev(y) || y->dtype() != DT || y->items() != self->items() || y->data() == mem_) return OP_OUTPUT_ERROR;
    const auto& s = self->shape();
    BR_OP(br_hip_transpose_0213(mem_, y->data(), (int)DataType_size(DT), (int64_t)s[0], (int64_t)s[1], (int64_t)s[2],
                                (int64_t)s[3], stream()));
    return OP_OK;
}

template <DataType DT>
ComputingReturn HIPTensor<DT>::op_qk(tensor_t self, tensor_t k, tensor_t qk) {
    if (self->shape().dim() != 4 || !dev(k) || k->items() != self->items()) return OP_INPUT_ERROR;
    const auto& s = self->shape();
    const int64_t bh = (int64_t)(s[0] * s[1]), t = (int64_t)s[2], hd = (int64_t)s[3];
    if (!dev(qk) || (int64_t)qk->items() != bh * t * t) return OP_OUTPUT_ERROR;
    const float alpha = (float)(1.0 / sqrt((double)hd));
    BR_OP(product(0, 1, t, t, hd, alpha, mem_, (int)DT, hd, t * hd, k->data(), code(k), hd, t * hd, 0, qk->data(),
                      code(qk), t, t * t, nullptr, bh, pick_compute({self, k})));
    return OP_OK;
}

template <DataType DT>
ComputingReturn HIPTensor<DT>::op_softmax(tensor_t self, tensor_t out) {
    if (DT != DataType::Float) return OP_TODO_ERROR;
    if (!dev_f32(out) || out->items() != self->items()) return OP_OUTPUT_ERROR;
    const int64_t cols = (int64_t)self->shape().vec().back();
    BR_OP(br_hip_softmax_fwd(static_cast<const float*>(mem_), static_cast<float*>(out->data()),
                             (int64_t)self->items() / cols, cols, stream()));
    return OP_OK;
}

template <DataType DT>
ComputingReturn HIPTensor<DT>::op_attn(tensor_t self, tensor_t v, tensor_t attn) {
    if (self->shape().dim() != 4 || v->shape().dim() != 4 || !dev(v)) return OP_INPUT_ERROR;
    const auto& s = self->shape();
    const int64_t bh = (int64_t)(s[0] * s[1]), t = (int64_t)s[2], hd = (int64_t)v->shape()[3];
    if ((int64_t)v->items() != bh * t * hd) return OP_INPUT_ERROR;
    if (!dev(attn) || (int64_t)attn->items() != bh * t * hd) return OP_OUTPUT_ERROR;
    BR_OP(product(0, 0, t, hd, t, 1.0f, mem_, (int)DT, t, t * t, v->data(), code(v), hd, t * hd, 0, attn->data(),
                      code(attn), hd, t * hd, nullptr, bh, pick_compute({self, v})));
    return OP_OK;
}

template <DataType DT>
ComputingReturn HIPTensor<DT>::op_gelu(tensor_t self, tensor_t dst) {
    if (DT == DataType::BF16) return OP_TODO_ERROR;
    if (!dev(dst) || dst->items() != self->items()) return OP_OUTPUT_ERROR;
    if (DT == DataType::Float && (dst->dtype() == DataType::F16 || dst->dtype() == DataType::BF16)) {
        // fp32 activation in, 16-bit operand buffer out
        BR_OP(br_hip_gelu_fwd_f32_to_16(static_cast<const float*>(mem_), dst->data(), code(dst), (int64_t)self->items(),
                                        stream()));
        return OP_OK;
    }
    if (dst->dtype() != DT) return OP_OUTPUT_ERROR;
    BR_OP(br_hip_gelu_fwd(mem_, dst->data(), (int)DT, (int64_t)self->items(), stream()));
    return OP_OK;
}

// Logits of the last real token of every sequence: the first position whose
// successor is padding, or position 0 when the row has no padding at all
// (that is what the reference computes, cuda_tensor.cpp:424-432).
template <DataType DT>
ComputingReturn HIPTensor<DT>::op_last_logits(tensor_t self, tensor_t mask_, tensor_t lm_head, tensor_t output) {
    if (DT != DataType::Float) return OP_TODO_ERROR;
    if (!mask_->is_cpu() || mask_->dtype() != DataType::Int || !dev(lm_head)) return OP_INPUT_ERROR;
    const int64_t batch = (int64_t)self->shape()[0], tokens = (int64_t)self->shape()[1];
    const int64_t hidden = (int64_t)self->shape()[2], vocab = (int64_t)lm_head->shape()[0];
    if (!dev_f32(output) || (int64_t)output->items() < batch * vocab) return OP_OUTPUT_ERROR;
    const int* mask = static_cast<const int*>(mask_->data());
    float* rows = static_cast<float*>(ComputingContext::workspace);
    br_assert((size_t)(batch * hidden) * sizeof(float) <= head_bytes(), "workspace too small for last_logits");
    for (int64_t b = 0; b < batch; b++) {
        const int* m = mask + b * tokens;
        int64_t target = 0;
        for (int64_t i = 0; i < tokens - 1; i++) {
            if (m[i + 1] == 0) {
                target = i;
                break;
            }
        }
        BR_OP(br_hip_memcpy_d2d(rows + b * hidden, static_cast<const float*>(mem_) + (b * tokens + target) * hidden,
                                hidden * sizeof(float), stream()));
    }
    BR_OP(product(0, 1, batch, vocab, hidden, 1.0f, rows, BR_F32, hidden, 0, lm_head->data(), code(lm_head),
                      hidden, 0, 0, output->data(), BR_F32, vocab, 0, nullptr, 1, pick_compute({self, lm_head})));
    return OP_OK;
}

// ------------------------------------------------------------- backward
// Shift-by-one masked cross entropy through the LM head, all on the device.
// Integer part (on the host, from the CPU ids / mask tensors, bit-exact):
//   position t < T-1 carries a loss iff mask[t] and mask[t+1] are non-zero;
//   its label is ids[t+1]; count = number of such positions.
// Float part, per chunk of rows that fits `all_logits`:
//   logits = x . W^T  ->  lse, log p(label)  ->  dlogits in place
//   x_g = dlogits . W          (x_g is zeroed first)
//   lm_head_g += dlogits^T . x
// Returns +mean log-prob of the labels (the reference's sign convention).
template <DataType DT>
TransformerComputing::loss_result_t HIPTensor<DT>::op_loss_backward(tensor_t self, tensor_t ids_, tensor_t mask_,
                                                                    tensor_t lm_head, tensor_t all_logits,
                                                                    tensor_t x_g, tensor_t lm_head_g) {
    if (DT != DataType::Float) return OP_TODO_ERROR;
    if (!ids_->is_cpu() || ids_->dtype() != DataType::Int || !mask_->is_cpu() || mask_->dtype() != DataType::Int)
        return OP_INPUT_ERROR;
    if (!dev(lm_head) || !dev_f32(all_logits)) return OP_INPUT_ERROR;
    if (!dev_f32(x_g) || x_g->items() != self->items()) return OP_OUTPUT_ERROR;
    if (lm_head_g->items() != lm_head->items() || lm_head_g->dtype() != DataType::Float) return OP_OUTPUT_ERROR;

    const int64_t batch = (int64_t)self->shape()[0], tokens = (int64_t)self->shape()[1];
    const int64_t hidden = (int64_t)self->shape()[2], vocab = (int64_t)lm_head->shape()[0];
    const int64_t n = batch * tokens;
    if ((int64_t)ids_->items() < n || (int64_t)mask_->items() < n) return OP_INPUT_ERROR;
    const int64_t cap = (int64_t)all_logits->items() / vocab;
    br_assert(cap >= 1, " logits workspace is not enough !");

    const int* ids = static_cast<const int*>(ids_->data());
    const int* mask = static_cast<const int*>(mask_->data());
    std::vector<int32_t> labels(n, -100), keep(n, 0);
    int64_t count = 0;
    for (int64_t b = 0; b < batch; b++) {
        for (int64_t t = 0; t + 1 < tokens; t++) {
            const int64_t i = b * tokens + t;
            if (mask[i] != 0 && mask[i + 1] != 0) {
                labels[i] = ids[i + 1];
                keep[i] = 1;
                count++;
            }
        }
    }
    const float scale = count > 0 ? 1.0f / (float)count : 0.0f;
    const int compute = pick_compute({self, lm_head});
    if (ComputingContext::grad_lift_auto) {
        // 16 * 2^ceil(log2(count)): undoes the mean over loss positions and leaves
        // four more bits of headroom below; no lift for fp32 products
        float lift_now = 1.0f;
        if (compute != BR_GEMM_F32 && count > 0) {
            lift_now = 16.0f;
            while (lift_now < 16.0f * (float)count) lift_now *= 2.0f;
        }
        ComputingContext::grad_lift = lift_now;
    }
    const float grad_lift = ComputingContext::grad_lift;   // x_g leaves carrying this factor

    // small per-row arrays in the workspace tail (slots 2..7)
    br_assert((size_t)n * 4 * sizeof(float) + 64 <= 6u * (1u << 20), "too many rows for the loss scratch");
    char* t0 = tail() + 2u * (1u << 20);
    int32_t* d_labels = reinterpret_cast<int32_t*>(t0);
    int32_t* d_keep = d_labels + n;
    float* d_lse = reinterpret_cast<float*>(d_keep + n);
    float* d_logp = d_lse + n;
    float* d_result = d_logp + n;
    BR_OP(br_hip_memcpy_h2d(d_labels, labels.data(), n * sizeof(int32_t), stream()));
    BR_OP(br_hip_memcpy_h2d(d_keep, keep.data(), n * sizeof(int32_t), stream()));

    // weight gradient target: the tensor itself when it lives on the device,
    // otherwise a zeroed device staging buffer that is added into the CPU
    // tensor at the end
    float* d_wg = nullptr;
    void* staging = nullptr;
    if (lm_head_g->is_cuda()) {
        d_wg = static_cast<float*>(lm_head_g->data());
    } else {
        staging = hip_tensor_alloc((size_t)(vocab * hidden) * sizeof(float));
        d_wg = static_cast<float*>(staging);
        BR_OP(br_hip_fill(d_wg, BR_F32, 0.f, vocab * hidden, stream()));
    }

    BR_OP(br_hip_fill(x_g->data(), BR_F32, 0.f, n * hidden, stream()));
    const float* x = static_cast<const float*>(mem_);
    float* dx = static_cast<float*>(x_g->data());
    float* logits = static_cast<float*>(all_logits->data());
    // lm_head_g is accumulated into, as the reference does; a driver that would
    // zero it right before (ComputingContext::loss_head_overwrite) gets the
    // first chunk written instead of added, which saves clearing and re-reading
    // a [vocab, hidden] tensor
    // (a host-resident gradient goes through the zeroed staging buffer either way;
    // in overwrite mode the staged sum is assigned to it instead of added)
    const bool overwrite_host = ComputingContext::loss_head_overwrite && !lm_head_g->is_cuda();
    bool overwrite = ComputingContext::loss_head_overwrite && lm_head_g->is_cuda();
    if (overwrite && count == 0) BR_OP(br_hip_fill(d_wg, BR_F32, 0.f, vocab * hidden, stream()));
    for (int64_t r0 = 0; r0 < n && count > 0; r0 += cap) {
        const int64_t rows = std::min(cap, n - r0);
        bool any = false;
        for (int64_t r = r0; r < r0 + rows; r++) any = any || keep[r] != 0;
        if (!any) continue;  // nothing but zero gradients in this chunk
        BR_OP(product(0, 1, rows, vocab, hidden, 1.0f, x + r0 * hidden, BR_F32, hidden, 0, lm_head->data(),
                          code(lm_head), hidden, 0, 0, logits, BR_F32, vocab, 0, nullptr, 1, compute));
        BR_OP(br_hip_logsoftmax_nll_fwd(logits, d_labels + r0, d_keep + r0, d_lse + r0, d_logp + r0, d_result, rows,
                                        vocab, stream()));
        // dlogits.  With fp32 products it is scaled by 1/count in place, as the
        // reference does.  With 16-bit products the stored operand leaves 1/count
        // out (p/count would fall below fp16's smallest subnormal at a real
        // vocabulary size) and, for fp16, carries an exact factor 2^14 that lifts
        // probabilities down to 4e-12 into range (|softmax - onehot| <= 1, so no
        // overflow); both factors go into the products' alpha.
        Operand dl{logits, BR_F32};
        float alpha = 1.0f;
        if (compute == BR_GEMM_F32) {
            BR_OP(br_hip_logsoftmax_nll_bwd(logits, d_labels + r0, d_keep + r0, d_lse + r0, logits, BR_F32, scale,
                                            rows, vocab, stream()));
        } else {
            const int native = compute == BR_GEMM_F16 ? BR_F16 : BR_BF16;
            const float lift = compute == BR_GEMM_F16 ? 16384.0f : 1.0f;
            alpha = scale / lift;
            if ((rows * vocab) % 8 == 0) {
                void* dl16 = ComputingContext::gemm_staging(1, (size_t)(rows * vocab) * 2);
                BR_OP(br_hip_logsoftmax_nll_bwd(logits, d_labels + r0, d_keep + r0, d_lse + r0, dl16, native, lift,
                                                rows, vocab, stream()));
                dl = Operand{dl16, native};
            } else {
                BR_OP(br_hip_logsoftmax_nll_bwd(logits, d_labels + r0, d_keep + r0, d_lse + r0, logits, BR_F32, lift,
                                                rows, vocab, stream()));
                dl = shared_operand(logits, BR_F32, rows * vocab, compute);
            }
        }
        BR_OP(product(0, 0, rows, hidden, vocab, alpha * grad_lift, dl.ptr, dl.dtype, vocab, 0, lm_head->data(), code(lm_head),
                      hidden, 0, 0, dx + r0 * hidden, BR_F32, hidden, 0, nullptr, 1, compute));
        BR_OP(product(1, 0, vocab, hidden, rows, alpha, dl.ptr, dl.dtype, vocab, 0, x + r0 * hidden, BR_F32, hidden,
                      0, overwrite ? 0 : 1, d_wg, BR_F32, hidden, 0, nullptr, 1, compute));
        overwrite = false;
    }
    // overwrite mode with no chunk carrying a label at all: the gradient is zero
    if (overwrite && count > 0) BR_OP(br_hip_fill(d_wg, BR_F32, 0.f, vocab * hidden, stream()));

    // sum of log p(label) in fp64 on the host, as the reference accumulates it
    std::vector<float> logp(n, 0.f);
    if (count > 0) BR_OP(br_hip_memcpy_d2h(logp.data(), d_logp, n * sizeof(float), stream()));
    ComputingContext::sync();
    double total = 0.0;
    for (int64_t i = 0; i < n; i++)
        if (keep[i]) total += (double)logp[i];

    if (staging) {
        float* host_g = static_cast<float*>(lm_head_g->data());
        float* bounce = static_cast<float*>(ComputingContext::host_workspace);
        const size_t per = ComputingContext::workspace_size / sizeof(float);
        const size_t all = (size_t)(vocab * hidden);
        for (size_t off = 0; off < all; off += per) {
            const size_t cnt = std::min(per, all - off);
            BR_OP(br_hip_memcpy_d2h(bounce, d_wg + off, cnt * sizeof(float), stream()));
            ComputingContext::sync();
            if (overwrite_host) {
                memcpy(host_g + off, bounce, cnt * sizeof(float));
            } else {
                for (size_t i = 0; i < cnt; i++) host_g[off + i] += bounce[i];
            }
        }
        hip_tensor_free(staging);
    }

    const float ret = count > 0 ? (float)(total / (double)count) : 0.0f;
    ComputingContext::last_loss = ret;
    if (ComputingContext::echo_loss) std::cout << "#################  " << count << " " << ret << std::endl;
    return ret;
}

template <DataType DT>
ComputingReturn HIPTensor<DT>::op_layernorm_backward(tensor_t self, tensor_t scale, tensor_t bias, tensor_t var,
                                                     tensor_t y, tensor_t dscale, tensor_t dbias, tensor_t din,
                                                     float eps) {
    if (DT != DataType::Float) return OP_TODO_ERROR;
    if (!dev_f32(scale) || !dev_f32(bias) || !dev_f32(var) || !dev_f32(y)) return OP_INPUT_ERROR;
    if (!dev_f32(dscale) || !dev_f32(dbias) || !dev_f32(din)) return OP_OUTPUT_ERROR;
    const int64_t rows = (int64_t)(self->shape()[0] * self->shape()[1]);
    const int64_t cols = (int64_t)self->shape()[2];
    if (y->items() != self->items() || (int64_t)var->items() < rows) return OP_INPUT_ERROR;
    if (din->items() != self->items() || (int64_t)dscale->items() != cols || (int64_t)dbias->items() != cols)
        return OP_OUTPUT_ERROR;
    const size_t need = br_hip_layernorm_bwd_workspace(rows, cols);
    void* ws = need <= head_bytes() ? ComputingContext::workspace : ComputingContext::scratch(need);
    BR_OP(br_hip_layernorm_bwd(static_cast<const float*>(mem_), static_cast<const float*>(y->data()),
                               static_cast<const float*>(scale->data()), static_cast<const float*>(bias->data()),
                               static_cast<const float*>(var->data()), static_cast<float*>(dscale->data()),
                               static_cast<float*>(dbias->data()), static_cast<float*>(din->data()), rows, cols, eps,
                               unlift(), ws, need, stream()));
    return OP_OK;
}

// self = dy[n,out].  Order matters: the bias and weight gradients read x
// before the input gradient may overwrite it (x_g aliases x in the scripts).
template <DataType DT>
ComputingReturn HIPTensor<DT>::op_linear_backward(tensor_t self, tensor_t x, tensor_t weight, tensor_t bias,
                                                  tensor_t x_g, tensor_t weight_g, tensor_t bias_g) {
    if (!dev(x) || !dev(weight)) return OP_INPUT_ERROR;
    if (!dev(x_g) || !dev(weight_g) || !dev_f32(bias_g)) return OP_OUTPUT_ERROR;
    const int64_t n = (int64_t)(self->shape()[0] * self->shape()[1]);
    const int64_t out = (int64_t)self->shape()[2], in = (int64_t)x->shape()[2];
    if ((int64_t)x->items() != n * in || (int64_t)weight->items() != out * in) return OP_INPUT_ERROR;
    if ((int64_t)x_g->items() != n * in || (int64_t)weight_g->items() != out * in || (int64_t)bias_g->items() != out)
        return OP_OUTPUT_ERROR;
    const int compute = pick_compute({self, x, weight});
    // bias_g[o] = sum_n dy[n,o]
    const size_t need = br_hip_colsum_workspace(n, out);
    void* ws = need <= head_bytes() ? ComputingContext::workspace : ComputingContext::scratch(need);
    Operand dy{mem_, (int)DT};
    if (DT == DataType::Float && compute != BR_GEMM_F32 && out % 8 == 0) {
        // one pass over dy: its column sums and the 16-bit copy both products read
        const int native = compute == BR_GEMM_F16 ? BR_F16 : BR_BF16;
        void* dy16 = ComputingContext::gemm_staging(1, (size_t)(n * out) * 2);
        BR_OP(br_hip_colsum_cast(static_cast<const float*>(mem_), static_cast<float*>(bias_g->data()), dy16, native, n,
                                 out, unlift(), ws, need, stream()));
        dy = Operand{dy16, native};
    } else {
        BR_OP(br_hip_colsum(mem_, (int)DT, static_cast<float*>(bias_g->data()), n, out, unlift(), ws, need, stream()));
        dy = shared_operand(mem_, (int)DT, n * out, compute);
    }
    BR_OP(linear_backward_products(dy, x, weight, x_g, weight_g, n, in, out, compute));
    return OP_OK;
}

template <DataType DT>
ComputingReturn HIPTensor<DT>::op_gelu_backward(tensor_t self, tensor_t x, tensor_t x_g) {
    if (DT == DataType::BF16) return OP_TODO_ERROR;
    if (!dev(x) || x->dtype() != DT || x->items() != self->items()) return OP_INPUT_ERROR;
    if (!dev(x_g) || x_g->dtype() != DT || x_g->items() != self->items()) return OP_OUTPUT_ERROR;
    BR_OP(br_hip_gelu_bwd(mem_, x->data(), x_g->data(), (int)DT, (int64_t)self->items(), stream()));
    return OP_OK;
}

namespace {
struct AttnDims {
    int64_t bh, t, hd;
};
bool attn_dims(const tensor_t& d_o, const tensor_t& attn, const tensor_t& v, AttnDims& d) {
    if (d_o->shape().dim() != 4) return false;
    const auto& s = d_o->shape();
    d.bh = (int64_t)(s[0] * s[1]);
    d.t = (int64_t)s[2];
    d.hd = (int64_t)s[3];
    return (int64_t)attn->items() == d.bh * d.t * d.t && (int64_t)v->items() == d.bh * d.t * d.hd;
}
}  // namespace

// self = dO[B,NH,T,HD]:  v_g = P^T . dO,  attn_g = dO . V^T
template <DataType DT>
ComputingReturn HIPTensor<DT>::op_attn_backward(tensor_t self, tensor_t attn, tensor_t v, tensor_t attn_g,
                                                tensor_t v_g) {
    AttnDims d;
    if (!dev(attn) || !dev(v) || !attn_dims(self, attn, v, d)) return OP_INPUT_ERROR;
    if (!dev(attn_g) || !dev(v_g) || attn_g->items() != attn->items() || v_g->items() != v->items())
        return OP_OUTPUT_ERROR;
    const int compute = pick_compute({self, attn, v});
    const Operand d_o = shared_operand(mem_, (int)DT, d.bh * d.t * d.hd, compute);
    BR_OP(product(1, 0, d.t, d.hd, d.t, 1.0f, attn->data(), code(attn), d.t, d.t * d.t, d_o.ptr, d_o.dtype, d.hd,
                  d.t * d.hd, 0, v_g->data(), code(v_g), d.hd, d.t * d.hd, nullptr, d.bh, compute));
    BR_OP(product(0, 1, d.t, d.t, d.hd, 1.0f, d_o.ptr, d_o.dtype, d.hd, d.t * d.hd, v->data(), code(v), d.hd,
                  d.t * d.hd, 0, attn_g->data(), code(attn_g), d.t, d.t * d.t, nullptr, d.bh, compute));
    return OP_OK;
}

template <DataType DT>
ComputingReturn HIPTensor<DT>::op_softmax_backward(tensor_t self, tensor_t out, tensor_t x_g) {
    if (DT != DataType::Float) return OP_TODO_ERROR;
    if (!dev_f32(out) || out->items() != self->items()) return OP_INPUT_ERROR;
    if (!dev(x_g) || x_g->items() != self->items()) return OP_OUTPUT_ERROR;
    const int64_t cols = (int64_t)self->shape().vec().back();
    const int64_t rows = (int64_t)self->items() / cols;
    const float* dy = static_cast<const float*>(mem_);
    const float* y = static_cast<const float*>(out->data());
    if (x_g->dtype() != DataType::Float) {
        // a 16-bit gradient for the score products: written directly when the
        // kernel can, otherwise fp32 into scratch memory and converted
        const int rc = br_hip_softmax_bwd_to16(dy, y, x_g->data(), code(x_g), rows, cols, stream());
        if (rc == BR_ERR_TODO) {
            float* tmp = static_cast<float*>(ComputingContext::scratch(self->items() * sizeof(float)));
            BR_OP(br_hip_softmax_bwd(dy, y, tmp, rows, cols, stream()));
            BR_OP(br_hip_cast(tmp, BR_F32, x_g->data(), code(x_g), (int64_t)self->items(), stream()));
        } else {
            BR_OP(rc);
        }
        return OP_OK;
    }
    BR_OP(br_hip_softmax_bwd(dy, y, static_cast<float*>(x_g->data()), rows, cols, stream()));
    return OP_OK;
}

// The two ops above in one: dP is staged in scratch memory so that attn_g may
// alias attn (it does in the scripts): dS = P o (dP - rowsum(dP o P)) is then
// written over P row by row, each row read completely before it is replaced.
template <DataType DT>
ComputingReturn HIPTensor<DT>::op_softmax_attn_backward(tensor_t self, tensor_t attn, tensor_t v, tensor_t attn_g,
                                                        tensor_t v_g) {
    AttnDims d;
    if (!dev_f32(attn) || !dev(v) || !attn_dims(self, attn, v, d)) return OP_INPUT_ERROR;
    if (!dev_f32(attn_g) || !dev(v_g) || attn_g->items() != attn->items() || v_g->items() != v->items())
        return OP_OUTPUT_ERROR;
    const int compute = pick_compute({self, attn, v});
    const Operand d_o = shared_operand(mem_, (int)DT, d.bh * d.t * d.hd, compute);
    BR_OP(product(1, 0, d.t, d.hd, d.t, 1.0f, attn->data(), code(attn), d.t, d.t * d.t, d_o.ptr, d_o.dtype, d.hd,
                  d.t * d.hd, 0, v_g->data(), code(v_g), d.hd, d.t * d.hd, nullptr, d.bh, compute));
    float* dp = static_cast<float*>(ComputingContext::scratch((size_t)(d.bh * d.t * d.t) * sizeof(float)));
    BR_OP(product(0, 1, d.t, d.t, d.hd, 1.0f, d_o.ptr, d_o.dtype, d.hd, d.t * d.hd, v->data(), code(v), d.hd,
                  d.t * d.hd, 0, dp, BR_F32, d.t, d.t * d.t, nullptr, d.bh, compute));
    BR_OP(br_hip_softmax_bwd(dp, static_cast<const float*>(attn->data()), static_cast<float*>(attn_g->data()),
                             d.bh * d.t, d.t, stream()));
    return OP_OK;
}

// self = dS[B,NH,T,T]:  q_g = dS . K / sqrt(HD),  k_g = dS^T . Q / sqrt(HD)
template <DataType DT>
ComputingReturn HIPTensor<DT>::op_qk_backward(tensor_t self, tensor_t q, tensor_t k, tensor_t q_g, tensor_t k_g) {
    if (q->shape().dim() != 4 || !dev(q) || !dev(k) || k->items() != q->items()) return OP_INPUT_ERROR;
    const auto& s = q->shape();
    const int64_t bh = (int64_t)(s[0] * s[1]), t = (int64_t)s[2], hd = (int64_t)s[3];
    if ((int64_t)self->items() != bh * t * t) return OP_INPUT_ERROR;
    if (!dev(q_g) || !dev(k_g) || q_g->items() != q->items() || k_g->items() != q->items()) return OP_OUTPUT_ERROR;
    const float alpha = (float)(1.0 / sqrt((double)hd));
    const int compute = pick_compute({self, q, k});
    const Operand ds = shared_operand(mem_, (int)DT, bh * t * t, compute);
    BR_OP(product(0, 0, t, hd, t, alpha, ds.ptr, ds.dtype, t, t * t, k->data(), code(k), hd, t * hd, 0, q_g->data(),
                  code(q_g), hd, t * hd, nullptr, bh, compute));
    BR_OP(product(1, 0, t, hd, t, alpha, ds.ptr, ds.dtype, t, t * t, q->data(), code(q), hd, t * hd, 0, k_g->data(),
                  code(k_g), hd, t * hd, nullptr, bh, compute));
    return OP_OK;
}

ComputingReturn hip_gelu_linear_backward(const tensor_t& dy, const tensor_t& u, const tensor_t& du, const tensor_t& x,
                                         const tensor_t& weight, const tensor_t& bias, const tensor_t& x_g,
                                         const tensor_t& weight_g, const tensor_t& bias_g) {
    bool fast = dev_f32(dy) && dev_f32(u) && dev_f32(du) && dev(x) && dev(weight) && dev(x_g) && dev(weight_g) &&
                dev_f32(bias_g) && du->shape().dim() == 3 && x->shape().dim() == 3 && u->items() == dy->items() &&
                du->items() == dy->items();
    if (fast) {
        const int64_t n = (int64_t)(du->shape()[0] * du->shape()[1]);
        const int64_t out = (int64_t)du->shape()[2], in = (int64_t)x->shape()[2];
        const int compute = pick_compute({du, x, weight});
        fast = compute != BR_GEMM_F32 && out % 8 == 0 && (int64_t)x->items() == n * in &&
               (int64_t)weight->items() == out * in && (int64_t)x_g->items() == n * in &&
               (int64_t)weight_g->items() == out * in && (int64_t)bias_g->items() == out;
        if (fast) {
            const int native = compute == BR_GEMM_F16 ? BR_F16 : BR_BF16;
            const size_t need = br_hip_colsum_workspace(n, out);
            void* ws = need <= head_bytes() ? ComputingContext::workspace : ComputingContext::scratch(need);
            void* dy16 = ComputingContext::gemm_staging(1, (size_t)(n * out) * 2);
            const int rc = br_hip_gelu_bwd_colsum_cast(
                static_cast<const float*>(dy->data()), static_cast<const float*>(u->data()),
                static_cast<float*>(du->data()), static_cast<float*>(bias_g->data()), dy16, native, n, out, unlift(), ws,
                need, stream());
            if (rc != BR_ERR_TODO) {
                BR_OP(rc);
                BR_OP(linear_backward_products(Operand{dy16, native}, x, weight, x_g, weight_g, n, in, out, compute));
                return OP_OK;
            }
        }
    }
    // everything already in the products' 16-bit type (the 4h activation and its gradient kept in the
    // products' type): one pass gives du and the bias gradient, du is the
    // products' operand as it stands
    const DataType gdt = dy->dtype();
    const bool half = dev(dy) && dev(u) && dev(du) && (gdt == DataType::F16 || gdt == DataType::BF16) &&
                      u->dtype() == gdt && du->dtype() == gdt && dev(x) && dev(weight) && dev(x_g) && dev(weight_g) &&
                      dev_f32(bias_g) && du->shape().dim() == 3 && x->shape().dim() == 3 &&
                      u->items() == dy->items() && du->items() == dy->items();
    if (half) {
        const int64_t n = (int64_t)(du->shape()[0] * du->shape()[1]);
        const int64_t out = (int64_t)du->shape()[2], in = (int64_t)x->shape()[2];
        const int compute = pick_compute({du, x, weight});
        const int native = compute == BR_GEMM_F16 ? BR_F16 : compute == BR_GEMM_BF16 ? BR_BF16 : BR_F32;
        if (native == (int)gdt && out % 8 == 0 && (int64_t)x->items() == n * in && (int64_t)weight->items() == out * in &&
            (int64_t)x_g->items() == n * in && (int64_t)weight_g->items() == out * in &&
            (int64_t)bias_g->items() == out) {
            const size_t need = br_hip_bias_gelu_bwd_workspace(n, out);
            void* ws = need <= head_bytes() ? ComputingContext::workspace : ComputingContext::scratch(need);
            BR_OP(br_hip_bias_gelu_bwd(dy->data(), u->data(), nullptr, du->data(), static_cast<float*>(bias_g->data()),
                                       native, n, out, unlift(), ws, need, stream()));
            BR_OP(linear_backward_products(Operand{du->data(), native}, x, weight, x_g, weight_g, n, in, out, compute));
            return OP_OK;
        }
    }
    ComputingReturn r = dy->op_gelu_backward(dy, u, du);
    if (r != OP_OK) return r;
    return du->op_linear_backward(du, x, weight, bias, x_g, weight_g, bias_g);
}

ComputingReturn hip_linear_gelu(const tensor_t& x, const tensor_t& w, const tensor_t& bias, const tensor_t& u,
                                const tensor_t& y) {
    if (!dev(x) || !dev(w) || !dev(bias) || x->shape().dim() != 3) return OP_INPUT_ERROR;
    if (!dev(u) || !dev(y) || u->items() != y->items() || u->data() == y->data()) return OP_OUTPUT_ERROR;
    const int64_t n = (int64_t)(x->shape()[0] * x->shape()[1]);
    const int64_t in = (int64_t)x->shape()[2];
    const int64_t out = (int64_t)w->shape()[0];
    if ((int64_t)w->shape()[1] != in || (int64_t)bias->items() != out) return OP_INPUT_ERROR;
    if ((int64_t)u->items() != n * out) return OP_OUTPUT_ERROR;
    const DataType dt = x->dtype();
    if ((dt == DataType::F16 || dt == DataType::BF16) && w->dtype() == dt && u->dtype() == dt && y->dtype() == dt) {
        const int rc = br_hip_linear_gelu(x->data(), w->data(), bias_f32(bias, 0), u->data(), y->data(), (int)dt, n, out,
                                          in, stream());
        if (rc != BR_ERR_TODO) return done(rc, "br_hip_linear_gelu");
    }
    // the two operators
    ComputingReturn r = x->op_linear(x, w, bias, u);
    if (r != OP_OK) return r;
    return u->op_gelu(u, y);
}

ComputingReturn hip_linear_accumulate(const tensor_t& x, const tensor_t& w, const tensor_t& bias, const tensor_t& y) {
    if (!dev(x) || !dev(w) || !dev(bias) || x->shape().dim() != 3) return OP_INPUT_ERROR;
    if (!dev_f32(y)) return OP_OUTPUT_ERROR;
    const int64_t n = (int64_t)(x->shape()[0] * x->shape()[1]);
    const int64_t in = (int64_t)x->shape()[2];
    const int64_t out = (int64_t)w->shape()[0];
    if ((int64_t)w->shape()[1] != in || (int64_t)bias->items() != out) return OP_INPUT_ERROR;
    if ((int64_t)y->items() != n * out) return OP_OUTPUT_ERROR;
    BR_OP(product(0, 1, n, out, in, 1.0f, x->data(), code(x), in, 0, w->data(), code(w), in, 0, 1, y->data(), BR_F32,
                  out, 0, bias_f32(bias, 0), 1, pick_compute({x, w, y})));
    return OP_OK;
}

// y = x . w^T + bias + residual in one product (the residual is read in the epilogue); y may be the residual.
ComputingReturn hip_linear_residual(const tensor_t& x, const tensor_t& w, const tensor_t& bias,
                                    const tensor_t& residual, const tensor_t& y) {
    if (!dev(x) || !dev(w) || !dev(bias) || !dev_f32(residual) || x->shape().dim() != 3) return OP_INPUT_ERROR;
    if (!dev_f32(y)) return OP_OUTPUT_ERROR;
    const int64_t n = (int64_t)(x->shape()[0] * x->shape()[1]);
    const int64_t in = (int64_t)x->shape()[2];
    const int64_t out = (int64_t)w->shape()[0];
    if ((int64_t)w->shape()[1] != in || (int64_t)bias->items() != out || (int64_t)residual->items() != n * out)
        return OP_INPUT_ERROR;
    if ((int64_t)y->items() != n * out) return OP_OUTPUT_ERROR;
    const int compute = pick_compute({x, w, y});
    const size_t need = compute == BR_GEMM_F32 ? 0 : br_hip_gemm_staged_workspace(0, 1, n, out, in, code(x), code(w), 1);
    void* ws = need ? ComputingContext::gemm_staging(0, need) : nullptr;
    BR_OP(br_hip_linear_residual(x->data(), code(x), w->data(), code(w), bias_f32(bias, 0), residual->data(), y->data(),
                                 BR_F32, n, out, in, compute, ws, need, stream()));
    return OP_OK;
}

ComputingReturn hip_layernorm_backward_add(const tensor_t& dy, const tensor_t& scale, const tensor_t& bias,
                                           const tensor_t& var, const tensor_t& y, const tensor_t& dscale,
                                           const tensor_t& dbias, const tensor_t& residual, const tensor_t& din,
                                           float eps) {
    bool fast = dev_f32(dy) && dev_f32(scale) && dev_f32(bias) && dev_f32(var) && dev_f32(y) && dev_f32(dscale) &&
                dev_f32(dbias) && dev_f32(residual) && dev_f32(din) && dy->shape().dim() == 3;
    if (fast) {
        const int64_t rows = (int64_t)(dy->shape()[0] * dy->shape()[1]);
        const int64_t cols = (int64_t)dy->shape()[2];
        fast = y->items() == dy->items() && (int64_t)var->items() >= rows && din->items() == dy->items() &&
               residual->items() == dy->items() && (int64_t)dscale->items() == cols && (int64_t)dbias->items() == cols &&
               (int64_t)scale->items() == cols && (int64_t)bias->items() == cols && din->data() != y->data();
        if (fast) {
            const size_t need = br_hip_layernorm_bwd_workspace(rows, cols);
            void* ws = need <= head_bytes() ? ComputingContext::workspace : ComputingContext::scratch(need);
            const int rc = br_hip_layernorm_bwd_residual(
                static_cast<const float*>(dy->data()), static_cast<const float*>(y->data()),
                static_cast<const float*>(scale->data()), static_cast<const float*>(bias->data()),
                static_cast<const float*>(var->data()), static_cast<const float*>(residual->data()),
                static_cast<float*>(dscale->data()), static_cast<float*>(dbias->data()),
                static_cast<float*>(din->data()), rows, cols, eps, unlift(), ws, need, stream());
            if (rc != BR_ERR_TODO) return done(rc, "br_hip_layernorm_bwd_residual");
        }
    }
    // the two operators; din must then be a buffer of its own
    if (din->data() == residual->data()) return OP_OUTPUT_ERROR;
    ComputingReturn r = dy->op_layernorm_backward(dy, scale, bias, var, y, dscale, dbias, din, eps);
    if (r != OP_OK) return r;
    return din->op_add(din, residual, din);
}

// `op.layernorm_backward_add` followed by the `op.linear_backward` whose dy is the LayerNorm's din: the
// LayerNorm kernel has every row of din in registers, so it also writes the 16-bit image the two products read
// and the partial column sums that make the bias gradient -- the pass over din that op.linear_backward starts
// with does not run.  Anything the fused kernel declines runs as the two operators.
ComputingReturn hip_layernorm_backward_add_linear_backward(
    const tensor_t& dy, const tensor_t& scale, const tensor_t& bias, const tensor_t& var, const tensor_t& y,
    const tensor_t& dscale, const tensor_t& dbias, const tensor_t& residual, const tensor_t& din, float eps,
    const tensor_t& x, const tensor_t& weight, const tensor_t& lbias, const tensor_t& x_g, const tensor_t& weight_g,
    const tensor_t& bias_g) {
    bool fast = dev_f32(dy) && dev_f32(scale) && dev_f32(bias) && dev_f32(var) && dev_f32(y) && dev_f32(dscale) &&
                dev_f32(dbias) && dev_f32(residual) && dev_f32(din) && dy->shape().dim() == 3 && dev(x) &&
                dev(weight) && dev(x_g) && dev(weight_g) && dev_f32(bias_g) && x->shape().dim() == 3 &&
                din->shape().dim() == 3;
    if (fast) {
        const int64_t rows = (int64_t)(dy->shape()[0] * dy->shape()[1]);
        const int64_t cols = (int64_t)dy->shape()[2], in = (int64_t)x->shape()[2];
        const int compute = pick_compute({din, x, weight});
        fast = y->items() == dy->items() && (int64_t)var->items() >= rows && din->items() == dy->items() &&
               residual->items() == dy->items() && (int64_t)dscale->items() == cols && (int64_t)dbias->items() == cols &&
               (int64_t)scale->items() == cols && (int64_t)bias->items() == cols && din->data() != y->data() &&
               compute != BR_GEMM_F32 && cols % 8 == 0 && (int64_t)x->items() == rows * in &&
               (int64_t)weight->items() == cols * in && (int64_t)x_g->items() == rows * in &&
               (int64_t)weight_g->items() == cols * in && (int64_t)bias_g->items() == cols &&
               // the gradients this call writes must not be each other or an input of the products
               bias_g->data() != dscale->data() && bias_g->data() != dbias->data();
        if (fast) {
            const int native = compute == BR_GEMM_F16 ? BR_F16 : BR_BF16;
            const size_t need = br_hip_layernorm_bwd_sums_workspace(rows, cols);
            void* ws = need <= head_bytes() ? ComputingContext::workspace : ComputingContext::scratch(need);
            void* d16 = ComputingContext::gemm_staging(1, (size_t)(rows * cols) * 2);
            const int rc = br_hip_layernorm_bwd_residual_sums(
                static_cast<const float*>(dy->data()), static_cast<const float*>(y->data()),
                static_cast<const float*>(scale->data()), static_cast<const float*>(bias->data()),
                static_cast<const float*>(var->data()), static_cast<const float*>(residual->data()),
                static_cast<float*>(dscale->data()), static_cast<float*>(dbias->data()),
                static_cast<float*>(din->data()), d16, native, static_cast<float*>(bias_g->data()), rows, cols, eps,
                unlift(), ws, need, stream());
            if (rc != BR_ERR_TODO) {
                BR_OP(rc);
                BR_OP(linear_backward_products(Operand{d16, native}, x, weight, x_g, weight_g, rows, in, cols, compute));
                return OP_OK;
            }
        }
    }
    const ComputingReturn r = hip_layernorm_backward_add(dy, scale, bias, var, y, dscale, dbias, residual, din, eps);
    if (r != OP_OK) return r;
    return din->op_linear_backward(din, x, weight, lbias, x_g, weight_g, bias_g);
}

template struct HIPTensor<DataType::Float>;
template struct HIPTensor<DataType::F16>;
template struct HIPTensor<DataType::BF16>;

tensor_t create_cuda_float(std::vector<size_t>& shape_) {
    ShapeType shape(shape_);
    return std::make_shared<TensorType>(new HIPTensor<DataType::Float>(shape), shape);
}

tensor_t create_cuda_f16(std::vector<size_t>& shape_) {
    ShapeType shape(shape_);
    return std::make_shared<TensorType>(new HIPTensor<DataType::F16>(shape), shape);
}

tensor_t create_cuda_bf16(std::vector<size_t>& shape_) {
    ShapeType shape(shape_);
    return std::make_shared<TensorType>(new HIPTensor<DataType::BF16>(shape), shape);
}

}  // namespace br
