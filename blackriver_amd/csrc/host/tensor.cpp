#include "tensor.hpp"

#include "hip_tensor.hpp"
#include "host_tensor.hpp"

namespace br {

template <typename F>
ComputingReturn TensorType::forward(const tensor_t& self, const char* what, F&& f) {
    br_assert(self.get() == this, "can't be here!");
    const ComputingReturn ret = f(impl());
    if (ret != OP_OK) br_panic(what);
    return ret;
}

TransformerComputing* TensorType::impl() {
    return std::visit([](auto* p) -> TransformerComputing* { return p; }, impl_);
}

void* TensorType::data() {
    return std::visit([](auto* p) -> void* { return p->data(); }, impl_);
}

TensorType::~TensorType() {
    // CPU storage lives in the bump arena and is never released individually;
    // the backend object itself is.
    std::visit([](auto* p) { delete p; }, impl_);
}

std::string TensorType::to_string() {
    std::stringstream ss;
    ss << device_name() << ":" << DataType_name(dtype_) << ":" << marker_ << ":[";
    for (size_t i = 0; i < shape_.dim(); i++) ss << shape_[(int)i] << (i + 1 == shape_.dim() ? "" : " ");
    ss << "]";
    return ss.str();
}

ComputingReturn TensorType::op_zero(tensor_t self) {
    marker_ = 0;
    return forward(self, "zero", [&](auto* b) { return b->op_zero(self); });
}

ComputingReturn TensorType::op_fill(tensor_t self, float value) {
    return forward(self, "fill", [&](auto* b) { return b->op_fill(self, value); });
}

ComputingReturn TensorType::op_copy(tensor_t self, tensor_t src) {
    br_assert(items() == src->items(), "copy must has same size");
    return forward(self, "copy", [&](auto* b) { return b->op_copy(self, src); });
}

// A single 0 in newShape stands for "whatever fits between offset and the end
// of this tensor" (blackriver/tensortype.cpp:28-58).
TensorType::view_result_t TensorType::op_view(tensor_t self, size_t offset, const std::vector<size_t>& wanted) {
    br_assert(self.get() == this, "can't be here!");
    std::vector<size_t> shape = wanted;
    int dynamic = -1;
    size_t fixed = 1;
    for (size_t i = 0; i < shape.size(); i++) {
        if (shape[i] != 0) {
            fixed *= shape[i];
        } else if (dynamic < 0) {
            dynamic = (int)i;
        } else {
            br_panic("dynamic view must has one zero shape");
        }
    }
    if (dynamic >= 0) shape[dynamic] = (items() - offset) / fixed;
    br_assert(offset + ShapeType(shape).numel() <= items(), "view out of shape!");
    auto result = impl()->op_view(self, offset, shape);
    if (result.index() == 0 && std::get<0>(result) != OP_OK) br_panic("view");
    return result;
}

ComputingReturn TensorType::op_add(tensor_t self, tensor_t b, tensor_t c) {
    return forward(self, "add", [&](auto* i) { return i->op_add(self, b, c); });
}

ComputingReturn TensorType::op_mul(tensor_t self, tensor_t b, tensor_t c) {
    return forward(self, "mul", [&](auto* i) { return i->op_mul(self, b, c); });
}

ComputingReturn TensorType::op_linear(tensor_t self, tensor_t w, tensor_t bias, tensor_t y) {
    return forward(self, "linear", [&](auto* i) { return i->op_linear(self, w, bias, y); });
}

ComputingReturn TensorType::op_layernorm(tensor_t self, tensor_t mean, tensor_t var, tensor_t scale, tensor_t bias,
                                         tensor_t y, float eps) {
    return forward(self, "layernorm",
                   [&](auto* i) { return i->op_layernorm(self, mean, var, scale, bias, y, eps); });
}

ComputingReturn TensorType::op_transpos_0213(tensor_t self, tensor_t y) {
    return forward(self, "transpose_0213", [&](auto* i) { return i->op_transpos_0213(self, y); });
}

ComputingReturn TensorType::op_qk(tensor_t self, tensor_t k, tensor_t qk) {
    return forward(self, "qk", [&](auto* i) { return i->op_qk(self, k, qk); });
}

ComputingReturn TensorType::op_softmax(tensor_t self, tensor_t out) {
    return forward(self, "softmax", [&](auto* i) { return i->op_softmax(self, out); });
}

ComputingReturn TensorType::op_attn(tensor_t self, tensor_t v, tensor_t attn) {
    return forward(self, "attn", [&](auto* i) { return i->op_attn(self, v, attn); });
}

ComputingReturn TensorType::op_gelu(tensor_t self, tensor_t dst) {
    return forward(self, "gelu", [&](auto* i) { return i->op_gelu(self, dst); });
}

ComputingReturn TensorType::op_last_logits(tensor_t self, tensor_t mask, tensor_t lm_head, tensor_t output) {
    return forward(self, "last_logits", [&](auto* i) { return i->op_last_logits(self, mask, lm_head, output); });
}

TensorType::loss_result_t TensorType::op_loss_backward(tensor_t self, tensor_t ids, tensor_t mask, tensor_t lm_head,
                                                       tensor_t all_logits, tensor_t x_g, tensor_t lm_head_g) {
    br_assert(self.get() == this, "can't be here!");
    auto result = impl()->op_loss_backward(self, ids, mask, lm_head, all_logits, x_g, lm_head_g);
    if (result.index() == 0 && std::get<0>(result) != OP_OK) br_panic("loss_backward");
    return result;
}

ComputingReturn TensorType::op_layernorm_backward(tensor_t self, tensor_t scale, tensor_t bias, tensor_t var,
                                                  tensor_t y, tensor_t dscale, tensor_t dbias, tensor_t din,
                                                  float eps) {
    return forward(self, "layernorm_backward", [&](auto* i) {
        return i->op_layernorm_backward(self, scale, bias, var, y, dscale, dbias, din, eps);
    });
}

ComputingReturn TensorType::op_linear_backward(tensor_t self, tensor_t x, tensor_t weight, tensor_t bias, tensor_t x_g,
                                               tensor_t weight_g, tensor_t bias_g) {
    return forward(self, "linear_backward",
                   [&](auto* i) { return i->op_linear_backward(self, x, weight, bias, x_g, weight_g, bias_g); });
}

ComputingReturn TensorType::op_gelu_backward(tensor_t self, tensor_t x, tensor_t x_g) {
    return forward(self, "gelu_backward", [&](auto* i) { return i->op_gelu_backward(self, x, x_g); });
}

ComputingReturn TensorType::op_attn_backward(tensor_t self, tensor_t attn, tensor_t v, tensor_t attn_g, tensor_t v_g) {
    return forward(self, "attn_backward", [&](auto* i) { return i->op_attn_backward(self, attn, v, attn_g, v_g); });
}

ComputingReturn TensorType::op_softmax_backward(tensor_t self, tensor_t out, tensor_t x_g) {
    return forward(self, "softmax_backward", [&](auto* i) { return i->op_softmax_backward(self, out, x_g); });
}

ComputingReturn TensorType::op_softmax_attn_backward(tensor_t self, tensor_t attn, tensor_t v, tensor_t attn_g,
                                                     tensor_t v_g) {
    return forward(self, "softmax_attn_backward",
                   [&](auto* i) { return i->op_softmax_attn_backward(self, attn, v, attn_g, v_g); });
}

ComputingReturn TensorType::op_qk_backward(tensor_t self, tensor_t q, tensor_t k, tensor_t q_g, tensor_t k_g) {
    return forward(self, "qk_backward", [&](auto* i) { return i->op_qk_backward(self, q, k, q_g, k_g); });
}

ComputingReturn TensorType::io_load(tensor_t self, const char* fileName) {
    return forward(self, "load", [&](auto* i) { return i->io_load(self, fileName); });
}

ComputingReturn TensorType::io_save(tensor_t self, const char* fileName) {
    return forward(self, "save", [&](auto* i) { return i->io_save(self, fileName); });
}

ComputingReturn TensorType::io_dump(tensor_t self) {
    return forward(self, "dump", [&](auto* i) { return i->io_dump(self); });
}

ComputingReturn TensorType::io_mpi_bcast(tensor_t self, int root) {
    return forward(self, "mpi_bcast", [&](auto* i) { return i->io_mpi_bcast(self, root); });
}

ComputingReturn TensorType::io_mpi_recv(tensor_t self, int source) {
    return forward(self, "mpi_recv", [&](auto* i) { return i->io_mpi_recv(self, source); });
}

ComputingReturn TensorType::io_mpi_send(tensor_t self, int dst) {
    return forward(self, "mpi_send", [&](auto* i) { return i->io_mpi_send(self, dst); });
}

ComputingReturn TensorType::io_nccl_recv(tensor_t self, int source) {
    return forward(self, "nccl_recv", [&](auto* i) { return i->io_nccl_recv(self, source); });
}

ComputingReturn TensorType::io_nccl_send(tensor_t self, int dst) {
    return forward(self, "nccl_send", [&](auto* i) { return i->io_nccl_send(self, dst); });
}

}  // namespace br
