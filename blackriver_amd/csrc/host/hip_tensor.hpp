// HIPTensor: the MI355X backend of the operator API.
//
// Takes the place of the reference's CUDATensor (blackriver/cuda_tensor.hpp,
// cuda_tensor.cpp): it owns (or borrows, for views) a device pointer and
// implements every operator by calling the br_hip C ABI on the context's one
// stream.  No HIP header is included on this side of the ABI.
//
// Element types: fp32 for everything; fp16 / bf16 for weights and any tensor
// that only feeds matrix products (the MFMA kernels convert fp32 operands on
// load, so fp32 activations and fp16 weights mix freely).
#pragma once

#include "computing.hpp"
#include "runtime.hpp"
#include "tensor.hpp"

namespace br {

void* hip_tensor_alloc(size_t bytes);
void hip_tensor_free(void* p);

template <DataType DT>
struct HIPTensor : public TransformerComputing {
    static_assert(DT == DataType::Float || DT == DataType::F16 || DT == DataType::BF16,
                  "device tensors are fp32, fp16 or bf16");

    explicit HIPTensor(const ShapeType& shape)
        : mem_(hip_tensor_alloc(shape.numel() * DataType_size(DT))), owner_(true) {}
    explicit HIPTensor(void* mem) : mem_(mem), owner_(false) {}
    ~HIPTensor() override {
        if (owner_ && mem_) hip_tensor_free(mem_);
    }

    void* data() { return mem_; }

    ComputingReturn io_dump(tensor_t self) override;
    ComputingReturn io_load(tensor_t self, const char* fileName) override;
    ComputingReturn io_save(tensor_t self, const char* fileName) override;
    ComputingReturn io_nccl_send(tensor_t self, int dst) override;
    ComputingReturn io_nccl_recv(tensor_t self, int src) override;

    ComputingReturn op_zero(tensor_t self) override;
    ComputingReturn op_fill(tensor_t self, float value) override;
    ComputingReturn op_copy(tensor_t self, tensor_t src) override;
    view_result_t op_view(tensor_t self, size_t offset, const std::vector<size_t>& newShape) override;
    ComputingReturn op_add(tensor_t self, tensor_t b, tensor_t c) override;
    ComputingReturn op_linear(tensor_t self, tensor_t w, tensor_t bias, tensor_t y) override;
    ComputingReturn op_layernorm(tensor_t self, tensor_t mean, tensor_t var, tensor_t scale, tensor_t bias, tensor_t y,
                                 float eps) override;
    ComputingReturn op_transpos_0213(tensor_t self, tensor_t y) override;
    ComputingReturn op_qk(tensor_t self, tensor_t k, tensor_t qk) override;
    ComputingReturn op_softmax(tensor_t self, tensor_t out) override;
    ComputingReturn op_attn(tensor_t self, tensor_t v, tensor_t attn) override;
    ComputingReturn op_gelu(tensor_t self, tensor_t dst) override;
    ComputingReturn op_last_logits(tensor_t self, tensor_t mask, tensor_t lm_head, tensor_t output) override;
    loss_result_t op_loss_backward(tensor_t self, tensor_t ids, tensor_t mask, tensor_t lm_head, tensor_t all_logits,
                                   tensor_t x_g, tensor_t lm_head_g) override;
    ComputingReturn op_layernorm_backward(tensor_t self, tensor_t scale, tensor_t bias, tensor_t var, tensor_t y,
                                          tensor_t dscale, tensor_t dbias, tensor_t din, float eps) override;
    ComputingReturn op_linear_backward(tensor_t self, tensor_t x, tensor_t weight, tensor_t bias, tensor_t x_g,
                                       tensor_t weight_g, tensor_t bias_g) override;
    ComputingReturn op_gelu_backward(tensor_t self, tensor_t x, tensor_t x_g) override;
    ComputingReturn op_attn_backward(tensor_t self, tensor_t attn, tensor_t v, tensor_t attn_g, tensor_t v_g) override;
    ComputingReturn op_softmax_backward(tensor_t self, tensor_t out, tensor_t x_g) override;
    ComputingReturn op_softmax_attn_backward(tensor_t self, tensor_t attn, tensor_t v, tensor_t attn_g,
                                             tensor_t v_g) override;
    ComputingReturn op_qk_backward(tensor_t self, tensor_t q, tensor_t k, tensor_t q_g, tensor_t k_g) override;

private:
    void* mem_;
    const bool owner_;
};

// op_gelu_backward(dy, u, du) followed by op_linear_backward(du, x, ...): with a
// 16-bit MFMA type one pass produces du, its 16-bit copy and the bias gradient
// (same bits as the two operators), then the two products run.
ComputingReturn hip_gelu_linear_backward(const tensor_t& dy, const tensor_t& u, const tensor_t& du, const tensor_t& x,
                                         const tensor_t& weight, const tensor_t& bias, const tensor_t& x_g,
                                         const tensor_t& weight_g, const tensor_t& bias_g);
// u = x . w^T + bias, y = gelu(u): op_linear (cuda_tensor.cpp:146-193) followed by
// op_gelu (:400-412).  With 16-bit tensors throughout, one product whose
// epilogue writes both (gelu of the fp32 sum); otherwise the two operators.
ComputingReturn hip_linear_gelu(const tensor_t& x, const tensor_t& w, const tensor_t& bias, const tensor_t& u,
                                const tensor_t& y);
// y += x . w^T + bias: op_linear (cuda_tensor.cpp:146-193) followed by
// op_add(y, ., y) with the addition done in the product's epilogue; the sum is
// formed from the same fp32 values, so the bits equal the two operators'.
ComputingReturn hip_linear_accumulate(const tensor_t& x, const tensor_t& w, const tensor_t& bias, const tensor_t& y);
ComputingReturn hip_linear_residual(const tensor_t& x, const tensor_t& w, const tensor_t& bias,
                                    const tensor_t& residual, const tensor_t& y);
// din = layernorm_backward(...) + residual in one pass where the row kernel
// applies, else the two operators one after the other (din may be residual).
ComputingReturn hip_layernorm_backward_add(const tensor_t& dy, const tensor_t& scale, const tensor_t& bias,
                                           const tensor_t& var, const tensor_t& y, const tensor_t& dscale,
                                           const tensor_t& dbias, const tensor_t& residual, const tensor_t& din,
                                           float eps);
// The same followed by the linear backward whose output gradient is din (x, weight, bias of that layer and its
// three gradients): din's 16-bit image and the bias gradient come out of the LayerNorm kernel.
ComputingReturn hip_layernorm_backward_add_linear_backward(
    const tensor_t& dy, const tensor_t& scale, const tensor_t& bias, const tensor_t& var, const tensor_t& y,
    const tensor_t& dscale, const tensor_t& dbias, const tensor_t& residual, const tensor_t& din, float eps,
    const tensor_t& x, const tensor_t& weight, const tensor_t& lbias, const tensor_t& x_g, const tensor_t& weight_g,
    const tensor_t& bias_g);

}  // namespace br
