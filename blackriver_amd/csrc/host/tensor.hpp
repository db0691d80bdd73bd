// TensorType: the one tensor handle scripts and operators pass around.
//
// A dense row-major shape, an element type and a pointer to the backend
// object that owns (or borrows) the storage.  Same public surface as the
// reference's br::TensorType / ShapeType / DataType
// (blackriver/tensortype.hpp:16-51, 54-123, 135-317): each operator asserts
// that `self` is this very handle, forwards to the backend and panics on any
// result other than OP_OK.  The device backend is HIPTensor; the accessor and
// factory names keep the word "cuda" because the model scripts create their
// tensors on a device called "cuda".
#pragma once

#include <algorithm>
#include <cstdint>
#include <iostream>
#include <memory>
#include <sstream>
#include <string>
#include <variant>
#include <vector>

#include "common.hpp"
#include "computing.hpp"

namespace br {

// Numbering shared with the kernel library's BR_F32 / BR_BF16 / BR_F16 / BR_I32.
enum DataType {
    Float = 0,
    BF16 = 1,
    F16 = 2,
    Int = 3,
};

inline size_t DataType_size(DataType t) {
    if (t == Float || t == Int) return 4;
    if (t == F16 || t == BF16) return 2;
    br_panic("Can't be here");
}

inline const char* DataType_name(DataType t) {
    switch (t) {
        case Float: return "f32";
        case F16: return "f16";
        case BF16: return "bf16";
        case Int: return "i32";
    }
    br_panic("Can't be here");
}

// Logical shape; numel is cached on first use.
struct ShapeType {
    ShapeType() = delete;
    ShapeType(const std::vector<size_t>& dims) : dims_(dims), numel_(0) {}

    size_t numel() const {
        if (numel_ == 0) {
            numel_ = 1;
            for (size_t d : dims_) numel_ *= d;
        }
        return numel_;
    }
    const std::vector<size_t>& vec() const { return dims_; }
    const size_t* dims() const { return dims_.data(); }
    size_t dim() const { return dims_.size(); }
    size_t operator[](int i) const { return dims_[i]; }
    bool operator==(const ShapeType& o) const { return dims_ == o.dims_; }
    bool operator!=(const ShapeType& o) const { return dims_ != o.dims_; }
    std::string to_string() const {
        std::stringstream ss;
        ss << "[";
        for (size_t d : dims_) ss << d << " ";
        ss << "]";
        return ss.str();
    }

private:
    std::vector<size_t> dims_;
    mutable size_t numel_;
};

template <DataType DT>
struct HostTensor;
template <DataType DT>
struct HIPTensor;
using cpu_float_t = HostTensor<DataType::Float>;
using cpu_int_t = HostTensor<DataType::Int>;
using cuda_float_t = HIPTensor<DataType::Float>;
using cuda_f16_t = HIPTensor<DataType::F16>;
using cuda_bf16_t = HIPTensor<DataType::BF16>;

struct TensorType : public TransformerComputing {
private:
    enum ImplType { CPU_FLOAT, CPU_INT, HIP_FLOAT, HIP_F16, HIP_BF16 };  // order of the variant below
    using TensorImpl = std::variant<cpu_float_t*, cpu_int_t*, cuda_float_t*, cuda_f16_t*, cuda_bf16_t*>;

    template <size_t I>
    std::variant_alternative_t<I, TensorImpl> get(const char* msg) {
        if (impl_.index() != I) br_panic(msg);
        return std::get<I>(impl_);
    }

public:
    TensorType() = delete;
    TensorType(cpu_float_t* t, const ShapeType& s) : shape_(s), dtype_(Float), marker_(0), impl_(t) {}
    TensorType(cpu_int_t* t, const ShapeType& s) : shape_(s), dtype_(Int), marker_(0), impl_(t) {}
    TensorType(cuda_float_t* t, const ShapeType& s) : shape_(s), dtype_(Float), marker_(0), impl_(t) {}
    TensorType(cuda_f16_t* t, const ShapeType& s) : shape_(s), dtype_(F16), marker_(0), impl_(t) {}
    TensorType(cuda_bf16_t* t, const ShapeType& s) : shape_(s), dtype_(BF16), marker_(0), impl_(t) {}
    ~TensorType() override;

    const ShapeType& shape() const { return shape_; }
    const DataType& dtype() const { return dtype_; }
    size_t items() const { return shape_.numel(); }
    size_t impl_index() const { return impl_.index(); }
    int64_t& marker() { return marker_; }  // free for callers to use; op_zero resets it

    cpu_float_t* cpu_float() { return get<CPU_FLOAT>("Cant get cpu_float from a tensor"); }
    cpu_int_t* cpu_int() { return get<CPU_INT>("Cant get cpu_int from a tensor"); }
    cuda_float_t* cuda_float() { return get<HIP_FLOAT>("Cant get cuda_float from a tensor"); }
    cuda_f16_t* cuda_f16() { return get<HIP_F16>("Cant get cuda_f16 from a tensor"); }
    cuda_bf16_t* cuda_bf16() { return get<HIP_BF16>("Cant get cuda_bf16 from a tensor"); }

    // Raw storage pointer whatever the backend (host pointer for CPU tensors,
    // device pointer for HIP tensors).
    void* data();

    bool is_cpu() const { return impl_.index() == CPU_FLOAT || impl_.index() == CPU_INT; }
    bool is_cuda() const { return !is_cpu(); }
    const char* device_name() const { return is_cpu() ? "cpu" : "cuda"; }
    bool same_impl(tensor_t& o) { return impl_index() == o->impl_index(); }
    bool same_dtype(tensor_t& o) { return dtype_ == o->dtype(); }
    bool same_shape(tensor_t& o) { return shape_ == o->shape(); }
    std::string to_string();

    TransformerComputing* impl();

    // TransformerComputing, forwarded to the backend
    ComputingReturn io_load(tensor_t self, const char* fileName) override;
    ComputingReturn io_save(tensor_t self, const char* fileName) override;
    ComputingReturn io_dump(tensor_t self) override;
    ComputingReturn io_mpi_bcast(tensor_t self, int root) override;
    ComputingReturn io_mpi_recv(tensor_t self, int source) override;
    ComputingReturn io_mpi_send(tensor_t self, int dst) override;
    ComputingReturn io_nccl_recv(tensor_t self, int source) override;
    ComputingReturn io_nccl_send(tensor_t self, int dst) override;
    ComputingReturn op_zero(tensor_t self) override;
    ComputingReturn op_fill(tensor_t self, float value) override;
    ComputingReturn op_copy(tensor_t self, tensor_t src) override;
    view_result_t op_view(tensor_t self, size_t offset, const std::vector<size_t>& newShape) override;
    ComputingReturn op_add(tensor_t self, tensor_t b, tensor_t c) override;
    ComputingReturn op_mul(tensor_t self, tensor_t b, tensor_t c) override;
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
    // assert ownership, run `f` on the backend, panic unless it returns OP_OK
    template <typename F>
    ComputingReturn forward(const tensor_t& self, const char* what, F&& f);

    ShapeType shape_;
    const DataType dtype_;
    int64_t marker_;
    TensorImpl impl_;
};

tensor_t create_cuda_float(std::vector<size_t>& shape);
tensor_t create_cuda_f16(std::vector<size_t>& shape);
tensor_t create_cuda_bf16(std::vector<size_t>& shape);
tensor_t create_cpu_float(std::vector<size_t>& shape);
tensor_t create_cpu_int(std::vector<size_t>& shape);

}  // namespace br
