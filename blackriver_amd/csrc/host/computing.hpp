// The tensor operator API: the boundary every backend implements.
//
// Signature-for-signature the interface of the reference's
// br::TransformerComputing (blackriver/operators.hpp:20-112) and its return
// codes (operators.hpp:12-18), so code written against the reference's
// operators compiles against this header unchanged.  Each operator receives
// the owning handle as `self` (a TensorType asserts self.get() == this before
// it forwards to its backend) and the other operands by value; every default
// returns OP_TODO_ERROR, which the TensorType wrapper turns into a panic.
#pragma once

#include <memory>
#include <variant>
#include <vector>

namespace br {

struct TensorType;
using tensor_t = std::shared_ptr<TensorType>;

enum ComputingReturn {
    OP_OK = 0,
    OP_TODO_ERROR = -1,    // not implemented for this backend / dtype
    OP_INPUT_ERROR = -2,
    OP_OUTPUT_ERROR = -3,
    OP_ATTR_ERROR = -4,
};

struct TransformerComputing {
    using view_result_t = std::variant<ComputingReturn, tensor_t>;
    using loss_result_t = std::variant<ComputingReturn, float>;

    virtual ~TransformerComputing() = default;

    // ---- storage and transport -------------------------------------------
    // raw little-endian file <-> tensor; file size must match exactly
    virtual ComputingReturn io_load(tensor_t self, const char* fileName) { return OP_TODO_ERROR; }
    virtual ComputingReturn io_save(tensor_t self, const char* fileName) { return OP_TODO_ERROR; }
    // print the first and last (up to) 8 values
    virtual ComputingReturn io_dump(tensor_t self) { return OP_TODO_ERROR; }
    // host-side control-plane transport
    virtual ComputingReturn io_mpi_bcast(tensor_t self, int root) { return OP_TODO_ERROR; }
    virtual ComputingReturn io_mpi_recv(tensor_t self, int source) { return OP_TODO_ERROR; }
    virtual ComputingReturn io_mpi_send(tensor_t self, int dst) { return OP_TODO_ERROR; }
    // device-side point-to-point transport
    virtual ComputingReturn io_nccl_recv(tensor_t self, int source) { return OP_TODO_ERROR; }
    virtual ComputingReturn io_nccl_send(tensor_t self, int dst) { return OP_TODO_ERROR; }

    // ---- plumbing --------------------------------------------------------
    virtual ComputingReturn op_zero(tensor_t self) { return OP_TODO_ERROR; }
    virtual ComputingReturn op_fill(tensor_t self, float value) { return OP_TODO_ERROR; }
    // self <- src (element counts must match; host <-> device allowed)
    virtual ComputingReturn op_copy(tensor_t self, tensor_t src) { return OP_TODO_ERROR; }
    // non-owning window of newShape elements starting at element `offset`
    virtual view_result_t op_view(tensor_t self, size_t offset, const std::vector<size_t>& newShape) {
        return OP_TODO_ERROR;
    }

    // ---- forward operators -----------------------------------------------
    // c = self + b, b broadcast where its extent is 1; c may alias self
    virtual ComputingReturn op_add(tensor_t self, tensor_t b, tensor_t c) { return OP_TODO_ERROR; }
    virtual ComputingReturn op_mul(tensor_t self, tensor_t b, tensor_t c) { return OP_TODO_ERROR; }
    // y[B,T,out] = self[B,T,in] . w[out,in]^T + bias[out]
    virtual ComputingReturn op_linear(tensor_t self, tensor_t w, tensor_t bias, tensor_t y) { return OP_TODO_ERROR; }
    // rows = B*T, cols = hidden; var receives sigma^2 + eps
    virtual ComputingReturn op_layernorm(tensor_t self, tensor_t mean, tensor_t var, tensor_t scale, tensor_t bias,
                                         tensor_t y, float eps) {
        return OP_TODO_ERROR;
    }
    // [s0,s1,s2,s3] -> [s0,s2,s1,s3]
    virtual ComputingReturn op_transpos_0213(tensor_t self, tensor_t y) { return OP_TODO_ERROR; }
    // qk[B,NH,T,T] = self[B,NH,T,HD] . k^T / sqrt(HD)
    virtual ComputingReturn op_qk(tensor_t self, tensor_t k, tensor_t qk) { return OP_TODO_ERROR; }
    // row softmax over the last dimension; out may alias self
    virtual ComputingReturn op_softmax(tensor_t self, tensor_t out) { return OP_TODO_ERROR; }
    // attn[B,NH,T,HD] = self[B,NH,T,T] . v[B,NH,T,HD]
    virtual ComputingReturn op_attn(tensor_t self, tensor_t v, tensor_t attn) { return OP_TODO_ERROR; }
    virtual ComputingReturn op_gelu(tensor_t self, tensor_t dst) { return OP_TODO_ERROR; }
    // logits of the last unmasked token of every sequence
    virtual ComputingReturn op_last_logits(tensor_t self, tensor_t mask, tensor_t lm_head, tensor_t output) {
        return OP_TODO_ERROR;
    }

    // ---- backward operators ----------------------------------------------
    // shift-by-one masked cross entropy through lm_head; returns +mean log-prob,
    // overwrites x_g, accumulates into lm_head_g
    virtual loss_result_t op_loss_backward(tensor_t self, tensor_t ids, tensor_t mask, tensor_t lm_head,
                                           tensor_t all_logits, tensor_t x_g, tensor_t lm_head_g) {
        return OP_TODO_ERROR;
    }
    // self = dy; y is the forward OUTPUT, var what the forward stored
    virtual ComputingReturn op_layernorm_backward(tensor_t self, tensor_t scale, tensor_t bias, tensor_t var,
                                                  tensor_t y, tensor_t dscale, tensor_t dbias, tensor_t din,
                                                  float eps) {
        return OP_TODO_ERROR;
    }
    // self = dy; bias_g, weight_g, x_g are overwritten in that order (x_g may alias x)
    virtual ComputingReturn op_linear_backward(tensor_t self, tensor_t x, tensor_t weight, tensor_t bias, tensor_t x_g,
                                               tensor_t weight_g, tensor_t bias_g) {
        return OP_TODO_ERROR;
    }
    // self = dy; x_g may alias x
    virtual ComputingReturn op_gelu_backward(tensor_t self, tensor_t x, tensor_t x_g) { return OP_TODO_ERROR; }
    // self = dO; attn_g = dO . v^T, v_g = attn^T . dO
    virtual ComputingReturn op_attn_backward(tensor_t self, tensor_t attn, tensor_t v, tensor_t attn_g, tensor_t v_g) {
        return OP_TODO_ERROR;
    }
    // self = dy, out = softmax output
    virtual ComputingReturn op_softmax_backward(tensor_t self, tensor_t out, tensor_t x_g) { return OP_TODO_ERROR; }
    // op_attn_backward followed by op_softmax_backward; attn_g may alias attn
    virtual ComputingReturn op_softmax_attn_backward(tensor_t self, tensor_t attn, tensor_t v, tensor_t attn_g,
                                                     tensor_t v_g) {
        return OP_TODO_ERROR;
    }
    // self = dS; q_g = dS . k / sqrt(HD), k_g = dS^T . q / sqrt(HD)
    virtual ComputingReturn op_qk_backward(tensor_t self, tensor_t q, tensor_t k, tensor_t q_g, tensor_t k_g) {
        return OP_TODO_ERROR;
    }
};

}  // namespace br
