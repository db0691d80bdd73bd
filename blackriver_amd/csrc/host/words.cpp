// io.* / op.* word bindings.  Each word pops its operands from the stack,
// last argument on top, and calls the TensorType operator of the same name;
// the stack effects are those of the reference bindings
// (blackriver/nn.cpp:16-337) so the model scripts run unchanged.
#include "words.hpp"

#include <cmath>

#include <vector>

#include "br_hip.h"
#include "hip_tensor.hpp"
#include "runtime.hpp"
#include "tensor.hpp"

namespace br {

namespace {

std::vector<size_t> pop_shape(Stack& stack) {
    std::vector<size_t> shape;
    for (double d : stack.pop_number_list()) shape.push_back((size_t)d);
    return shape;
}

// Pops N tensors; t[0] is the deepest (first pushed), t[N-1] was on top.
template <size_t N>
struct Tensors {
    tensor_t t[N];
    explicit Tensors(Stack& stack) {
        for (size_t i = N; i-- > 0;) t[i] = stack.pop_tensor();
    }
    tensor_t& operator[](size_t i) { return t[i]; }
};

#define BR_WORD(CLS, ...)                                 \
    struct CLS : public NativeWord {                      \
        void run(Stack& stack) override { __VA_ARGS__ }   \
        NWORD_CREATOR_DEFINE_LR(CLS)                      \
    };

// Free-function operators follow the TensorType wrappers' convention: anything
// but OP_OK is fatal.
void op_check_word(ComputingReturn r, const char* what) {
    if (r != OP_OK) br_panic(what);
}

// True when `dst <- src` is the 16-bit device image of the fp32 device tensor
// `produced` (src is that very tensor).
bool copy16_of(const tensor_t& dst, const tensor_t& src, const tensor_t& produced) {
    return dst && src && dst->is_cuda() && (dst->dtype() == DataType::F16 || dst->dtype() == DataType::BF16) &&
           src->is_cuda() && src->dtype() == DataType::Float && src->data() == produced->data() &&
           src->items() == produced->items() && dst->items() == src->items();
}

// ( -- )  wait for everything queued on the compute stream
BR_WORD(Sync, (void)stack; ComputingContext::sync();)

// ( d0 .. dn-1 n device dtype -- tensor )
BR_WORD(Create,
    const std::string dtype = stack.pop_string();
    const std::string device = stack.pop_string();
    auto shape = pop_shape(stack);
    tensor_t t;
    if (device == "cuda" && dtype == "float") t = create_cuda_float(shape);
    else if (device == "cuda" && dtype == "f16") t = create_cuda_f16(shape);
    else if (device == "cuda" && dtype == "bf16") t = create_cuda_bf16(shape);
    else if (device == "cpu" && dtype == "float") t = create_cpu_float(shape);
    else if (device == "cpu" && dtype == "int") t = create_cpu_int(shape);
    else br_panic("Can' be here!");
    stack.push_tensor(t);
)

// ( "f32" | "f16" | "bf16" -- )  MFMA type for products whose operands are all
// stored as fp32 (extension; fp32 is the default and matches the reference)
BR_WORD(GemmPrecision,
    const std::string p = stack.pop_string();
    if (p == "f32" || p == "float") ComputingContext::fp32_gemm_compute = BR_GEMM_F32;
    else if (p == "f16") ComputingContext::fp32_gemm_compute = BR_GEMM_F16;
    else if (p == "bf16") ComputingContext::fp32_gemm_compute = BR_GEMM_BF16;
    else br_panic("op.gemm_precision takes \"f32\", \"f16\" or \"bf16\"");
)

// ( S -- )  gradient lift for the backward pass (extension): S > 0 must be a
// power of two and is used as given; 0 lets op.loss_backward choose it from the
// number of loss positions; 1 (the default) switches it off.
BR_WORD(GradLift,
    const double v = stack.pop_number();
    if (v == 0.0) {
        ComputingContext::grad_lift_auto = true;
        ComputingContext::grad_lift = 1.0f;
    } else {
        int e = 0;
        br_assert(v > 0.0 && std::frexp(v, &e) == 0.5 && v <= 16777216.0 && v >= 1.0 / 16777216.0,
                  "op.grad_lift takes 0 (choose per step) or a power of two");
        ComputingContext::grad_lift_auto = false;
        ComputingContext::grad_lift = (float)v;
    }
)

BR_WORD(Zero, tensor_t t = stack.pop_tensor(); t->op_zero(t);)
// ( tensor value -- )
BR_WORD(Fill, const double v = stack.pop_number(); tensor_t t = stack.pop_tensor(); t->op_fill(t, (float)v);)
// ( tensor offset d0 .. dn-1 n -- view )
BR_WORD(View,
    auto shape = pop_shape(stack);
    const size_t offset = (size_t)stack.pop_number();
    tensor_t t = stack.pop_tensor();
    auto ret = t->op_view(t, offset, shape);
    stack.push_tensor(std::get<1>(ret));
)
// ( dst src -- )
BR_WORD(Copy, Tensors<2> a(stack); a[0]->op_copy(a[0], a[1]);)
// ( x w b y -- )
BR_WORD(Linear, Tensors<4> a(stack); a[0]->op_linear(a[0], a[1], a[2], a[3]);)
// ( x mean var scale bias y eps -- )
BR_WORD(Layernorm,
    const float eps = (float)stack.pop_number();
    Tensors<6> a(stack);
    a[0]->op_layernorm(a[0], a[1], a[2], a[3], a[4], a[5], eps);
)
// ( x y -- )
BR_WORD(Transpos0213, Tensors<2> a(stack); a[0]->op_transpos_0213(a[0], a[1]);)
// ( q k qk -- )
BR_WORD(QueryKey, Tensors<3> a(stack); a[0]->op_qk(a[0], a[1], a[2]);)
// ( a b c -- )
BR_WORD(Add, Tensors<3> a(stack); a[0]->op_add(a[0], a[1], a[2]);)
// ( x out -- )
BR_WORD(Softmax, Tensors<2> a(stack); a[0]->op_softmax(a[0], a[1]);)
// ( s alibi s  s xmask s  s p -- )  the operands of `op.add op.add op.softmax`
// as bloomz-7b/train.words:158-162 strings them together on the attention
// scores.  When they have that shape (one fp32 device tensor [B,NH,T,T] updated
// in place, alibi [1,NH,1,T], xmask [B,1,T,T]) the three passes run as one
// kernel that applies the same operations in the same order (bit-identical);
// anything else runs the three operators one after the other.
// `copy_dst` / `copy_src` (both null, or the operands of an `op.copy` that
// follows): when the copy is a 16-bit image of the softmax output, the fused
// kernel writes it too.
void add_add_softmax(Tensors<8>& a, const tensor_t& copy_dst, const tensor_t& copy_src) {
    auto same = [](const tensor_t& x, const tensor_t& y) { return x->data() == y->data() && x->items() == y->items(); };
    auto f32dev = [](const tensor_t& x) { return x->is_cuda() && x->dtype() == DataType::Float; };
    bool fast = f32dev(a[0]) && f32dev(a[1]) && f32dev(a[4]) && f32dev(a[7]) && a[0]->shape().dim() == 4 &&
                a[1]->shape().dim() == 4 && a[4]->shape().dim() == 4 && same(a[0], a[2]) && same(a[0], a[3]) &&
                same(a[0], a[5]) && same(a[0], a[6]) && a[7]->items() == a[0]->items();
    bool copied = false;
    if (fast) {
        const auto& xs = a[0]->shape();
        const auto& as = a[1]->shape();
        const auto& ms = a[4]->shape();
        fast = as[0] == 1 && as[1] == xs[1] && as[2] == 1 && as[3] == xs[3] && ms[0] == xs[0] && ms[1] == 1 &&
               ms[2] == xs[2] && ms[3] == xs[3];
        if (fast) {
            const float* x = static_cast<const float*>(a[0]->data());
            const float* alibi = static_cast<const float*>(a[1]->data());
            const float* mask = static_cast<const float*>(a[4]->data());
            float* out = static_cast<float*>(a[7]->data());
            if (copy_dst && copy16_of(copy_dst, copy_src, a[7])) {
                const int rc = br_hip_alibi_masked_softmax_fwd_copy16(
                    x, alibi, mask, out, copy_dst->data(), (int)copy_dst->dtype(), (int64_t)xs[0], (int64_t)xs[1],
                    (int64_t)xs[2], (int64_t)xs[3], ComputingContext::stream);
                if (rc != BR_ERR_TODO) {
                    BR_HIP_CHECK(rc);
                    copied = true;
                }
            }
            if (!copied)
                BR_HIP_CHECK(br_hip_alibi_masked_softmax_fwd(x, alibi, mask, out, (int64_t)xs[0], (int64_t)xs[1],
                                                             (int64_t)xs[2], (int64_t)xs[3],
                                                             ComputingContext::stream));
        }
    }
    if (!fast) {
        a[0]->op_add(a[0], a[1], a[2]);
        a[3]->op_add(a[3], a[4], a[5]);
        a[6]->op_softmax(a[6], a[7]);
    }
    if (copy_dst && !copied) copy_dst->op_copy(copy_dst, copy_src);
}
BR_WORD(AddAddSoftmax, Tensors<8> a(stack); add_add_softmax(a, nullptr, nullptr);)
// ( x a x  x m x  x y  dst src -- )  the same followed by `op.copy`
BR_WORD(AddAddSoftmaxCopy,
    Tensors<2> c(stack);
    Tensors<8> a(stack);
    add_add_softmax(a, c[0], c[1]);
)
// ( x mean var scale bias y eps  dst src -- )  `op.layernorm` followed by
// `op.copy`: when the copy is a 16-bit image of y the forward kernel writes
// both; anything else runs the two operators one after the other.
BR_WORD(LayernormCopy,
    Tensors<2> c(stack);
    const float eps = (float)stack.pop_number();
    Tensors<6> a(stack);
    auto f32dev = [](const tensor_t& x) { return x->is_cuda() && x->dtype() == DataType::Float; };
    bool done = false;
    bool fast = copy16_of(c[0], c[1], a[5]) && a[0]->shape().dim() == 3;
    for (size_t i = 0; i < 6; i++) fast = fast && f32dev(a[i]);
    if (fast) {
        const int64_t rows = (int64_t)(a[0]->shape()[0] * a[0]->shape()[1]);
        const int64_t cols = (int64_t)a[0]->shape()[2];
        fast = (int64_t)a[1]->items() >= rows && (int64_t)a[2]->items() >= rows && (int64_t)a[3]->items() == cols &&
               (int64_t)a[4]->items() == cols && a[5]->items() == a[0]->items();
        if (fast) {
            const int rc = br_hip_layernorm_fwd_copy16(
                static_cast<const float*>(a[0]->data()), static_cast<const float*>(a[3]->data()),
                static_cast<const float*>(a[4]->data()), static_cast<float*>(a[5]->data()), c[0]->data(),
                (int)c[0]->dtype(), static_cast<float*>(a[1]->data()), static_cast<float*>(a[2]->data()), rows, cols,
                eps, ComputingContext::stream);
            if (rc != BR_ERR_TODO) {
                BR_HIP_CHECK(rc);
                done = true;
            }
        }
    }
    if (!done) {
        a[0]->op_layernorm(a[0], a[1], a[2], a[3], a[4], a[5], eps);
        c[0]->op_copy(c[0], c[1]);
    }
)
// ( p v out -- )
BR_WORD(Attn, Tensors<3> a(stack); a[0]->op_attn(a[0], a[1], a[2]);)
// ( x out -- )
BR_WORD(Gelu, Tensors<2> a(stack); a[0]->op_gelu(a[0], a[1]);)
// ( x mask lm_head out -- )
BR_WORD(LastLogits, Tensors<4> a(stack); a[0]->op_last_logits(a[0], a[1], a[2], a[3]);)
// ( x ids mask lm_head workspace x_g lm_head_g -- )
BR_WORD(LossBackward, Tensors<7> a(stack); a[0]->op_loss_backward(a[0], a[1], a[2], a[3], a[4], a[5], a[6]);)
// ( x ids mask lm_head workspace x_g lm_head_g -- )  the same with lm_head_g
// overwritten: `'lm_head_g' @ op.zero` followed by op.loss_backward without
// the clearing pass and the re-read of a [vocab, hidden] tensor (extension)
BR_WORD(LossBackwardSet,
    Tensors<7> a(stack);
    // the flag is this call's only, also when the operator leaves by an exception
    struct Overwrite {
        Overwrite() { ComputingContext::loss_head_overwrite = true; }
        ~Overwrite() { ComputingContext::loss_head_overwrite = false; }
    } guard;
    a[0]->op_loss_backward(a[0], a[1], a[2], a[3], a[4], a[5], a[6]);
)
// ( dy scale bias var y dscale dbias din eps -- )
BR_WORD(LayernormBackward,
    const float eps = (float)stack.pop_number();
    Tensors<8> a(stack);
    a[0]->op_layernorm_backward(a[0], a[1], a[2], a[3], a[4], a[5], a[6], a[7], eps);
)
// ( dy x w b x_g w_g b_g -- )
BR_WORD(LinearBackward, Tensors<7> a(stack); a[0]->op_linear_backward(a[0], a[1], a[2], a[3], a[4], a[5], a[6]);)
// ( dy x x_g -- )
BR_WORD(GeluBackward, Tensors<3> a(stack); a[0]->op_gelu_backward(a[0], a[1], a[2]);)
// ( dO attn v attn_g v_g -- )
BR_WORD(AttnBackward, Tensors<5> a(stack); a[0]->op_attn_backward(a[0], a[1], a[2], a[3], a[4]);)
// ( dy out x_g -- )
BR_WORD(SoftmaxBackward, Tensors<3> a(stack); a[0]->op_softmax_backward(a[0], a[1], a[2]);)
// ( dO attn v attn_g v_g -- )
BR_WORD(SoftmaxAttnBackward, Tensors<5> a(stack); a[0]->op_softmax_attn_backward(a[0], a[1], a[2], a[3], a[4]);)
// ( dS q k q_g k_g -- )
BR_WORD(QueryKeyBackward, Tensors<5> a(stack); a[0]->op_qk_backward(a[0], a[1], a[2], a[3], a[4]);)

// Fused attention (no counterpart in the reference, which runs the chain
// op.querykey, op.add, op.add, op.softmax, op.attn and its backward through
// [B, heads, T, T] tensors).  q, k, v, o, dO are 16-bit device tensors laid out
// [B, T, heads, 128] (the projections' own output, no 0213 transposes); only
// q's shape is consulted.  `valid` comes from bloom.valid (sequences padded on
// the right), `alibi` is the table bloom.alibi builds.
struct FlashOperands {
    int64_t batch, tokens, heads, head_dim;
    const int32_t* valid;  // device, [batch]
};
// `valid` is the tensor bloom.valid fills: per sequence the number of leading
// real tokens, int32 values kept in the storage of a 4-byte-element device tensor.
FlashOperands flash_operands(const tensor_t& q, const tensor_t& valid, const tensor_t& alibi) {
    br_assert(q->shape().dim() == 4, "fused attention: q must be [batch, tokens, heads, head size]");
    FlashOperands f;
    f.batch = (int64_t)q->shape()[0];
    f.tokens = (int64_t)q->shape()[1];
    f.heads = (int64_t)q->shape()[2];
    f.head_dim = (int64_t)q->shape()[3];
    br_assert(valid->is_cuda() && valid->dtype() == DataType::Float && (int64_t)valid->items() >= f.batch,
              "fused attention: valid must be the device tensor bloom.valid fills");
    br_assert(alibi->is_cuda() && alibi->dtype() == DataType::Float && (int64_t)alibi->items() == f.heads * f.tokens,
              "fused attention: alibi must be the fp32 [heads, tokens] table");
    f.valid = static_cast<const int32_t*>(valid->data());
    return f;
}
bool flash_16(const tensor_t& t, const tensor_t& q) {
    return t->is_cuda() && t->dtype() == q->dtype() && t->items() == q->items();
}
bool flash_f32(const tensor_t& t, size_t items) {
    return t->is_cuda() && t->dtype() == DataType::Float && t->items() == items;
}
// ( q k v alibi valid o lse -- )
BR_WORD(FlashAttn,
    Tensors<7> a(stack);
    const tensor_t& q = a[0];
    br_assert(q->is_cuda() && (q->dtype() == DataType::F16 || q->dtype() == DataType::BF16),
              "op.flash_attn: 16-bit device tensors");
    const FlashOperands f = flash_operands(q, a[4], a[3]);
    br_assert(flash_16(a[1], q) && flash_16(a[2], q) && flash_16(a[5], q), "op.flash_attn: k, v, o must match q");
    br_assert(flash_f32(a[6], (size_t)(f.batch * f.heads * f.tokens)), "op.flash_attn: lse is fp32 [batch, heads, tokens]");
    BR_HIP_CHECK(br_hip_flash_attn_fwd(q->data(), a[1]->data(), a[2]->data(), (int)q->dtype(),
                                       static_cast<const float*>(a[3]->data()), f.valid, a[5]->data(),
                                       static_cast<float*>(a[6]->data()), f.batch, f.heads, f.tokens, f.head_dim,
                                       f.heads * f.head_dim, f.head_dim, f.tokens * f.heads * f.head_dim,
                                       f.heads * f.head_dim, f.tokens * f.heads * f.head_dim, ComputingContext::stream));
)
// ( q k v o dO alibi valid lse dq dk dv -- )   dq, dk, dv: fp32 or q's type, same layout
BR_WORD(FlashAttnBackward,
    Tensors<11> a(stack);
    const tensor_t& q = a[0];
    br_assert(q->is_cuda() && (q->dtype() == DataType::F16 || q->dtype() == DataType::BF16),
              "op.flash_attn_backward: 16-bit device tensors");
    const FlashOperands f = flash_operands(q, a[6], a[5]);
    float* delta = static_cast<float*>(ComputingContext::scratch((size_t)(f.batch * f.heads * f.tokens) * sizeof(float)));
    br_assert(flash_16(a[1], q) && flash_16(a[2], q) && flash_16(a[3], q) && flash_16(a[4], q),
              "op.flash_attn_backward: k, v, o, dO must match q");
    br_assert(flash_f32(a[7], (size_t)(f.batch * f.heads * f.tokens)), "op.flash_attn_backward: lse");
    const bool g32 = flash_f32(a[8], q->items()) && flash_f32(a[9], q->items()) && flash_f32(a[10], q->items());
    const bool g16 = flash_16(a[8], q) && flash_16(a[9], q) && flash_16(a[10], q);
    br_assert(g32 || g16, "op.flash_attn_backward: dq, dk, dv are tensors of q's size, all fp32 or all of q's type");
    BR_HIP_CHECK(br_hip_flash_attn_bwd(q->data(), a[1]->data(), a[2]->data(), a[3]->data(), a[4]->data(),
                                       (int)q->dtype(), static_cast<const float*>(a[5]->data()), f.valid,
                                       static_cast<const float*>(a[7]->data()), delta, a[8]->data(), a[9]->data(),
                                       a[10]->data(), g32 ? BR_F32 : (int)q->dtype(), f.batch, f.heads, f.tokens,
                                       f.head_dim,
                                       f.heads * f.head_dim, f.head_dim, f.tokens * f.heads * f.head_dim,
                                       f.heads * f.head_dim, f.tokens * f.heads * f.head_dim, ComputingContext::stream));
)
// The same on a packed projection: qkv is the [B, T, 3 * hidden] output of ONE
// linear layer over the fused query_key_value weight (rows ordered q | k | v,
// each [heads, 128]); o is [B, T, heads, 128] and its shape is the one consulted.
// ( qkv alibi valid o lse -- )
BR_WORD(FlashAttnQkv,
    Tensors<5> a(stack);
    const tensor_t& o = a[3];
    br_assert(o->is_cuda() && (o->dtype() == DataType::F16 || o->dtype() == DataType::BF16),
              "op.flash_attn_qkv: 16-bit device tensors");
    const FlashOperands f = flash_operands(o, a[2], a[1]);
    const int64_t hidden = f.heads * f.head_dim;
    br_assert(a[0]->is_cuda() && a[0]->dtype() == o->dtype() && a[0]->items() == 3 * o->items(),
              "op.flash_attn_qkv: qkv must hold three tensors of o's size and type");
    br_assert(flash_f32(a[4], (size_t)(f.batch * f.heads * f.tokens)), "op.flash_attn_qkv: lse is fp32 [batch, heads, tokens]");
    const char* qkv = static_cast<const char*>(a[0]->data());
    BR_HIP_CHECK(br_hip_flash_attn_fwd(qkv, qkv + 2 * hidden, qkv + 4 * hidden, (int)o->dtype(),
                                       static_cast<const float*>(a[1]->data()), f.valid, o->data(),
                                       static_cast<float*>(a[4]->data()), f.batch, f.heads, f.tokens, f.head_dim,
                                       3 * hidden, f.head_dim, f.tokens * 3 * hidden, hidden, f.tokens * hidden,
                                       ComputingContext::stream));
)
// ( qkv o dO alibi valid lse dqkv -- )   dqkv: [B, T, 3 * hidden] packed like qkv, fp32 or qkv's type
BR_WORD(FlashAttnQkvBackward,
    Tensors<7> a(stack);
    const tensor_t& o = a[1];
    br_assert(o->is_cuda() && (o->dtype() == DataType::F16 || o->dtype() == DataType::BF16),
              "op.flash_attn_qkv_backward: 16-bit device tensors");
    const FlashOperands f = flash_operands(o, a[4], a[3]);
    const int64_t hidden = f.heads * f.head_dim;
    br_assert(a[0]->is_cuda() && a[0]->dtype() == o->dtype() && a[0]->items() == 3 * o->items() && flash_16(a[2], o),
              "op.flash_attn_qkv_backward: qkv holds three tensors of o's size and type, dO matches o");
    br_assert(flash_f32(a[5], (size_t)(f.batch * f.heads * f.tokens)), "op.flash_attn_qkv_backward: lse");
    const bool g32 = flash_f32(a[6], 3 * o->items());
    br_assert(g32 || (a[6]->is_cuda() && a[6]->dtype() == o->dtype() && a[6]->items() == 3 * o->items()),
              "op.flash_attn_qkv_backward: dqkv has qkv's size and is fp32 or of qkv's type");
    float* delta = static_cast<float*>(ComputingContext::scratch((size_t)(f.batch * f.heads * f.tokens) * sizeof(float)));
    const char* qkv = static_cast<const char*>(a[0]->data());
    char* g = static_cast<char*>(a[6]->data());
    const int64_t gs = hidden * (g32 ? 4 : 2);  // bytes from dq to dk to dv
    BR_HIP_CHECK(br_hip_flash_attn_bwd(qkv, qkv + 2 * hidden, qkv + 4 * hidden, o->data(), a[2]->data(), (int)o->dtype(),
                                       static_cast<const float*>(a[3]->data()), f.valid,
                                       static_cast<const float*>(a[5]->data()), delta, g, g + gs, g + 2 * gs,
                                       g32 ? BR_F32 : (int)o->dtype(), f.batch, f.heads, f.tokens, f.head_dim,
                                       3 * hidden, f.head_dim,
                                       f.tokens * 3 * hidden, hidden, f.tokens * hidden, ComputingContext::stream));
)

// Two operator pairs of the model scripts with the addition folded into the
// producing kernel (same bits as the pair; no counterpart word in the reference):
// ( dy u du   du' x w b x_g w_g b_g -- )  `op.gelu_backward` followed by the
// `op.linear_backward` of the layer below; fused when du' is du
BR_WORD(GeluLinearBackward,
    Tensors<7> l(stack);
    Tensors<3> g(stack);
    if (l[0]->data() == g[2]->data() && l[0]->items() == g[2]->items()) {
        op_check_word(hip_gelu_linear_backward(g[0], g[1], g[2], l[1], l[2], l[3], l[4], l[5], l[6]),
                      "op.gelu_backward + op.linear_backward");
    } else {
        g[0]->op_gelu_backward(g[0], g[1], g[2]);
        l[0]->op_linear_backward(l[0], l[1], l[2], l[3], l[4], l[5], l[6]);
    }
)
// ( x w b u y -- )   u = x . w^T + b,  y = gelu(u)      `op.linear` + `op.gelu`
BR_WORD(LinearGelu,
    Tensors<5> a(stack);
    op_check_word(hip_linear_gelu(a[0], a[1], a[2], a[3], a[4]), "op.linear_gelu");
)
// ( x w b y -- )   y += x . w^T + b          `op.linear` into a temporary + `op.add`
BR_WORD(LinearAdd,
    Tensors<4> a(stack);
    op_check_word(hip_linear_accumulate(a[0], a[1], a[2], a[3]), "op.linear_add");
)
// ( x w b r y -- )   y = x . w^T + b + r        `op.linear` into a temporary + `op.add` of the residual r
BR_WORD(LinearResidual,
    Tensors<5> a(stack);
    op_check_word(hip_linear_residual(a[0], a[1], a[2], a[3], a[4]), "op.linear_residual");
)
// ( dy scale bias var y dscale dbias residual din eps -- )   din = dLN + residual
BR_WORD(LayernormBackwardAdd,
    const float eps = (float)stack.pop_number();
    Tensors<9> a(stack);
    op_check_word(hip_layernorm_backward_add(a[0], a[1], a[2], a[3], a[4], a[5], a[6], a[7], a[8], eps),
                  "op.layernorm_backward_add");
)
// ( dy scale bias var y dscale dbias residual din eps   din' x w b x_g w_g b_g -- )  `op.layernorm_backward_add`
// followed by the `op.linear_backward` of the layer below; fused when din' is din
BR_WORD(LayernormBackwardAddLinearBackward,
    Tensors<7> l(stack);
    const float eps = (float)stack.pop_number();
    Tensors<9> a(stack);
    if (l[0]->data() == a[8]->data() && l[0]->items() == a[8]->items()) {
        op_check_word(hip_layernorm_backward_add_linear_backward(a[0], a[1], a[2], a[3], a[4], a[5], a[6], a[7], a[8], eps,
                                                                 l[1], l[2], l[3], l[4], l[5], l[6]),
                      "op.layernorm_backward_add + op.linear_backward");
    } else {
        op_check_word(hip_layernorm_backward_add(a[0], a[1], a[2], a[3], a[4], a[5], a[6], a[7], a[8], eps),
                      "op.layernorm_backward_add");
        l[0]->op_linear_backward(l[0], l[1], l[2], l[3], l[4], l[5], l[6]);
    }
)

// AdamW on one parameter tensor.  The reference stops at the gradients; these
// two words are what a training loop runs after them.
// ( param [master] grad m v lr beta1 beta2 eps weight_decay step -- )
void adamw(Stack& stack, bool with_master) {
    const double step = stack.pop_number();
    const float wd = (float)stack.pop_number();
    const float eps = (float)stack.pop_number();
    const float beta2 = (float)stack.pop_number();
    const float beta1 = (float)stack.pop_number();
    const float lr = (float)stack.pop_number();
    tensor_t v = stack.pop_tensor();
    tensor_t m = stack.pop_tensor();
    tensor_t grad = stack.pop_tensor();
    tensor_t master = with_master ? stack.pop_tensor() : nullptr;
    tensor_t param = stack.pop_tensor();
    auto f32dev = [](const tensor_t& x) { return x->is_cuda() && x->dtype() == DataType::Float; };
    br_assert(param->is_cuda() && f32dev(grad) && f32dev(m) && f32dev(v), "op.adamw: device tensors, fp32 state");
    br_assert(grad->items() == param->items() && m->items() == param->items() && v->items() == param->items(),
              "op.adamw: parameter, gradient and moments differ in size");
    br_assert(step >= 1, "op.adamw: steps count from 1");
    float* master_ptr = nullptr;
    if (with_master) {
        br_assert(f32dev(master) && master->items() == param->items() && param->dtype() != DataType::Float,
                  "op.adamw_master: an fp32 master copy of a 16-bit parameter");
        master_ptr = static_cast<float*>(master->data());
    }
    BR_HIP_CHECK(br_hip_adamw(param->data(), (int)param->dtype(), master_ptr, static_cast<const float*>(grad->data()),
                              static_cast<float*>(m->data()), static_cast<float*>(v->data()), (int64_t)param->items(),
                              lr, beta1, beta2, eps, wd, (int64_t)step, ComputingContext::stream));
}
BR_WORD(AdamW, adamw(stack, false);)
BR_WORD(AdamWMaster, adamw(stack, true);)

BR_WORD(Dump, tensor_t t = stack.pop_tensor(); t->io_dump(t);)
// ( tensor filename -- )
BR_WORD(Load, const std::string f = stack.pop_string(); tensor_t t = stack.pop_tensor(); t->io_load(t, f.c_str());)
BR_WORD(Save, const std::string f = stack.pop_string(); tensor_t t = stack.pop_tensor(); t->io_save(t, f.c_str());)
// ( tensor peer -- )
BR_WORD(MPIRecv, const int p = (int)stack.pop_number(); tensor_t t = stack.pop_tensor(); t->io_mpi_recv(t, p);)
BR_WORD(MPIBcast, const int p = (int)stack.pop_number(); tensor_t t = stack.pop_tensor(); t->io_mpi_bcast(t, p);)
BR_WORD(NcclRecv, const int p = (int)stack.pop_number(); tensor_t t = stack.pop_tensor(); t->io_nccl_recv(t, p);)
BR_WORD(NcclSend, const int p = (int)stack.pop_number(); tensor_t t = stack.pop_tensor(); t->io_nccl_send(t, p);)

}  // namespace

void load_nn_words(Enviroment& env) {
    static const struct {
        const char* name;
        NativeCreator* creator;
    } table[] = {
        {"io.dump", Dump::creator},
        {"io.load", Load::creator},
        {"io.save", Save::creator},
        {"io.mpi.bcast", MPIBcast::creator},
        {"io.mpi.recv", MPIRecv::creator},
        {"io.nccl.send", NcclSend::creator},
        {"io.nccl.recv", NcclRecv::creator},
        {"op.sync", Sync::creator},
        {"op.create", Create::creator},
        {"op.gemm_precision", GemmPrecision::creator},
        {"op.grad_lift", GradLift::creator},
        {"op.zero", Zero::creator},
        {"op.fill", Fill::creator},
        {"op.view", View::creator},
        {"op.copy", Copy::creator},
        {"op.linear", Linear::creator},
        {"op.layernorm", Layernorm::creator},
        {"op.transpos_0213", Transpos0213::creator},
        {"op.add", Add::creator},
        {"op.querykey", QueryKey::creator},
        {"op.softmax", Softmax::creator},
        {"op.add_add_softmax", AddAddSoftmax::creator},
        {"op.add_add_softmax_copy", AddAddSoftmaxCopy::creator},
        {"op.layernorm_copy", LayernormCopy::creator},
        {"op.attn", Attn::creator},
        {"op.gelu", Gelu::creator},
        {"op.last_logits", LastLogits::creator},
        {"op.loss_backward", LossBackward::creator},
        {"op.loss_backward_set", LossBackwardSet::creator},
        {"op.layernorm_backward", LayernormBackward::creator},
        {"op.linear_backward", LinearBackward::creator},
        {"op.gelu_backward", GeluBackward::creator},
        {"op.attn_backward", AttnBackward::creator},
        {"op.softmax_backward", SoftmaxBackward::creator},
        {"op.softmax_attn_backward", SoftmaxAttnBackward::creator},
        {"op.qk_backward", QueryKeyBackward::creator},
        {"op.gelu_linear_backward", GeluLinearBackward::creator},
        {"op.linear_add", LinearAdd::creator},
        {"op.linear_gelu", LinearGelu::creator},
        {"op.linear_residual", LinearResidual::creator},
        {"op.layernorm_backward_add", LayernormBackwardAdd::creator},
        {"op.layernorm_backward_add_linear_backward", LayernormBackwardAddLinearBackward::creator},
        {"op.flash_attn", FlashAttn::creator},
        {"op.flash_attn_backward", FlashAttnBackward::creator},
        {"op.flash_attn_qkv", FlashAttnQkv::creator},
        {"op.flash_attn_qkv_backward", FlashAttnQkvBackward::creator},
        {"op.adamw", AdamW::creator},
        {"op.adamw_master", AdamWMaster::creator},
    };
    for (const auto& e : table) env.insert_native_word(e.name, e.creator);
    // longer patterns first: a pass only sees what earlier passes left unfused
    env.insert_fusion({"op.add", "op.add", "op.softmax", "op.copy"}, "op.add_add_softmax_copy");
    env.insert_fusion({"op.add", "op.add", "op.softmax"}, "op.add_add_softmax");
    env.insert_fusion({"op.layernorm", "op.copy"}, "op.layernorm_copy");
    env.insert_fusion({"op.gelu_backward", "op.linear_backward"}, "op.gelu_linear_backward");
    env.insert_fusion({"op.layernorm_backward_add", "op.linear_backward"}, "op.layernorm_backward_add_linear_backward");
}

}  // namespace br
