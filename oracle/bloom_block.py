"""Oracle composition of one BLOOM block, op by op as the reference's word
scripts sequence it.  TEST INFRASTRUCTURE ONLY.

``layer_forward`` restates bloomz-7b/train.words:137-192 and
``layer_backward`` restates bloomz-7b/train.words:194-248; each numbered
comment names the script line it follows.  Buffers are named as the script's
arena views are (xa, xb, xc, x4a, x4b, xll, zquery ...), so a device run of
the unchanged script can be compared buffer by buffer.
"""
from __future__ import annotations

import numpy as np

import oracle as orc

WEIGHT_NAMES = [
    "input_layernorm.weight", "input_layernorm.bias",
    "query.weight", "query.bias", "key.weight", "key.bias",
    "value.weight", "value.bias",
    "dense.weight", "dense.bias",
    "post_attention_layernorm.weight", "post_attention_layernorm.bias",
    "dense_h_to_4h.weight", "dense_h_to_4h.bias",
    "dense_4h_to_h.weight", "dense_4h_to_h.bias",
]


def make_weights(rng, hidden, std=0.02, dtype=np.float32):
    """Random-init block weights (q/k/v as three [H,H] slices, the layout
    bloomz-7b/init.words:32-44 gives them)."""
    h = hidden
    w = {}
    for ln in ("input_layernorm", "post_attention_layernorm"):
        w[ln + ".weight"] = (1.0 + std * rng.standard_normal(h)).astype(dtype)
        w[ln + ".bias"] = (std * rng.standard_normal(h)).astype(dtype)
    for name, (o, i) in {
        "query": (h, h), "key": (h, h), "value": (h, h), "dense": (h, h),
        "dense_h_to_4h": (4 * h, h), "dense_4h_to_h": (h, 4 * h),
    }.items():
        w[name + ".weight"] = (std * rng.standard_normal((o, i))).astype(dtype)
        w[name + ".bias"] = (std * rng.standard_normal(o)).astype(dtype)
    return w


def layer_forward(w, xinput, alibi, xmask, heads, eps=1e-5):
    b, t, h = xinput.shape
    hd = h // heads
    s = {}
    # :139 input layernorm
    s["xattn_in"], _, s["input_ln_var"] = orc.layernorm_fwd(
        xinput, w["input_layernorm.weight"], w["input_layernorm.bias"], eps)
    # :143-145 q, k, v projections
    xa = orc.linear_fwd(s["xattn_in"], w["query.weight"], w["query.bias"])
    xb = orc.linear_fwd(s["xattn_in"], w["key.weight"], w["key.bias"])
    xc = orc.linear_fwd(s["xattn_in"], w["value.weight"], w["value.bias"])
    # :147-149 [B,T,NH,HD] -> [B,NH,T,HD]
    s["zquery"] = orc.transpose_0213(xa.reshape(b, t, heads, hd))
    s["zkey"] = orc.transpose_0213(xb.reshape(b, t, heads, hd))
    s["zvalue"] = orc.transpose_0213(xc.reshape(b, t, heads, hd))
    # :155 scores, :158-159 alibi and mask, :162 softmax
    xll = orc.qk(s["zquery"], s["zkey"])
    xll = orc.add_bcast(xll, alibi.reshape(1, heads, 1, t))
    xll = orc.add_bcast(xll, xmask.reshape(b, 1, t, t))
    s["xll"] = orc.softmax_fwd(xll)
    # :165-166 context and transpose back
    zc = orc.attn(s["xll"], s["zvalue"])
    s["xattn_out"] = orc.transpose_0213(zc).reshape(b, t, h)
    # :170-171 dense + residual
    xb = orc.linear_fwd(s["xattn_out"], w["dense.weight"], w["dense.bias"])
    xa = orc.add_bcast(xb, xinput)
    s["residual1"] = xa
    # :174 post-attention layernorm
    s["xb"], _, s["post_ln_var"] = orc.layernorm_fwd(
        xa, w["post_attention_layernorm.weight"], w["post_attention_layernorm.bias"], eps)
    # :182-186 MLP
    s["x4a"] = orc.linear_fwd(s["xb"], w["dense_h_to_4h.weight"], w["dense_h_to_4h.bias"])
    s["x4b"] = orc.gelu_fwd(s["x4a"])
    xc = orc.linear_fwd(s["x4b"], w["dense_4h_to_h.weight"], w["dense_4h_to_h.bias"])
    # :189 residual
    s["xa"] = orc.add_bcast(xa, xc)
    return s


def layer_backward(w, s, xinput, yout_g, heads, eps=1e-5):
    """Returns (dx, grads) where grads maps '<name>_g' to arrays."""
    b, t, h = xinput.shape
    hd = h // heads
    g = {}
    yout_g = np.array(yout_g, np.float32)
    # :198 4h->h backward
    d4b, g["dense_4h_to_h.weight_g"], g["dense_4h_to_h.bias_g"] = orc.linear_bwd(
        yout_g, s["x4b"], w["dense_4h_to_h.weight"])
    # :200 gelu backward
    d4a = orc.gelu_bwd(d4b, s["x4a"])
    # :202 h->4h backward
    xa, g["dense_h_to_4h.weight_g"], g["dense_h_to_4h.bias_g"] = orc.linear_bwd(
        d4a, s["xb"], w["dense_h_to_4h.weight"])
    # :207 post layernorm backward, :208 add into yout_g
    xc, g["post_attention_layernorm.weight_g"], g["post_attention_layernorm.bias_g"] = \
        orc.layernorm_bwd(xa, s["xb"], w["post_attention_layernorm.weight"],
                          w["post_attention_layernorm.bias"], s["post_ln_var"], eps)
    yout_g = orc.add_bcast(yout_g, xc)
    # :211 dense backward
    xa, g["dense.weight_g"], g["dense.bias_g"] = orc.linear_bwd(
        yout_g, s["xattn_out"], w["dense.weight"])
    # :215 transpose, :217 fused softmax/attn backward, :219 qk backward
    zb = orc.transpose_0213(xa.reshape(b, t, heads, hd))
    ds, dv = orc.softmax_attn_bwd(zb, s["xll"], s["zvalue"])
    dq, dk = orc.qk_bwd(ds, s["zquery"], s["zkey"])
    # :225-227 back to [B,T,H]
    xvalue = orc.transpose_0213(dv).reshape(b, t, h)
    xquery = orc.transpose_0213(dq).reshape(b, t, h)
    xkey = orc.transpose_0213(dk).reshape(b, t, h)
    # :229-238 three projections backward, summed
    xa = np.zeros((b, t, h), np.float32)
    for name, dy in (("query", xquery), ("key", xkey), ("value", xvalue)):
        xb, g[name + ".weight_g"], g[name + ".bias_g"] = orc.linear_bwd(
            dy, s["xattn_in"], w[name + ".weight"])
        xa = orc.add_bcast(xa, xb)
    # :240 input layernorm backward, :243 residual
    xb, g["input_layernorm.weight_g"], g["input_layernorm.bias_g"] = orc.layernorm_bwd(
        xa, s["xattn_in"], w["input_layernorm.weight"], w["input_layernorm.bias"],
        s["input_ln_var"], eps)
    dx = orc.add_bcast(xb, yout_g)
    return dx, g
