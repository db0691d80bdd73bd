"""Pins the oracle's block composition (oracle/bloom_block.py, which follows
the reference's layer_forward / layer_backward word sequence) against an
independent textbook pre-LN BLOOM block written with torch fp64 ops and
differentiated by autograd.  CPU only.

Differences that are part of the reference and are accounted for here:
ALiBi as key_index*slope plus an additive -FLT_MAX mask (equal to the
relative-position / masked_fill form by shift invariance), and the second eps
in the LayerNorm backward (a relative 1e-5-scale effect at eps=1e-5, inside
the 1e-4 bound used for gradients).
"""
import numpy as np
import torch

import oracle as orc
from oracle import bloom_block as blk
from conftest import assert_close


def textbook_block(w, x, heads, mask, eps):
    F = torch.nn.functional
    b, t, h = x.shape
    hd = h // heads
    ln1 = F.layer_norm(x, (h,), w["input_layernorm.weight"], w["input_layernorm.bias"], eps)

    def proj(name):
        y = F.linear(ln1, w[name + ".weight"], w[name + ".bias"])
        return y.view(b, t, heads, hd).transpose(1, 2)

    q, k, v = proj("query"), proj("key"), proj("value")
    s = q @ k.transpose(-1, -2) / np.sqrt(hd)
    slopes = torch.tensor(2.0 ** (-8.0 * np.arange(1, heads + 1) / heads), dtype=x.dtype)
    pos = torch.arange(t, dtype=x.dtype)
    s = s + (pos[None, :] - pos[:, None])[None, None] * slopes[None, :, None, None]
    valid = torch.tensor(mask.sum(1))
    open_ = (pos[None, None, :] <= pos[None, :, None]) & (pos[None, None, :] < valid[:, None, None])
    s = s.masked_fill(~open_[:, None], float("-inf"))
    p = torch.softmax(s, -1)
    ctx = (p @ v).transpose(1, 2).reshape(b, t, h)
    r1 = F.linear(ctx, w["dense.weight"], w["dense.bias"]) + x
    ln2 = F.layer_norm(r1, (h,), w["post_attention_layernorm.weight"],
                       w["post_attention_layernorm.bias"], eps)
    m = F.gelu(F.linear(ln2, w["dense_h_to_4h.weight"], w["dense_h_to_4h.bias"]), approximate="tanh")
    return r1 + F.linear(m, w["dense_4h_to_h.weight"], w["dense_4h_to_h.bias"])


def test_block_forward_backward_against_textbook_autograd():
    rng = np.random.default_rng(3)
    b, t, h, heads, eps = 2, 12, 32, 4, 1e-5
    w = blk.make_weights(rng, h, std=0.2)
    x = rng.standard_normal((b, t, h)).astype(np.float32)
    dy = rng.standard_normal((b, t, h)).astype(np.float32)
    mask = np.ones((b, t), np.int32)
    mask[1, 9:] = 0

    wt = {k: torch.tensor(v.astype(np.float64), requires_grad=True) for k, v in w.items()}
    xt = torch.tensor(x.astype(np.float64), requires_grad=True)
    out = textbook_block(wt, xt, heads, mask, eps)
    out.backward(torch.tensor(dy.astype(np.float64)))

    alibi = orc.alibi(heads, t)
    xmask = orc.xmask(mask)
    s = blk.layer_forward(w, x, alibi, xmask, heads, eps)
    assert_close(s["xa"], out.detach().numpy(), 5e-6, "block output")
    dx, g = blk.layer_backward(w, s, x, dy, heads, eps)
    assert_close(dx, xt.grad.numpy(), 1e-4, "block dx")
    for name in blk.WEIGHT_NAMES:
        if name == "key.bias":
            continue
        assert_close(g[name + "_g"], wt[name].grad.numpy(), 1e-4, name + "_g")
    # a constant added to every key shifts each score row by a constant, which
    # softmax ignores: the key bias gradient is zero up to fp32 rounding
    scale = float(np.sqrt(np.mean(g["query.bias_g"].astype(np.float64) ** 2)))
    assert np.max(np.abs(g["key.bias_g"])) < 1e-5 * scale
    assert np.max(np.abs(wt["key.bias"].grad.numpy())) < 1e-12 * scale
