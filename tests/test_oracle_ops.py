"""Pins the CPU oracle (oracle/br_oracle.c) against evidence that does not
share its code: torch's fp64 autograd, numpy's broadcasting / einsum, closed
forms and invariants.  CPU only.

Where the reference deviates from the textbook (stored variance includes eps,
the backward adds eps again, +log-prob sign), the test derives the exact
factor by which the textbook answer must change and checks that.
"""
import numpy as np
import pytest
import torch

import oracle as orc
from conftest import assert_close

T64 = torch.float64


def t64(a, grad=False):
    x = torch.tensor(np.asarray(a, np.float64), dtype=T64)
    x.requires_grad_(grad)
    return x


# ------------------------------------------------------------------ LayerNorm
@pytest.mark.parametrize("rows,cols,eps", [(7, 64, 1e-5), (3, 1000, 1e-5), (5, 32, 0.1)])
def test_layernorm_fwd_against_torch(rows, cols, eps):
    rng = np.random.default_rng(0)
    x = rng.standard_normal((rows, cols)).astype(np.float32) * 3 + 0.5
    g = (1 + 0.02 * rng.standard_normal(cols)).astype(np.float32)
    b = (0.02 * rng.standard_normal(cols)).astype(np.float32)
    y, mean, var = orc.layernorm_fwd(x, g, b, eps)
    ref = torch.nn.functional.layer_norm(t64(x), (cols,), t64(g), t64(b), eps).numpy()
    assert_close(y, ref, 2e-7, "ln y")
    assert_close(mean, x.astype(np.float64).mean(1), 2e-7, "ln mean")
    # the stored statistic is the biased variance PLUS eps
    assert_close(var, x.astype(np.float64).var(1) + eps, 2e-7, "ln var+eps")


@pytest.mark.parametrize("eps", [1e-5, 0.1])
def test_layernorm_bwd_against_autograd_with_double_eps_factor(eps):
    """Autograd of y = xhat*g + b gives dgamma, dbeta exactly and dx up to the
    factor sqrt(var_stored / (var_stored + eps)) that the second eps causes."""
    rng = np.random.default_rng(1)
    rows, cols = 6, 48
    x = rng.standard_normal((rows, cols)).astype(np.float32) * 2
    g = (1 + 0.3 * rng.standard_normal(cols)).astype(np.float32)
    b = (0.3 * rng.standard_normal(cols)).astype(np.float32)
    dy = rng.standard_normal((rows, cols)).astype(np.float32)

    xt, gt, bt = t64(x, True), t64(g, True), t64(b, True)
    yt = torch.nn.functional.layer_norm(xt, (cols,), gt, bt, eps)
    yt.backward(t64(dy))
    var_stored = x.astype(np.float64).var(1) + eps
    factor = np.sqrt(var_stored / (var_stored + eps))[:, None]

    # feed the oracle the exact fp64 forward output rounded once to fp32
    y32 = yt.detach().numpy().astype(np.float32)
    dx, dgamma, dbeta = orc.layernorm_bwd(dy, y32, g, b, var_stored.astype(np.float32), eps)
    assert_close(dbeta, bt.grad.numpy(), 1e-6, "dbeta")
    assert_close(dgamma, gt.grad.numpy(), 1e-5, "dgamma")
    assert_close(dx, xt.grad.numpy() * factor, 1e-5, "dx")
    if eps == 0.1:
        # the factor is far from one here, so a single-eps oracle would fail
        assert np.max(np.abs(factor - 1)) > 1e-2


def test_layernorm_bwd_row_invariants_and_tiny_gamma_guard():
    rng = np.random.default_rng(2)
    rows, cols, eps = 4, 64, 1e-5
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    g = np.ones(cols, np.float32)
    b = np.zeros(cols, np.float32)
    y, _, var = orc.layernorm_fwd(x, g, b, eps)
    dy = rng.standard_normal((rows, cols)).astype(np.float32)
    dx, dgamma, dbeta = orc.layernorm_bwd(dy, y, g, b, var, eps)
    assert np.max(np.abs(dx.astype(np.float64).sum(1))) < 1e-4
    assert np.max(np.abs((dx.astype(np.float64) * y).sum(1))) < 1e-3
    assert_close(dbeta, dy.astype(np.float64).sum(0), 1e-6, "dbeta=colsum(dy)")
    # |gamma| <= eps is replaced by +-eps in the xhat division
    g2 = g.copy()
    g2[0], g2[1] = 1e-7, -1e-7
    y2 = (y * g2).astype(np.float32)
    _, dgamma2, _ = orc.layernorm_bwd(dy, y2, g2, b, var, eps)
    exp0 = (dy[:, 0].astype(np.float64) * (y2[:, 0].astype(np.float64) / eps)).sum()
    exp1 = (dy[:, 1].astype(np.float64) * (y2[:, 1].astype(np.float64) / -eps)).sum()
    assert_close(dgamma2[:2], np.array([exp0, exp1]), 1e-6, "add_eps guard")


# ----------------------------------------------------------------------- GELU
def test_gelu_fwd_against_torch_tanh_gelu():
    x = np.linspace(-9, 9, 4001).astype(np.float32)
    ref = torch.nn.functional.gelu(t64(x), approximate="tanh").numpy()
    y = orc.gelu_fwd(x)
    assert_close(y, ref, 1e-6, "gelu")
    # g(x) - g(-x) = x
    assert_close(y - orc.gelu_fwd(-x), x, 1e-6, "odd part")
    # the folded constant really is the product of the two textbook ones
    assert abs(0.03567741 - 0.79788456 * 0.044715) < 5e-9


def test_gelu_bwd_against_autograd():
    rng = np.random.default_rng(3)
    x = (1.5 * rng.standard_normal(5000)).astype(np.float32)
    dy = rng.standard_normal(5000).astype(np.float32)
    xt = t64(x, True)
    torch.nn.functional.gelu(xt, approximate="tanh").backward(t64(dy))
    dx = orc.gelu_bwd(dy, x)
    # tanh is rounded to fp32 in the reference (gelu.cu:66): absolute noise of
    # about 6e-8 * |x| on the derivative, hence the rms-scaled floor
    assert_close(dx, xt.grad.numpy(), 2e-6, "gelu bwd")


def test_bias_gelu_is_gelu_of_sum_and_dbias_is_colsum():
    rng = np.random.default_rng(4)
    x = rng.standard_normal((9, 40)).astype(np.float32)
    bias = rng.standard_normal(40).astype(np.float32)
    dy = rng.standard_normal((9, 40)).astype(np.float32)
    xt, bt = t64(x, True), t64(bias, True)
    yt = torch.nn.functional.gelu(xt + bt, approximate="tanh")
    yt.backward(t64(dy))
    assert_close(orc.bias_gelu_fwd(x, bias), yt.detach().numpy(), 1e-6, "bias gelu")
    dx, dbias = orc.bias_gelu_bwd(dy, x, bias)
    assert_close(dx, xt.grad.numpy(), 2e-6, "bias gelu dx")
    assert_close(dbias, bt.grad.numpy(), 2e-6, "bias gelu dbias")


# --------------------------------------------------------------------- Linear
def test_linear_fwd_bwd_against_autograd():
    rng = np.random.default_rng(5)
    n, inn, out = 10, 24, 17
    x = rng.standard_normal((2, 5, inn)).astype(np.float32)
    w = rng.standard_normal((out, inn)).astype(np.float32)
    b = rng.standard_normal(out).astype(np.float32)
    dy = rng.standard_normal((2, 5, out)).astype(np.float32)
    xt, wt, bt = t64(x, True), t64(w, True), t64(b, True)
    yt = torch.nn.functional.linear(xt, wt, bt)
    yt.backward(t64(dy))
    assert_close(orc.linear_fwd(x, w, b), yt.detach().numpy(), 1e-6, "linear")
    dx, dw, db = orc.linear_bwd(dy, x, w)
    assert_close(dx, xt.grad.numpy(), 1e-6, "dx")
    assert_close(dw, wt.grad.numpy(), 1e-6, "dw")
    assert_close(db, bt.grad.numpy(), 1e-6, "db")
    assert n == x.size // inn


# ----------------------------------------------------------- transpose / add
def test_transpose_0213_is_numpy_transpose_and_involution():
    rng = np.random.default_rng(6)
    x = rng.standard_normal((2, 5, 3, 8)).astype(np.float32)
    y = orc.transpose_0213(x)
    assert np.array_equal(y, np.ascontiguousarray(x.transpose(0, 2, 1, 3)))
    assert np.array_equal(orc.transpose_0213(y), x)


@pytest.mark.parametrize("ashape,bshape", [
    ((2, 4, 6, 6), (1, 4, 1, 6)),   # alibi onto scores
    ((2, 4, 6, 6), (2, 1, 6, 6)),   # xmask onto scores
    ((2, 6, 8), (2, 6, 8)),         # residual
    ((3, 5), (1, 5)),
])
def test_add_bcast_is_numpy_broadcast(ashape, bshape):
    rng = np.random.default_rng(7)
    a = rng.standard_normal(ashape).astype(np.float32)
    b = rng.standard_normal(bshape).astype(np.float32)
    assert np.array_equal(orc.add_bcast(a, b), a + b)


def test_add_bcast_mask_absorbs_finite_scores():
    a = np.array([[[[1.5, -2.0, 3.0]]]], np.float32)
    m = np.array([[[[0.0, -np.finfo(np.float32).max, -np.finfo(np.float32).max]]]], np.float32)
    c = orc.add_bcast(a, m)
    assert c[0, 0, 0, 0] == 1.5 and c[0, 0, 0, 1] == -np.finfo(np.float32).max
    # a fully masked row softmaxes to uniform
    full = np.full((1, 4), -np.finfo(np.float32).max, np.float32)
    assert_close(orc.softmax_fwd(full), np.full((1, 4), 0.25), 1e-7, "uniform")


# ------------------------------------------------------------------ attention
def test_attention_chain_against_autograd():
    rng = np.random.default_rng(8)
    b, h, t, hd = 2, 3, 7, 8
    q = rng.standard_normal((b, h, t, hd)).astype(np.float32)
    k = rng.standard_normal((b, h, t, hd)).astype(np.float32)
    v = rng.standard_normal((b, h, t, hd)).astype(np.float32)
    d_o = rng.standard_normal((b, h, t, hd)).astype(np.float32)
    qt, kt, vt = t64(q, True), t64(k, True), t64(v, True)
    alpha = float(np.float32(1.0 / np.sqrt(hd)))   # rounded to fp32 as in cuda_tensor.cpp:292
    st = (qt @ kt.transpose(-1, -2)) * alpha
    st.retain_grad()
    pt = torch.softmax(st, -1)
    pt.retain_grad()
    ot = pt @ vt
    ot.backward(t64(d_o))

    s = orc.qk(q, k)
    assert_close(s, st.detach().numpy(), 1e-6, "qk")
    p = orc.softmax_fwd(s)
    assert_close(p, pt.detach().numpy(), 1e-6, "softmax")
    assert_close(p.astype(np.float64).sum(-1), np.ones((b, h, t)), 1e-6, "rows sum to 1")
    assert_close(orc.softmax_fwd(s + 5.0), p, 2e-6, "shift invariance")
    o = orc.attn(p, v)
    assert_close(o, ot.detach().numpy(), 1e-6, "attn")

    dp, dv = orc.attn_bwd(d_o, p, v)
    assert_close(dp, pt.grad.numpy(), 2e-6, "dP")
    assert_close(dv, vt.grad.numpy(), 2e-6, "dV")
    ds = orc.softmax_bwd(dp, p)
    assert_close(ds, st.grad.numpy(), 5e-6, "dS")
    assert np.max(np.abs(ds.astype(np.float64).sum(-1))) < 1e-5
    ds2, dv2 = orc.softmax_attn_bwd(d_o, p, v)
    assert_close(ds2, st.grad.numpy(), 5e-6, "fused dS")
    assert_close(dv2, vt.grad.numpy(), 2e-6, "fused dV")
    dq, dk = orc.qk_bwd(ds, q, k)
    assert_close(dq, qt.grad.numpy(), 1e-5, "dQ")
    assert_close(dk, kt.grad.numpy(), 1e-5, "dK")


# ------------------------------------------------------------------ loss head
def test_logsoftmax_nll_against_torch_cross_entropy():
    rng = np.random.default_rng(9)
    rows, vocab = 11, 37
    logits = (2 * rng.standard_normal((rows, vocab))).astype(np.float32)
    target = rng.integers(0, vocab, rows).astype(np.int32)
    keep = (rng.random(rows) < 0.7).astype(np.int32)
    keep[0] = 1
    lt = t64(logits, True)
    tt = torch.tensor(np.where(keep != 0, target, -100), dtype=torch.long)
    ce = torch.nn.functional.cross_entropy(lt, tt, ignore_index=-100)
    ce.backward()
    loss, lse, dl = orc.logsoftmax_nll(logits, target, keep)
    # the reference reports +mean log-prob, i.e. minus the cross entropy ...
    assert abs(loss + ce.item()) < 1e-6
    # ... while its gradient is the cross entropy's
    assert_close(dl, lt.grad.numpy(), 2e-6, "dlogits")
    assert_close(lse, torch.logsumexp(lt.detach(), -1).numpy(), 1e-6, "lse")
    assert np.all(dl[keep == 0] == 0)


def test_loss_backward_against_autograd_and_accumulates_weight_grad():
    rng = np.random.default_rng(10)
    b, t, h, v = 2, 9, 16, 29
    x = rng.standard_normal((b, t, h)).astype(np.float32)
    w = (0.3 * rng.standard_normal((v, h))).astype(np.float32)
    ids = rng.integers(0, v, (b, t)).astype(np.int32)
    mask = np.ones((b, t), np.int32)
    mask[0, 6:] = 0
    mask[1, 4] = 0          # a hole: positions 3 and 4 both drop out
    xt, wt = t64(x, True), t64(w, True)
    logits = xt @ wt.T
    labels = np.full((b, t), -100, np.int64)
    for bb in range(b):
        for tt in range(t - 1):
            if mask[bb, tt] != 0 and mask[bb, tt + 1] != 0:
                labels[bb, tt] = ids[bb, tt + 1]
    ce = torch.nn.functional.cross_entropy(logits.reshape(-1, v), torch.tensor(labels.reshape(-1)),
                                           ignore_index=-100)
    ce.backward()
    g0 = rng.standard_normal((v, h)).astype(np.float32)
    loss, x_g, w_g, dl = orc.loss_backward(x, ids, mask, w, lm_head_g=g0, want_dlogits=True)
    assert abs(loss + ce.item()) < 1e-6
    assert_close(x_g, xt.grad.numpy(), 5e-6, "x_g")
    assert_close(w_g, g0.astype(np.float64) + wt.grad.numpy(), 5e-6, "lm_head_g accumulates")
    lab, count = orc.loss_labels(ids, mask)
    assert np.array_equal(lab, labels.astype(np.int32))
    assert count == int((labels >= 0).sum())
    assert np.all(x_g[:, -1, :] == 0)


def test_last_logits_picks_last_unmasked_and_zero_without_padding():
    rng = np.random.default_rng(11)
    b, t, h, v = 3, 6, 8, 13
    x = rng.standard_normal((b, t, h)).astype(np.float32)
    w = rng.standard_normal((v, h)).astype(np.float32)
    mask = np.ones((b, t), np.int32)
    mask[0, 4:] = 0       # last real token is 3
    mask[1, 1:] = 0       # last real token is 0
    # row 2 has no padding: the reference then picks position 0, not T-1
    out = orc.last_logits(x, mask, w)
    exp = np.stack([w.astype(np.float64) @ x[0, 3], w.astype(np.float64) @ x[1, 0],
                    w.astype(np.float64) @ x[2, 0]])
    assert_close(out, exp, 1e-6, "last logits")


# ------------------------------------------------------------------ fp16 glue
def test_f16_converters_match_numpy_bit_for_bit():
    allh = np.arange(65536, dtype=np.uint16)
    f = orc.f16_bits_to_f32(allh)
    ref = allh.view(np.float16).astype(np.float32)
    nan = np.isnan(ref)
    assert np.array_equal(f[~nan], ref[~nan]) and np.all(np.isnan(f[nan]))
    rng = np.random.default_rng(12)
    x = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * 10.0 ** rng.integers(-9, 6, 200000),
        ref[~nan],
        np.array([65504, 65519.99, 65520, 1e9, -1e9, 2.0 ** -25, 2.0 ** -25 * 1.0001, 2.0 ** -24,
                  0.0, -0.0, np.inf, -np.inf, 6.1e-5, 6.0975e-5], np.float32),
    ]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(orc.f32_to_f16_bits(x), want)


def test_embedding_scatter_add_against_brute_force_and_numpy():
    """grad[ids[i]] += dx[i] in ascending i: the same as numpy's unbuffered
    np.add.at (also sequential, hence bit-exact) and, within rounding, as the
    one-hot matrix product onehot(ids)^T . dx; ids outside the table are skipped."""
    rng = np.random.default_rng(9)
    n, hidden, vocab = 50, 12, 7
    ids = rng.integers(0, vocab, n).astype(np.int32)
    dx = rng.standard_normal((n, hidden)).astype(np.float32)
    grad = rng.standard_normal((vocab, hidden)).astype(np.float32)
    got = orc.embedding_scatter_add(grad, dx, ids)
    want = grad.copy()
    np.add.at(want, ids, dx)
    assert np.array_equal(got, want)
    onehot = np.zeros((n, vocab))
    onehot[np.arange(n), ids] = 1
    assert_close(got, grad + onehot.T @ dx.astype(np.float64), 1e-5, "one-hot product")
    bad = ids.copy()
    bad[0], bad[1] = -3, vocab
    got = orc.embedding_scatter_add(grad, dx, bad)
    want = grad.copy()
    np.add.at(want, bad[2:], dx[2:])
    assert np.array_equal(got, want)


def test_adamw_step_against_torch_optim():
    """The oracle's AdamW restatement against torch.optim.AdamW on the CPU over
    several steps (so the bias corrections and the moment recurrences are
    exercised), with weight decay on and off."""
    rng = np.random.default_rng(4)
    for wd in (0.0, 0.1):
        p0 = rng.standard_normal(1000).astype(np.float32)
        tp = torch.nn.Parameter(torch.from_numpy(p0.copy()))
        opt = torch.optim.AdamW([tp], lr=3e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=wd)
        p, m, v = p0, np.zeros_like(p0), np.zeros_like(p0)
        for step in range(1, 6):
            g = (rng.standard_normal(1000) * 10.0 ** int(rng.integers(-3, 2))).astype(np.float32)
            tp.grad = torch.from_numpy(g.copy())
            opt.step()
            p, m, v = orc.adamw_step(p, g, m, v, 3e-3, 0.9, 0.95, 1e-8, wd, step)
            assert_close(p, tp.detach().numpy(), 1e-6, "parameter after step %d" % step)
            st = opt.state[tp]
            assert_close(m, st["exp_avg"].numpy(), 1e-6, "first moment")
            assert_close(v, st["exp_avg_sq"].numpy(), 1e-6, "second moment")
    # a plain descent direction: positive gradient lowers the parameter
    p, _, _ = orc.adamw_step(np.ones(4, np.float32), np.ones(4, np.float32), np.zeros(4), np.zeros(4), 1e-2, 0.9,
                             0.999, 1e-8, 0.0, 1)
    assert np.all(p < 1.0) and np.allclose(p, 1.0 - 1e-2, rtol=1e-5)
