"""Softmax-family HIP kernels against the CPU oracle through the C ABI:
attention softmax fwd/bwd, the fused ALiBi + mask + softmax (table and
analytic forms) and the vocabulary log-softmax + NLL forward / backward."""
import ctypes

import numpy as np
import pytest
import torch

import oracle as orc
from conftest import assert_close
from gpu_util import BF16, F16, F32, assert_close_f16, call, dev, empty, host, ptr, stream
from blackriver_amd import hip

pytestmark = pytest.mark.gpu
RTOL = 1e-5
FLT_MAX = np.finfo(np.float32).max
VOCAB = 250880


@pytest.mark.parametrize("rows,cols", [(4 * 32 * 64, 512), (10, 8), (33, 100), (7, 1001), (5, 2048), (3, 5000)])
def test_softmax_fwd_bwd(rows, cols):
    rng = np.random.default_rng(0)
    x = (3 * rng.standard_normal((rows, cols))).astype(np.float32)
    dy = rng.standard_normal((rows, cols)).astype(np.float32)
    dx_ = dev(x)
    y = empty((rows, cols))
    call("br_hip_softmax_fwd", ptr(dx_), ptr(y), rows, cols, stream())
    y_ref = orc.softmax_fwd(x)
    assert_close(host(y), y_ref, RTOL, "softmax")
    # in place (train.words:162)
    call("br_hip_softmax_fwd", ptr(dx_), ptr(dx_), rows, cols, stream())
    assert np.array_equal(host(dx_), host(y))
    g = empty((rows, cols))
    dyd = dev(dy)
    dyr = dev(y_ref)
    call("br_hip_softmax_bwd", ptr(dyd), ptr(dyr), ptr(g), rows, cols, stream())
    assert_close(host(g), orc.softmax_bwd(dy, y_ref), RTOL, "softmax bwd")
    # in place on dy (what the fused attention backward does, cuda_tensor.cpp:984-990)
    call("br_hip_softmax_bwd", ptr(dyd), ptr(dyr), ptr(dyd), rows, cols, stream())
    assert np.array_equal(host(dyd), host(g))


@pytest.mark.parametrize("b,h,t", [(2, 32, 512), (2, 4, 12), (1, 3, 37)])
def test_alibi_masked_softmax_table_and_analytic_forms(b, h, t, fixture_ids_mask):
    rng = np.random.default_rng(1)
    _, fmask = fixture_ids_mask
    mask = np.ones((b, t), np.int32)
    if t == 512:
        mask = fmask.copy()
    else:
        mask[0, t - 3:] = 0
    s = rng.standard_normal((b, h, t, t)).astype(np.float32)
    alibi = orc.alibi(h, t)
    xmask = orc.xmask(mask)
    ref = orc.softmax_fwd(orc.add_bcast(orc.add_bcast(s, alibi.reshape(1, h, 1, t)), xmask.reshape(b, 1, t, t)))

    ds, dalibi, dxmask = dev(s), dev(alibi), dev(xmask)
    p = empty(s.shape)
    call("br_hip_alibi_masked_softmax_fwd", ptr(ds), ptr(dalibi), ptr(dxmask), ptr(p), b, h, t, t, stream())
    got = host(p)
    assert_close(got, ref, RTOL, "fused alibi/mask softmax")
    # masked keys get exactly zero probability
    q, k = np.meshgrid(np.arange(t), np.arange(t), indexing="ij")
    valid = np.array([int(np.argmax(m == 0)) if (m == 0).any() else t for m in mask])
    closed = ~((k[None] <= q[None]) & (k[None] < valid[:, None, None]))
    assert np.all(got[np.broadcast_to(closed[:, None], got.shape)] == 0)

    # the three separate kernels give the same bits as the fused one
    tmp = empty(s.shape)
    call("br_hip_add_bcast", ptr(ds), ptr(dalibi), ptr(tmp), F32, hip.shape4(s.shape), hip.shape4((1, h, 1, t)), stream())
    call("br_hip_add_bcast", ptr(tmp), ptr(dxmask), ptr(tmp), F32, hip.shape4(s.shape), hip.shape4((b, 1, t, t)), stream())
    call("br_hip_softmax_fwd", ptr(tmp), ptr(tmp), b * h * t, t, stream())
    assert np.array_equal(host(tmp), got)

    # the analytic form (slopes + valid lengths, no tables) gives the same bits too
    slopes = (ctypes.c_double * h)()
    hip.load().br_hip_alibi_slopes(slopes, h)
    p2 = empty(s.shape)
    dslopes, dvalid = dev(np.array(slopes[:], np.float64)), dev(valid.astype(np.int32))
    call("br_hip_alibi_causal_softmax_fwd", ptr(ds), ptr(dslopes), ptr(dvalid), ptr(p2), b, h, t, t, stream())
    assert np.array_equal(host(p2), got)


def test_fully_masked_row_is_uniform():
    t = 16
    s = np.random.default_rng(2).standard_normal((1, 1, t, t)).astype(np.float32)
    mask = np.zeros((1, t), np.int32)          # first token already padding
    xmask = orc.xmask(mask)
    p = empty(s.shape)
    ds, dxmask = dev(s), dev(xmask)
    call("br_hip_alibi_masked_softmax_fwd", ptr(ds), None, ptr(dxmask), ptr(p), 1, 1, t, t, stream())
    assert_close(host(p), np.full(s.shape, 1.0 / t), 1e-6, "uniform")


def nll_run(logits, target, keep, out_dtype=F32):
    rows, vocab = logits.shape
    dl, dt, dk = dev(logits), dev(target), dev(keep)
    lse, rowlp, res = empty(rows), empty(rows), empty(2)
    call("br_hip_logsoftmax_nll_fwd", ptr(dl), ptr(dt), ptr(dk), ptr(lse), ptr(rowlp), ptr(res), rows, vocab, stream())
    r = host(res)
    count = int(r[1])
    g = empty((rows, vocab), torch.float32 if out_dtype == F32 else torch.float16)
    call("br_hip_logsoftmax_nll_bwd", ptr(dl), ptr(dt), ptr(dk), ptr(lse), ptr(g), out_dtype,
         1.0 / max(count, 1), rows, vocab, stream())
    return float(r[0]), count, host(lse), host(g), dl, dt, dk, lse


@pytest.mark.parametrize("rows,vocab", [(48, VOCAB), (17, 1000), (5, 1003), (300, 64)])
def test_logsoftmax_nll_against_oracle(rows, vocab):
    rng = np.random.default_rng(3)
    logits = (2 * rng.standard_normal((rows, vocab))).astype(np.float32)
    target = rng.integers(0, vocab, rows).astype(np.int32)
    keep = (rng.random(rows) < 0.9).astype(np.int32)
    keep[0] = 1
    loss_ref, lse_ref, dl_ref = orc.logsoftmax_nll(logits, target, keep)
    loss, count, lse, g, dl, dt, dk, dlse = nll_run(logits, target, keep)
    assert count == int((keep != 0).sum())                   # integer part: exact
    assert abs(loss - loss_ref) <= RTOL * abs(loss_ref)
    assert_close(lse, lse_ref, RTOL, "lse")
    assert_close(g, dl_ref, RTOL, "dlogits")
    assert np.all(g[keep == 0] == 0)
    # fp16 gradient storage
    _, _, _, g16, *_ = nll_run(logits, target, keep, F16)
    assert_close_f16(g16, dl_ref, RTOL, "dlogits fp16")
    # in place: dlogits over logits
    call("br_hip_logsoftmax_nll_bwd", ptr(dl), ptr(dt), ptr(dk), ptr(dlse), ptr(dl), F32, 1.0 / count, rows, vocab,
         stream())
    assert np.array_equal(host(dl), g)


def test_logsoftmax_nll_headline_shape_properties_and_sampled_rows():
    """logits[2048, 250880] fp32 ~N(0,2), targets uniform, mask Bernoulli(0.9),
    seed 2.  Too large for a full oracle pass in seconds: rows are independent,
    so a random sample of rows is checked exactly against the oracle and the
    whole tensor through invariants."""
    rows, vocab = 2048, VOCAB
    gen = torch.Generator(device="cuda").manual_seed(2)
    logits = torch.randn((rows, vocab), generator=gen, device="cuda", dtype=torch.float32) * 2.0
    target = torch.randint(0, vocab, (rows,), generator=gen, device="cuda", dtype=torch.int32)
    keep = (torch.rand((rows,), generator=gen, device="cuda") < 0.9).to(torch.int32)
    lse, rowlp, res = empty(rows), empty(rows), empty(2)
    call("br_hip_logsoftmax_nll_fwd", ptr(logits), ptr(target), ptr(keep), ptr(lse), ptr(rowlp), ptr(res), rows,
         vocab, stream())
    r = host(res)
    count = int(r[1])
    assert count == int(keep.sum().item())
    g = empty((rows, vocab))
    call("br_hip_logsoftmax_nll_bwd", ptr(logits), ptr(target), ptr(keep), ptr(lse), ptr(g), F32, 1.0 / count, rows,
         vocab, stream())
    torch.cuda.synchronize()
    k = host(keep)
    # invariants: each kept row of the gradient sums to zero, dropped rows are zero,
    # the label entry is the only negative one
    rs = g.double().sum(1).cpu().numpy()
    assert np.max(np.abs(rs)) < 1e-5 / count * 50
    assert float(g[torch.from_numpy(k == 0).cuda()].abs().max().item()) == 0.0
    neg = (g < 0).sum(1).cpu().numpy()
    assert np.array_equal(neg, (k != 0).astype(np.int64))
    # exact parity on sampled rows
    pick = np.sort(np.random.default_rng(0).choice(rows, 24, replace=False))
    sub = host(logits[torch.from_numpy(pick).cuda()])
    tsub, ksub = host(target)[pick], k[pick]
    _, lse_ref, dl_ref = orc.logsoftmax_nll(sub, tsub, ksub)
    assert_close(host(lse)[pick], lse_ref, RTOL, "lse on sampled rows")
    nk = max(int((ksub != 0).sum()), 1)
    assert_close(host(g[torch.from_numpy(pick).cuda()]) * count, dl_ref * nk, RTOL, "dlogits on sampled rows")
    # the loss is the mean over kept rows of logit[target] - lse
    lg = host(logits[torch.arange(rows, device="cuda"), target.long()])
    want = float(((lg.astype(np.float64) - host(lse).astype(np.float64)) * (k != 0)).sum() / count)
    assert abs(r[0] - want) <= RTOL * abs(want)


def test_fused_add_add_softmax_word_is_bit_identical_to_the_three_words(runtime):
    """The word machine fuses `op.add op.add op.softmax`; the fused word must
    give exactly what the three words give (each run as its own program, which
    the fusion pass cannot see across), on the attention-score pattern and, via
    its fallback, on operands that do not have that pattern."""
    from blackriver_amd import host
    rng = np.random.default_rng(12)
    b, h, t = 2, 4, 96
    s = rng.standard_normal((b, h, t, t)).astype(np.float32)
    alibi = rng.standard_normal((1, h, 1, t)).astype(np.float32)
    xmask = np.where(rng.random((b, 1, t, t)) < 0.3, -3.4028234663852886e38, 0.0).astype(np.float32)
    env = host.Env(1)
    try:
        env.execute("%d %d %d %d 4 'cuda' 'float' op.create 's' !  %d %d %d %d 4 'cuda' 'float' op.create 'p' !"
                    % (b, h, t, t, b, h, t, t))
        env.execute("1 %d 1 %d 4 'cuda' 'float' op.create 'a' !  %d 1 %d %d 4 'cuda' 'float' op.create 'm' !"
                    % (h, t, b, t, t))
        env.write("a", alibi)
        env.write("m", xmask)
        three = ["'s' @ 'a' @ 's' @ op.add", "'s' @ 'm' @ 's' @ op.add", "'s' @ 'p' @ op.softmax"]
        env.write("s", s)
        for w in three:
            env.execute(w)
        p_separate, s_separate = env.read("p"), env.read("s")
        env.write("s", s)
        env.execute("  ".join(three))
        assert np.array_equal(env.read("p"), p_separate)
        # in place, as the model script does it
        env.write("s", s)
        for w in three[:2] + ["'s' @ 's' @ op.softmax"]:
            env.execute(w)
        in_place = env.read("s")
        env.write("s", s)
        env.execute("  ".join(three[:2] + ["'s' @ 's' @ op.softmax"]))
        assert np.array_equal(env.read("s"), in_place)
        assert np.array_equal(in_place, p_separate) and s_separate.shape == s.shape
        # operands without the pattern (second add not in place): the fused word falls back
        env.execute("%d %d %d %d 4 'cuda' 'float' op.create 'q' !" % (b, h, t, t))
        other = ["'s' @ 'a' @ 's' @ op.add", "'s' @ 'm' @ 'q' @ op.add", "'q' @ 'p' @ op.softmax"]
        env.write("s", s)
        for w in other:
            env.execute(w)
        expect_p, expect_q = env.read("p"), env.read("q")
        env.write("s", s)
        env.execute("'p' @ op.zero 'q' @ op.zero")
        env.execute("  ".join(other))
        assert np.array_equal(env.read("p"), expect_p) and np.array_equal(env.read("q"), expect_q)
    finally:
        env.close()


@pytest.mark.parametrize("dtype,tdtype", [(F16, torch.float16), (BF16, torch.bfloat16)])
@pytest.mark.parametrize("b,h,t", [(2, 32, 512), (1, 3, 36), (1, 2, 2048)])
def test_softmax_16_bit_outputs_are_the_cast_of_the_fp32_outputs(b, h, t, dtype, tdtype):
    """The fused score softmax with a 16-bit image of p, and the softmax
    backward that stores only a 16-bit gradient, against the plain kernels
    followed by a cast: identical bits."""
    print("case b=%d h=%d t=%d dtype=%d" % (b, h, t, dtype), flush=True)
    rng = np.random.default_rng(21)
    s = rng.standard_normal((b, h, t, t)).astype(np.float32)
    alibi = orc.alibi(h, t)
    mask = np.ones((b, t), np.int32)
    mask[0, t - 5:] = 0
    xmask = orc.xmask(mask)
    ds, da, dm = dev(s), dev(alibi), dev(xmask)
    p_plain = empty(s.shape)
    call("br_hip_alibi_masked_softmax_fwd", ptr(ds), ptr(da), ptr(dm), ptr(p_plain), b, h, t, t, stream())
    p, p16 = empty(s.shape), empty(s.shape, tdtype)
    call("br_hip_alibi_masked_softmax_fwd_copy16", ptr(ds), ptr(da), ptr(dm), ptr(p), ptr(p16), dtype, b, h, t, t,
         stream())
    assert torch.equal(p, p_plain)
    assert torch.equal(p16, p_plain.to(tdtype))
    # in place on the scores, as the scripts run it
    call("br_hip_alibi_masked_softmax_fwd_copy16", ptr(ds), ptr(da), ptr(dm), ptr(ds), ptr(p16), dtype, b, h, t, t,
         stream())
    assert torch.equal(ds, p_plain) and torch.equal(p16, p_plain.to(tdtype))

    dp = dev(rng.standard_normal(s.shape).astype(np.float32))
    g_plain = empty(s.shape)
    call("br_hip_softmax_bwd", ptr(dp), ptr(p_plain), ptr(g_plain), b * h * t, t, stream())
    g16 = empty(s.shape, tdtype)
    call("br_hip_softmax_bwd_to16", ptr(dp), ptr(p_plain), ptr(g16), dtype, b * h * t, t, stream())
    assert torch.equal(g16, g_plain.to(tdtype))
    torch.cuda.synchronize()


def test_softmax_16_bit_outputs_decline_rows_the_wave_kernel_cannot_hold():
    lib = hip.load()
    rows, cols = 3, 1001
    t = empty(rows * cols)
    h16 = empty(rows * cols, torch.float16)
    assert lib.br_hip_softmax_bwd_to16(ptr(t), ptr(t), ptr(h16), F16, rows, cols, stream()) == -1
    assert lib.br_hip_softmax_bwd_to16(ptr(t), ptr(t), ptr(h16), F32, rows, 1000, stream()) == -1
    assert lib.br_hip_alibi_masked_softmax_fwd_copy16(ptr(t), None, None, ptr(t), ptr(h16), F16, 1, 1, rows, cols,
                                                      stream()) == -1
    assert lib.br_hip_alibi_masked_softmax_fwd_copy16(ptr(t), None, None, ptr(t), None, F16, 1, 1, rows, 1000,
                                                      stream()) == -3
    torch.cuda.synchronize()


def test_fused_words_with_a_16_bit_copy_match_the_separate_words(runtime):
    """`op.layernorm op.copy` and `op.add op.add op.softmax op.copy` are fused
    when the copy is the 16-bit image of the output; run fused (one program)
    and separately (one program per word) they must leave identical tensors.
    A copy of something else leaves the sequence to the fallback.  A 16-bit
    `op.softmax_backward` output equals the cast of the fp32 one."""
    from blackriver_amd import host
    rng = np.random.default_rng(5)
    b, h, t, hid = 2, 4, 96, 256
    env = host.Env(1)
    try:
        env.execute("%d %d %d 3 'cuda' 'float' op.create 'x' !  %d %d %d 3 'cuda' 'float' op.create 'y' !"
                    % (b, t, hid, b, t, hid))
        env.execute("%d %d %d 3 'cuda' 'f16' op.create 'y.h' !  %d %d %d 3 'cuda' 'f16' op.create 'z.h' !"
                    % (b, t, hid, b, t, hid))
        env.execute("%d 1 'cuda' 'float' op.create 'mean' !  %d 1 'cuda' 'float' op.create 'var' !" % (b * t, b * t))
        env.execute("%d 1 'cuda' 'float' op.create 'g' !  %d 1 'cuda' 'float' op.create 'bb' !" % (hid, hid))
        env.write("x", rng.standard_normal((b, t, hid)).astype(np.float32))
        env.write("g", (1 + 0.1 * rng.standard_normal(hid)).astype(np.float32))
        env.write("bb", (0.1 * rng.standard_normal(hid)).astype(np.float32))
        ln = "'x' @ 'mean' @ 'var' @ 'g' @ 'bb' @ 'y' @ 1e-5 op.layernorm"
        for cp in ("'y.h' @ 'y' @ op.copy", "'z.h' @ 'x' @ op.copy"):
            dst = cp.split("'")[1]
            env.execute(ln)
            env.execute(cp)
            y_sep, c_sep = env.read("y"), env.read(dst)
            env.execute("'y' @ op.zero '%s' @ op.zero" % dst)
            env.execute(ln + "  " + cp)
            assert np.array_equal(env.read("y"), y_sep)
            assert np.array_equal(env.read(dst).view(np.int16), c_sep.view(np.int16))

        env.execute("%d %d %d %d 4 'cuda' 'float' op.create 's' !  %d %d %d %d 4 'cuda' 'f16' op.create 's.h' !"
                    % (b, h, t, t, b, h, t, t))
        env.execute("1 %d 1 %d 4 'cuda' 'float' op.create 'a' !  %d 1 %d %d 4 'cuda' 'float' op.create 'm' !"
                    % (h, t, b, t, t))
        s = rng.standard_normal((b, h, t, t)).astype(np.float32)
        env.write("a", rng.standard_normal((1, h, 1, t)).astype(np.float32))
        env.write("m", np.where(rng.random((b, 1, t, t)) < 0.3, -3.4028234663852886e38, 0.0).astype(np.float32))
        words = ["'s' @ 'a' @ 's' @ op.add", "'s' @ 'm' @ 's' @ op.add", "'s' @ 's' @ op.softmax",
                 "'s.h' @ 's' @ op.copy"]
        env.write("s", s)
        for w in words:
            env.execute(w)
        p_sep, h_sep = env.read("s"), env.read("s.h")
        env.write("s", s)
        env.execute("'s.h' @ op.zero")
        env.execute("  ".join(words))
        assert np.array_equal(env.read("s"), p_sep)
        assert np.array_equal(env.read("s.h").view(np.int16), h_sep.view(np.int16))

        # softmax backward straight into a 16-bit tensor
        env.execute("%d %d %d %d 4 'cuda' 'float' op.create 'dp' !  %d %d %d %d 4 'cuda' 'float' op.create 'ds' !"
                    % (b, h, t, t, b, h, t, t))
        env.write("dp", rng.standard_normal((b, h, t, t)).astype(np.float32))
        env.execute("'dp' @ 's' @ 'ds' @ op.softmax_backward  's.h' @ 'ds' @ op.copy")
        want = env.read("s.h")
        env.execute("'s.h' @ op.zero  'dp' @ 's' @ 's.h' @ op.softmax_backward")
        assert np.array_equal(env.read("s.h").view(np.int16), want.view(np.int16))
    finally:
        env.close()
