"""The BLOOM block through the whole product path on the GPU: word script ->
word machine -> TensorType -> HIPTensor -> br_hip kernels, compared buffer by
buffer with the CPU oracle's composition of the same operator sequence.

Two modes:
  fp32   weights stored as fp32, products on the fp32 MFMA kernel
         (bound 1e-4: a chain of ~20 fp32 operators, each within 1e-5)
  f16    weights stored as fp16, every product on the fp16 MFMA kernel with
         fp32 accumulation (bound 2e-2, the stated fp16-GEMM tolerance)
"""
import numpy as np
import pytest
import torch

import oracle as orc
from oracle import bloom_block as blk
from conftest import assert_close, print_ledger
from blackriver_amd import host

pytestmark = pytest.mark.gpu


def setup_block(runtime, hidden, heads, batch, tokens, mode, vocab=1024, seed=3):
    rng = np.random.default_rng(seed)
    env = host.Env(2)
    env.execute(host.words_text("bloom.words"))
    env.execute("%d %d %d 1e-05 model_dims" % (hidden, heads, vocab))
    env.set("$DEVICE", "cuda")
    env.set("$WDTYPE", {"f16": "f16", "bf16": "bf16"}.get(mode, "float"))
    env.execute("'%s' op.gemm_precision  1 op.grad_lift" % {"f16": "f16", "bf16": "bf16"}.get(mode, "f32"))
    env.execute("create_layer_weight create_layer_grad zero_layer_grad")
    env.execute("%d %d dynamic_floats" % (batch, tokens))
    floats = int(env.pop_number()) + 64 * vocab
    env.execute("%d create_var  %d %d create_dynamic" % (floats, batch, tokens))

    w = blk.make_weights(rng, hidden, std=0.02)
    if mode in ("f16", "bf16"):   # the oracle sees the weights exactly as the device stores them
        for k in w:
            if k.endswith(".weight") and "layernorm" not in k:
                if mode == "f16":
                    w[k] = w[k].astype(np.float16).astype(np.float32)
                else:
                    w[k] = torch.from_numpy(w[k]).to(torch.bfloat16).to(torch.float32).numpy()
    env.write("query_key_value.weight", np.concatenate([w["query.weight"], w["key.weight"], w["value.weight"]]))
    env.write("query_key_value.bias", np.concatenate([w["query.bias"], w["key.bias"], w["value.bias"]]))
    for name in blk.WEIGHT_NAMES:
        if not name.startswith(("query.", "key.", "value.")):
            env.write(name, w[name])
    x = rng.standard_normal((batch, tokens, hidden)).astype(np.float32)
    dy = rng.standard_normal((batch, tokens, hidden)).astype(np.float32)
    mask = np.ones((batch, tokens), np.int32)
    mask[-1, tokens - tokens // 4:] = 0          # right padding on the last sequence
    ids = rng.integers(0, vocab, (batch, tokens)).astype(np.int32)
    env.write("mask_", mask)
    env.write("ids_", ids)
    env.write("xinput", x)
    env.write("yout_g", dy)
    env.execute("prepare_batch")
    return env, w, x, dy, mask, ids


@pytest.mark.parametrize("mode,hidden,heads,batch,tokens", [
    ("fp32", 256, 4, 2, 24),
    ("fp32", 1024, 8, 2, 128),
    ("f16", 256, 4, 2, 24),
    ("f16", 1024, 8, 2, 128),
    ("bf16", 1024, 8, 2, 128),
])
def test_block_forward_backward_against_oracle(runtime, mode, hidden, heads, batch, tokens):
    print("case", mode, hidden, heads, batch, tokens, flush=True)
    # bf16 multiplicands carry 8 significant bits: operand rounding alone is 4x fp16's at these magnitudes
    tol = {"fp32": 1e-4, "f16": 2e-2, "bf16": 6e-2}[mode]
    env, w, x, dy, mask, _ = setup_block(runtime, hidden, heads, batch, tokens, mode)
    # the device-built tables are bit-exact
    assert np.array_equal(env.read("alibi").reshape(heads, tokens), orc.alibi(heads, tokens))
    assert np.array_equal(env.read("xmask").reshape(batch, tokens, tokens), orc.xmask(mask))

    s = blk.layer_forward(w, x, orc.alibi(heads, tokens), orc.xmask(mask), heads)
    env.execute("layer_forward op.sync")
    for name in ("xattn_in", "zquery", "zkey", "zvalue", "xll", "xattn_out", "x4a", "x4b", "xa"):
        assert_close(env.read(name).reshape(s[name].shape), s[name], tol, "forward " + name)
    assert_close(env.read("input_ln_var")[: batch * tokens], s["input_ln_var"], tol, "input_ln_var")
    assert_close(env.read("post_ln_var")[: batch * tokens], s["post_ln_var"], tol, "post_ln_var")

    dx_ref, g_ref = blk.layer_backward(w, s, x, dy, heads)
    env.execute("layer_backward_core op.sync")
    assert_close(env.read("xa"), dx_ref, tol, "backward dx")
    for name in blk.WEIGHT_NAMES:
        if name == "key.bias":
            continue
        assert_close(env.read(name + "_g").reshape(g_ref[name + "_g"].shape), g_ref[name + "_g"], tol, name + "_g")
    # key bias gradient is zero in exact arithmetic (softmax shift invariance)
    scale = float(np.sqrt(np.mean(g_ref["query.bias_g"].astype(np.float64) ** 2)))
    assert np.max(np.abs(env.read("key.bias_g"))) < {"fp32": 1e-3, "f16": 5e-2, "bf16": 2e-1}[mode] * scale
    env.close()


def test_block_step_is_repeatable(runtime):
    """Running the step twice from the same inputs gives the same bits: no
    operator reads state it did not write in this step."""
    env, w, x, dy, mask, _ = setup_block(runtime, 256, 4, 2, 24, "f16")
    env.execute("block_step op.sync")
    first = {n: env.read(n) for n in ("xa", "dense.weight_g", "query_key_value.weight_g", "input_layernorm.bias_g")}
    env.write("yout_g", dy)       # layer_backward accumulates into yout_g in place
    env.execute("block_step op.sync")
    for n, v in first.items():
        assert np.array_equal(env.read(n), v), n
    env.close()


@pytest.mark.parametrize("mode,hidden,heads,batch,tokens", [("f16", 256, 4, 2, 24), ("f16", 1024, 8, 2, 128),
                                                            ("bf16", 512, 8, 2, 64)])
def test_operand_buffer_words_give_the_same_bits(runtime, mode, hidden, heads, batch, tokens):
    """layer_forward_mixed / layer_backward_mixed keep product-only operands in
    fp16 buffers; since a product rounds its fp32 operands to fp16 the same way,
    every output and gradient must equal the fp32-arena words' bit for bit."""
    env, w, x, dy, mask, _ = setup_block(runtime, hidden, heads, batch, tokens, mode)
    env.execute("create_operand_buffers")
    env.execute("block_step op.sync")
    names = ["xa", "xattn_in", "x4a", "xll", "input_ln_var", "post_ln_var"] + [n + "_g" for n in blk.WEIGHT_NAMES
                                                                              if not n.startswith(("query.", "key.", "value."))]
    names += ["query_key_value.weight_g", "query_key_value.bias_g"]
    plain = {n: env.read(n) for n in names}
    for n in names:
        if n.endswith("_g"):
            env.execute("'%s' @ op.zero" % n)
    env.write("yout_g", dy)
    env.write("xinput", x)
    env.execute("block_step_mixed op.sync")
    for n in names:
        if n != "xll":
            assert np.array_equal(env.read(n), plain[n]), n
    # the buffers hold what the fp32 tensors round to; the score gradient, which
    # the fp32-arena words leave in xll, exists only as its 16-bit image here
    if mode == "f16":
        assert np.array_equal(env.read("xattn_in.h"), env.read("xattn_in").astype(np.float16).astype(np.float32))
        assert np.array_equal(env.read("xll.h"), plain["xll"].astype(np.float16).astype(np.float32))
    env.close()


@pytest.mark.parametrize("mode", ["fp32", "f16"])
def test_loss_head_against_oracle(runtime, mode):
    hidden, heads, batch, tokens, vocab = 256, 4, 2, 24, 1536
    tol = 1e-4 if mode == "fp32" else 2e-2
    env, _, x, _, mask, ids = setup_block(runtime, hidden, heads, batch, tokens, mode, vocab=vocab)
    rng = np.random.default_rng(5)
    lm = (0.05 * rng.standard_normal((vocab, hidden))).astype(np.float32)
    if mode == "f16":
        lm = lm.astype(np.float16).astype(np.float32)
    g0 = rng.standard_normal((vocab, hidden)).astype(np.float32)
    mask[0, 5] = 0                       # a hole: positions 4 and 5 carry no loss
    env.write("mask_", mask)
    env.execute("%d %d 2 'cuda' '%s' op.create 'lm_head.weight' !" % (vocab, hidden, "f16" if mode == "f16" else "float"))
    env.execute("%d %d 2 'cuda' 'float' op.create 'lm_head.weight_g' !" % (vocab, hidden))
    env.write("lm_head.weight", lm)
    env.write("lm_head.weight_g", g0)
    env.execute("'xinput' @ 'ids_' @ 'mask_' @ 'lm_head.weight' @ 'all_logits' @ 'xa' @ 'lm_head.weight_g' @ "
                "op.loss_backward op.sync")
    loss_ref, xg_ref, wg_ref, _ = orc.loss_backward(x, ids, mask, lm, lm_head_g=g0)
    assert_close(env.read("xa"), xg_ref, tol, "x_g")
    assert_close(env.read("lm_head.weight_g"), wg_ref, tol, "lm_head_g (accumulated)")
    # the overwriting form: whatever the gradient tensor held is gone, the result is the sum alone
    env.write("lm_head.weight_g", g0 * 7)
    env.execute("'xinput' @ 'ids_' @ 'mask_' @ 'lm_head.weight' @ 'all_logits' @ 'xb' @ 'lm_head.weight_g' @ "
                "op.loss_backward_set op.sync")
    assert_close(env.read("lm_head.weight_g"), wg_ref - g0, tol, "lm_head_g (overwritten)")
    assert np.array_equal(env.read("xb"), env.read("xa"))
    # a second call with a CPU gradient tensor, as the reference keeps it
    env.execute("%d %d 2 'cpu' 'float' op.create 'lm_g_cpu' !  'lm_g_cpu' @ op.zero" % (vocab, hidden))
    env.execute("'xinput' @ 'ids_' @ 'mask_' @ 'lm_head.weight' @ 'all_logits' @ 'xb' @ 'lm_g_cpu' @ op.loss_backward")
    assert_close(env.read("lm_g_cpu"), wg_ref - g0, tol, "lm_head_g on the host")
    assert np.array_equal(env.read("xb"), env.read("xa"))
    # the same tensor again: the plain word adds to what it holds, the overwriting word replaces it
    once = env.read("lm_g_cpu")
    env.execute("'xinput' @ 'ids_' @ 'mask_' @ 'lm_head.weight' @ 'all_logits' @ 'xb' @ 'lm_g_cpu' @ op.loss_backward")
    assert_close(env.read("lm_g_cpu"), 2 * once, 1e-6, "lm_head_g on the host, accumulated")
    env.execute("'xinput' @ 'ids_' @ 'mask_' @ 'lm_head.weight' @ 'all_logits' @ 'xb' @ 'lm_g_cpu' @ op.loss_backward_set")
    assert np.array_equal(env.read("lm_g_cpu"), once), "op.loss_backward_set left stale contents in a host gradient"
    env.close()


def test_loss_head_at_the_true_vocabulary_keeps_small_probabilities(runtime):
    """V = 250880, one 512-token sequence, fp16 products, a PEAKED head (logits
    ~ N(0, 6)): most probabilities are far below 1e-5, and p / count would
    fall under fp16's smallest subnormal.  The stored 16-bit gradient therefore
    leaves 1/count to the products' alpha; checked on x_g, on the whole
    lm_head_g, and row by row on vocabulary entries that are nobody's label and
    whose largest probability lies in [1e-7, 1e-5] -- rows that a gradient
    rounded to fp16 after the 1/count scaling would return as zeros."""
    hidden, heads, batch, tokens, vocab = 1024, 8, 1, 512, 250880
    env, _, x, _, mask, ids = setup_block(runtime, hidden, heads, batch, tokens, "f16", vocab=vocab)
    rng = np.random.default_rng(15)
    lm = (6.0 / np.sqrt(hidden) * rng.standard_normal((vocab, hidden))).astype(np.float16).astype(np.float32)
    env.execute("%d %d 2 'cuda' 'f16' op.create 'lm_head.weight' !" % (vocab, hidden))
    env.execute("%d %d 2 'cuda' 'float' op.create 'lm_head.weight_g' !  'lm_head.weight_g' @ op.zero" % (vocab, hidden))
    env.write("lm_head.weight", lm)
    env.execute("'xinput' @ 'ids_' @ 'mask_' @ 'lm_head.weight' @ 'all_logits' @ 'xa' @ 'lm_head.weight_g' @ "
                "op.loss_backward op.sync")
    loss_ref, xg_ref, wg_ref, _ = orc.loss_backward(x, ids, mask, lm)
    labels, count = orc.loss_labels(ids, mask)
    assert count == (tokens - tokens // 4) - 1
    assert_close(env.read("xa"), xg_ref, 2e-2, "x_g at V=250880")
    wg = env.read("lm_head.weight_g")
    assert_close(wg, wg_ref, 2e-2, "lm_head_g at V=250880")
    # selection only: probabilities from a plain numpy product
    logits = x.reshape(tokens, hidden)[labels.reshape(-1) >= 0] @ lm.T
    logits -= logits.max(axis=1, keepdims=True)
    prob = np.exp(logits)
    prob /= prob.sum(axis=1, keepdims=True)
    largest = prob.max(axis=0)
    rare = (largest >= 1e-7) & (largest <= 1e-5)
    rare[labels[labels >= 0]] = False
    assert rare.sum() > 1000
    ref_rows = wg_ref[rare].astype(np.float64)
    err = np.linalg.norm(wg[rare] - ref_rows, axis=1) / np.linalg.norm(ref_rows, axis=1)
    assert float(err.max()) <= 2e-2, "rare-token rows of lm_head_g: worst relative row error %.3g" % float(err.max())
    env.close()


def test_gradient_lift_scales_activation_gradients_only(runtime):
    """`S op.grad_lift`: the loss head hands out S * x_g, the block's backward
    passes the factor on and takes it out of every parameter gradient.  With
    fp32 products a power-of-two S commutes with every rounding, so parameter
    gradients equal the unlifted run's bit for bit and activation gradients are
    exactly S times as large; `0 op.grad_lift` picks S from the loss count only
    when products run in 16 bit."""
    hidden, heads, batch, tokens, vocab = 256, 4, 2, 24, 512
    env, _, x, dy, mask, ids = setup_block(runtime, hidden, heads, batch, tokens, "fp32", vocab=vocab)
    try:
        rng = np.random.default_rng(21)
        lm = (0.05 * rng.standard_normal((vocab, hidden))).astype(np.float32)
        env.execute("%d %d 2 'cuda' 'float' op.create 'lm_head.weight' !" % (vocab, hidden))
        env.execute("%d %d 2 'cuda' 'float' op.create 'lm_head.weight_g' !" % (vocab, hidden))
        env.write("lm_head.weight", lm)
        names = [n + "_g" for n in blk.WEIGHT_NAMES] + ["lm_head.weight_g"]
        step = ("'lm_head.weight_g' @ op.zero  layer_forward  'xa' @ 'ids_' @ 'mask_' @ 'lm_head.weight' @ 'all_logits' @ "
                "'yout_g' @ 'lm_head.weight_g' @ op.loss_backward  layer_backward_core op.sync")
        env.execute(step)
        plain = {n: env.read(n) for n in names + ["xa"]}
        env.write("xinput", x)
        env.execute("256 op.grad_lift  bloom.grad_lift")
        assert env.pop_number() == 256.0
        env.execute(step)
        for n in names:
            assert np.array_equal(env.read(n), plain[n]), n
        assert np.array_equal(env.read("xa"), plain["xa"] * np.float32(256)), "dx carries the lift"
        # choosing per step: fp32 products need no lift
        env.write("xinput", x)
        env.execute("0 op.grad_lift")
        env.execute(step)
        env.execute("bloom.grad_lift")
        assert env.pop_number() == 1.0
        assert np.array_equal(env.read("xa"), plain["xa"])
        with pytest.raises(host.HostError, match="power of two"):
            env.execute("3 op.grad_lift")
    finally:
        env.execute("1 op.grad_lift")
        env.close()


def test_loss_value_and_chunking(runtime, capfd):
    """The printed / returned value is +mean log-prob; a logits workspace that
    holds only a few rows forces the chunked path."""
    hidden, heads, batch, tokens, vocab = 256, 4, 2, 24, 512
    env, _, x, _, mask, ids = setup_block(runtime, hidden, heads, batch, tokens, "fp32", vocab=vocab)
    rng = np.random.default_rng(6)
    lm = (0.05 * rng.standard_normal((vocab, hidden))).astype(np.float32)
    env.execute("%d %d 2 'cuda' 'float' op.create 'lm_head.weight' !" % (vocab, hidden))
    env.execute("%d %d 2 'cuda' 'float' op.create 'lm_head.weight_g' !  'lm_head.weight_g' @ op.zero" % (vocab, hidden))
    env.write("lm_head.weight", lm)
    env.execute("'all_logits' @ 0 7 %d 2 op.view 'few_rows' !" % vocab)       # room for 7 rows only
    env.execute("'xinput' @ 'ids_' @ 'mask_' @ 'lm_head.weight' @ 'few_rows' @ 'xa' @ 'lm_head.weight_g' @ "
                "op.loss_backward op.sync")
    loss_ref, xg_ref, wg_ref, _ = orc.loss_backward(x, ids, mask, lm)
    out = capfd.readouterr().out
    line = [l for l in out.splitlines() if l.startswith("#################")][-1].split()
    _, count = orc.loss_labels(ids, mask)
    assert int(line[1]) == count
    assert abs(float(line[2]) - loss_ref) <= 2e-5 * abs(loss_ref) + 1e-5
    assert_close(env.read("xa"), xg_ref, 1e-4, "x_g (chunked)")
    assert_close(env.read("lm_head.weight_g"), wg_ref, 1e-4, "lm_head_g (chunked)")
    env.close()


def test_unfused_attention_backward_and_last_logits(runtime):
    hidden, heads, batch, tokens, vocab = 256, 4, 2, 24, 512
    env, w, x, dy, mask, ids = setup_block(runtime, hidden, heads, batch, tokens, "fp32", vocab=vocab)
    rng = np.random.default_rng(7)
    hd = hidden // heads
    p = orc.softmax_fwd(rng.standard_normal((batch, heads, tokens, tokens)).astype(np.float32))
    v = rng.standard_normal((batch, heads, tokens, hd)).astype(np.float32)
    d_o = rng.standard_normal((batch, heads, tokens, hd)).astype(np.float32)
    env.write("xll", p)
    env.write("zvalue", v)
    env.write("zb", d_o)
    env.execute("%d %d %d %d 4 'cuda' 'float' op.create 'dP' !" % (batch, heads, tokens, tokens))
    env.execute("'zb' @ 'xll' @ 'zvalue' @ 'dP' @ 'za' @ op.attn_backward")
    dp_ref, dv_ref = orc.attn_bwd(d_o, p, v)
    assert_close(env.read("dP"), dp_ref, 1e-5, "dP")
    assert_close(env.read("za"), dv_ref, 1e-5, "dV")
    env.execute("'dP' @ 'xll' @ 'dP' @ op.softmax_backward")
    assert_close(env.read("dP"), orc.softmax_bwd(dp_ref, p), 2e-5, "dS")

    lm = (0.05 * rng.standard_normal((vocab, hidden))).astype(np.float32)
    env.execute("%d %d 2 'cuda' 'float' op.create 'lm_head.weight' !" % (vocab, hidden))
    env.execute("%d %d 2 'cuda' 'float' op.create 'last' !" % (batch, vocab))
    env.write("lm_head.weight", lm)
    env.execute("'xinput' @ 'mask_' @ 'lm_head.weight' @ 'last' @ op.last_logits")
    assert_close(env.read("last"), orc.last_logits(x, mask, lm), 1e-5, "last logits")
    env.close()


def test_device_tensor_plumbing(runtime, tmp_path, capfd):
    env = host.Env(1)
    env.execute("2048 1 'cuda' 'float' op.create 'd' !  'd' @ 1.5 op.fill")
    assert env.info("d")[1] and (env.read("d") == 1.5).all()
    x = np.arange(2048, dtype=np.float32) / 7
    f = tmp_path / "x.bin"
    x.tofile(f)
    env.execute("'d' @ '%s' io.load  'd' @ io.dump" % f)
    assert np.array_equal(env.read("d"), x)
    out = capfd.readouterr().out
    assert "First 8 : 0 0.142857" in out and "Last 8 :" in out
    # fp16 tensor: converted on load, on copy and on save
    env.execute("2048 1 'cuda' 'f16' op.create 'h' !  'h' @ 'd' @ op.copy  'h' @ '%s' io.save" % (tmp_path / "h.bin"))
    assert np.array_equal(np.fromfile(tmp_path / "h.bin", dtype=np.float32), x.astype(np.float16).astype(np.float32))
    # host <-> device copies and views
    env.execute("2048 1 'cpu' 'float' op.create 'c' !  'c' @ 'd' @ op.copy")
    assert np.array_equal(env.read("c"), x)
    env.execute("'d' @ op.zero  'd' @ 1024 2 512 2 op.view 'dv' !  'dv' @ 'c' @ 0 2 512 2 op.view op.copy")
    got = env.read("d")
    assert (got[:1024] == 0).all() and np.array_equal(got[1024:], x[:1024])
    # in-process pipeline hand-off
    env.execute("'d' @ 0 io.nccl.send  'd' @ op.zero  'd' @ 0 io.nccl.recv")
    assert np.array_equal(env.read("d"), got)
    with pytest.raises(host.HostError, match="nccl_recv"):
        env.execute("'d' @ 1 io.nccl.recv")
    # wrong size file
    with pytest.raises(host.HostError, match="same size"):
        env.execute("1024 1 'cuda' 'float' op.create '%s' io.load" % f)
    env.close()


@pytest.mark.parametrize("dtype", ["float", "f16"])
def test_qkv_relayout_words_match_the_offline_converter(runtime, dtype):
    """qkv_*_from_hf reorder the rows of a Hugging Face fused query_key_value
    tensor, [head, q|k|v, d], into BlackRiver's [q|k|v, head, d]: the view /
    transpose / reshape of bloomz-7b/dump_weights.py:23-44, restated here with
    numpy.  qkv_*_to_hf is the inverse.  Pure data movement: exact."""
    hidden, heads = 256, 4
    hd = hidden // heads
    rng = np.random.default_rng(2)
    env = host.Env(1)
    try:
        env.execute(host.words_text("bloom.words"))
        env.execute("%d %d 1024 1e-05 model_dims" % (hidden, heads))
        for name, shape in (("w", "%d %d 2" % (3 * hidden, hidden)), ("b", "%d 1" % (3 * hidden))):
            for sfx in (".hf", "", ".back"):
                env.execute("%s 'cuda' '%s' op.create '%s%s' !" % (shape, dtype, name, sfx))
        w = rng.standard_normal((3 * hidden, hidden)).astype(np.float16).astype(np.float32)
        b = rng.standard_normal(3 * hidden).astype(np.float16).astype(np.float32)
        env.write("w.hf", w)
        env.write("b.hf", b)
        env.execute("'w.hf' @ 'w' @ qkv_weight_from_hf   'b.hf' @ 'b' @ qkv_bias_from_hf")
        want_w = w.reshape(heads, 3, hd, hidden).transpose(1, 0, 2, 3).reshape(3 * hidden, hidden)
        want_b = b.reshape(heads, 3, hd).transpose(1, 0, 2).reshape(3 * hidden)
        assert np.array_equal(env.read("w"), want_w)
        assert np.array_equal(env.read("b"), want_b)
        # the first third is the query projection of every head, heads in order
        assert np.array_equal(env.read("w")[:hd], w[:hd]) and np.array_equal(env.read("w")[hd:2 * hd], w[3 * hd:4 * hd])
        env.execute("'w' @ 'w.back' @ qkv_weight_to_hf   'b' @ 'b.back' @ qkv_bias_to_hf")
        assert np.array_equal(env.read("w.back"), w) and np.array_equal(env.read("b.back"), b)
    finally:
        env.close()


@pytest.mark.parametrize("mode,tol", [("f16", 2e-2), ("bf16", 6e-2)])
def test_block_with_fused_attention_matches_oracle(runtime, mode, tol):
    """layer_forward_flash / layer_backward_flash (attention as one fused kernel
    per direction, head size 128) against the oracle's operator-by-operator
    block, and against the operand-buffer words within the same bound."""
    hidden, heads, batch, tokens = 512, 4, 2, 64
    env, w, x, dy, mask, _ = setup_block(runtime, hidden, heads, batch, tokens, mode)
    env.execute("create_operand_buffers create_flash_buffers prepare_batch_flash")
    env.execute("block_step_flash op.sync")
    saved = blk.layer_forward(w, x, orc.alibi(heads, tokens), orc.xmask(mask), heads, 1e-5)
    dx_ref, g_ref = blk.layer_backward(w, saved, x, dy, heads, 1e-5)
    assert_close(env.read("xa"), dx_ref, tol, "dx")
    got = {n: env.read(n) for n in ["xa"] + [k for k in g_ref]}
    for name, ref in g_ref.items():
        if name.startswith("key.bias"):
            continue
        if name.startswith(("query.", "key.", "value.")):
            continue          # thirds of query_key_value, compared below
        assert_close(got[name], ref, tol, name)
    qkv_w = np.concatenate([g_ref["query.weight_g"], g_ref["key.weight_g"], g_ref["value.weight_g"]])
    assert_close(env.read("query_key_value.weight_g"), qkv_w, tol, "query_key_value.weight_g")
    # the forward output, from a fresh forward pass
    env.write("xinput", x)
    env.execute("layer_forward_flash op.sync")
    assert_close(env.read("xa"), saved["xa"], tol, "block output")
    flash_out = env.read("xa")
    env.write("xinput", x)
    env.execute("layer_forward_mixed op.sync")
    assert_close(flash_out, env.read("xa"), tol, "flash vs operator chain")
    env.close()


def test_linear_add_and_layernorm_backward_add_words_equal_the_operator_pairs(runtime):
    """`op.linear_add` = `op.linear` into a temporary + `op.add`;
    `op.layernorm_backward_add` = `op.layernorm_backward` + `op.add`: same bits,
    in fp32 and fp16 product modes, also on a width the row kernel declines."""
    rng = np.random.default_rng(8)
    for mode, hidden in (("f32", 256), ("f16", 256), ("f32", 102)):
        b, t = 2, 24
        env = host.Env(1)
        try:
            env.execute("'%s' op.gemm_precision" % mode)
            wdt = "f16" if mode == "f16" else "float"
            env.execute("%d %d %d 3 'cuda' '%s' op.create 'x' !" % (b, t, 4 * hidden, wdt))
            env.execute("%d %d 2 'cuda' '%s' op.create 'w' !  %d 1 'cuda' 'float' op.create 'bias' !"
                        % (hidden, 4 * hidden, wdt, hidden))
            for n in ("y", "tmp", "acc", "dy", "ln", "res", "din", "din2"):
                env.execute("%d %d %d 3 'cuda' 'float' op.create '%s' !" % (b, t, hidden, n))
            for n in ("var", "g", "be", "dg", "db", "dg2", "db2"):
                env.execute("%d 1 'cuda' 'float' op.create '%s' !" % (max(hidden, b * t), n))
            env.execute("%d 1 'cuda' 'float' op.create 'gam' !  %d 1 'cuda' 'float' op.create 'bet' !" % (hidden, hidden))
            env.execute("%d 1 'cuda' 'float' op.create 'dgam' !  %d 1 'cuda' 'float' op.create 'dbet' !" % (hidden, hidden))
            env.execute("%d 1 'cuda' 'float' op.create 'dgam2' !  %d 1 'cuda' 'float' op.create 'dbet2' !" % (hidden, hidden))
            env.write("x", rng.standard_normal((b, t, 4 * hidden)).astype(np.float32))
            env.write("w", (0.05 * rng.standard_normal((hidden, 4 * hidden))).astype(np.float32))
            env.write("bias", rng.standard_normal(hidden).astype(np.float32))
            acc0 = rng.standard_normal((b, t, hidden)).astype(np.float32)
            env.write("acc", acc0)
            env.execute("'x' @ 'w' @ 'bias' @ 'tmp' @ op.linear  'acc' @ 'tmp' @ 'y' @ op.add")
            env.execute("'x' @ 'w' @ 'bias' @ 'acc' @ op.linear_add")
            assert np.array_equal(env.read("acc"), env.read("y")), mode
            # the three-operand form: the residual stays as it is, or is the output itself
            env.write("acc", acc0)
            env.execute("'x' @ 'w' @ 'bias' @ 'acc' @ 'din' @ op.linear_residual")
            assert np.array_equal(env.read("din"), env.read("y")), mode
            assert np.array_equal(env.read("acc"), acc0), mode
            env.execute("'x' @ 'w' @ 'bias' @ 'acc' @ 'acc' @ op.linear_residual")
            assert np.array_equal(env.read("acc"), env.read("y")), mode

            env.write("gam", (1 + 0.1 * rng.standard_normal(hidden)).astype(np.float32))
            env.write("bet", (0.1 * rng.standard_normal(hidden)).astype(np.float32))
            env.write("dy", rng.standard_normal((b, t, hidden)).astype(np.float32))
            env.write("res", rng.standard_normal((b, t, hidden)).astype(np.float32))
            env.execute("'acc' @ 'g' @ 'var' @ 'gam' @ 'bet' @ 'ln' @ 1e-5 op.layernorm")
            env.execute("'dy' @ 'gam' @ 'bet' @ 'var' @ 'ln' @ 'dgam' @ 'dbet' @ 'din' @ 1e-5 op.layernorm_backward"
                        "  'din' @ 'res' @ 'din' @ op.add")
            env.execute("'dy' @ 'gam' @ 'bet' @ 'var' @ 'ln' @ 'dgam2' @ 'dbet2' @ 'res' @ 'din2' @ 1e-5 "
                        "op.layernorm_backward_add")
            assert np.array_equal(env.read("din2"), env.read("din")), (mode, hidden)
            assert np.array_equal(env.read("dgam2"), env.read("dgam")) and np.array_equal(env.read("dbet2"), env.read("dbet"))
        finally:
            env.close()


def test_linear_residual_on_a_product_that_is_split_along_k(runtime):
    """512 rows against a [4096, 16384] weight: few output tiles and a long K, which the backend runs as slices
    of K summed by a second kernel; the residual then joins in that kernel."""
    rng = np.random.default_rng(18)
    rows, out, k = 512, 4096, 16384
    env = host.Env(1)
    try:
        env.execute("'f16' op.gemm_precision")
        env.execute("1 %d %d 3 'cuda' 'f16' op.create 'x' !  %d %d 2 'cuda' 'f16' op.create 'w' !" % (rows, k, out, k))
        env.execute("%d 1 'cuda' 'float' op.create 'bias' !" % out)
        for n in ("tmp", "y", "res", "y2"):
            env.execute("1 %d %d 3 'cuda' 'float' op.create '%s' !" % (rows, out, n))
        env.write("x", rng.standard_normal((1, rows, k)).astype(np.float32))
        env.write("w", (0.02 * rng.standard_normal((out, k))).astype(np.float32))
        env.write("bias", rng.standard_normal(out).astype(np.float32))
        res = rng.standard_normal((1, rows, out)).astype(np.float32)
        env.write("res", res)
        env.execute("'x' @ 'w' @ 'bias' @ 'tmp' @ op.linear  'tmp' @ 'res' @ 'y' @ op.add")
        env.execute("'x' @ 'w' @ 'bias' @ 'res' @ 'y2' @ op.linear_residual op.sync")
        assert np.array_equal(env.read("y2"), env.read("y"))
        assert np.array_equal(env.read("res"), res)
    finally:
        env.close()


@pytest.mark.parametrize("mode", ["f16", "f32"])
def test_fused_gelu_backward_linear_backward_equals_the_two_words(runtime, mode):
    """The fusion pass turns `op.gelu_backward op.linear_backward` (the pair of
    bloomz-7b/train.words:200-202) into one word; run as one program (fused)
    and as two programs (not fused) it must leave identical tensors, in the
    16-bit product mode (fused kernel) and in fp32 mode (the word's fallback)."""
    rng = np.random.default_rng(13)
    b, t, hidden = 2, 24, 128
    env = host.Env(1)
    try:
        env.execute("'%s' op.gemm_precision" % mode)
        wdt = "f16" if mode == "f16" else "float"
        env.execute("%d %d %d 3 'cuda' 'float' op.create 'dy' !  %d %d %d 3 'cuda' 'float' op.create 'u' !"
                    % (b, t, 4 * hidden, b, t, 4 * hidden))
        env.execute("%d %d %d 3 'cuda' 'float' op.create 'x' !  %d %d %d 3 'cuda' 'float' op.create 'xg' !"
                    % (b, t, hidden, b, t, hidden))
        env.execute("%d %d 2 'cuda' '%s' op.create 'w' !  %d %d 2 'cuda' 'float' op.create 'wg' !"
                    % (4 * hidden, hidden, wdt, 4 * hidden, hidden))
        env.execute("%d 1 'cuda' 'float' op.create 'bias' !  %d 1 'cuda' 'float' op.create 'bg' !"
                    % (4 * hidden, 4 * hidden))
        u0 = (1.5 * rng.standard_normal((b, t, 4 * hidden))).astype(np.float32)
        env.write("dy", rng.standard_normal((b, t, 4 * hidden)).astype(np.float32))
        env.write("x", rng.standard_normal((b, t, hidden)).astype(np.float32))
        env.write("w", (0.05 * rng.standard_normal((4 * hidden, hidden))).astype(np.float32))
        gelu = "'dy' @ 'u' @ 'u' @ op.gelu_backward"
        lin = "'u' @ 'x' @ 'w' @ 'bias' @ 'xg' @ 'wg' @ 'bg' @ op.linear_backward"
        assert "W:op.gelu_linear_backward" in env.disassemble(gelu + "  " + lin, fused=True)
        env.write("u", u0)
        env.execute(gelu)
        env.execute(lin)
        want = {n: env.read(n) for n in ("u", "xg", "wg", "bg")}
        env.write("u", u0)
        env.execute("'xg' @ op.zero 'wg' @ op.zero 'bg' @ op.zero")
        env.execute(gelu + "  " + lin)
        for n, v in want.items():
            assert np.array_equal(env.read(n), v), (mode, n)
    finally:
        env.close()


@pytest.mark.parametrize("mode,hidden", [("f16", 256), ("bf16", 256), ("f32", 256), ("f16", 8192)])
def test_fused_layernorm_backward_add_linear_backward_equals_the_two_words(runtime, mode, hidden):
    """The fusion pass turns `op.layernorm_backward_add op.linear_backward` (the post-attention LayerNorm's
    backward followed by the dense layer's in the block's backward) into one word when the second reads the
    gradient the first writes.  Fused (one program) and unfused (two programs) must agree: the LayerNorm's
    outputs, the 16-bit products' results (they read the same 16-bit image) bit for bit, the bias gradient to
    the rounding of a different summation order; in fp32 mode and on rows wider than the fused kernel takes the
    word falls back to the two operators (same bits throughout); a pair that is not chained is left alone."""
    rng = np.random.default_rng(23)
    b, t, inner = 2, 24, 128
    env = host.Env(1)
    try:
        env.execute("'%s' op.gemm_precision" % mode)
        wdt = {"f16": "f16", "bf16": "bf16", "f32": "float"}[mode]
        for n in ("dy", "ln", "res", "din", "other"):
            env.execute("%d %d %d 3 'cuda' 'float' op.create '%s' !" % (b, t, hidden, n))
        env.execute("%d %d %d 3 'cuda' '%s' op.create 'x' !  %d %d %d 3 'cuda' 'float' op.create 'xg' !"
                    % (b, t, inner, wdt, b, t, inner))
        env.execute("%d %d 2 'cuda' '%s' op.create 'w' !  %d %d 2 'cuda' 'float' op.create 'wg' !"
                    % (hidden, inner, wdt, hidden, inner))
        for n in ("gam", "bet", "dgam", "dbet", "bias", "bg"):
            env.execute("%d 1 'cuda' 'float' op.create '%s' !" % (hidden, n))
        env.execute("%d 1 'cuda' 'float' op.create 'var' !  %d 1 'cuda' 'float' op.create 'mean' !" % (b * t, b * t))
        env.write("gam", (1 + 0.1 * rng.standard_normal(hidden)).astype(np.float32))
        env.write("bet", (0.1 * rng.standard_normal(hidden)).astype(np.float32))
        env.write("other", rng.standard_normal((b, t, hidden)).astype(np.float32))
        env.execute("'other' @ 'mean' @ 'var' @ 'gam' @ 'bet' @ 'ln' @ 1e-5 op.layernorm")
        env.write("dy", rng.standard_normal((b, t, hidden)).astype(np.float32))
        env.write("res", rng.standard_normal((b, t, hidden)).astype(np.float32))
        env.write("x", rng.standard_normal((b, t, inner)).astype(np.float32))
        env.write("w", (0.05 * rng.standard_normal((hidden, inner))).astype(np.float32))
        ln = "'dy' @ 'gam' @ 'bet' @ 'var' @ 'ln' @ 'dgam' @ 'dbet' @ 'res' @ 'din' @ 1e-5 op.layernorm_backward_add"
        lin = "'din' @ 'x' @ 'w' @ 'bias' @ 'xg' @ 'wg' @ 'bg' @ op.linear_backward"
        assert "W:op.layernorm_backward_add_linear_backward" in env.disassemble(ln + "  " + lin, fused=True)
        # a switch of the name scope between the two (the model driver goes from one block's words to the next
        # block's that way) does not hide the pair; anything else does
        assert "W:op.layernorm_backward_add_linear_backward" in env.disassemble(ln + "  0 #  " + lin, fused=True)
        assert "W:op.layernorm_backward_add_linear_backward" not in env.disassemble(ln + "  op.sync  " + lin, fused=True)
        assert "W:op.layernorm_backward_add_linear_backward" not in env.disassemble(ln + "  7  " + lin, fused=True)
        outs = ("din", "dgam", "dbet", "xg", "wg", "bg")
        zero = "  ".join("'%s' @ op.zero" % n for n in outs)
        env.execute(zero)
        env.execute(ln)
        env.execute(lin)
        want = {n: env.read(n) for n in outs}
        env.execute(zero)
        env.execute(ln + "  0 #  " + lin)
        for n in outs:
            got = env.read(n)
            if n == "bg" and mode != "f32" and hidden <= 4096:
                # the fused kernel's column sums: another fixed order
                mag = np.abs(want["din"]).reshape(-1, hidden).sum(0)
                assert np.all(np.abs(got - want[n]) <= 2e-6 * mag + 1e-30), (mode, n)
            else:
                assert np.array_equal(got, want[n]), (mode, hidden, n)
        # the linear backward of some other gradient: the word must run the pair as written
        lin2 = "'other' @ 'x' @ 'w' @ 'bias' @ 'xg' @ 'wg' @ 'bg' @ op.linear_backward"
        env.execute(zero)
        env.execute(ln)
        env.execute(lin2)
        want = {n: env.read(n) for n in outs}
        env.execute(zero)
        env.execute(ln + "  " + lin2)
        for n in outs:
            assert np.array_equal(env.read(n), want[n]), (mode, hidden, n, "unchained")
    finally:
        env.close()


def test_fused_attention_follows_the_mask_tables_prefix_rule(runtime):
    """A mask with a hole: the reference's table closes every key from the
    first zero on (train_bloom.cpp:73-90), so `bloom.valid` must report the
    length of the leading run of non-zeros, and the fused path must match the
    operator chain that reads the table."""
    hidden, heads, batch, tokens = 256, 2, 2, 32
    env, w, x, dy, mask, _ = setup_block(runtime, hidden, heads, batch, tokens, "f16")
    mask = np.ones((batch, tokens), np.int32)
    mask[0, 10] = 0          # a hole: keys 10.. are closed although 11.. are non-zero
    mask[1, 0] = 0           # nothing open at all: uniform probabilities
    env.write("mask_", mask)
    env.execute("create_operand_buffers create_flash_buffers prepare_batch_flash")
    assert list(env.read("xvalid").view(np.int32)[:batch]) == [10, 0]
    env.execute("layer_forward_flash op.sync")
    flash = env.read("xa")
    saved = blk.layer_forward(w, x, orc.alibi(heads, tokens), orc.xmask(mask), heads, 1e-5)
    assert_close(flash, saved["xa"], 2e-2, "block output against the oracle")
    env.write("xinput", x)
    env.execute("layer_forward_mixed op.sync")
    assert_close(flash, env.read("xa"), 2e-2, "block output against the operator chain")
    env.close()


def test_flash_attention_words_on_separate_and_packed_projections_agree(runtime):
    """`op.flash_attn` / `op.flash_attn_backward` take q, k, v as three
    [B, T, heads, 128] tensors, the `_qkv` forms one packed [B, T, 3H] tensor
    read through strides: same kernels, so the same bits."""
    rng = np.random.default_rng(17)
    b, t, nh, hd = 2, 48, 2, 128
    h = nh * hd
    env = host.Env(1)
    try:
        for n in ("q", "k", "v", "o", "o2", "g"):
            env.execute("%d %d %d %d 4 'cuda' 'f16' op.create '%s' !" % (b, t, nh, hd, n))
        env.execute("%d %d %d 3 'cuda' 'f16' op.create 'qkv' !" % (b, t, 3 * h))
        env.execute("%d %d %d 3 'cuda' 'float' op.create 'dqkv' !" % (b, t, 3 * h))
        for n in ("dq", "dk", "dv"):
            env.execute("%d %d %d %d 4 'cuda' 'float' op.create '%s' !" % (b, t, nh, hd, n))
        env.execute("%d %d %d 3 'cuda' 'float' op.create 'lse' !  %d %d %d 3 'cuda' 'float' op.create 'lse2' !"
                    % (b, nh, t, b, nh, t))
        env.execute("1 %d 1 %d 4 'cuda' 'float' op.create 'alibi' !  %d 1 'cuda' 'float' op.create 'valid' !" % (nh, t, b))
        env.execute("%d %d 2 'cpu' 'int' op.create 'mask' !" % (b, 1024 // b))   # cpu tensors come in 1024-item granules
        q, k, v, g = (rng.standard_normal((b, t, nh, hd)).astype(np.float16).astype(np.float32) for _ in range(4))
        for n, a in (("q", q), ("k", k), ("v", v), ("g", g)):
            env.write(n, a)
        env.write("qkv", np.concatenate([q.reshape(b, t, h), k.reshape(b, t, h), v.reshape(b, t, h)], axis=2))
        m = np.zeros((b, 1024 // b), np.int32)
        m[0, :t] = 1
        m[1, :t - 7] = 1
        env.execute("'alibi' @ bloom.alibi")
        # bloom.valid reads [batch, tokens] rows of the mask it is given: a [B, T] view of the granule-sized tensor
        env.execute("'mask' @ 0 %d %d 2 op.view 'mask_bt' !" % (b, t))
        env.write("mask_bt", np.ascontiguousarray(m[:, :t]))
        env.execute("'mask_bt' @ 'valid' @ bloom.valid")
        assert list(env.read("valid").view(np.int32)[:b]) == [t, t - 7]
        env.execute("'q' @ 'k' @ 'v' @ 'alibi' @ 'valid' @ 'o' @ 'lse' @ op.flash_attn")
        env.execute("'qkv' @ 'alibi' @ 'valid' @ 'o2' @ 'lse2' @ op.flash_attn_qkv")
        assert np.array_equal(env.read("o"), env.read("o2")) and np.array_equal(env.read("lse"), env.read("lse2"))
        assert np.all(np.isfinite(env.read("o"))) and np.any(env.read("o") != 0)
        env.execute("'q' @ 'k' @ 'v' @ 'o' @ 'g' @ 'alibi' @ 'valid' @ 'lse' @ 'dq' @ 'dk' @ 'dv' @ op.flash_attn_backward")
        env.execute("'qkv' @ 'o' @ 'g' @ 'alibi' @ 'valid' @ 'lse' @ 'dqkv' @ op.flash_attn_qkv_backward")
        packed = env.read("dqkv")
        for i, n in enumerate(("dq", "dk", "dv")):
            assert np.array_equal(packed[:, :, i * h:(i + 1) * h], env.read(n).reshape(b, t, h)), n
    finally:
        env.close()


def test_block_at_the_full_headline_size_against_oracle(runtime):
    """Config C4 exactly: hidden 4096, 32 heads x 128, FFN 16384, batch 4 x 512
    tokens, fp16 weights (the last sequence right-padded).  The oracle's block
    is computed once; the fp32-arena operator words (`block_step`) and the
    fused-attention words the benchmark quotes (`block_step_flash`) are each
    held to 2e-2 on the block output, the input gradient and every parameter
    gradient.  This is the shape where the 256x256 GEMM tiles, split-K and the
    8-key-tile attention loops run."""
    hidden, heads, batch, tokens = 4096, 32, 4, 512
    tol = 2e-2
    print("case C4 full size", flush=True)
    env, w, x, dy, mask, _ = setup_block(runtime, hidden, heads, batch, tokens, "f16")
    saved = blk.layer_forward(w, x, orc.alibi(heads, tokens), orc.xmask(mask), heads, 1e-5)
    dx_ref, g_ref = blk.layer_backward(w, saved, x, dy, heads, 1e-5)
    out_ref = saved["xa"]
    qkv_w = np.concatenate([g_ref["query.weight_g"], g_ref["key.weight_g"], g_ref["value.weight_g"]])
    qkv_b = np.concatenate([g_ref["query.bias_g"], g_ref["key.bias_g"], g_ref["value.bias_g"]])
    v_only = slice(2 * hidden, 3 * hidden)
    del saved

    def check(step_word, forward_word, what):
        print("  path", what, flush=True)
        ledger = {}
        env.write("xinput", x)
        env.write("yout_g", dy)
        env.execute("zero_layer_grad")
        env.execute(step_word + " op.sync")
        assert_close(env.read("xa"), dx_ref, tol, what + ": dx", ledger)
        for name, ref in g_ref.items():
            if name.startswith(("query.", "key.", "value.")):
                continue
            assert_close(env.read(name).reshape(ref.shape), ref, tol, what + ": " + name, ledger)
        assert_close(env.read("query_key_value.weight_g"), qkv_w, tol, what + ": query_key_value.weight_g", ledger)
        # the key third of the bias gradient is zero up to rounding; query and value thirds are checked
        got_b = env.read("query_key_value.bias_g")
        assert_close(got_b[:hidden], qkv_b[:hidden], tol, what + ": query bias_g", ledger)
        assert_close(got_b[v_only], qkv_b[v_only], tol, what + ": value bias_g", ledger)
        env.write("xinput", x)
        env.execute(forward_word + " op.sync")
        assert_close(env.read("xa"), out_ref, tol, what + ": block output", ledger)
        print_ledger("C4 block, " + what, ledger)

    check("block_step", "layer_forward", "operator words")
    env.execute("create_operand_buffers create_flash_buffers prepare_batch_flash")
    check("block_step_flash", "layer_forward_flash", "fused-attention words")
    env.close()
