"""A whole BLOOM model (embedding LayerNorm, blocks, final LayerNorm, tied LM
head with the shift-by-one masked loss) stepped through the product path on
the GPU by the C++ driver, compared with the CPU oracle's composition
(oracle/bloom_model.py) on the same weights, ids and mask.

  fp32 mode: fp32 weights, fp32 MFMA products; bound 2e-4 (a chain of
             3 x ~20 fp32 operators plus the head, each within 1e-5)
  f16 mode:  fp16 weights, fp16 MFMA products, fp32 accumulation; bound 2e-2
  bf16 mode: bf16 weights and products; bound 1e-1 (8 times coarser rounding)
"""
import numpy as np
import pytest

import oracle as orc
from oracle import bloom_block as blk
from oracle import bloom_model as mdl
from conftest import assert_close, assert_rows_close, print_ledger
from blackriver_amd import host

pytestmark = pytest.mark.gpu

MODEL_NAMES = ["word_embeddings.weight", "word_embeddings_layernorm.weight", "word_embeddings_layernorm.bias",
               "ln_f.weight", "ln_f.bias"]


def build(mode, layers, batch, tokens, hidden, heads, vocab, seed, std=0.05, read_layers=True):
    rng = np.random.default_rng(seed)
    wdtype = {"f16": "f16", "bf16": "bf16"}.get(mode, "float")
    model = host.BloomModel(layers, batch, tokens, hidden, heads, vocab, 1e-5, wdtype,
                            wdtype if wdtype != "float" else "f32")
    model.init(seed, std)
    # LayerNorm parameters and biases away from their 1 / 0 defaults
    for i in range(1, layers + 1):
        for name in ("input_layernorm", "post_attention_layernorm"):
            model.write(i, name + ".weight", 1 + 0.1 * rng.standard_normal(hidden))
            model.write(i, name + ".bias", 0.1 * rng.standard_normal(hidden))
        model.write(i, "query_key_value.bias", 0.05 * rng.standard_normal(3 * hidden))
        model.write(i, "dense_h_to_4h.bias", 0.05 * rng.standard_normal(4 * hidden))
    model.write(0, "ln_f.weight", 1 + 0.1 * rng.standard_normal(hidden))
    model.write(0, "word_embeddings_layernorm.bias", 0.1 * rng.standard_normal(hidden))
    # the oracle sees the weights exactly as the device holds them
    model_w = {n: model.read(0, n) for n in MODEL_NAMES}
    layer_ws = [{n: model.read(i, n) for n in blk.WEIGHT_NAMES} for i in range(1, layers + 1)] if read_layers else None
    ids = rng.integers(0, vocab, (batch, tokens)).astype(np.int32)
    mask = np.ones((batch, tokens), np.int32)
    mask[-1, tokens - tokens // 4:] = 0
    return model, model_w, layer_ws, ids, mask


@pytest.mark.parametrize("mode,layers,batch,tokens,hidden,heads,vocab", [
    ("fp32", 3, 2, 32, 256, 4, 1024),
    ("f16", 2, 2, 64, 512, 8, 2048),
    ("f16", 2, 2, 64, 512, 4, 2048),      # head size 128: attention runs as the fused kernels
    ("bf16", 2, 2, 64, 512, 4, 2048),     # the same in bf16 (8-bit mantissa; see the bound below)
    # config C5's shapes with two of its thirty blocks: one 512-token sequence, hidden 4096, 32 heads,
    # the 250880-word tied table (products with M = 512: few output tiles, split along K; one logits
    # row per position)
    ("f16", 2, 1, 512, 4096, 32, 250880),
])
def test_model_step_matches_oracle(runtime, mode, layers, batch, tokens, hidden, heads, vocab):
    print("case %s layers=%d batch=%d tokens=%d hidden=%d" % (mode, layers, batch, tokens, hidden), flush=True)
    # the full-width case takes config C5's N(0, 0.02) matrices; at hidden 4096 a standard deviation of 0.05
    # gives attention scores of +-10 and probabilities whose fp16-operand error alone exceeds the bound
    std = 0.02 if hidden >= 4096 else 0.05
    model, model_w, layer_ws, ids, mask = build(mode, layers, batch, tokens, hidden, heads, vocab, seed=7, std=std)
    # bf16: one block holds 6e-2 (tests/test_gpu_block.py); two blocks, the head and the tied
    # table's gradient (a sum of two bf16-product results) compound to just under 1e-1
    tol = {"fp32": 2e-4, "f16": 2e-2, "bf16": 1e-1}[mode]
    ledger = {}
    try:
        # different initial matrices per block (a seed slip would make them equal)
        assert not np.array_equal(layer_ws[0]["dense.weight"], layer_ws[1]["dense.weight"])
        assert 0.6 * std < float(np.std(layer_ws[0]["dense_h_to_4h.weight"])) < 1.4 * std
        loss = model.step(ids, mask)
        ref_loss, ref = mdl.model_step(model_w, layer_ws, ids, mask, heads, 1e-5)
        assert abs(loss - ref_loss) <= tol * abs(ref_loss), (loss, ref_loss)
        for i in range(1, layers + 1):
            for name in blk.WEIGHT_NAMES:
                if name == "key.bias":      # zero up to rounding (softmax shift invariance)
                    continue
                assert_close(model.read(i, name + "_g"), ref[i][name + "_g"], tol, "block %d %s_g" % (i, name), ledger)
        for name in ("ln_f.weight", "ln_f.bias", "word_embeddings_layernorm.weight", "word_embeddings_layernorm.bias"):
            assert_close(model.read(0, name + "_g"), ref[0][name + "_g"], tol, name + "_g", ledger)
        # The tied table's gradient: rows of the batch's ids (the scattered embedding-row gradients on top
        # of the head's) and all other rows (the head's alone) are held to the bound separately, each
        # against its own scale -- at 250880 rows the rms of the whole table says nothing about the
        # few hundred rows the scatter touches.
        table, table_ref = model.read(0, "word_embeddings.weight_g"), ref[0]["word_embeddings.weight_g"]
        touched = np.zeros(vocab, bool)
        touched[ids.reshape(-1)] = True
        assert_close(table[touched], table_ref[touched], tol, "word_embeddings.weight_g, rows of the batch", ledger)
        if vocab * hidden < (1 << 28):
            assert_close(table[~touched], table_ref[~touched], tol, "word_embeddings.weight_g, other rows", ledger)
        else:
            # a billion entries: the bound is held row by row, as a pure relative one (see assert_rows_close); the
            # largest single-entry error is recorded next to it, against the usual bound, for the record only
            assert_rows_close(table[~touched], table_ref[~touched], tol, "word_embeddings.weight_g, other rows (by row)",
                              ledger)
            assert_close(table[~touched], table_ref[~touched], 2 * tol,
                         "word_embeddings.weight_g, other rows (largest entry, of 4e-2)", ledger)
        del table, table_ref
        # activation gradients are left carrying the step's gradient lift (a power of two; 1 in fp32 mode)
        lift = model.grad_lift()
        assert lift == (1.0 if mode == "fp32" else 16.0 * 2 ** int(np.ceil(np.log2(orc.loss_labels(ids, mask)[1]))))
        assert_close(model.read(0, "xc") / np.float32(lift), ref[0]["embedding_rows_g"], tol,
                     "gradient of the embedding rows", ledger)
        print_ledger("model step %s hidden %d" % (mode, hidden), ledger)
        # the head is tied to the table: one gradient tensor under both names
        assert np.array_equal(model.read(0, "lm_head.weight_g"), model.read(0, "word_embeddings.weight_g"))
        # a second step on the same batch: gradients are overwritten, the head's
        # accumulator is cleared, so everything repeats exactly
        g1 = model.read(0, "lm_head.weight_g")
        d1 = model.read(1, "dense.weight_g")
        loss2 = model.step(ids, mask)
        assert loss2 == loss
        assert np.array_equal(model.read(0, "lm_head.weight_g"), g1)
        assert np.array_equal(model.read(1, "dense.weight_g"), d1)
    finally:
        model.close()


@pytest.mark.timeout(900)
def test_full_depth_model_step_against_oracle(runtime):
    """BLOOM-7B1 at its real depth: 30 blocks, hidden 4096, 32 heads, the
    250880-word tied table, one 512-token sequence whose last 0..64 tokens are
    masked, fp16 weights ~N(0, 0.02), seed 4.  The oracle runs the forward pass
    through all thirty blocks and the backward pass of the head, the final
    LayerNorm and block 30 (a full backward pass on the host cores would take
    several minutes more and add nothing a two-block case does not cover);
    what depth adds -- error growth of the fp16 forward over 30 blocks, thirty
    arenas chained by name, the gradient lift carried down 30 backward blocks --
    shows in the loss, in the gradients next to the head and in every block's
    gradients being finite, non-zero and bit-repeatable."""
    layers, batch, tokens, hidden, heads, vocab = 30, 1, 512, 4096, 32, 250880
    print("case f16 layers=30 batch=1 tokens=512 hidden=4096 vocab=250880", flush=True)
    model, model_w, _, ids, _ = build("f16", layers, batch, tokens, hidden, heads, vocab, seed=4, std=0.02,
                                      read_layers=False)
    rng = np.random.default_rng(4)
    mask = np.ones((batch, tokens), np.int32)
    masked = int(rng.integers(0, 65))
    if masked:
        mask[0, tokens - masked:] = 0
    tol, ledger = 2e-2, {}
    try:
        loss = model.step(ids, mask)
        # oracle forward, one block's weights on the host at a time
        alibi, xmask = orc.alibi(heads, tokens), orc.xmask(mask)
        rows = orc.embedding_gather(model_w["word_embeddings.weight"], ids.reshape(-1)).reshape(batch, tokens, hidden)
        x, _, _ = orc.layernorm_fwd(rows, model_w["word_embeddings_layernorm.weight"],
                                    model_w["word_embeddings_layernorm.bias"], 1e-5)
        for i in range(1, layers + 1):
            w = {n: model.read(i, n) for n in blk.WEIGHT_NAMES}
            last_in, saved = x, blk.layer_forward(w, x, alibi, xmask, heads, 1e-5)
            x = saved["xa"]
            print("oracle forward: block %d" % i, flush=True)
        # the device's block outputs chain by name: block 30's output is hash 0's xa before the head overwrote it,
        # so the forward pass is compared through the loss and through the final LayerNorm's input statistics
        y, _, f_var = orc.layernorm_fwd(x, model_w["ln_f.weight"], model_w["ln_f.bias"], 1e-5)
        ref_loss, y_g, head_g, _ = orc.loss_backward(y, ids, mask, model_w["word_embeddings.weight"])
        assert abs(loss - ref_loss) <= tol * abs(ref_loss), (loss, ref_loss)
        ledger["loss"] = abs(loss - ref_loss) / (tol * abs(ref_loss))
        dx, lnw_g, lnb_g = orc.layernorm_bwd(y_g, y, model_w["ln_f.weight"], model_w["ln_f.bias"], f_var, 1e-5)
        assert_close(model.read(0, "ln_f.weight_g"), lnw_g, tol, "ln_f.weight_g", ledger)
        assert_close(model.read(0, "ln_f.bias_g"), lnb_g, tol, "ln_f.bias_g", ledger)
        # Block 30's gradients against the oracle's own chain: the two chains enter block 30 thirty-odd fp16
        # roundings per element apart (29 blocks of forward pass), which the attention scores amplify, so these
        # are held to three times the single-block bound -- a block fed the same input on both sides is held to
        # 2e-2 itself by the two-block case above and by tests/test_gpu_block.py at full size.  Ratios below are
        # fractions of 6e-2 (measured: 0.65 for key.weight_g and 0.53 for query.weight_g, the two tensors that
        # sit behind the softmax; under 0.2 for every other one, i.e. inside 2e-2 even across the depth).
        _, g30 = blk.layer_backward(w, saved, last_in, dx, heads, 1e-5)
        deep = {}
        for name in blk.WEIGHT_NAMES:
            if name == "key.bias":
                continue
            assert_close(model.read(layers, name + "_g"), g30[name + "_g"], 3 * tol, "block 30 %s_g" % name, deep)
        print_ledger("full-depth model step, block 30 against the oracle's chain (fractions of 6e-2)", deep, top=16)
        del saved, g30, w
        # rows of the tied table that no position of the batch looks up hold the head's gradient alone
        table = model.read(0, "word_embeddings.weight_g")
        touched = np.zeros(vocab, bool)
        touched[ids.reshape(-1)] = True
        assert_rows_close(table[~touched], head_g[~touched], tol, "word_embeddings.weight_g, rows outside the batch (by row)",
                          ledger)
        del head_g
        print_ledger("full-depth model step", ledger, top=8)
        # every block's gradients arrived: finite and not all zero, all the way down
        first = {}
        for i in range(1, layers + 1):
            g = model.read(i, "dense.weight_g")
            assert np.all(np.isfinite(g)) and float(np.abs(g).max()) > 0.0, "block %d dense.weight_g" % i
            if i in (1, 15, 30):
                first[i] = g
        emb_g = model.read(0, "word_embeddings_layernorm.weight_g")
        assert np.all(np.isfinite(emb_g)) and float(np.abs(emb_g).max()) > 0.0
        # a second step on the same batch repeats bit for bit
        assert model.step(ids, mask) == loss
        assert np.array_equal(model.read(0, "word_embeddings.weight_g"), table)
        for i, g in first.items():
            assert np.array_equal(model.read(i, "dense.weight_g"), g), "block %d dense.weight_g differs on a second step" % i
    finally:
        model.close()


@pytest.mark.parametrize("mode", ["fp32", "f16"])
def test_adamw_updates_every_parameter_and_training_raises_the_log_probability(runtime, mode):
    """After one step + optimizer step every parameter tensor equals the
    oracle's AdamW applied to the gradients the device holds (wiring: names,
    master copies, step count); repeating on one batch raises the mean
    log-probability of its labels."""
    layers, batch, tokens, hidden, heads, vocab = 2, 2, 32, 256, 4, 512
    model, model_w, layer_ws, ids, mask = build(mode, layers, batch, tokens, hidden, heads, vocab, seed=9)
    lr, b1, b2, eps, wd = 2e-3, 0.9, 0.95, 1e-8, 0.01
    names0 = ["word_embeddings.weight", "word_embeddings_layernorm.weight", "word_embeddings_layernorm.bias",
              "ln_f.weight", "ln_f.bias"]
    names_i = ["input_layernorm.weight", "input_layernorm.bias", "post_attention_layernorm.weight",
               "post_attention_layernorm.bias", "query_key_value.weight", "query_key_value.bias", "dense.weight",
               "dense.bias", "dense_h_to_4h.weight", "dense_h_to_4h.bias", "dense_4h_to_h.weight", "dense_4h_to_h.bias"]
    every = [(0, n) for n in names0] + [(i, n) for i in range(1, layers + 1) for n in names_i]
    try:
        model.create_optimizer(lr, b1, b2, eps, wd)
        before = {k: model.read(*k) for k in every}
        first = model.step(ids, mask)
        model.optimizer_step()
        for k in every:
            g = model.read(k[0], k[1] + "_g")
            want, m, v = orc.adamw_step(before[k], g, np.zeros_like(g), np.zeros_like(g), lr, b1, b2, eps, wd, 1)
            got = model.read(*k)
            assert not np.array_equal(got, before[k]), k
            matrix16 = mode == "f16" and k[1].endswith(".weight") and "layernorm" not in k[1] and "ln_f" not in k[1]
            if matrix16:
                assert_close(model.read(k[0], k[1] + "_w32"), want, 1e-5, "%d %s master" % k)
                assert np.array_equal(got, model.read(k[0], k[1] + "_w32").astype(np.float16).astype(np.float32))
            else:
                assert_close(got, want, 1e-5, "%d %s" % k)
            assert_close(model.read(k[0], k[1] + "_m"), m, 1e-5, "%d %s first moment" % k)
        losses = [first]
        for _ in range(8):
            losses.append(model.step(ids, mask))
            model.optimizer_step()
        assert losses[-1] > losses[0] + 0.5, losses      # log-probability rises
        assert all(np.isfinite(losses))
    finally:
        model.close()
