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
from conftest import assert_close
from blackriver_amd import host

pytestmark = pytest.mark.gpu

MODEL_NAMES = ["word_embeddings.weight", "word_embeddings_layernorm.weight", "word_embeddings_layernorm.bias",
               "ln_f.weight", "ln_f.bias"]


def build(mode, layers, batch, tokens, hidden, heads, vocab, seed, std=0.05):
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
    layer_ws = [{n: model.read(i, n) for n in blk.WEIGHT_NAMES} for i in range(1, layers + 1)]
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
                assert_close(model.read(i, name + "_g"), ref[i][name + "_g"], tol, "block %d %s_g" % (i, name))
        for name in ("ln_f.weight", "ln_f.bias", "word_embeddings_layernorm.weight", "word_embeddings_layernorm.bias"):
            assert_close(model.read(0, name + "_g"), ref[0][name + "_g"], tol, name + "_g")
        # The tied table's gradient: rows of the batch's ids (the scattered embedding-row gradients on top
        # of the head's) and all other rows (the head's alone) are held to the bound separately, each
        # against its own scale -- at 250880 rows the rms of the whole table says nothing about the
        # few hundred rows the scatter touches.
        table, table_ref = model.read(0, "word_embeddings.weight_g"), ref[0]["word_embeddings.weight_g"]
        touched = np.zeros(vocab, bool)
        touched[ids.reshape(-1)] = True
        assert_close(table[touched], table_ref[touched], tol, "word_embeddings.weight_g, rows of the batch")
        assert_close(table[~touched], table_ref[~touched], tol, "word_embeddings.weight_g, other rows")
        del table, table_ref
        # activation gradients are left carrying the step's gradient lift (a power of two; 1 in fp32 mode)
        lift = model.grad_lift()
        assert lift == (1.0 if mode == "fp32" else 16.0 * 2 ** int(np.ceil(np.log2(orc.loss_labels(ids, mask)[1]))))
        assert_close(model.read(0, "xc") / np.float32(lift), ref[0]["embedding_rows_g"], tol,
                     "gradient of the embedding rows")
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
