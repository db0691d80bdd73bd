"""A whole BLOOM model (embedding LayerNorm, blocks, final LayerNorm, tied LM
head with the shift-by-one masked loss) stepped through the product path on
the GPU by the C++ driver, compared with the CPU oracle's composition
(oracle/bloom_model.py) on the same weights, ids and mask.

  fp32 mode: fp32 weights, fp32 MFMA products; bound 2e-4 (a chain of
             3 x ~20 fp32 operators plus the head, each within 1e-5)
  f16 mode:  fp16 weights, fp16 MFMA products, fp32 accumulation; bound 2e-2
"""
import numpy as np
import pytest

from oracle import bloom_block as blk
from oracle import bloom_model as mdl
from conftest import assert_close
from blackriver_amd import host

pytestmark = pytest.mark.gpu

MODEL_NAMES = ["word_embeddings.weight", "word_embeddings_layernorm.weight", "word_embeddings_layernorm.bias",
               "ln_f.weight", "ln_f.bias"]


def build(mode, layers, batch, tokens, hidden, heads, vocab, seed):
    rng = np.random.default_rng(seed)
    f16 = mode == "f16"
    model = host.BloomModel(layers, batch, tokens, hidden, heads, vocab, 1e-5, "f16" if f16 else "float",
                            "f16" if f16 else "f32")
    model.init(seed, 0.05)
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
])
def test_model_step_matches_oracle(runtime, mode, layers, batch, tokens, hidden, heads, vocab):
    print("case %s layers=%d batch=%d tokens=%d hidden=%d" % (mode, layers, batch, tokens, hidden), flush=True)
    model, model_w, layer_ws, ids, mask = build(mode, layers, batch, tokens, hidden, heads, vocab, seed=7)
    tol = 2e-4 if mode == "fp32" else 2e-2
    try:
        # different initial matrices per block (a seed slip would make them equal)
        assert not np.array_equal(layer_ws[0]["dense.weight"], layer_ws[1]["dense.weight"])
        assert 0.03 < float(np.std(layer_ws[0]["dense_h_to_4h.weight"])) < 0.07
        loss = model.step(ids, mask)
        ref_loss, ref = mdl.model_step(model_w, layer_ws, ids, mask, heads, 1e-5)
        assert abs(loss - ref_loss) <= tol * abs(ref_loss), (loss, ref_loss)
        for i in range(1, layers + 1):
            for name in blk.WEIGHT_NAMES:
                if name == "key.bias":      # zero up to rounding (softmax shift invariance)
                    continue
                assert_close(model.read(i, name + "_g"), ref[i][name + "_g"], tol, "block %d %s_g" % (i, name))
        for name in ("ln_f.weight", "ln_f.bias", "word_embeddings_layernorm.weight",
                     "word_embeddings_layernorm.bias", "word_embeddings.weight"):
            assert_close(model.read(0, name + "_g"), ref[0][name + "_g"], tol, name + "_g")
        assert_close(model.read(0, "xc"), ref[0]["embedding_rows_g"], tol, "gradient of the embedding rows")
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
