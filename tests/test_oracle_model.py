"""Pins the oracle's whole-model composition (oracle/bloom_model.py: embedding
LayerNorm, blocks, final LayerNorm, tied LM head, shift-by-one masked loss and
the backward chain) against a textbook BLOOM written with torch fp64 ops and
differentiated by autograd.  CPU only.

Reference conventions accounted for: the loss is the MEAN LOG-PROBABILITY of
the labels (positive-log-prob sign), a position counts iff its own and the next
mask entry are non-zero, and LayerNorm backward adds eps twice (a 1e-5-scale
relative effect, inside the 1e-4 bound)."""
import numpy as np
import torch

from oracle import bloom_block as blk
from oracle import bloom_model as mdl
from conftest import assert_close
from test_oracle_block import textbook_block


def test_model_step_against_textbook_autograd():
    rng = np.random.default_rng(11)
    b, t, h, heads, v, layers, eps = 2, 10, 32, 4, 48, 2, 1e-5
    layer_ws = [blk.make_weights(rng, h, std=0.2) for _ in range(layers)]
    model_w = {
        "word_embeddings.weight": (0.5 * rng.standard_normal((v, h))).astype(np.float32),
        "word_embeddings_layernorm.weight": (1 + 0.1 * rng.standard_normal(h)).astype(np.float32),
        "word_embeddings_layernorm.bias": (0.1 * rng.standard_normal(h)).astype(np.float32),
        "ln_f.weight": (1 + 0.1 * rng.standard_normal(h)).astype(np.float32),
        "ln_f.bias": (0.1 * rng.standard_normal(h)).astype(np.float32),
    }
    ids = rng.integers(0, v, (b, t)).astype(np.int32)
    mask = np.ones((b, t), np.int32)
    mask[1, 7:] = 0

    F = torch.nn.functional
    mt = {k: torch.tensor(a.astype(np.float64), requires_grad=True) for k, a in model_w.items()}
    lt = [{k: torch.tensor(a.astype(np.float64), requires_grad=True) for k, a in w.items()} for w in layer_ws]
    rows = mt["word_embeddings.weight"][torch.tensor(ids.astype(np.int64))]
    rows.retain_grad()
    x = F.layer_norm(rows, (h,), mt["word_embeddings_layernorm.weight"], mt["word_embeddings_layernorm.bias"], eps)
    for w in lt:
        x = textbook_block(w, x, heads, mask, eps)
    y = F.layer_norm(x, (h,), mt["ln_f.weight"], mt["ln_f.bias"], eps)
    logp = torch.log_softmax(y @ mt["word_embeddings.weight"].T, -1)
    total, count = 0.0, 0
    for bi in range(b):
        for ti in range(t - 1):
            if mask[bi, ti] and mask[bi, ti + 1]:
                total = total + logp[bi, ti, int(ids[bi, ti + 1])]
                count += 1
    loss_t = total / count
    # the reference's head produces gradients of MINUS the mean log-probability
    (-loss_t).backward()

    loss, grads = mdl.model_step(model_w, layer_ws, ids, mask, heads, eps)
    assert abs(loss - float(loss_t.detach())) < 1e-5 * abs(float(loss_t.detach()))
    for i in range(layers):
        for name in blk.WEIGHT_NAMES:
            if name == "key.bias":
                continue
            assert_close(grads[i + 1][name + "_g"], lt[i][name].grad.numpy(), 2e-4, "layer %d %s" % (i, name))
    for name in ("ln_f.weight", "ln_f.bias", "word_embeddings_layernorm.weight", "word_embeddings_layernorm.bias"):
        assert_close(grads[0][name + "_g"], mt[name].grad.numpy(), 2e-4, name)
    assert_close(grads[0]["embedding_rows_g"], rows.grad.numpy(), 2e-4, "embedding rows gradient")
    # tied table: autograd's gradient = head part + scatter of the row gradients
    head = mt["word_embeddings.weight"].grad.numpy().copy()
    np.subtract.at(head, ids.reshape(-1), rows.grad.numpy().reshape(-1, h))
    assert_close(grads[0]["lm_head.weight_g"], head, 2e-4, "lm_head gradient")
    assert_close(grads[0]["word_embeddings.weight_g"], mt["word_embeddings.weight"].grad.numpy(), 2e-4,
                 "tied table gradient")
