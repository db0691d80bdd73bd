"""CPU oracle of one whole-model training step (TEST INFRASTRUCTURE ONLY, like
everything under oracle/): embedding gather + embedding LayerNorm, N decoder
blocks, final LayerNorm, LM-head loss, and the backward chain, composed from
the operator restatements exactly as BlackRiver's model script composes them
(bloomz-7b/train.words:250-318 for rank 0's head and tail, :137-248 per block),
plus the gradient of the embedding table, which the reference keeps frozen.

Pinned by: the per-operator checks of the functions it calls, and a central
finite difference of the whole loss with respect to a few weights
(tests/test_oracle_model.py)."""
import numpy as np

import oracle as orc
from oracle import bloom_block as blk


def model_step(model_w, layer_ws, ids, mask, heads, eps=1e-5):
    """model_w: word_embeddings.weight [V,H] (the LM head is tied to it),
    word_embeddings_layernorm.{weight,bias}, ln_f.{weight,bias}.
    Returns (loss, grads) with grads[0] the model-level and grads[i] block i's."""
    ids = np.ascontiguousarray(ids, np.int32)
    mask = np.ascontiguousarray(mask, np.int32)
    b, t = ids.shape
    emb = model_w["word_embeddings.weight"]
    h = emb.shape[1]
    alibi = orc.alibi(heads, t)
    xmask = orc.xmask(mask)
    # train.words:264-268: gathered rows -> embedding LayerNorm -> first block's input
    rows = orc.embedding_gather(emb, ids.reshape(-1)).reshape(b, t, h)
    x, _, emb_var = orc.layernorm_fwd(rows, model_w["word_embeddings_layernorm.weight"],
                                      model_w["word_embeddings_layernorm.bias"], eps)
    emb_y = x
    saved, inputs = [], []
    for w in layer_ws:
        inputs.append(x)
        s = blk.layer_forward(w, x, alibi, xmask, heads, eps)
        saved.append(s)
        x = s["xa"]
    # train.words:305-311: final LayerNorm, loss head, LayerNorm backward
    y, _, f_var = orc.layernorm_fwd(x, model_w["ln_f.weight"], model_w["ln_f.bias"], eps)
    loss, y_g, head_g, _ = orc.loss_backward(y, ids, mask, emb)
    g0 = {"lm_head.weight_g": head_g}
    dx, g0["ln_f.weight_g"], g0["ln_f.bias_g"] = orc.layernorm_bwd(y_g, y, model_w["ln_f.weight"], model_w["ln_f.bias"],
                                                                   f_var, eps)
    grads = [None] * (len(layer_ws) + 1)
    for i in range(len(layer_ws) - 1, -1, -1):
        dx, grads[i + 1] = blk.layer_backward(layer_ws[i], saved[i], inputs[i], dx, heads, eps)
    dx, g0["word_embeddings_layernorm.weight_g"], g0["word_embeddings_layernorm.bias_g"] = orc.layernorm_bwd(
        dx, emb_y, model_w["word_embeddings_layernorm.weight"], model_w["word_embeddings_layernorm.bias"], emb_var, eps)
    g0["embedding_rows_g"] = dx
    # the table is tied: its gradient is the head's plus the scatter of the row gradients
    g0["word_embeddings.weight_g"] = orc.embedding_scatter_add(head_g, dx.reshape(-1, h), ids.reshape(-1))
    grads[0] = g0
    return loss, grads
