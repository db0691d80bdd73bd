"""Pins the integer / gather half of the path (loss-token rule, labels, group
walk, embedding gather, ALiBi table, additive mask) on the two data fixtures
the reference ships, by brute force and closed forms.  CPU only."""
import numpy as np

import oracle as orc
from conftest import assert_close

FLT_MAX = np.finfo(np.float32).max


def test_fixture_shape_and_padding(fixture_ids_mask):
    ids, mask = fixture_ids_mask
    assert ids.shape == mask.shape == (2, 512)
    assert mask.sum(1).tolist() == [48, 22]
    for b, valid in enumerate((48, 22)):
        assert np.all(mask[b, :valid] == 1) and np.all(mask[b, valid:] == 0)
        assert np.all(ids[b, valid:] == 3)          # pad id


def test_loss_labels_on_fixture(fixture_ids_mask):
    ids, mask = fixture_ids_mask
    labels, count = orc.loss_labels(ids, mask)
    assert count == (48 - 1) + (22 - 1) == 68
    for b, valid in enumerate((48, 22)):
        assert np.array_equal(labels[b, :valid - 1], ids[b, 1:valid])
        assert np.all(labels[b, valid - 1:] == -100)


def test_loss_groups_on_fixture(fixture_ids_mask):
    _, mask = fixture_ids_mask
    # 133 = 128 MiB / (250880 * 4 B), the reference's group size
    groups = orc.loss_groups(mask, 133)
    # row 0: the first group [0,133) is trimmed back to t in [0,47]; the later
    # groups are all padding and vanish.  Row 1 likewise: t in [0,21].
    assert groups.tolist() == [[0, 0, 48], [1, 0, 22]]
    # a smaller group size splits the real tokens
    assert orc.loss_groups(mask, 20).tolist() == [[0, 0, 20], [0, 20, 20], [0, 40, 8],
                                                  [1, 0, 20], [1, 20, 2]]


def test_loss_token_rule_differs_from_next_label_rule_on_holes():
    mask = np.array([[1, 1, 0, 1, 1, 0]], np.int32)
    ids = np.array([[10, 11, 12, 13, 14, 15]], np.int32)
    labels, count = orc.loss_labels(ids, mask)
    # both m[t] and m[t+1] must be set: t=0 (1,1) and t=3 (1,1) only
    assert labels.tolist() == [[11, -100, -100, 14, -100, -100]] and count == 2


def test_embedding_gather_is_row_copy(fixture_ids_mask):
    ids, _ = fixture_ids_mask
    rng = np.random.default_rng(0)
    small_ids = (ids % 997).astype(np.int32)
    vocab = rng.standard_normal((997, 32)).astype(np.float32)
    out = orc.embedding_gather(vocab, small_ids)
    assert out.shape == (2, 512, 32)
    assert np.array_equal(out, vocab[small_ids])


def test_alibi_slopes_closed_form():
    a = orc.alibi(32, 512)
    k = np.arange(512, dtype=np.float64)
    for h in (0, 1, 15, 31):
        slope = 2.0 ** (-(h + 1) / 4.0)
        assert np.array_equal(a[h], (k * slope).astype(np.float32))
    assert abs(a[0, 1] - 0.8408964) < 1e-6 and a[31, 1] == 2.0 ** -8
    # key index times slope, NOT relative distance: column 0 is zero for every head
    assert np.all(a[:, 0] == 0)
    a8 = orc.alibi(8, 4)
    assert np.array_equal(a8[:, 1], (2.0 ** -(np.arange(1, 9))).astype(np.float32))


def test_xmask_on_fixture(fixture_ids_mask):
    _, mask = fixture_ids_mask
    xm = orc.xmask(mask)
    t = 512
    for b, valid in enumerate((48, 22)):
        q, k = np.meshgrid(np.arange(t), np.arange(t), indexing="ij")
        open_ = (k <= q) & (k < valid)
        want = np.where(open_, 0.0, -FLT_MAX).astype(np.float32)
        assert np.array_equal(xm[b], want)


def test_xmask_prefix_rule_with_hole():
    mask = np.array([[1, 1, 0, 1]], np.int32)
    xm = orc.xmask(mask)[0]
    # the walk over n stops at the first zero, so key 3 stays masked although mask[3]=1
    want = np.array([[0, -FLT_MAX, -FLT_MAX, -FLT_MAX],
                     [0, 0, -FLT_MAX, -FLT_MAX],
                     [0, 0, -FLT_MAX, -FLT_MAX],
                     [0, 0, -FLT_MAX, -FLT_MAX]], np.float32)
    assert np.array_equal(xm, want)


def test_masked_softmax_equals_textbook_causal_padding_softmax(fixture_ids_mask):
    """scores + alibi + xmask -> softmax equals a masked_fill softmax with a
    relative-position ALiBi (softmax is shift invariant per row)."""
    _, mask = fixture_ids_mask
    rng = np.random.default_rng(1)
    t, heads = 64, 4
    m = mask[:, :t].copy()
    m[0, 40:] = 0
    s = rng.standard_normal((2, heads, t, t)).astype(np.float32)
    a = orc.alibi(heads, t)
    x = orc.add_bcast(orc.add_bcast(s, a.reshape(1, heads, 1, t)), orc.xmask(m).reshape(2, 1, t, t))
    p = orc.softmax_fwd(x)
    slopes = 2.0 ** (-8.0 * np.arange(1, heads + 1) / heads)
    q, k = np.meshgrid(np.arange(t), np.arange(t), indexing="ij")
    rel = (k - q)[None, None] * slopes[None, :, None, None]
    valid = m.sum(1)
    open_ = (k[None] <= q[None]) & (k[None] < valid[:, None, None])
    z = np.where(open_[:, None], s.astype(np.float64) + rel, -np.inf)
    z = z - z.max(-1, keepdims=True)
    ref = np.exp(z) / np.exp(z).sum(-1, keepdims=True)
    assert_close(p, ref, 2e-6, "masked alibi softmax")
