"""Pins oracle/lut_attention_oracle.py without the reference's code: known answers
worked out by hand and invariants that a wrong mask, a wrong softmax axis or a
transposed operand would break."""
import math

import numpy as np

import lut_attention_oracle as att


def test_layout_to_lut_hand_example():
    # 1 head, 4 blocks: rows keep {0}, {0,1}, {1,2}, {0,2,3} -> nnz 3, ascending, padded with the last kept index
    layout = np.zeros((1, 4, 4), dtype=bool)
    for i, cols in enumerate(([0], [0, 1], [1, 2], [0, 2, 3])):
        layout[0, i, cols] = True
    lut = att.layout_to_lut(layout)
    assert lut.dtype == np.int64
    assert lut.tolist() == [[[0, 0, 0], [0, 1, 1], [1, 2, 2], [0, 2, 3]]]
    assert np.array_equal(att.lut_to_layout(lut, 4), layout)


def test_synth_layout_properties():
    for causal in (False, True):
        lay = att.synth_layout(3, 16, 0.25, causal, seed=1)
        assert np.all(lay[:, np.arange(16), np.arange(16)])          # diagonal always kept
        if causal:
            assert not np.any(np.triu(lay, 1))
            assert np.all(lay.sum(-1) == np.minimum(4, np.arange(16) + 1))
        else:
            assert np.all(lay.sum(-1) == 4)


def test_two_key_softmax_closed_form():
    # S = 2 inside one block, D = 1: scores q*k*scale -> weights sigmoid of the score gap
    q = np.array([[[[1.0], [2.0]]]])
    k = np.array([[[[0.0], [1.0]]]])
    v = np.array([[[[10.0], [20.0]]]])
    lut = np.zeros((1, 1, 1), dtype=np.int64)
    out = att.attention_ref(q, k, v, lut, sm_scale=1.0, causal=False)[0, 0, :, 0]
    for m, qv in enumerate((1.0, 2.0)):
        w1 = 1.0 / (1.0 + math.exp(-qv))         # weight of key 1 (score qv) against key 0 (score 0)
        assert abs(out[m] - (10.0 * (1 - w1) + 20.0 * w1)) < 1e-12
    causal = att.attention_ref(q, k, v, lut, sm_scale=1.0, causal=True)[0, 0, :, 0]
    assert causal[0] == 10.0                      # query 0 sees only key 0


def test_invariants_on_random_sparse_case():
    rng = np.random.default_rng(0)
    z, h, s, d = 2, 3, 200, 8                     # ragged: 200 = 3 blocks + 8 rows
    nb = 4
    q = rng.normal(size=(z, h, s, d))
    k = rng.normal(size=(z, h, s, d))
    v = rng.normal(size=(z, h, s, d))
    lay = att.synth_layout(h, nb, 0.5, causal=False, seed=3)
    lut = att.layout_to_lut(lay)
    out = att.attention_ref(q, k, v, lut, 0.3, causal=False)
    # constant V -> constant output
    vc = np.broadcast_to(np.arange(d, dtype=np.float64), v.shape)
    assert np.allclose(att.attention_ref(q, k, vc, lut, 0.3, False), vc)
    # outputs are convex combinations of visible V rows, recomputed here row by row
    for (b, a, m) in [(0, 0, 5), (1, 2, 130), (0, 1, 199)]:
        cols = [n for j in np.flatnonzero(lay[a, m // 64]) for n in range(64 * j, min(64 * j + 64, s))]
        sc = np.array([q[b, a, m] @ k[b, a, n] for n in cols]) * 0.3
        w = np.exp(sc - sc.max())
        w /= w.sum()
        assert np.allclose(out[b, a, m], sum(wi * v[b, a, n] for wi, n in zip(w, cols)))
    # all blocks kept == plain softmax attention
    full = att.layout_to_lut(np.ones((h, nb, nb), dtype=bool))
    dense = att.attention_ref(q, k, v, full, 0.3, causal=True)
    b, a, m = 1, 1, 77
    sc = (k[b, a, :m + 1] @ q[b, a, m]) * 0.3
    w = np.exp(sc - sc.max())
    w /= w.sum()
    assert np.allclose(dense[b, a, m], w @ v[b, a, :m + 1])


def test_single_visible_key_returns_its_value_row():
    # causal, query 0 of any head sees exactly key 0
    rng = np.random.default_rng(1)
    q = rng.normal(size=(1, 2, 70, 4))
    k = rng.normal(size=(1, 2, 70, 4))
    v = rng.normal(size=(1, 2, 70, 4))
    lut = att.layout_to_lut(att.synth_layout(2, 2, 1.0, causal=True))
    out = att.attention_ref(q, k, v, lut, 1.0, causal=True)
    assert np.array_equal(out[0, :, 0], v[0, :, 0])


# ---- decode branch ----

def test_decode_equal_keys_give_mean_of_values():
    rng = np.random.default_rng(0)
    b, h, l, d = 2, 3, 8, 16  # 1/8 is exact in fp16
    q = rng.normal(size=(b, h, d))
    k = np.broadcast_to(rng.normal(size=(b, h, 1, d)), (b, h, l, d))
    v = rng.normal(size=(b, h, l, d))
    out = att.decode_attention_ref(q, k, v, 0.3)
    assert np.allclose(out, v.mean(axis=2), rtol=0, atol=1e-12)


def test_decode_dominating_key_returns_its_value_row():
    rng = np.random.default_rng(1)
    b, h, l, d = 1, 2, 37, 8
    q = np.zeros((b, h, d)); q[..., 0] = 1.0
    k = np.zeros((b, h, l, d)); k[:, :, 5, 0] = 60.0   # score gap 60 -> all other probabilities round to 0
    v = rng.normal(size=(b, h, l, d))
    out = att.decode_attention_ref(q, k, v, 1.0)
    assert np.array_equal(out, v[:, :, 5])


def test_decode_two_key_closed_form():
    # scores (a, 0): p0 = 1/(1+e^-a); P is rounded to fp16 before it meets v
    a = 0.75
    q = np.array([[[1.0, 0.0]]]); k = np.array([[[[a, 0.0], [0.0, 0.0]]]])
    v = np.array([[[[1.0, 0.0], [0.0, 1.0]]]])
    out = att.decode_attention_ref(q, k, v, 1.0)
    p0 = 1.0 / (1.0 + np.exp(-a))
    want = np.array([np.float16(p0), np.float16(1 - p0)], dtype=np.float64)
    assert np.array_equal(out[0, 0], want)


def test_decode_minus_inf_mask_equals_attention_over_remaining_rows():
    rng = np.random.default_rng(2)
    b, h, l, d = 2, 2, 21, 8
    q = rng.normal(size=(b, h, d)); k = rng.normal(size=(b, h, l, d)); v = rng.normal(size=(b, h, l, d))
    keep = np.array([0, 3, 4, 9, 20])
    mask = np.full((b, l), -np.inf); mask[:, keep] = 0.0
    got = att.decode_attention_ref(q, k, v, 0.35, mask)
    want = att.decode_attention_ref(q, k[:, :, keep], v[:, :, keep], 0.35)
    assert np.allclose(got, want, rtol=0, atol=1e-12)


def test_decode_against_elementwise_loops():
    import math
    rng = np.random.default_rng(3)
    b, h, l, d = 1, 2, 5, 4
    q = rng.normal(size=(b, h, d)); k = rng.normal(size=(b, h, l, d)); v = rng.normal(size=(b, h, l, d))
    mask = rng.normal(size=(b, l))
    got = att.decode_attention_ref(q, k, v, 0.5, mask)
    for hh in range(h):
        s = [sum(q[0, hh, t] * k[0, hh, j, t] for t in range(d)) * 0.5 + mask[0, j] for j in range(l)]
        m = max(s)
        e = [math.exp(x - m) for x in s]
        tot = sum(e)
        p = [float(np.float16(x / tot)) for x in e]
        for t in range(d):
            assert abs(got[0, hh, t] - sum(p[j] * v[0, hh, j, t] for j in range(l))) < 1e-12


def test_package_lut_builder_agrees_with_the_oracle():
    import torch
    from sqamd.lut_layout import layout2lut_single_density, synth_layout
    for causal in (False, True):
        lay = synth_layout(3, 9, 0.4, causal, seed=5)
        assert bool(lay.diagonal(dim1=1, dim2=2).all())
        if causal:
            assert not bool(torch.triu(lay, diagonal=1).any())
        lut = layout2lut_single_density(lay[None])[0]
        assert np.array_equal(lut.numpy(), att.layout_to_lut(lay.numpy()))


def test_repeated_block_after_a_different_one_counts_twice():
    """Padding rule: only an entry equal to its predecessor is skipped.  A row [1, 2, 1] therefore
    attends the keys of block 1 twice; pinned against textbook softmax attention over the explicit
    concatenation of the visited blocks.  An immediate repeat [1, 1, 2] counts block 1 once."""
    rng = np.random.default_rng(3)
    s, d, nb = 192, 16, 3
    q = rng.normal(size=(1, 1, s, d))
    k = rng.normal(size=(1, 1, s, d))
    v = rng.normal(size=(1, 1, s, d))
    blocks = lambda a, idx: np.concatenate([a[0, 0, 64 * j:64 * j + 64] for j in idx], axis=0)

    def textbook(rows, idx):
        kk, vv = blocks(k, idx), blocks(v, idx)
        sc = q[0, 0, rows] @ kk.T * 0.3
        p = np.exp(sc - sc.max(axis=-1, keepdims=True))
        return (p / p.sum(axis=-1, keepdims=True)) @ vv

    lut = np.array([[[0, 0, 0], [1, 2, 1], [1, 1, 2]]])
    counts = att.lut_to_counts(lut, nb)
    assert counts[0].tolist() == [[1, 0, 0], [0, 2, 1], [0, 1, 1]]
    out = att.attention_ref(q, k, v, lut, 0.3, False)
    assert np.allclose(out[0, 0, 64:128], textbook(slice(64, 128), [1, 2, 1]), rtol=1e-12, atol=1e-12)
    assert np.allclose(out[0, 0, 128:192], textbook(slice(128, 192), [1, 2]), rtol=1e-12, atol=1e-12)
    assert np.allclose(out[0, 0, :64], textbook(slice(0, 64), [0]), rtol=1e-12, atol=1e-12)
    # more entries than key blocks: only the first nb are read
    lut4 = np.array([[[0, 1, 2, 0], [1, 1, 1, 0], [2, 2, 2, 2]]])
    assert att.lut_to_counts(lut4, nb)[0].tolist() == [[1, 1, 1], [0, 1, 0], [0, 0, 1]]


def test_row_without_visible_key_is_nan():
    # causal, query block 0 pointed at key block 1 only: nothing visible
    rng = np.random.default_rng(4)
    q = rng.normal(size=(1, 1, 128, 8))
    lut = np.array([[[1], [1]]])
    with np.errstate(invalid="ignore"):
        out = att.attention_ref(q, q, q, lut, 1.0, True)
    assert np.all(np.isnan(out[0, 0, :64])) and np.all(np.isfinite(out[0, 0, 64:]))
