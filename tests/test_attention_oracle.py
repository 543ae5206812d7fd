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
