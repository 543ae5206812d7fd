"""CPU oracle for the LUT block-sparse attention.  TEST INFRASTRUCTURE ONLY.

Restates in numpy what the reference's prefill kernel computes
(sparse-attention/nvidia/playground/kernels/block_sparse_attention_lut.py:22-172):
for query block i of head h, softmax over the keys of the 64-wide key blocks
lut[h, i, :NNZ] of q.k^T * sm_scale, optionally causal, times v -- i.e. dense
attention under the mask the LUT describes (test/nvidia/module/mask/
sparse_attention.py:562-595, layout_to_mask).  The kernel's online softmax, its
base-2 exponentials and its fp16 roundings of q*scale and p are implementation
detail; the oracle computes the same quantity in float64.

Pinning (tests/test_attention_oracle.py): hand-written LUT known answer; a two-key
softmax with weights known in closed form; single-visible-key rows return that V
row exactly; constant V returns the constant; an all-blocks LUT equals unmasked
softmax attention computed with a different formulation (per-row loops); a row that names
a block again after a different one equals textbook attention over the concatenation of the
visited blocks' keys and values (the block counted twice), while an immediate repeat counts once.
A row without any visible key is 0/0 = NaN here; the reference's running sums give NaN as well.
decode_attention_ref restates the decode branch of the same entry point (:272-300): dense
attention of one query row over the whole cache, softmax in fp32, probabilities cast to fp16
before the product with v.  Pinning: equal keys give the mean of v; a dominating key returns
its v row; -inf mask entries equal attention over the remaining rows; a per-element Python
loop formulation on a small case; the two-key closed form.
No function here is "parity unpinned".
"""
import numpy as np

BLOCK = 64


def layout_to_lut(layout):
    """bool [H, nb, nb] -> int64 [H, nb, nnz], nnz = max kept blocks over all rows.

    Follows layout2lut_single_density (test/nvidia/module/mask/sparse_attention.py:
    509-539): each row lists its kept key-block indices in ascending order and is
    right-padded with the largest kept index of that row.
    """
    layout = np.asarray(layout, dtype=bool)
    h, nb, _ = layout.shape
    nnz = int(layout.sum(axis=-1).max())
    lut = np.zeros((h, nb, nnz), dtype=np.int64)
    for a in range(h):
        for i in range(nb):
            idx = np.flatnonzero(layout[a, i])
            assert idx.size > 0, "every query block must keep at least one key block"
            row = np.full(nnz, idx[-1], dtype=np.int64)
            row[:idx.size] = idx
            lut[a, i] = row
    return lut


def lut_to_counts(lut, nb):
    """int [H, nb, nnz] -> int64 [H, nb, nb]: how often the kernel's loop visits key block j for
    query block i.  At most nb entries of a row are read and an entry is skipped only when it
    equals its predecessor in the row (block_sparse_attention_lut.py:96,134,163: last_nnz_id
    starts at -1 and p is multiplied by last_nnz_id != present_nnz_id), so a block that shows up
    again after a different one is visited, and weighted, again.  Entries outside [0, nb) select
    keys beyond the sequence, which the kernel masks completely."""
    lut = np.asarray(lut)
    h = lut.shape[0]
    counts = np.zeros((h, nb, nb), dtype=np.int64)
    visit = min(lut.shape[-1], nb)
    for a in range(h):
        for i in range(nb):
            last = -1
            for j in lut[a, i, :visit]:
                j = int(j)
                if j != last and 0 <= j < nb:
                    counts[a, i, j] += 1
                last = j
    return counts


def lut_to_layout(lut, nb):
    """int [H, nb, nnz] -> bool [H, nb, nb]: the key blocks a row visits at least once."""
    return lut_to_counts(lut, nb) > 0


def synth_layout(h, nb, density, causal, seed=0):
    """Diagonal block always kept; the rest sampled uniformly without replacement so
    that every row keeps round(density * nb) blocks (at least 1; at most i+1 if causal)."""
    rng = np.random.default_rng(seed)
    layout = np.zeros((h, nb, nb), dtype=bool)
    keep = max(1, int(round(density * nb)))
    for a in range(h):
        for i in range(nb):
            cand = np.arange(i) if causal else np.delete(np.arange(nb), i)
            extra = min(keep - 1, cand.size)
            layout[a, i, i] = True
            if extra > 0:
                layout[a, i, rng.choice(cand, size=extra, replace=False)] = True
    return layout


def attention_ref(q, k, v, lut, sm_scale, causal):
    """q, k, v float [Z,H,S,D]; lut int [H, ceil(S/64), nnz] -> float64 [Z,H,S,D]."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    z, h, s, d = q.shape
    nb = (s + BLOCK - 1) // BLOCK
    counts = lut_to_counts(lut, nb)
    weight = np.repeat(np.repeat(counts, BLOCK, axis=1), BLOCK, axis=2)[:, :s, :s].astype(np.float64)
    if causal:
        weight = weight * np.tril(np.ones((s, s)))[None]
    mask = weight > 0
    out = np.empty_like(q)
    for b in range(z):
        scores = np.einsum("hmd,hnd->hmn", q[b], k[b]) * sm_scale
        scores = np.where(mask, scores, -np.inf)
        scores -= scores.max(axis=-1, keepdims=True)
        p = np.exp(scores) * weight  # a key block visited c times enters the running sums c times
        p /= p.sum(axis=-1, keepdims=True)
        out[b] = np.einsum("hmn,hnd->hmd", p, v[b])
    return out


def decode_attention_ref(q, k, v, sm_scale, mask=None):
    """q float [B,H,D]; k, v float [B,H,L,D]; mask None or additive float [B,L] -> float64 [B,H,D].

    Follows block_sparse_attention_lut.py:279-298: weights = q k^T * sm_scale (+ mask), softmax,
    cast of the probabilities to fp16, product with v."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    w = np.einsum("bhd,bhld->bhl", q, k) * sm_scale
    if mask is not None:
        w = w + np.asarray(mask, dtype=np.float64)[:, None, :]
    w = w - w.max(axis=-1, keepdims=True)
    p = np.exp(w)
    p /= p.sum(axis=-1, keepdims=True)
    p = p.astype(np.float16).astype(np.float64)
    return np.einsum("bhl,bhld->bhd", p, v)
