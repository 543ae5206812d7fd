"""Block layouts and look-up tables for the LUT attention: host-side mirror of the reference's
mask utilities (test/nvidia/module/mask/sparse_attention.py:509-539, layout2lut_single_density)."""
import torch


def layout2lut_single_density(layout):
    """bool [layers, H, nb, nb] -> tuple of int64 [H, nb, nnz] per layer.

    Each row lists its kept key-block indices in ascending order and is right-padded with the
    largest kept index of the row; nnz is the largest number of kept blocks in any row of the layer."""
    assert layout.dim() == 4, "The layout should have 4 dimensions: (layer, num_heads, num_block, num_block)"
    nb = layout.shape[-1]
    cols = torch.arange(nb, device=layout.device)
    luts = ()
    for lay in layout.bool():
        nnz = int(lay.sum(dim=-1).max().item())
        last = torch.where(lay, cols, torch.full_like(cols, -1)).max(dim=-1, keepdim=True)[0]
        assert int(last.min().item()) >= 0, "every query block must keep at least one key block"
        keyed = torch.where(lay, cols.expand_as(lay), last.expand_as(lay))
        luts += (torch.sort(keyed, dim=-1)[0][..., :nnz].to(torch.int64).contiguous(),)
    return luts


def synth_layout(heads, nb, density, causal=False, seed=0):
    """bool [H, nb, nb]: the diagonal block always kept, the others sampled uniformly without replacement
    so that a row keeps round(density * nb) blocks (at least 1, at most i + 1 when causal)."""
    gen = torch.Generator().manual_seed(seed)
    keep = max(1, int(round(density * nb)))
    layout = torch.zeros((heads, nb, nb), dtype=torch.bool)
    for a in range(heads):
        for i in range(nb):
            layout[a, i, i] = True
            cand = torch.arange(i) if causal else torch.cat([torch.arange(i), torch.arange(i + 1, nb)])
            extra = min(keep - 1, cand.numel())
            if extra > 0:
                layout[a, i, cand[torch.randperm(cand.numel(), generator=gen)[:extra]]] = True
    return layout
