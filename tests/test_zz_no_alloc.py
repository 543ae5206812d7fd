"""The entry point that allocates nothing (sq_w4a16_gemm_static_ws): same results as
sq_w4a16_gemm_ws with a caller-owned workspace, bit for bit, and within the linear path's bar of
the oracle, on two calls in a row, the second with a smaller input; shapes beyond the static
buffer are rejected."""
import ctypes

import numpy as np
import pytest
import torch

import w4a16_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def capi(built_lib):
    from sqamd import capi as c
    c.lib()
    return c


def to_dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def test_static_workspace_entry_point_matches_the_caller_workspace_one(capi):
    g = 128
    before = torch.cuda.memory_allocated()
    # (M, N, K): split-K decode kernel on a large weight, then a smaller problem on a small weight, then a
    # K-split tiled GEMM and a shape that needs no workspace at all
    # (the last two: a single token and 2048 tokens on an lm_head-sized weight, N = 50272, which need no workspace
    # although the query for decode batches on that weight exceeds the static buffer); 24 tokens on 13824 x 5120 take
    # the tiled GEMM with K split four ways (7 MiB of partial tiles)
    cases = [(16, 8192, 4096), (20, 1024, 2048), (8, 8192, 4096), (96, 1024, 4096), (3, 512, 1024), (1, 50272, 1024),
             (2048, 50272, 1024), (24, 13824, 5120)]
    data = {}
    for m, n, k in cases:
        if (n, k) not in data:
            d = orc.synth_linear(n, k, g, seed=n + k)
            data[(n, k)] = (to_dev(d["w_l1"]), to_dev(d["zs_l1"]), orc.dequant_l1(d["w_l1"], d["zs_l1"], g))
    outs = {c: torch.empty((c[0], c[1]), dtype=torch.float16, device=DEV) for c in cases}
    xs = {c: to_dev(orc.synth_x(c[0], c[2], seed=c[0])) for c in cases}
    refs = {c: capi.gemm_ws(xs[c], data[c[1:]][0], data[c[1:]][1], c[1], c[2], g) for c in cases}
    torch.cuda.synchronize()
    held = torch.cuda.memory_allocated()
    for c in cases:  # back to back on one stream, no allocation in between
        m, n, k = c
        w, zs, _ = data[(n, k)]
        capi.gemm_static_ws(xs[c], w, zs, n, k, g, out=outs[c])
    assert torch.cuda.memory_allocated() == held
    torch.cuda.synchronize()
    for c in cases:
        m, n, k = c
        assert torch.equal(outs[c], refs[c]), "static workspace result differs at %s" % (c,)
        y_ref = orc.gemm_ref(xs[c].cpu().numpy(), data[(n, k)][2])
        err = np.max(np.abs(outs[c].float().cpu().numpy() - y_ref))
        assert err <= 1e-2 * np.max(np.abs(y_ref)), "%s: %.3e" % (c, err)
    assert before <= held


def test_static_workspace_entry_point_rejects_what_does_not_fit(capi):
    L = capi.lib()
    p = ctypes.c_void_p(4096)
    # 32 tokens on N = 32768 need 32 MiB of partial sums: beyond the static buffer
    assert L.sq_w4a16_workspace_bytes(32, 32768, 4096) > capi.SQ_STATIC_WS_BYTES
    assert L.sq_w4a16_gemm_static_ws(p, p, p, p, 32, 32768, 4096, 128, 1, 0, None) == capi.SQ_ERR_STATIC_WS
    assert L.sq_w4a16_workspace_bytes(32, 50272, 1024) > capi.SQ_STATIC_WS_BYTES  # yet one token on it is served (above)
    assert "static" in capi.strerror(capi.SQ_ERR_STATIC_WS)
    assert L.sq_w4a16_gemm_static_ws(None, p, p, p, 8, 4096, 4096, 128, 1, 0, None) == capi.SQ_ERR_NULL_POINTER
    assert L.sq_w4a16_gemm_static_ws(p, p, p, p, 8, 4096, 4096, 100, 1, 0, None) == capi.SQ_ERR_BAD_GROUP
