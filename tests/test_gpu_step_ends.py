"""GPU tests of the launches around the quantised layers of a greedy decode step (sq_embed_rows, sq_f16_gemv,
sq_greedy_feedback) and of the harness step that uses them.  Bars: the embedding sum is bit-exact against
torch's fp16 gather + add; the fp16 product satisfies max|y - y_ref| <= 1e-2 * max|y_ref| against the float64
product of the same fp16 operands; the chosen token is exactly the first index of the largest stored logit."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def capi(built_lib):
    from sqamd import capi as c
    c.lib()
    return c


@pytest.mark.parametrize("rows,hidden", [(1, 64), (3, 4096), (8, 4096), (8, 5120)])
def test_embed_rows_bit_exact(capi, rows, hidden):
    g = torch.Generator(device=DEV)
    g.manual_seed(rows + hidden)
    vocab, positions = 1000, 300
    embed = torch.randn((vocab, hidden), device=DEV, generator=g).half()
    table = torch.randn((positions, hidden), device=DEV, generator=g).half()
    tok = torch.randint(0, vocab, (rows,), device=DEV, generator=g)
    for p in (0, 17, positions - 3):
        pos = torch.tensor([p], device=DEV, dtype=torch.long)
        out = capi.embed_rows(embed, table, tok, pos, 2)
        ref = embed[tok] + table[p + 2]
        assert torch.equal(out, ref)
    # indices outside the tables are clamped, not followed
    out = capi.embed_rows(embed, table, torch.full((rows,), vocab + 5, device=DEV), torch.tensor([positions + 9], device=DEV), 0)
    assert torch.equal(out, (embed[vocab - 1] + table[positions - 1]).expand(rows, hidden))


@pytest.mark.parametrize("m", [1, 2, 4, 5, 8])
@pytest.mark.parametrize("n,k", [(50272, 4096), (1000, 512), (33, 1024), (4096, 8192), (257, 1536), (8200, 2048)])
def test_f16_gemv_and_greedy_choice(capi, m, n, k):
    g = torch.Generator(device=DEV)
    g.manual_seed(m * 7 + n + k)
    w = (torch.randn((n, k), device=DEV, generator=g) * 0.05).half()
    x = torch.randn((m, k), device=DEV, generator=g).half()
    parts = capi.f16_gemv_parts(n, DEV)
    y = capi.f16_gemv(x, w, parts=parts)
    ref = x.double() @ w.double().t()
    err = (y.double() - ref).abs().max().item()
    assert err <= 1e-2 * ref.abs().max().item()
    assert torch.equal(y, capi.f16_gemv(x, w))  # the candidates are a by-product, not another product
    tok = torch.full((m,), -1, device=DEV, dtype=torch.long)
    pos = torch.tensor([40], device=DEV, dtype=torch.long)
    step = torch.tensor([1], device=DEV, dtype=torch.long)
    hist = torch.full((3, m), -7, device=DEV, dtype=torch.long)
    capi.greedy_feedback(parts, m, tok, pos=pos, history=hist, step=step)
    torch.cuda.synchronize()
    assert torch.equal(tok, y.float().argmax(-1))
    assert pos.item() == 41 and step.item() == 2
    assert torch.equal(hist[1], tok) and (hist[0] == -7).all() and (hist[2] == -7).all()
    # a step beyond the history writes nothing there
    step.fill_(3)
    capi.greedy_feedback(parts, m, tok, history=hist, step=step)
    torch.cuda.synchronize()
    assert (hist[0] == -7).all() and (hist[2] == -7).all() and step.item() == 4 and pos.item() == 41


def test_greedy_choice_takes_the_first_of_equal_logits(capi):
    n, k, m = 5000, 512, 3
    g = torch.Generator(device=DEV)
    g.manual_seed(5)
    w = (torch.randn((n, k), device=DEV, generator=g) * 0.05).half()
    x = torch.randn((m, k), device=DEV, generator=g).half()
    y0 = capi.f16_gemv(x, w)
    best = y0.float().argmax(-1)
    # copies of token 0's winning row further down and further up: equal logits in several workgroups
    r = int(best[0])
    for dup in (r + 1, r + 40, n - 1, max(r - 33, 0)):
        if 0 <= dup < n:
            w[dup] = w[r]
    parts = capi.f16_gemv_parts(n, DEV)
    y = capi.f16_gemv(x, w, parts=parts)
    tok = torch.zeros((m,), device=DEV, dtype=torch.long)
    capi.greedy_feedback(parts, m, tok)
    torch.cuda.synchronize()
    yf = y.float()
    for i in range(m):
        first = int((yf[i] == yf[i].max()).nonzero()[0])
        assert int(tok[i]) == first


def test_step_ends_rejections(capi):
    L = capi.lib()
    x = torch.zeros((9, 512), device=DEV, dtype=torch.float16)
    w = torch.zeros((64, 512), device=DEV, dtype=torch.float16)
    y = torch.zeros((9, 64), device=DEV, dtype=torch.float16)
    assert L.sq_f16_gemv(x.data_ptr(), w.data_ptr(), y.data_ptr(), None, None, 9, 64, 512, None) == capi.SQ_ERR_BAD_SHAPE
    assert L.sq_f16_gemv(x.data_ptr(), w.data_ptr(), y.data_ptr(), None, None, 4, 64, 640, None) == capi.SQ_ERR_BAD_SHAPE
    assert L.sq_f16_gemv(x.data_ptr(), w.data_ptr(), y.data_ptr(), y.data_ptr(), None, 4, 64, 512, None) == capi.SQ_ERR_NULL_POINTER
    assert L.sq_f16_gemv(None, w.data_ptr(), y.data_ptr(), None, None, 4, 64, 512, None) == capi.SQ_ERR_NULL_POINTER
    assert L.sq_embed_rows(w.data_ptr(), w.data_ptr(), x.data_ptr(), x.data_ptr(), 0, y.data_ptr(), 2, 252, 64, 64, None) == capi.SQ_ERR_BAD_SHAPE
    assert L.sq_greedy_feedback(y.data_ptr(), y.data_ptr(), 4, 9, x.data_ptr(), None, None, None, 0, None) == capi.SQ_ERR_BAD_SHAPE
    assert L.sq_greedy_feedback(y.data_ptr(), None, 4, 2, x.data_ptr(), None, None, None, 0, None) == capi.SQ_ERR_NULL_POINTER


def test_harness_step_with_library_ends_generates_the_same_tokens(capi):
    """The greedy step whose ends are library launches (graph replay) against the step whose ends are torch ops
    (eager): same tokens.  The logits of the two differ only in the order of fp32 sums."""
    from sqamd import opt_decode
    a = opt_decode.run_e2e(batch=8, prompt=64, new_tokens=10, layers=2, use_graph=False, return_tokens=True,
                           lut_density=None, fused_ends=False)
    b = opt_decode.run_e2e(batch=8, prompt=64, new_tokens=10, layers=2, use_graph=True, return_tokens=True,
                           lut_density=None, fused_ends=True)
    c = opt_decode.run_e2e(batch=8, prompt=64, new_tokens=10, layers=2, use_graph=False, return_tokens=True,
                           lut_density=None, fused_ends=True)
    assert torch.equal(b["tokens"], c["tokens"])
    assert torch.equal(a["tokens"], b["tokens"])
