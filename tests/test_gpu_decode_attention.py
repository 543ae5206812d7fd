"""GPU parity of the dense decode attention kernel (through the C ABI) against the float64
oracle of the reference's decode branch.  Bar: max|out - ref| <= 2e-3 * max(1, max|ref|) (fp16
inputs and output, fp32 scores and softmax, fp16 probabilities, fp32 accumulation); the
appended cache row is checked bit for bit."""
import numpy as np
import pytest
import torch

import lut_attention_oracle as att

pytestmark = pytest.mark.gpu
TOL = 2e-3


@pytest.fixture(scope="module")
def capi(built_lib):
    from sqamd import capi as c
    c.lib()
    return c


def make(b, h, l, d, seed, lmax=None):
    rng = np.random.default_rng(seed)
    lmax = lmax or l
    q = rng.normal(size=(b, h, d)).astype(np.float16)
    k = rng.normal(size=(b, h, lmax, d)).astype(np.float16)
    v = rng.normal(size=(b, h, lmax, d)).astype(np.float16)
    return q, k, v


def check(out, ref, what=""):
    out = out.float().cpu().numpy().astype(np.float64).reshape(ref.shape)
    assert np.all(np.isfinite(out)), what
    err = np.max(np.abs(out - ref))
    assert err <= TOL * max(1.0, np.max(np.abs(ref))), "%s: err %.3e" % (what, err)


@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("l", [1, 5, 64, 127, 640, 1000, 2049])
def test_decode_parity(capi, d, l):
    b, h = 2, 3
    q, k, v = make(b, h, l, d, seed=l + d)
    scale = 1.0 / np.sqrt(d)
    ref = att.decode_attention_ref(q, k, v, scale)
    out = capi.decode_attention(torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(),
                                l, scale)
    torch.cuda.synchronize()
    assert out.shape == (b, 1, h * d)
    check(out, ref, "d=%d l=%d" % (d, l))


def test_decode_opt67_shape_with_unused_cache_rows(capi):
    # batch 8 x 32 heads x 128, 640 of 1024 cache rows valid; the unused rows hold NaN and must not matter
    b, h, l, d, lmax = 8, 32, 640, 128, 1024
    q, k, v = make(b, h, l, d, seed=1, lmax=lmax)
    k[:, :, l:] = np.nan
    v[:, :, l:] = np.nan
    scale = 1.0 / np.sqrt(d)
    ref = att.decode_attention_ref(q, k[:, :, :l], v[:, :, :l], scale)
    kc, vc = torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda()
    out = capi.decode_attention(torch.from_numpy(q).cuda(), kc, vc, l, scale)
    check(out, ref, "host length")
    out = capi.decode_attention(torch.from_numpy(q).cuda(), kc, vc, torch.tensor([l], device="cuda"), scale)
    check(out, ref, "device length")
    # a slice of the cache, as the reference's caller passes it
    out = capi.decode_attention(torch.from_numpy(q).cuda(), kc[:, :, :l], vc[:, :, :l], l, scale)
    check(out, ref, "sliced cache")


@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("n0", [0, 3, 255, 256, 700])
def test_decode_append_writes_the_row_and_attends_it(capi, d, n0):
    b, h, lmax = 3, 4, 768
    q, k, v = make(b, h, n0 + 1, d, seed=n0 + d, lmax=lmax)
    kc, vc = torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda()
    # the new rows arrive as a strided view of a fused [b, 1, 3, h, d] projection output
    rng = np.random.default_rng(7)
    qkv = torch.from_numpy(rng.normal(size=(b, 1, 3, h, d)).astype(np.float16)).cuda()
    qg, kn, vn = (qkv[:, :, j].transpose(1, 2) for j in range(3))
    k_full, v_full = k.copy(), v.copy()
    k_full[:, :, n0] = kn.cpu().numpy().reshape(b, h, d)
    v_full[:, :, n0] = vn.cpu().numpy().reshape(b, h, d)
    scale = 1.0 / np.sqrt(d)
    ref = att.decode_attention_ref(qg.cpu().numpy().reshape(b, h, d), k_full[:, :, :n0 + 1], v_full[:, :, :n0 + 1], scale)
    out = capi.decode_attention(qg, kc, vc, torch.tensor([n0], device="cuda"), scale, k_new=kn, v_new=vn)
    torch.cuda.synchronize()
    check(out, ref, "append at %d" % n0)
    assert np.array_equal(kc.cpu().numpy(), k_full) and np.array_equal(vc.cpu().numpy(), v_full)


def test_decode_additive_mask(capi):
    b, h, l, d = 4, 2, 300, 64
    q, k, v = make(b, h, l, d, seed=11)
    rng = np.random.default_rng(12)
    mask = np.where(rng.random((b, l)) < 0.3, -np.inf, 0.0)
    mask[:, 0] = 0.0
    mask += rng.normal(size=(b, l)) * 0.1 * np.isfinite(mask)
    mask = mask.astype(np.float16)
    ref = att.decode_attention_ref(q, k, v, 0.2, mask.astype(np.float64))
    out = capi.decode_attention(torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(), l, 0.2,
                                mask=torch.from_numpy(mask).cuda().view(b, 1, 1, l))
    check(out, ref, "mask")


def test_decode_properties(capi):
    b, h, l, d = 2, 2, 333, 128
    q, k, v = make(b, h, l, d, seed=21)
    qt = torch.from_numpy(q).cuda()
    # equal keys: the mean of the value rows; constant values: the constant
    kk = np.broadcast_to(k[:, :, :1], k.shape).copy()
    out = capi.decode_attention(qt, torch.from_numpy(kk).cuda(), torch.from_numpy(v).cuda(), l, 0.1)
    p = float(np.float16(1.0 / l))
    check(out, v.astype(np.float64).sum(axis=2) * p, "equal keys")
    vv = np.full_like(v, 0.5)
    out = capi.decode_attention(qt, torch.from_numpy(k).cuda(), torch.from_numpy(vv).cuda(), l, 0.1)
    check(out, np.full((b, h, d), 0.5), "constant values")
    # a dominating key returns its value row bit for bit
    qd = np.zeros_like(q); qd[..., 0] = 8.0
    kd = np.zeros_like(k); kd[:, :, 77, 0] = 8.0
    out = capi.decode_attention(torch.from_numpy(qd).cuda(), torch.from_numpy(kd).cuda(), torch.from_numpy(v).cuda(), l, 1.0)
    assert np.array_equal(out.cpu().numpy().reshape(b, h, d), v[:, :, 77])


def test_decode_graph_replays_follow_a_growing_cache(capi):
    b, h, d, lmax, n0 = 2, 4, 128, 256, 100
    q, k, v = make(b, h, lmax, d, seed=31)
    kc, vc = torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda()
    rng = np.random.default_rng(32)
    qkv = torch.zeros((b, 1, 3, h, d), dtype=torch.float16, device="cuda")
    qg, kn, vn = (qkv[:, :, j].transpose(1, 2) for j in range(3))
    pos = torch.tensor([n0], device="cuda")
    out = torch.empty((b, 1, h * d), dtype=torch.float16, device="cuda")
    scale = 1.0 / np.sqrt(d)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            capi.decode_attention(qg, kc, vc, pos, scale, k_new=kn, v_new=vn, out=out)
    k_ref, v_ref = k.copy(), v.copy()
    for step in range(4):
        new = rng.normal(size=(b, 1, 3, h, d)).astype(np.float16)
        qkv.copy_(torch.from_numpy(new).cuda())
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        n = n0 + step
        k_ref[:, :, n] = new[:, 0, 1]
        v_ref[:, :, n] = new[:, 0, 2]
        ref = att.decode_attention_ref(new[:, 0, 0], k_ref[:, :, :n + 1], v_ref[:, :, :n + 1], scale)
        check(out, ref, "replay %d" % step)
        pos += 1
    assert np.array_equal(kc.cpu().numpy(), k_ref)


def test_decode_rejections(capi):
    L = capi.lib()
    q = torch.zeros((1, 2, 128), dtype=torch.float16, device="cuda")
    kc = torch.zeros((1, 2, 64, 128), dtype=torch.float16, device="cuda")
    with pytest.raises(capi.SqError):
        capi.decode_attention(q, kc, kc.clone(), 65, 1.0)       # more rows than the cache holds
    with pytest.raises(capi.SqError):
        capi.decode_attention(q, kc, kc.clone(), 0, 1.0)        # nothing to attend to
    with pytest.raises(capi.SqError):
        capi.decode_attention(q, kc, kc.clone(), 64, 1.0, k_new=q, v_new=q)  # no room for the new row
    q96 = torch.zeros((1, 2, 96), dtype=torch.float16, device="cuda")
    kc96 = torch.zeros((1, 2, 64, 96), dtype=torch.float16, device="cuda")
    with pytest.raises(capi.SqError):
        capi.decode_attention(q96, kc96, kc96.clone(), 64, 1.0)  # head dim
    assert L.sq_decode_attention(None, None, None, None, None, None, None, 1, 1, 128, 64, 0, 0, 0, 0, 0, 8192, 0, 1, None,
                                 1.0, None, 0, None) == capi.SQ_ERR_NULL_POINTER


def test_sparse_attention_entry_point_decode_branch(capi):
    from sqamd.block_sparse_attention_lut import sparse_attention
    b, h, l, d = 2, 4, 200, 64
    q, k, v = make(b, h, l, d, seed=41)
    mask = np.zeros((b, 1, 1, l), dtype=np.float16)
    mask[1, ..., :50] = -np.inf
    out = sparse_attention(torch.from_numpy(q).cuda().view(b, h, 1, d), torch.from_numpy(k).cuda(),
                           torch.from_numpy(v).cuda(), 0.125, None, attention_mask=torch.from_numpy(mask).cuda())
    assert out.shape == (b, h, 1, d)
    ref = att.decode_attention_ref(q, k, v, 0.125, mask.reshape(b, l).astype(np.float64))
    check(out, ref, "entry point")


def test_decoder_step_with_the_kernel_matches_the_torch_attention_path(capi):
    """Two-layer OPT-shaped decoder: a decode step through sq_decode_attention (device-side position,
    fused append) against the same step through the harness's torch attention path (host position)."""
    from sqamd.opt_decode import OPTDecoder
    model = OPTDecoder(layers=2, hidden=512, heads=4, ffn=1024, vocab=1000, max_pos=128, group=128, dev="cuda", seed=3)
    for layer in model.layers:
        layer.fuse_qkv()
    gen = torch.Generator(device="cuda")
    gen.manual_seed(4)
    ids = torch.randint(0, 1000, (3, 20), device="cuda", generator=gen)
    cache_a = model.new_cache(3, 32)
    cache_b = model.new_cache(3, 32)
    la = model(ids, cache_a, 0)
    lb = model(ids, cache_b, 0)
    assert torch.equal(la, lb)
    tok = la.argmax(-1)
    pos = torch.tensor([20], device="cuda")
    for step in range(3):
        want = model(tok, cache_a, 20 + step)
        got = model(tok, cache_b, pos, pos_ids=pos + 2)
        torch.cuda.synchronize()
        err = (got.float() - want.float()).abs().max().item()
        assert err <= 1e-2 * max(1.0, want.float().abs().max().item()), "step %d: %.3e" % (step, err)
        for (ka, va), (kb, vb) in zip(cache_a[:1], cache_b[:1]):  # layer 0 sees identical inputs
            assert torch.equal(ka, kb) and torch.equal(va, vb)
        tok = want.argmax(-1)
        pos += 1


@pytest.mark.parametrize("rows,cols", [(1, 8), (8, 4096), (3, 5120), (5, 1000), (2, 8192), (4, 16384), (4096, 4096)])
def test_layernorm_parity(capi, rows, cols):
    import w4a16_oracle as orc
    rng = np.random.default_rng(rows + cols)
    x = (rng.normal(size=(rows, cols)) * 2 + 0.5).astype(np.float16)
    gamma = rng.normal(size=cols).astype(np.float16)
    beta = rng.normal(size=cols).astype(np.float16)
    ref = orc.layernorm_ref(x, gamma, beta, 1e-5)
    xt = torch.from_numpy(x).cuda()
    out = capi.layernorm(xt, torch.from_numpy(gamma).cuda(), torch.from_numpy(beta).cuda(), 1e-5)
    torch.cuda.synchronize()
    got = out.float().cpu().numpy().astype(np.float64)
    # one rounding to fp16 at the end: half an ulp of the result, plus fp32 arithmetic noise
    tol = np.abs(ref) * 2.0 ** -11 + 1e-3
    assert np.all(np.abs(got - ref) <= tol), np.max(np.abs(got - ref))
    # without affine parameters, and in place
    ref0 = orc.layernorm_ref(x, None, None, 1e-5)
    capi.layernorm(xt, None, None, 1e-5, out=xt)
    got0 = xt.float().cpu().numpy().astype(np.float64)
    assert np.all(np.abs(got0 - ref0) <= np.abs(ref0) * 2.0 ** -11 + 1e-3)


def test_layernorm_rejections(capi):
    x = torch.zeros((2, 12), dtype=torch.float16, device="cuda")
    with pytest.raises(capi.SqError) as ei:
        capi.layernorm(x, None, None)
    assert ei.value.code == capi.SQ_ERR_BAD_SHAPE


def test_decode_long_cache(capi):
    # 40000 rows: far beyond what a score buffer in LDS could hold
    b, h, l, d = 1, 2, 40000, 64
    q, k, v = make(b, h, l, d, seed=51)
    ref = att.decode_attention_ref(q, k, v, 0.125)
    out = capi.decode_attention(torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(), l, 0.125)
    check(out, ref, "long cache")


@pytest.mark.parametrize("b,h,d,l", [(1, 32, 128, 640), (1, 4, 64, 5000), (2, 16, 128, 300), (1, 1, 128, 2049), (3, 5, 64, 129)])
def test_decode_split_over_cache_rows(capi, b, h, d, l):
    """Few heads: several workgroups share a head through the workspace; same result as one workgroup per
    head, bit-reproducible, the workspace counters back at zero, append still lands in the cache."""
    lmax = l + 3
    q, k, v = make(b, h, l, d, seed=l + h, lmax=lmax)
    scale = 1.0 / np.sqrt(d)
    rng = np.random.default_rng(l)
    kn = rng.normal(size=(b, h, d)).astype(np.float16)
    vn = rng.normal(size=(b, h, d)).astype(np.float16)
    k_full, v_full = k.copy(), v.copy()
    k_full[:, :, l] = kn
    v_full[:, :, l] = vn
    ref = att.decode_attention_ref(q, k_full[:, :, :l + 1], v_full[:, :, :l + 1], scale)
    qt = torch.from_numpy(q).cuda()
    need = capi.lib().sq_decode_attention_workspace_bytes(b, h, d)
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    outs = []
    for length in (l, torch.tensor([l], device="cuda")):   # host length: shares sized by l; device length: by Lmax
        kc, vc = torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda()
        out = capi.decode_attention(qt, kc, vc, length, scale, k_new=torch.from_numpy(kn).cuda(),
                                    v_new=torch.from_numpy(vn).cuda(), ws=ws)
        torch.cuda.synchronize()
        check(out, ref, "split b=%d h=%d l=%d" % (b, h, l))
        assert np.array_equal(kc.cpu().numpy(), k_full) and np.array_equal(vc.cpu().numpy(), v_full)
        assert torch.count_nonzero(ws[:b * h * 4]).item() == 0
        again = capi.decode_attention(qt, kc, vc, l + 1, scale, ws=ws)
        assert torch.equal(again, capi.decode_attention(qt, kc, vc, l + 1, scale, ws=ws))
        outs.append(again)
    single = capi.decode_attention(qt, torch.from_numpy(k_full).cuda(), torch.from_numpy(v_full).cuda(), l + 1, scale,
                                   use_workspace=False)
    check(single, ref, "one workgroup per head")
    for o in outs:
        assert (o.float() - single.float()).abs().max().item() <= 2e-3


def test_decode_split_with_mask_and_fully_masked_share(capi):
    # batch 1 x 8 heads, 1024 rows: 8 shares of 128 rows; the mask hides the whole of shares 2 and 5
    b, h, l, d = 1, 8, 1024, 128
    q, k, v = make(b, h, l, d, seed=61)
    mask = np.zeros((b, l), dtype=np.float16)
    mask[:, 256:384] = -np.inf
    mask[:, 640:768] = -np.inf
    mask[:, 5] = -1.5
    ref = att.decode_attention_ref(q, k, v, 0.09, mask.astype(np.float64))
    out = capi.decode_attention(torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(), l, 0.09,
                                mask=torch.from_numpy(mask).cuda())
    check(out, ref, "masked shares")


def test_decode_split_workspace_shared_across_head_counts(capi):
    """One zeroed workspace used with B*H = 128, then 32, then 128 again: the counters sit in a fixed
    region in front of the partial states, so a call with fewer heads cannot leave partial states
    where a later call with more heads reads its counters."""
    d, l, h = 128, 640, 32
    need = capi.lib().sq_decode_attention_workspace_bytes(4, h, d)
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    scale = 1.0 / np.sqrt(d)
    for b in (4, 1, 4):
        q, k, v = make(b, h, l, d, seed=70 + b)
        qt, kc, vc = torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda()
        ref = att.decode_attention_ref(q, k, v, scale)
        out = capi.decode_attention(qt, kc, vc, l, scale, ws=ws)
        single = capi.decode_attention(qt, kc, vc, l, scale, use_workspace=False)
        torch.cuda.synchronize()
        check(out, ref, "shared workspace, b=%d" % b)
        assert (out.float() - single.float()).abs().max().item() <= 2e-3
        assert torch.count_nonzero(ws[:1024]).item() == 0
