"""GPU parity of sq_w4a16_gemv_sequence (several decode linears in one persistent launch) against the
CPU oracle and against the one-launch-per-linear path.  Bar as for every linear:
max|Y - Y_ref| <= 1e-2 * max|Y_ref| against the oracle's fp32 result; repeated launches are bit-identical."""
import ctypes

import numpy as np
import pytest
import torch

import w4a16_oracle as orc

pytestmark = pytest.mark.gpu
TOL = 1e-2
DEV = "cuda:0"


@pytest.fixture(scope="module")
def capi(built_lib):
    from sqamd import capi as c
    c.lib()
    return c


def to_dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def make_linear(n, k, g, seed, scale_mul=1.0):
    d = orc.synth_linear(n, k, g, seed=seed)
    if scale_mul != 1.0:
        d["s"] = (d["s"].astype(np.float32) * scale_mul).astype(np.float16)
        d["zs_l1"] = orc.zeros_scales_l1(d["z"], d["s"])
    d["w_hat"] = orc.dequant_l1(d["w_l1"], d["zs_l1"], g)
    d["w_dev"], d["zs_dev"] = to_dev(d["w_l1"]), to_dev(d["zs_l1"])
    return d


def rel_err(y, y_ref):
    y = np.asarray(y, dtype=np.float64)
    assert np.all(np.isfinite(y))
    return float(np.max(np.abs(y - y_ref)) / max(np.max(np.abs(y_ref)), 1e-30))


def oracle_linear(x, d, bias=None, residual=None, act=0):
    y = orc.gemm_ref(x, d["w_hat"]).astype(np.float64)
    if bias is not None:
        y = y + bias.astype(np.float64)[None, :]
    if act:
        y = np.maximum(y, 0.0)
    if residual is not None:
        y = y + residual.astype(np.float64)
    return y


@pytest.mark.parametrize("m", [1, 2, 3, 4])
def test_independent_linears_of_mixed_shapes(capi, m):
    """Linears that share nothing: ragged N, K that is no multiple of the 2048-wide sub-unit, every group size."""
    shapes = [(200, 1536, 64), (1024, 2048, 128), (72, 32, 32), (2056, 4096, 128), (264, 704, 32), (8, 6144, 64)]
    lin, xs, ys, refs = [], [], [], []
    for idx, (n, k, g) in enumerate(shapes):
        d = make_linear(n, k, g, seed=10 * m + idx)
        x = orc.synth_x(m, k, seed=50 + idx)
        xs.append(to_dev(x))
        ys.append(torch.full((m, n), float("nan"), dtype=torch.float16, device=DEV))
        refs.append(oracle_linear(x, d))
        lin.append(dict(x=xs[-1], w=d["w_dev"], zs=d["zs_dev"], y=ys[-1], n=n, k=k, group_size=g))
    seq = capi.LinearSequence(lin, m, DEV)
    seq.run()
    torch.cuda.synchronize()
    for y, ref, sh in zip(ys, refs, shapes):
        assert rel_err(y.float().cpu().numpy(), ref) <= TOL, sh
    assert seq.error_flag() == 0 and capi.workspace_is_clean(seq.ws)  # counters; partial tiles may stay
    first = [y.clone() for y in ys]
    seq.run()
    torch.cuda.synchronize()
    for y, f in zip(ys, first):
        assert torch.equal(y, f)


@pytest.mark.parametrize("mode", ["auto", "one_launch"])
@pytest.mark.parametrize("m", [1, 2, 3, 4])
def test_dependent_chain_with_epilogues(capi, m, mode):
    """y0 = relu(x W0 + b0); y1 = y0 W1 + b1 + x; y2 = y1 W2; y3 = relu(y1 W3) + y2: every linear consumes what an
    earlier one of the same launch wrote (input and residual), against the same chain through the oracle with
    every intermediate rounded to fp16 as the kernel stores it."""
    h, f, g = 1024, 3072, 128
    d0, d1 = make_linear(f, h, g, 1, 0.2), make_linear(h, f, g, 2, 0.2)
    d2, d3 = make_linear(h, h, g, 3, 0.2), make_linear(h, h, g, 4, 0.2)
    rng = np.random.default_rng(5)
    b0 = rng.normal(0, 0.5, size=f).astype(np.float16)
    b1 = rng.normal(0, 0.5, size=h).astype(np.float16)
    x = orc.synth_x(m, h, seed=6)
    f16 = lambda a: a.astype(np.float16)
    r0 = f16(oracle_linear(x, d0, bias=b0, act=1))
    r1 = f16(oracle_linear(r0, d1, bias=b1, residual=x))
    r2 = f16(oracle_linear(r1, d2))
    r3 = oracle_linear(r1, d3, residual=r2, act=1)
    xd = to_dev(x)
    y = [torch.full((m, n), float("nan"), dtype=torch.float16, device=DEV) for n in (f, h, h, h)]
    lin = [dict(x=xd, w=d0["w_dev"], zs=d0["zs_dev"], y=y[0], n=f, k=h, group_size=g, bias=to_dev(b0), act=capi.SQ_ACT_RELU),
           dict(x=y[0], w=d1["w_dev"], zs=d1["zs_dev"], y=y[1], n=h, k=f, group_size=g, bias=to_dev(b1), residual=xd,
                depends=True),
           dict(x=y[1], w=d2["w_dev"], zs=d2["zs_dev"], y=y[2], n=h, k=h, group_size=g, depends=True),
           dict(x=y[1], w=d3["w_dev"], zs=d3["zs_dev"], y=y[3], n=h, k=h, group_size=g, residual=y[2], act=capi.SQ_ACT_RELU,
                depends=True)]
    seq = capi.LinearSequence(lin, m, DEV, mode=capi.SQ_SEQ_ONE_LAUNCH if mode == "one_launch" else capi.SQ_SEQ_AUTO)
    for rep in range(3):
        for t in y:
            t.fill_(float("nan"))
        seq.run()
        torch.cuda.synchronize()
        assert rel_err(y[0].float().cpu().numpy(), r0.astype(np.float64)) <= TOL
        assert rel_err(y[1].float().cpu().numpy(), r1.astype(np.float64)) <= TOL
        assert rel_err(y[2].float().cpu().numpy(), r2.astype(np.float64)) <= TOL
        assert rel_err(y[3].float().cpu().numpy(), r3) <= TOL
    assert seq.error_flag() == 0 and capi.workspace_is_clean(seq.ws)  # counters; partial tiles may stay
    # the same chain with one launch per linear (no workspace: the fallback inside the entry point)
    y2 = [torch.empty_like(t) for t in y]
    lin2 = [dict(l) for l in lin]
    lin2[0]["y"], lin2[1]["y"], lin2[2]["y"], lin2[3]["y"] = y2
    lin2[1]["x"], lin2[2]["x"], lin2[3]["x"], lin2[3]["residual"] = y2[0], y2[1], y2[1], y2[2]
    capi.LinearSequence(lin2, m, DEV, workspace=False).run()
    torch.cuda.synchronize()
    for a, b in zip(y, y2):
        assert (a.float() - b.float()).abs().max().item() <= 2e-2 * max(1.0, b.float().abs().max().item())


@pytest.mark.parametrize("mode", ["auto", "one_launch"])
@pytest.mark.parametrize("m", [1, 4])
def test_opt67_layer_linears_in_one_launch(capi, m, mode):
    """The six linears of an OPT-6.7B decoder layer (group 128): q/k/v share their input; out_proj, fc1 and fc2
    are marked as depending on earlier outputs (as in the layer).  Oracle on sampled output rows of each."""
    g = 128
    shapes = [(4096, 4096), (4096, 4096), (4096, 4096), (4096, 4096), (16384, 4096), (4096, 16384)]
    depends = [False, False, False, True, True, True]
    rng = np.random.default_rng(9)
    x4 = orc.synth_x(m, 4096, seed=1)
    x16 = orc.synth_x(m, 16384, seed=2)
    gen = torch.Generator(device=DEV)
    gen.manual_seed(3)
    lin, ys, checks = [], [], []
    xs = {4096: to_dev(x4), 16384: to_dev(x16)}
    for idx, (n, k) in enumerate(shapes):
        w = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device=DEV, generator=gen)
        z = torch.randint(0, 16, (n, k // g), device=DEV, generator=gen).half() + 64
        s = (torch.randn((n, k // g), device=DEV, generator=gen).abs() * 0.02 + 1e-3).half()
        zs = torch.stack([z, s], dim=-1).reshape(n, 2 * (k // g)).contiguous()
        y = torch.full((m, n), float("nan"), dtype=torch.float16, device=DEV)
        ys.append(y)
        lin.append(dict(x=xs[k], w=w, zs=zs, y=y, n=n, k=k, group_size=g, depends=depends[idx]))
        rows = np.sort(rng.choice(n, size=96, replace=False))
        rows[0], rows[-1] = 0, n - 1
        ridx = torch.from_numpy(rows).to(DEV)
        w_hat = orc.dequant_l1(w[ridx].cpu().numpy(), zs[ridx].cpu().numpy(), g)
        checks.append((rows, orc.gemm_ref(x4 if k == 4096 else x16, w_hat)))
    seq = capi.LinearSequence(lin, m, DEV, mode=capi.SQ_SEQ_ONE_LAUNCH if mode == "one_launch" else capi.SQ_SEQ_AUTO)
    seq.run()
    torch.cuda.synchronize()
    for y, (rows, ref), sh in zip(ys, checks, shapes):
        assert torch.isfinite(y).all(), sh
        assert rel_err(y[:, torch.from_numpy(rows).to(DEV)].float().cpu().numpy(), ref) <= 5e-3, sh
    # one launch per linear through the product dispatch gives the same numbers up to summation order
    for l, y in zip(lin, ys):
        single = capi.gemm(l["x"], l["w"], l["zs"], l["n"], l["k"], g)
        assert (single.float() - y.float()).abs().max().item() <= 5e-3 * y.float().abs().max().item()
    # HIP-graph replays of the launch: same bits every time, counters back at zero
    first = [y.clone() for y in ys]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        seq.run(stream=side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            seq.run(stream=side)
    for rep in range(4):
        for y in ys:
            y.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for y, f in zip(ys, first):
            assert torch.equal(y, f)
    assert seq.error_flag() == 0 and capi.workspace_is_clean(seq.ws)  # counters; partial tiles may stay


def _chained_opt_layer(capi, m, seed=11, x_scale=1.0 / 64):
    """The six linears of an OPT-6.7B decoder layer wired as a chain of real buffers: q, k, v read x; out_proj reads
    q's output, fc1 (ReLU, bias) reads out_proj's, fc2 reads fc1's and adds out_proj's output as residual."""
    g = 128
    shapes = [(4096, 4096), (4096, 4096), (4096, 4096), (4096, 4096), (16384, 4096), (4096, 16384)]
    gen = torch.Generator(device=DEV)
    gen.manual_seed(seed)
    x = (torch.randn((m, 4096), device=DEV, generator=gen) * x_scale).half()
    ys = [torch.full((m, n), float("nan"), dtype=torch.float16, device=DEV) for n, _ in shapes]
    xin = [x, x, x, ys[0], ys[3], ys[4]]
    lin = []
    for idx, (n, k) in enumerate(shapes):
        w = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device=DEV, generator=gen)
        z = torch.randint(0, 16, (n, k // g), device=DEV, generator=gen).half() + 64
        s = (torch.randn((n, k // g), device=DEV, generator=gen).abs() * 0.02 + 1e-3).half()
        zs = torch.stack([z, s], dim=-1).reshape(n, 2 * (k // g)).contiguous()
        lin.append(dict(x=xin[idx], w=w, zs=zs, y=ys[idx], n=n, k=k, group_size=g, depends=idx >= 3))
    lin[4]["bias"] = (torch.randn(16384, device=DEV, generator=gen) * 0.1).half()
    lin[4]["act"] = capi.SQ_ACT_RELU
    lin[5]["residual"] = ys[3]
    return lin, ys, x


def _check_chain_against_oracle(lin, rng, tol=5e-3):
    """Every linear against the oracle on sampled output rows, fed with the input the device actually read."""
    for l in lin:
        n, k, g = l["n"], l["k"], l["group_size"]
        rows = np.sort(rng.choice(n, size=64, replace=False))
        rows[0], rows[-1] = 0, n - 1
        ridx = torch.from_numpy(rows).to(DEV)
        w_hat = orc.dequant_l1(l["w"][ridx].cpu().numpy(), l["zs"][ridx].cpu().numpy(), g)
        ref = orc.gemm_ref(l["x"].cpu().numpy(), w_hat).astype(np.float64)
        if l.get("bias") is not None:
            ref = ref + l["bias"][ridx].float().cpu().numpy()[None, :]
        if l.get("act"):
            ref = np.maximum(ref, 0.0)
        if l.get("residual") is not None:
            ref = ref + l["residual"][:, ridx].float().cpu().numpy()
        assert torch.isfinite(l["y"]).all()
        assert rel_err(l["y"][:, ridx].float().cpu().numpy(), ref) <= tol, (n, k)


@pytest.mark.parametrize("m", [1, 2, 3, 4])
def test_opt67_layer_chained_in_one_launch(capi, m):
    """The decoder layer's linears with their real data flow in ONE persistent launch: the outputs that later
    linears read travel between workgroups as tagged words.  Oracle per linear on the inputs the device read;
    eager launches and HIP-graph replays give the same bits; the launch counter advances, nothing times out."""
    lin, ys, _ = _chained_opt_layer(capi, m)
    seq = capi.LinearSequence(lin, m, DEV, mode=capi.SQ_SEQ_ONE_LAUNCH)
    seq.run()
    torch.cuda.synchronize()
    _check_chain_against_oracle(lin, np.random.default_rng(m))
    first = [y.clone() for y in ys]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        seq.run(stream=side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            seq.run(stream=side)
    for rep in range(4):
        for y in ys:
            y.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for y, f in zip(ys, first):
            assert torch.equal(y, f)
    assert seq.error_flag() == 0 and capi.workspace_is_clean(seq.ws)
    # the same chain through a launch per dependent linear
    lin2, ys2, _ = _chained_opt_layer(capi, m)
    capi.LinearSequence(lin2, m, DEV, mode=capi.SQ_SEQ_AUTO).run()
    torch.cuda.synchronize()
    for a, b in zip(ys, ys2):
        assert (a.float() - b.float()).abs().max().item() <= 1e-2 * max(b.float().abs().max().item(), 1e-3)


def test_one_launch_gives_up_cleanly(capi):
    """With no polls allowed, a wait for another workgroup's output gives up at once: the launch still ends, the
    sticky error word is reported, the split-K counters in front of it stay zero and a split-K launch on the same
    workspace is right; after the word is cleared and polls are allowed again the same sequence is right."""
    m = 2  # (with 3 or 4 tokens the activations of fc2 leave no room for the weight ring: launch per linear)
    lin, ys, x = _chained_opt_layer(capi, m)
    seq = capi.LinearSequence(lin, m, DEV, mode=capi.SQ_SEQ_ONE_LAUNCH)
    try:
        capi.sequence_tune(spin_limit=0)
        seq.run()
        torch.cuda.synchronize()
    finally:
        capi.sequence_tune()
    assert seq.error_flag() == 1
    assert capi.workspace_is_clean(seq.ws)
    # a split-K decode launch (8 tokens, K = 16384) on the same workspace
    l5 = lin[5]
    x8 = (torch.randn((8, 16384), device=DEV) * 0.1).half()
    y8 = capi.gemm_ws(x8, l5["w"], l5["zs"], 4096, 16384, 128, ws=seq.ws)
    torch.cuda.synchronize()
    rows = torch.arange(0, 4096, 67, device=DEV)
    ref = orc.gemm_ref(x8.cpu().numpy(), orc.dequant_l1(l5["w"][rows].cpu().numpy(), l5["zs"][rows].cpu().numpy(), 128))
    assert rel_err(y8[:, rows].float().cpu().numpy(), ref.astype(np.float64)) <= 5e-3
    assert capi.workspace_is_clean(seq.ws)
    assert seq.error_flag(clear=True) == 1 and seq.error_flag() == 0
    for y in ys:
        y.fill_(float("nan"))
    seq.run()
    torch.cuda.synchronize()
    _check_chain_against_oracle(lin, np.random.default_rng(0))
    assert seq.error_flag() == 0


@pytest.mark.parametrize("m", [5, 8, 16, 32])
def test_grouped_launch_for_decode_batches(capi, m):
    """5..32 tokens: q, k and v (three weights, one input) share one launch of the split-K decode kernel, a
    dependent linear follows in a launch of its own; against the oracle on sampled rows and against one
    sq_w4a16_gemm_ws launch per linear (same kernel, same arithmetic: bit-identical)."""
    g, h = 128, 4096
    rng = np.random.default_rng(m)
    x = orc.synth_x(m, h, seed=60 + m)
    xd = to_dev(x)
    gen = torch.Generator(device=DEV)
    gen.manual_seed(m)
    lin, ys, checks = [], [], []
    for idx, n in enumerate((4096, 4096, 4096, 2112)):
        w = torch.randint(0, 256, (n, h // 2), dtype=torch.uint8, device=DEV, generator=gen)
        z = torch.randint(0, 16, (n, h // g), device=DEV, generator=gen).half() + 64
        s = (torch.randn((n, h // g), device=DEV, generator=gen).abs() * 0.02 + 1e-3).half()
        zs = torch.stack([z, s], dim=-1).reshape(n, 2 * (h // g)).contiguous()
        y = torch.full((m, n), float("nan"), dtype=torch.float16, device=DEV)
        bias = (torch.randn(n, device=DEV, generator=gen) * 0.5).half() if idx == 1 else None
        ys.append(y)
        lin.append(dict(x=xd, w=w, zs=zs, y=y, n=n, k=h, group_size=g, bias=bias, depends=(idx == 3)))
        rows = np.sort(rng.choice(n, size=64, replace=False))
        ridx = torch.from_numpy(rows).to(DEV)
        ref = orc.gemm_ref(x, orc.dequant_l1(w[ridx].cpu().numpy(), zs[ridx].cpu().numpy(), g)).astype(np.float64)
        if bias is not None:
            ref = ref + bias[ridx].float().cpu().numpy()[None, :]
        checks.append((ridx, ref))
    seq = capi.LinearSequence(lin, m, DEV)
    assert seq.ws.numel() >= capi.lib().sq_w4a16_workspace_bytes(m, 3 * 4096, h)
    for rep in range(2):
        seq.run()
        torch.cuda.synchronize()
        for y, (ridx, ref) in zip(ys, checks):
            assert torch.isfinite(y).all()
            assert rel_err(y[:, ridx].float().cpu().numpy(), ref) <= 5e-3
        assert capi.workspace_is_clean(seq.ws)
    for l, y in zip(lin, ys):
        single = capi.gemm_fused(l["x"], l["w"], l["zs"], l["n"], l["k"], g, bias=l["bias"])
        assert (single.float() - y.float()).abs().max().item() <= 5e-3 * y.float().abs().max().item()
    # without a workspace the same call launches linear by linear
    ys2 = [torch.empty_like(y) for y in ys]
    lin2 = [dict(l, y=y2) for l, y2 in zip(lin, ys2)]
    capi.LinearSequence(lin2, m, DEV, workspace=False).run()
    torch.cuda.synchronize()
    for a, b in zip(ys, ys2):
        assert (a.float() - b.float()).abs().max().item() <= 5e-3 * b.float().abs().max().item()


def test_llama_mlp_shapes_and_more_than_four_tokens(capi):
    g = 128
    d1, d2 = make_linear(11008, 4096, g, 21), make_linear(4096, 11008, g, 22, 0.05)
    for m in (2, 6):  # 6 tokens: served by one launch per linear inside the entry point
        x = orc.synth_x(m, 4096, seed=m)
        r1 = oracle_linear(x, d1, act=1).astype(np.float16)
        r2 = oracle_linear(r1, d2)
        xd = to_dev(x)
        y1 = torch.empty((m, 11008), dtype=torch.float16, device=DEV)
        y2 = torch.empty((m, 4096), dtype=torch.float16, device=DEV)
        seq = capi.LinearSequence([dict(x=xd, w=d1["w_dev"], zs=d1["zs_dev"], y=y1, n=11008, k=4096, group_size=g,
                                        act=capi.SQ_ACT_RELU),
                                   dict(x=y1, w=d2["w_dev"], zs=d2["zs_dev"], y=y2, n=4096, k=11008, group_size=g,
                                        depends=True)], m, DEV, mode=capi.SQ_SEQ_ONE_LAUNCH)
        seq.run()
        torch.cuda.synchronize()
        assert rel_err(y1.float().cpu().numpy(), r1.astype(np.float64)) <= TOL
        assert rel_err(y2.float().cpu().numpy(), r2) <= TOL
        assert seq.error_flag() == 0


def test_sequence_rejections(capi):
    L = capi.lib()
    p = 4096
    descs = (capi.LinearDesc * 2)()
    for d in descs:
        d.x = d.w = d.zs = d.y = p
        d.N, d.K, d.group_size = 64, 128, 64
    ws = ctypes.c_void_p(p)
    call = lambda count, m, layout=1, mode=0: L.sq_w4a16_gemv_sequence(descs, count, m, layout, mode, ws, 256, None)
    # 64 KiB for the split-K kernels' counters, then the one-launch kernel's control block (nothing to exchange here)
    assert L.sq_w4a16_gemv_sequence_workspace_bytes(descs, 2, 1) == 65536 + 256
    assert call(2, 1, mode=5) == capi.SQ_ERR_BAD_ALGO
    assert call(9, 1) == capi.SQ_ERR_BAD_SHAPE
    assert call(0, 1) == capi.SQ_OK
    assert call(2, 0) == capi.SQ_OK
    assert call(2, 1, layout=2) == capi.SQ_ERR_BAD_LAYOUT
    descs[1].group_size = 48
    assert call(2, 1) == capi.SQ_ERR_BAD_GROUP
    descs[1].group_size = 64
    descs[1].y = None
    assert call(2, 1) == capi.SQ_ERR_NULL_POINTER
    descs[1].y = p + 2
    assert call(2, 1) == capi.SQ_ERR_MISALIGNED
    descs[1].y = p
    descs[0].act = 7
    assert call(2, 1) == capi.SQ_ERR_BAD_ALGO
    assert L.sq_w4a16_gemv_sequence(None, 2, 1, 1, 0, ws, 256, None) == capi.SQ_ERR_NULL_POINTER
