"""GPU parity of the streaming decode kernel (SQ_ALGO_STREAM: up to 16 tokens, group size 128 or 64) against the
CPU oracle, through the C ABI: every workgroup shape and K split it can be launched with, ragged row counts,
K ranges that do not fill a workgroup's chunk slots, the fused epilogue, the grouped launch behind
sq_w4a16_gemv_sequence, and the properties that do not depend on the size (determinism, exact doubling,
one-hot rows returning W_hat bit for bit, counters left at zero).

Bar: max|Y - Y_ref| <= 1e-2 * max|Y_ref| with Y_ref the oracle's fp32 product of the dequantised weight."""
import numpy as np
import pytest
import torch

import w4a16_oracle as orc

pytestmark = pytest.mark.gpu

TOL = 1e-2
DEV = "cuda:0"
G = 128


@pytest.fixture(scope="module")
def capi(built_lib):
    from sqamd import capi as c
    c.lib()
    return c


def to_dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


_cache = {}


def linear(n, k, seed=0):
    key = (n, k, seed)
    if key not in _cache:
        d = orc.synth_linear(n, k, G, seed=seed)
        d["w_hat"] = orc.dequant_l1(d["w_l1"], d["zs_l1"], G)
        d["w_dev"] = to_dev(d["w_l1"])
        d["zs_dev"] = to_dev(d["zs_l1"])
        if len(_cache) > 4:
            _cache.pop(next(iter(_cache)))
        _cache[key] = d
    return _cache[key]


def tunings(k):
    """0 = heuristic; rows per workgroup (1: 16, 3: 48, 4: 64) | ksplit << 4 for every split whose K range fits."""
    chunks = k // 128
    out = [0]
    for rt in (1, 3, 4):
        for ks in (1, 2, 3, 4, 8):
            cps = -(-chunks // ks)
            if rt == 3 and (ks != 1 or cps <= 16):
                continue  # 48-row workgroups: full-length K ranges without a split only
            if cps <= 32 and (ks - 1) * cps < chunks:
                out.append(rt | (ks << 4))
    return out


SHAPES = [(256, 1024), (264, 2048), (200, 1536), (520, 4096), (1048, 3200), (72, 4224), (1000, 5120), (264, 11008), (136, 16384)]


@pytest.mark.parametrize("n,k", SHAPES)
@pytest.mark.parametrize("m", [1, 4, 5, 8, 9, 13, 16])
def test_stream_parity(capi, n, k, m):
    d = linear(n, k, seed=41)
    x = orc.synth_x(m, k, seed=42 + m)
    y_ref = orc.gemm_ref(x, d["w_hat"])
    xd = to_dev(x)
    ws = capi.workspace(16, n, k, xd.device)
    for tune in tunings(k):
        y = torch.full((m, n), float("nan"), dtype=torch.float16, device=DEV)
        capi.gemm_ws(xd, d["w_dev"], d["zs_dev"], n, k, G, algo=capi.SQ_ALGO_STREAM | (tune << 8), out=y, ws=ws)
        torch.cuda.synchronize()
        got = y.float().cpu().numpy()
        assert np.all(np.isfinite(got)), (m, n, k, hex(tune))
        assert np.max(np.abs(got - y_ref)) <= TOL * np.max(np.abs(y_ref)), (m, n, k, hex(tune))
    assert capi.workspace_is_clean(ws)


def test_stream_without_workspace_up_to_4096_columns(capi):
    n, k = 264, 4096
    d = linear(n, k, seed=43)
    x = orc.synth_x(8, k, seed=44)
    y_ref = orc.gemm_ref(x, d["w_hat"])
    y = capi.gemm(to_dev(x), d["w_dev"], d["zs_dev"], n, k, G, algo=capi.SQ_ALGO_STREAM).float().cpu().numpy()
    assert np.max(np.abs(y - y_ref)) <= TOL * np.max(np.abs(y_ref))
    # a longer K needs the K split and with it the workspace
    d2 = linear(n, 8192, seed=45)
    with pytest.raises(capi.SqError):
        capi.gemm(to_dev(orc.synth_x(8, 8192, seed=46)), d2["w_dev"], d2["zs_dev"], n, 8192, G, algo=capi.SQ_ALGO_STREAM)


@pytest.mark.parametrize("n,k", [(256, 1024), (200, 1536), (520, 4096), (4096, 4096), (264, 8192)])
@pytest.mark.parametrize("m", [3, 5, 8, 13, 16])
def test_stream_group_size_64(capi, n, k, m):
    """Group size 64 (two (zero, scale) pairs per 128-wide chunk): explicit kernel id with 16- and 64-row
    workgroups and K splits, and the automatic dispatch, against the oracle."""
    dd = orc.synth_linear(n, k, 64, seed=90)
    w_hat = orc.dequant_l1(dd["w_l1"], dd["zs_l1"], 64)
    wd, zd = to_dev(dd["w_l1"]), to_dev(dd["zs_l1"])
    x = orc.synth_x(m, k, seed=91 + m)
    rows = np.arange(n) if n <= 1024 else np.sort(np.random.default_rng(92).choice(n, size=256, replace=False))
    y_ref = orc.gemm_ref(x, w_hat[rows])
    xd = to_dev(x)
    ws = capi.workspace(16, n, k, xd.device)
    for tune in [t for t in tunings(k) if (t & 0xF) != 3]:
        y = torch.full((m, n), float("nan"), dtype=torch.float16, device=DEV)
        capi.gemm_ws(xd, wd, zd, n, k, 64, algo=capi.SQ_ALGO_STREAM | (tune << 8), out=y, ws=ws)
        torch.cuda.synchronize()
        got = y.float().cpu().numpy()[:, rows]
        assert np.all(np.isfinite(got)), (m, n, k, hex(tune))
        assert np.max(np.abs(got - y_ref)) <= TOL * np.max(np.abs(y_ref)), (m, n, k, hex(tune))
    if m >= 5:  # the automatic choice at this group size too
        y_auto = capi.gemm_ws(xd, wd, zd, n, k, 64, ws=ws)
        y_stream = capi.gemm_ws(xd, wd, zd, n, k, 64, algo=capi.SQ_ALGO_STREAM, ws=ws)
        assert torch.equal(y_auto, y_stream)
    assert capi.workspace_is_clean(ws)


def test_stream_rejects_what_it_cannot_run(capi):
    d = linear(256, 1024, seed=47)
    with pytest.raises(capi.SqError):  # more than 16 tokens on a weight too small for the two-tile variant
        capi.gemm(to_dev(orc.synth_x(17, 1024, seed=48)), d["w_dev"], d["zs_dev"], 256, 1024, G, algo=capi.SQ_ALGO_STREAM)
    d32 = orc.synth_linear(256, 1024, 32, seed=49)
    with pytest.raises(capi.SqError):  # group size 32
        capi.gemm(to_dev(orc.synth_x(8, 1024, seed=50)), to_dev(d32["w_l1"]), to_dev(d32["zs_l1"]), 256, 1024, 32,
                  algo=capi.SQ_ALGO_STREAM)


@pytest.mark.parametrize("n,k", [(4096, 4096), (16384, 4096), (4096, 16384), (11008, 4096), (4096, 11008)])
@pytest.mark.parametrize("m", [5, 8, 16])
def test_stream_is_the_automatic_choice_at_full_size(capi, n, k, m):
    """The automatic dispatch and the explicit kernel id give the same bits on the decode shapes, within the
    bar of the oracle on 256 sampled output rows."""
    d = linear(n, k, seed=51)
    x = orc.synth_x(m, k, seed=52)
    xd = to_dev(x)
    ws = capi.workspace(m, n, k, xd.device)
    y_auto = capi.gemm_ws(xd, d["w_dev"], d["zs_dev"], n, k, G, ws=ws)
    y_stream = capi.gemm_ws(xd, d["w_dev"], d["zs_dev"], n, k, G, algo=capi.SQ_ALGO_STREAM, ws=ws)
    assert torch.equal(y_auto, y_stream)
    rows = np.sort(np.random.default_rng(53).choice(n, size=256, replace=False))
    y_ref = orc.gemm_ref(x, d["w_hat"][rows])
    got = y_auto.float().cpu().numpy()[:, rows]
    assert np.max(np.abs(got - y_ref)) <= TOL * np.max(np.abs(y_ref))
    assert capi.workspace_is_clean(ws)


@pytest.mark.parametrize("n,k", [(8192, 1024), (8200, 3200), (16384, 4096), (4096, 16384), (4096, 11008)])
@pytest.mark.parametrize("m", [17, 24, 31, 32])
def test_stream_two_token_tiles(capi, n, k, m):
    """17..32 tokens: two token tiles per weight word, every wave moving the activations of its own chunks into LDS
    (short K ranges leave chunk slots empty, long ones are split through the workspace, ragged N and K); explicit
    kernel id and automatic dispatch against the oracle on sampled rows, with bias, ReLU and residual on the way out."""
    d = linear(n, k, seed=95)
    rng = np.random.default_rng(96 + m)
    x = orc.synth_x(m, k, seed=97 + m)
    bias = rng.normal(0, 1.0, size=n).astype(np.float16)
    res = rng.normal(0, 1.0, size=(m, n)).astype(np.float16)
    rows = np.sort(rng.choice(n, size=256, replace=False))
    rows[0], rows[-1] = 0, n - 1
    plain = orc.gemm_ref(x, d["w_hat"][rows]).astype(np.float64)
    ref = np.maximum(plain + bias[rows].astype(np.float64)[None, :], 0.0) + res[:, rows].astype(np.float64)
    xd, bd, rd = to_dev(x), to_dev(bias), to_dev(res)
    ws = capi.workspace(m, n, k, xd.device)
    y = capi.gemm_fused(xd, d["w_dev"], d["zs_dev"], n, k, G, bias=bd, residual=rd, act=1, algo=capi.SQ_ALGO_STREAM, ws=ws)
    y_auto = capi.gemm_fused(xd, d["w_dev"], d["zs_dev"], n, k, G, bias=bd, residual=rd, act=1, ws=ws)
    torch.cuda.synchronize()
    assert torch.equal(y, y_auto)
    got = y.float().cpu().numpy()[:, rows]
    assert np.all(np.isfinite(got))
    assert np.max(np.abs(got - ref)) <= TOL * np.max(np.abs(plain))
    # fixed summation order: the same bits on a second call, counters back at zero
    assert torch.equal(y, capi.gemm_fused(xd, d["w_dev"], d["zs_dev"], n, k, G, bias=bd, residual=rd, act=1, ws=ws))
    assert capi.workspace_is_clean(ws)


def test_stream_properties(capi):
    n, k = 4096, 16384  # K split four ways through the workspace
    d = linear(n, k, seed=54)
    x = to_dev(orc.synth_x(8, k, seed=55))
    ws = capi.workspace(16, n, k, x.device)
    algo = capi.SQ_ALGO_STREAM
    y1 = capi.gemm_ws(x, d["w_dev"], d["zs_dev"], n, k, G, algo=algo, ws=ws)
    for _ in range(3):  # fixed summation order: the same bits every time, counters back at zero
        assert torch.equal(y1, capi.gemm_ws(x, d["w_dev"], d["zs_dev"], n, k, G, algo=algo, ws=ws))
    assert capi.workspace_is_clean(ws)
    y2 = capi.gemm_ws(x * 2, d["w_dev"], d["zs_dev"], n, k, G, algo=algo, ws=ws)
    normal = y1.abs() >= 2.0 ** -13
    assert torch.equal(y2[normal], (y1 * 2)[normal])
    e = torch.zeros((16, k), dtype=torch.float16, device=DEV)
    cols = [(977 * i + 5) % k for i in range(16)]
    for i, c in enumerate(cols):
        e[i, c] = 1.0
    ye = capi.gemm_ws(e, d["w_dev"], d["zs_dev"], n, k, G, algo=algo, ws=ws).cpu().numpy()
    for i, c in enumerate(cols):  # a one-hot row returns W_hat bit for bit
        assert np.array_equal(ye[i].view(np.int16), d["w_hat"][:, c].view(np.int16))
    # rows of a batch do not depend on the other rows
    y_one = capi.gemm_ws(x[3:4].repeat(5, 1), d["w_dev"], d["zs_dev"], n, k, G, algo=algo, ws=ws)
    assert torch.equal(y_one[0], y1[3]) and torch.equal(y_one[4], y1[3])


@pytest.mark.parametrize("m,n,k,tune", [(5, 264, 2048, 0), (8, 520, 4096, 4), (16, 136, 16384, 0), (9, 1000, 5120, 1 | (2 << 4))])
@pytest.mark.parametrize("use_bias,use_res,act", [(True, False, 0), (False, True, 0), (True, True, 1), (False, False, 1)])
def test_stream_fused_epilogue(capi, m, n, k, tune, use_bias, use_res, act):
    d = linear(n, k, seed=56)
    rng = np.random.default_rng(57)
    x = orc.synth_x(m, k, seed=58)
    bias = rng.normal(0, 2.0, size=n).astype(np.float16) if use_bias else None
    res = rng.normal(0, 2.0, size=(m, n)).astype(np.float16) if use_res else None
    y_ref = orc.gemm_ref(x, d["w_hat"]).astype(np.float64)
    if bias is not None:
        y_ref = y_ref + bias.astype(np.float64)[None, :]
    if act:
        y_ref = np.maximum(y_ref, 0.0)
    if res is not None:
        y_ref = y_ref + res.astype(np.float64)
    y = capi.gemm_fused(to_dev(x), d["w_dev"], d["zs_dev"], n, k, G, bias=None if bias is None else to_dev(bias),
                        residual=None if res is None else to_dev(res), act=act, algo=capi.SQ_ALGO_STREAM | (tune << 8))
    torch.cuda.synchronize()
    y = y.float().cpu().numpy()
    scale = np.max(np.abs(orc.gemm_ref(x, d["w_hat"])))
    assert np.max(np.abs(y - y_ref)) <= TOL * scale
    if act and not use_res:
        assert y.min() >= 0.0


@pytest.mark.parametrize("m", [5, 8, 16])
@pytest.mark.parametrize("k,ns", [(1024, (256, 136, 264)), (4096, (520, 520)), (5120, (264, 200, 72, 136))])
def test_grouped_stream_launch_behind_the_sequence(capi, m, k, ns):
    """Independent linears of equal K go out as one launch of the streaming kernel; each keeps its own
    activations, bias, residual and output."""
    rng = np.random.default_rng(59)
    lin, refs = [], []
    for i, n in enumerate(ns):
        d = linear(n, k, seed=60 + i)
        x = orc.synth_x(m, k, seed=70 + i)
        bias = rng.normal(0, 1.0, size=n).astype(np.float16)
        res = rng.normal(0, 1.0, size=(m, n)).astype(np.float16)
        ref = orc.gemm_ref(x, d["w_hat"]).astype(np.float64) + bias.astype(np.float64)[None, :]
        if i % 2:
            ref = np.maximum(ref, 0.0)
        ref = ref + res.astype(np.float64)
        refs.append((ref, np.max(np.abs(orc.gemm_ref(x, d["w_hat"])))))
        lin.append(dict(x=to_dev(x), w=d["w_dev"], zs=d["zs_dev"], bias=to_dev(bias), residual=to_dev(res),
                        y=torch.full((m, n), float("nan"), dtype=torch.float16, device=DEV), n=n, k=k, group_size=G,
                        act=i % 2, depends=False))
    seq = capi.LinearSequence(lin, m, torch.device(DEV))
    seq.run()
    torch.cuda.synchronize()
    for l, (ref, scale) in zip(lin, refs):
        got = l["y"].float().cpu().numpy()
        assert np.all(np.isfinite(got))
        assert np.max(np.abs(got - ref)) <= TOL * scale
    if seq.ws is not None:
        assert capi.workspace_is_clean(seq.ws)


def ln_linear_ref(x, gamma, beta, eps, w_hat, bias, res, act):
    """The oracle's composition: LayerNorm in float64, rounded to fp16 as the reference's module boundary does,
    then the fp32 product with the dequantised weight, bias, activation, residual."""
    h = orc.layernorm_ref(x, gamma, beta, eps).astype(np.float16)
    y = orc.gemm_ref(h, w_hat).astype(np.float64)
    scale = np.max(np.abs(y))
    if bias is not None:
        y = y + bias.astype(np.float64)[None, :]
    if act:
        y = np.maximum(y, 0.0)
    if res is not None:
        y = y + res.astype(np.float64)
    return y, scale


@pytest.mark.parametrize("n,k", [(264, 4096), (520, 2176), (72, 3200), (1000, 4096)])
@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 7, 8])
def test_layernorm_inside_the_linear(capi, n, k, m):
    """sq_w4a16_gemm_ln_fused where the normalisation happens in the kernel, against the oracle's composition."""
    assert capi.lib().sq_w4a16_ln_fusable(m, n, k, G, capi.SQ_LAYOUT_L1) == 1
    d = linear(n, k, seed=80)
    rng = np.random.default_rng(81 + m)
    x = (rng.normal(0.7, 1.0, size=(m, k)) * rng.uniform(0.2, 8.0, size=(m, 1))).astype(np.float16)
    gamma = rng.normal(1.0, 0.3, size=k).astype(np.float16)
    beta = rng.normal(0.0, 0.3, size=k).astype(np.float16)
    bias = rng.normal(0, 1.0, size=n).astype(np.float16)
    res = rng.normal(0, 1.0, size=(m, n)).astype(np.float16)
    for use_affine, use_epi, act in ((True, True, 1), (True, False, 0), (False, True, 0)):
        ga, be = (gamma, beta) if use_affine else (None, None)
        bi, re = (bias, res) if use_epi else (None, None)
        ref, scale = ln_linear_ref(x, ga, be, 1e-5, d["w_hat"], bi, re, act)
        y = capi.gemm_ln_fused(to_dev(x), None if ga is None else to_dev(ga), None if be is None else to_dev(be), 1e-5,
                               d["w_dev"], d["zs_dev"], n, k, G, bias=None if bi is None else to_dev(bi),
                               residual=None if re is None else to_dev(re), act=act)
        torch.cuda.synchronize()
        got = y.float().cpu().numpy()
        assert np.all(np.isfinite(got))
        assert np.max(np.abs(got - ref)) <= TOL * scale, (m, n, k, use_affine, use_epi, act)


def test_layernorm_linear_matches_the_two_step_path(capi):
    """Fused and unfused give the same result up to the rounding of the normalised row (one fp16 ulp in rare
    elements): on the OPT-6.7B fc1 shape the two differ by far less than either differs from the oracle's bar."""
    n, k, m = 16384, 4096, 8
    d = linear(n, k, seed=82)
    rng = np.random.default_rng(83)
    x = to_dev(rng.normal(0.1, 1.5, size=(m, k)).astype(np.float16))
    gamma = to_dev(rng.normal(1.0, 0.2, size=k).astype(np.float16))
    beta = to_dev(rng.normal(0.0, 0.2, size=k).astype(np.float16))
    y_fused = capi.gemm_ln_fused(x, gamma, beta, 1e-5, d["w_dev"], d["zs_dev"], n, k, G)
    h = capi.layernorm(x, gamma, beta, 1e-5)
    y_two = capi.gemm_ws(h, d["w_dev"], d["zs_dev"], n, k, G)
    torch.cuda.synchronize()
    diff = (y_fused.float() - y_two.float()).abs().max().item()
    assert diff <= 2e-3 * y_two.float().abs().max().item()
    # determinism
    assert torch.equal(y_fused, capi.gemm_ln_fused(x, gamma, beta, 1e-5, d["w_dev"], d["zs_dev"], n, k, G))


@pytest.mark.parametrize("m,n,k,g", [(8, 264, 1024, 128), (9, 264, 4096, 128), (40, 264, 4096, 128), (8, 136, 8192, 128), (5, 136, 640, 32),
                                     (300, 264, 4096, 128)])
def test_layernorm_linear_fallback(capi, m, n, k, g):
    """Shapes the kernel cannot normalise in place go through the LayerNorm kernel and a scratch tensor."""
    assert capi.lib().sq_w4a16_ln_fusable(m, n, k, g, capi.SQ_LAYOUT_L1) == 0
    dd = orc.synth_linear(n, k, g, seed=84)
    w_hat = orc.dequant_l1(dd["w_l1"], dd["zs_l1"], g)
    rng = np.random.default_rng(85)
    x = rng.normal(0.3, 2.0, size=(m, k)).astype(np.float16)
    gamma = rng.normal(1.0, 0.3, size=k).astype(np.float16)
    beta = rng.normal(0.0, 0.3, size=k).astype(np.float16)
    res = rng.normal(0, 1.0, size=(m, n)).astype(np.float16)
    ref, scale = ln_linear_ref(x, gamma, beta, 1e-5, w_hat, None, res, 0)
    y = capi.gemm_ln_fused(to_dev(x), to_dev(gamma), to_dev(beta), 1e-5, to_dev(dd["w_l1"]), to_dev(dd["zs_l1"]), n, k, g,
                           residual=to_dev(res))
    torch.cuda.synchronize()
    assert np.max(np.abs(y.float().cpu().numpy() - ref)) <= TOL * scale
    # without the scratch rows the call is refused
    rc = capi.lib().sq_w4a16_gemm_ln_fused(to_dev(x).data_ptr(), None, None, 1e-5, None, to_dev(dd["w_l1"]).data_ptr(),
                                           to_dev(dd["zs_l1"]).data_ptr(), None, None, y.data_ptr(), m, n, k, g,
                                           capi.SQ_LAYOUT_L1, 0, None, 0, None)
    assert rc == 1  # SQ_ERR_NULL_POINTER
