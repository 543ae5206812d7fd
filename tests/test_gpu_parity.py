"""GPU parity tests: the HIP path (through the C ABI and through the `quant`
extension) against the CPU oracle on the same seeded inputs.

Bars: int4 unpack / dequant and every repack are bit-exact; GEMM outputs satisfy
max|Y - Y_ref| <= 1e-2 * max|Y_ref| with Y_ref the oracle's fp32 result (the
tolerance the task states; observed errors are about 1e-3, dominated by the final
fp16 rounding)."""
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


def bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy()


_cache = {}


def linear(n, k, g, seed=0):
    key = (n, k, g, seed)
    if key not in _cache:
        d = orc.synth_linear(n, k, g, seed=seed)
        d["w_hat"] = orc.dequant_l1(d["w_l1"], d["zs_l1"], g)
        d["w_dev"] = to_dev(d["w_l1"])
        d["zs_dev"] = to_dev(d["zs_l1"])
        if len(_cache) > 6:
            _cache.pop(next(iter(_cache)))
        _cache[key] = d
    return _cache[key]


def check_gemm(capi, m, n, k, g, algo, seed=0, tol=TOL):
    d = linear(n, k, g, seed)
    x = orc.synth_x(m, k, seed=seed + 100)
    y_ref = orc.gemm_ref(x, d["w_hat"])
    y = capi.gemm(to_dev(x), d["w_dev"], d["zs_dev"], n, k, g, algo=algo)
    torch.cuda.synchronize()
    y = y.float().cpu().numpy()
    assert np.all(np.isfinite(y))
    err = np.max(np.abs(y - y_ref))
    ref = np.max(np.abs(y_ref))
    assert err <= tol * ref, "m=%d n=%d k=%d g=%d algo=%#x: err %.3e vs %.3e" % (m, n, k, g, algo, err, tol * ref)
    return err / ref


# ------------------------------------------------------------------ dequant
@pytest.mark.parametrize("n,k,g", [(8, 32, 32), (16, 128, 64), (40, 1024, 128), (4096, 4096, 64),
                                   (4096, 4096, 128), (4096, 11008, 128)])
def test_dequant_l1_bit_exact(capi, n, k, g):
    d = linear(n, k, g, seed=3)
    out = capi.dequant(d["w_dev"], d["zs_dev"], n, k, g)
    torch.cuda.synchronize()
    assert np.array_equal(bits(out), d["w_hat"].view(np.int16))


def test_dequant_handmade_word(capi):
    # nibbles 0,2,4,6,1,3,5,7 -> q = 0..7 in natural order; z = 3, s = 0.5
    w = np.array([[0x20, 0x64, 0x31, 0x75] * 4] * 8, dtype=np.uint8)
    zs = orc.zeros_scales_l1(np.full((8, 1), 3), np.full((8, 1), 0.5))
    out = capi.dequant(to_dev(w), to_dev(zs), 8, 32, 32).float().cpu().numpy()
    assert out[0, :8].tolist() == [(q - 3) * 0.5 for q in range(8)]


# ------------------------------------------------------------------ GEMM parity
SMALL_SHAPES = [(64, 512, 64), (256, 1024, 128), (136, 640, 32), (48, 2816, 128)]


@pytest.mark.parametrize("n,k,g", SMALL_SHAPES)
@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 8])
@pytest.mark.parametrize("algo_name", ["GEMV", "GEMV_FIXUP"])
def test_gemv_parity_small(capi, n, k, g, m, algo_name):
    check_gemm(capi, m, n, k, g, getattr(capi, "SQ_ALGO_" + algo_name))


@pytest.mark.parametrize("tune", [nr | (ks << 4) for nr in (2, 4, 8) for ks in (1, 2, 4)])
def test_gemv_every_tuning_is_correct(capi, tune):
    # tune = row groups per workgroup | k ranges per workgroup << 4
    for m in (1, 4, 7):
        check_gemm(capi, m, 200, 1536, 64, capi.SQ_ALGO_GEMV | (tune << 8))
        check_gemm(capi, m, 200, 1536, 128, capi.SQ_ALGO_GEMV_FIXUP | (tune << 8))


@pytest.mark.parametrize("n,k,g", SMALL_SHAPES)
@pytest.mark.parametrize("m", [1, 9, 16, 17, 32, 33, 64])
def test_skinny_parity_small(capi, n, k, g, m):
    check_gemm(capi, m, n, k, g, capi.SQ_ALGO_SKINNY)
    check_gemm(capi, m, n, k, g, capi.SQ_ALGO_SKINNY | ((8 | (1 << 8)) << 8))  # exact mode


@pytest.mark.parametrize("n,k,g", SMALL_SHAPES + [(520, 1056, 32)])
@pytest.mark.parametrize("m", [1, 31, 33, 64, 100, 128, 129, 300])
def test_gemm_parity_small(capi, n, k, g, m):
    check_gemm(capi, m, n, k, g, capi.SQ_ALGO_GEMM)


@pytest.mark.parametrize("mi", [1, 2, 4, 8, 9, 10])
def test_gemm_every_tile_height_is_correct(capi, mi):
    for m in (5, 70, 260):
        check_gemm(capi, m, 264, 704, 64, capi.SQ_ALGO_GEMM | (mi << 8))


# The benchmark's decode shapes (OPT-6.7B linears) and prefill shapes (plus the Llama-2-7B MLP).
@pytest.mark.parametrize("n,k,g", [(4096, 4096, 64), (4096, 4096, 128), (16384, 4096, 128), (4096, 16384, 128)])
@pytest.mark.parametrize("m", [1, 4, 8, 16, 32])
def test_decode_shapes_auto_dispatch(capi, n, k, g, m):
    rel = check_gemm(capi, m, n, k, g, capi.SQ_ALGO_AUTO)
    assert rel < 5e-3


@pytest.mark.parametrize("n,k", [(4096, 4096), (11008, 4096), (4096, 11008)])
def test_prefill_shapes_auto_dispatch(capi, n, k):
    rel = check_gemm(capi, 512, n, k, 128, capi.SQ_ALGO_AUTO)
    assert rel < 5e-3


# ------------------------------------------------------------------ size-independent properties at full size
@pytest.mark.parametrize("algo_name,m", [("GEMV", 1), ("GEMV_FIXUP", 1), ("GEMV_FIXUP", 8), ("SKINNY", 16),
                                         ("GEMM", 200)])
def test_properties_full_size(capi, algo_name, m):
    n, k, g = 4096, 4096, 128
    algo = getattr(capi, "SQ_ALGO_" + algo_name)
    d = linear(n, k, g, seed=7)
    x = to_dev(orc.synth_x(m, k, seed=8))
    y1 = capi.gemm(x, d["w_dev"], d["zs_dev"], n, k, g, algo=algo)
    # determinism: the same launch twice gives the same bits
    y1b = capi.gemm(x, d["w_dev"], d["zs_dev"], n, k, g, algo=algo)
    assert torch.equal(y1, y1b)
    # scaling the activations by 2 is exact in fp16 and fp32, so the output doubles bit for bit
    y2 = capi.gemm(x * 2, d["w_dev"], d["zs_dev"], n, k, g, algo=algo)
    # (outputs in the fp16 subnormal range are excluded: there 2*round(a) != round(2a))
    normal = y1.abs() >= 2.0 ** -13
    assert torch.equal(y2[normal], (y1 * 2)[normal])
    # a one-hot activation row returns a column of W_hat, exactly
    e = torch.zeros((m, k), dtype=torch.float16, device=DEV)
    cols = [(37 * i + 5) % k for i in range(m)]
    for i, c in enumerate(cols):
        e[i, c] = 1.0
    ye = capi.gemm(e, d["w_dev"], d["zs_dev"], n, k, g, algo=algo).cpu().numpy()
    for i, c in enumerate(cols):
        assert np.array_equal(ye[i].view(np.int16), d["w_hat"][:, c].view(np.int16))


@pytest.mark.parametrize("algo_name,m", [("GEMV", 3), ("SKINNY", 20), ("GEMM", 70)])
def test_zero_output_when_q_equals_z(capi, algo_name, m):
    n, k, g = 512, 2048, 64
    rng = np.random.default_rng(5)
    z = rng.integers(0, 16, size=(n, k // g), dtype=np.uint8)
    s = (np.abs(rng.normal(0, 0.02, size=(n, k // g))) + 1e-3).astype(np.float16)
    w = to_dev(orc.pack_l1(np.repeat(z, g, axis=1)))
    zs = to_dev(orc.zeros_scales_l1(z, s))
    algo = getattr(capi, "SQ_ALGO_" + algo_name)
    if algo_name == "SKINNY":
        algo |= (8 | (1 << 8)) << 8  # exact arithmetic mode
    y = capi.gemm(to_dev(orc.synth_x(m, k)), w, zs, n, k, g, algo=algo)
    assert torch.count_nonzero(y).item() == 0


def test_gemv_rows_do_not_depend_on_batch(capi):
    # A token's output does not depend on which other tokens share the launch, as long as the launches
    # use the same workgroup shape (the split of K decides the order of the fp32 additions; the tuning
    # word pins it here) and the same arithmetic path (the fixup mode has one for up to 4 tokens and one
    # for 5 to 8).
    n, k, g = 1024, 4096, 128
    d = linear(n, k, g, seed=9)
    x = to_dev(orc.synth_x(8, k, seed=10))
    pinned = (4 | (1 << 4)) << 8  # 4 row groups x 1 k range per workgroup
    run = lambda t, algo: capi.gemm(t.contiguous(), d["w_dev"], d["zs_dev"], n, k, g, algo=algo | pinned)
    y4 = run(x[:4], capi.SQ_ALGO_GEMV_FIXUP)
    for m in (0, 3):
        assert torch.equal(run(x[m:m + 1], capi.SQ_ALGO_GEMV_FIXUP)[0], y4[m])
    y8 = run(x, capi.SQ_ALGO_GEMV_FIXUP)
    y5 = run(x[3:8], capi.SQ_ALGO_GEMV_FIXUP)
    assert torch.equal(y5, y8[3:8])
    y8e = run(x, capi.SQ_ALGO_GEMV)
    for m in (0, 3, 7):
        assert torch.equal(run(x[m:m + 1], capi.SQ_ALGO_GEMV)[0], y8e[m])


# ------------------------------------------------------------------ edge cases
def test_empty_and_minimal(capi):
    d = linear(8, 32, 32, seed=1)
    y = capi.gemm(torch.empty((0, 32), dtype=torch.float16, device=DEV), d["w_dev"], d["zs_dev"], 8, 32, 32)
    assert tuple(y.shape) == (0, 8)
    for algo in (capi.SQ_ALGO_GEMV, capi.SQ_ALGO_GEMV_FIXUP, capi.SQ_ALGO_SKINNY, capi.SQ_ALGO_GEMM):
        check_gemm(capi, 1, 8, 32, 32, algo, seed=1)


def test_extreme_codes(capi):
    # all-15 weights with zero point 0 and all-0 weights with zero point 15, large activations
    n, k, g = 64, 1024, 128
    for qv, zv in ((15, 0), (0, 15)):
        q = np.full((n, k), qv, dtype=np.uint8)
        z = np.full((n, k // g), zv, dtype=np.uint8)
        s = np.full((n, k // g), 0.01, dtype=np.float16)
        w_l1, zs_l1 = orc.pack_l1(q), orc.zeros_scales_l1(z, s)
        x = (orc.synth_x(4, k, seed=2).astype(np.float32) * 8).astype(np.float16)
        y_ref = orc.gemm_ref(x, orc.dequant_l1(w_l1, zs_l1, g))
        for algo in (capi.SQ_ALGO_GEMV, capi.SQ_ALGO_GEMV_FIXUP, capi.SQ_ALGO_SKINNY, capi.SQ_ALGO_GEMM):
            y = capi.gemm(to_dev(x), to_dev(w_l1), to_dev(zs_l1), n, k, g, algo=algo).float().cpu().numpy()
            assert np.max(np.abs(y - y_ref)) <= TOL * np.max(np.abs(y_ref))


# ------------------------------------------------------------------ layout L2 and converters
def test_l2_converters_bit_exact(capi):
    n, k, g = 96, 256, 128
    d = orc.synth_linear(n, k, g, seed=13)
    ours = orc.pack_ours(d["q"])
    awq = capi.convert_ours_to_awq(to_dev(ours), k, n)
    assert np.array_equal(awq.cpu().numpy().view(np.uint32).reshape(k, n // 8), orc.ours_to_awq(ours, k, n))
    l2 = capi.convert_awq_to_lmdeploy(awq, k, n)
    want = orc.pack_l2(d["q"])
    assert np.array_equal(l2.cpu().numpy(), want)
    zs2 = capi.transpose_merge_zeros_scales(to_dev(d["z"].astype(np.float16)), to_dev(d["s"]), k, n, g)
    zs2_want = orc.transpose_merge_zeros_scales(d["z"].astype(np.float16), d["s"], k, n, g)
    assert np.array_equal(bits(zs2), zs2_want.view(np.int16))
    # dequant straight from L2, and L2 -> L1 repack
    out = capi.dequant(l2, zs2, n, k, g, layout=capi.SQ_LAYOUT_L2)
    assert np.array_equal(bits(out), orc.dequant_l1(d["w_l1"], d["zs_l1"], g).view(np.int16))
    w1, zs1 = capi.repack_l2_to_l1(l2, zs2, n, k, g)
    assert np.array_equal(w1.cpu().numpy(), d["w_l1"])
    assert np.array_equal(bits(zs1), d["zs_l1"].view(np.int16))


def test_two_bit_expansion(capi):
    rng = np.random.default_rng(17)
    w2 = rng.integers(0, 256, size=(16, 64), dtype=np.uint8)
    out = capi.convert_2bit_to_4bit(to_dev(w2)).cpu().numpy()
    assert np.array_equal(out, orc.convert_2bit_to_4bit_l1(w2))


def test_two_bit_int32_layout_words(capi):
    """Layout L2 with 2-bit storage: the packer and the expander against the oracle's
    restatement of the reference's word arithmetic, bit for bit."""
    rng = np.random.default_rng(29)
    for k, n in ((32, 64), (96, 1040), (1, 16)):
        w4 = rng.integers(0, 2**32, size=(k, n // 8), dtype=np.uint64).astype(np.uint32).view(np.int32)
        packed = capi.l2_convert_4bit_to_2bit(to_dev(w4))
        assert packed.dtype == torch.int32 and tuple(packed.shape) == (k, n // 16)
        assert np.array_equal(packed.cpu().numpy(), orc.convert_4bit_to_2bit_l2(w4))
        w2 = rng.integers(0, 2**32, size=(k, n // 16), dtype=np.uint64).astype(np.uint32).view(np.int32)
        wide = capi.l2_convert_2bit_to_4bit(to_dev(w2))
        assert wide.dtype == torch.int32 and tuple(wide.shape) == (k, n // 8)
        assert np.array_equal(wide.cpu().numpy(), orc.convert_2bit_to_4bit_l2(w2))


# ------------------------------------------------------------------ the `quant` extension and WALinear
def test_quant_extension_matches_reference_recipe():
    """The reference's own kernel check: allclose(x @ W_hat.T, gemm_awq_ut(...), atol = rtol = 2e-2)
    (quantization/muxi/script/gemm_awq_test.py:80-109), run on seeded data."""
    import quant
    from sqamd import quant_funcs as qf
    torch.manual_seed(0)
    for bs, seq, k, n, g in [(1, 1, 4096, 4096, 128), (1, 16, 4096, 4096, 64), (2, 128, 1024, 2048, 128)]:
        x = torch.empty((bs, seq, k), dtype=torch.float16, device=DEV).normal_(mean=0.0, std=0.5)
        lin = torch.nn.Linear(k, n, bias=False, device=DEV, dtype=torch.float16)
        qweight, zeros_scales = qf.quant_muxi(lin.weight.data, k, n, n_bit=4, group_size=g)
        w_fp16 = qf.dequant_to_fp16(lin.weight.data, 4, g)
        ref = torch.matmul(x.float(), w_fp16.float().t())
        out = quant.gemm_awq_ut(x, qweight, zeros_scales, bs * seq, n, k, g)
        assert tuple(out.shape) == (bs, seq, n) and out.dtype == torch.float16
        assert torch.allclose(ref, out.float(), atol=2e-2, rtol=2e-2)
        # dequant op: bit-identical to the torch fp16 recipe
        assert torch.equal(quant.dequant(qweight, zeros_scales, n, k, g), w_fp16)


def test_quant_extension_l2_weights():
    import quant
    from sqamd import quant_funcs as qf
    torch.manual_seed(1)
    k, n, g = 1024, 512, 128
    lin = torch.nn.Linear(k, n, bias=False, device=DEV, dtype=torch.float16)
    qw2, zs2, w_fake = qf.quant_lmdeploy(lin.weight.data, k, n, group_size=g, n_bit=4)
    assert w_fake.dtype == torch.float16 and tuple(w_fake.shape) == (n, k)
    assert qw2.dtype == torch.int32 and tuple(qw2.shape) == (k, n // 8) and tuple(zs2.shape) == (k // g, 2 * n)
    w_fp16 = qf.dequant_to_fp16(lin.weight.data, 4, g)
    assert torch.equal(quant.dequant(qw2, zs2, n, k, g), w_fp16)
    x = torch.randn((1, 5, k), dtype=torch.float16, device=DEV)
    ref = torch.matmul(x.float(), w_fp16.float().t())
    quant.clear_repack_cache()
    out = quant.gemm_awq_ut(x, qw2, zs2, 5, n, k, g)
    out2 = quant.gemm_awq_ut(x, qw2, zs2, 5, n, k, g)  # second call is served from the repack cache
    assert quant.repack_cache_size() == 1
    assert torch.equal(out, out2)
    assert (out.float() - ref).abs().max() <= TOL * ref.abs().max()
    with pytest.raises(RuntimeError, match="unsupported group size"):
        quant.gemm_awq_ut(x, qw2, zs2, 5, n, k, 64)
    del qw2
    quant.clear_repack_cache()


def test_quant_extension_argument_errors_on_device():
    import quant
    k, n, g = 256, 64, 64
    x = torch.zeros((2, 2, k), dtype=torch.float16, device=DEV)
    w = torch.zeros((n, k // 2), dtype=torch.uint8, device=DEV)
    zs = torch.zeros((n, 2 * k // g), dtype=torch.float16, device=DEV)
    with pytest.raises(RuntimeError, match="contiguous"):
        quant.gemm_awq_ut(x.transpose(0, 1), w, zs, 4, n, k, g)
    with pytest.raises(RuntimeError, match="dtype"):
        quant.gemm_awq_ut(x.float(), w, zs, 2, n, k, g)
    with pytest.raises(RuntimeError, match="dimension"):
        quant.gemm_awq_ut(x[0], w, zs, 2, n, k, g)
    with pytest.raises(RuntimeError, match="dtype"):
        quant.gemm_awq_ut(x, w.to(torch.int64), zs, 2, n, k, g)
    with pytest.raises(ValueError, match="output dim mismatch"):
        quant.gemm_awq_ut(x, w, zs, 2, n + 8, k, g)
    with pytest.raises(ValueError):
        quant.gemm_awq_ut(x, w, zs, 2, n, k, 48)
    with pytest.raises(ValueError, match="zeros_scales"):
        quant.gemm_awq_ut(x, w, zs[:, :2].contiguous(), 2, n, k, g)
    y = quant.gemm_awq_ut(x[:, :0].contiguous(), w, zs, 0, n, k, g)
    assert tuple(y.shape) == (2, 0, n)


def test_walinear_module():
    from sqamd.qlinear import WALinear
    torch.manual_seed(2)
    k, n = 1024, 768
    lin = torch.nn.Linear(k, n, bias=True, device=DEV, dtype=torch.float16)
    for layout, g in (("l1", 64), ("l2", 128)):
        q = WALinear.from_float(lin, {"n_bit": 4, "group_size": g}, None, layout=layout)
        sd = q.state_dict()
        assert set(sd) == {"weight", "zeros_scales", "bias"} and tuple(sd["bias"].shape) == (1, n)
        fresh = WALinear(k, n, w_bit=4, group_size=g, bias=True, dev=DEV, layout=layout)
        fresh.load_state_dict(sd)
        x = torch.randn((2, 3, k), dtype=torch.float16, device=DEV)
        from sqamd import quant_funcs as qf
        ref = torch.matmul(x.float(), qf.dequant_to_fp16(lin.weight.data, 4, g).float().t()) + lin.bias.float()
        out = fresh(x)
        assert tuple(out.shape) == (2, 3, n)
        assert (out.float() - ref).abs().max() <= TOL * ref.abs().max()
    # the 2-bit layer: weights stored 2-bit packed, expanded to nibbles in front of the same GEMM
    q2 = WALinear.from_float(lin, {"n_bit": 2, "group_size": 64}, None)
    assert tuple(q2.weight.shape) == (n, k // 4)
    x = torch.randn((1, 4, k), dtype=torch.float16, device=DEV)
    ref = torch.matmul(x.float(), qf.dequant_to_fp16(lin.weight.data, 2, 64).float().t()) + lin.bias.float()
    assert (q2(x).float() - ref).abs().max() <= TOL * ref.abs().max()


def test_walinear_two_bit_int32_layout():
    """A 2-bit layer in layout L2 computes what the reference's module computes: four-level codes
    packed into the tensor-core layout, the reference's 4-bit -> 2-bit -> 4-bit word arithmetic
    (which returns half of the codes in their neighbours' places), then the 4-bit GEMM on the result.
    Expected value from the oracle's chain on the same fp16 weight."""
    import quant
    from sqamd.qlinear import WALinear
    from sqamd import quant_funcs as qf
    rng = np.random.default_rng(31)
    k, n, g = 512, 256, 128
    w = (rng.normal(0, 0.05, size=(n, k))).astype(np.float16)
    bias = rng.normal(0, 0.1, size=n).astype(np.float16)
    lin = torch.nn.Linear(k, n, bias=True, device=DEV, dtype=torch.float16)
    lin.weight.data.copy_(torch.from_numpy(w))
    lin.bias.data.copy_(torch.from_numpy(bias))
    layer = WALinear.from_float(lin, {"n_bit": 2, "group_size": g}, None, layout="l2")
    assert layer.weight.dtype == torch.int32 and tuple(layer.weight.shape) == (k, n * 2 // 32)
    # the packer's side of the chain
    q, s, z = orc.rtn_quantize(w, 2, g, dtype=np.float16)
    assert q.max() <= 3
    stored = orc.convert_4bit_to_2bit_l2(orc.pack_l2(q))
    assert np.array_equal(layer.weight.cpu().numpy(), stored)
    zs = orc.transpose_merge_zeros_scales(z.astype(np.float16), s.astype(np.float16), k, n, g)
    assert np.array_equal(layer.zeros_scales.cpu().numpy().view(np.uint16), zs.view(np.uint16))
    # the module's side: expand, then the 4-bit GEMM
    w4 = orc.convert_2bit_to_4bit_l2(stored)
    assert np.array_equal(qf.convert_2bit_to_4bit(layer.weight).cpu().numpy(), w4)
    x = rng.normal(0, 0.5, size=(2, 3, k)).astype(np.float16)
    want = orc.gemm_l2(x.reshape(-1, k), w4, zs, g, k, n)[0].astype(np.float64) + bias.astype(np.float64)
    fresh = WALinear(k, n, w_bit=2, group_size=g, bias=True, dev=DEV, layout="l2")
    fresh.load_state_dict(layer.state_dict())
    for _ in range(2):  # the second call reuses the kept expansion
        got = fresh(to_dev(x)).cpu().numpy().astype(np.float64).reshape(-1, n)
        assert np.abs(got - want).max() <= TOL * np.abs(want).max()
    # half of the codes are not where a lossless 2-bit format would put them
    assert not np.array_equal(w4, orc.pack_l2(q))
    quant.clear_repack_cache()


# ------------------------------------------------------------------ workspace-backed split-K kernel (5 <= M <= 32)
def check_gemm_ws(capi, m, n, k, g, algo, seed=0):
    d = linear(n, k, g, seed)
    x = orc.synth_x(m, k, seed=seed + 100)
    y_ref = orc.gemm_ref(x, d["w_hat"])
    y = capi.gemm_ws(to_dev(x), d["w_dev"], d["zs_dev"], n, k, g, algo=algo)
    torch.cuda.synchronize()
    y = y.float().cpu().numpy()
    assert np.all(np.isfinite(y))
    assert np.max(np.abs(y - y_ref)) <= TOL * np.max(np.abs(y_ref)), (m, n, k, g, hex(algo))


@pytest.mark.parametrize("n,k,g", SMALL_SHAPES + [(520, 1056, 32), (4096, 4096, 128)])
@pytest.mark.parametrize("m", [5, 8, 16, 17, 32])
def test_skinny_ws_parity(capi, n, k, g, m):
    check_gemm_ws(capi, m, n, k, g, capi.SQ_ALGO_AUTO)
    for ksplit in (1, 2, 4, 8):
        for mode in (1, 2):
            check_gemm_ws(capi, m, n, k, g, capi.SQ_ALGO_SKINNY_WS | ((ksplit | (mode << 8)) << 8))
            # 4-wave workgroups
            check_gemm_ws(capi, m, n, k, g, capi.SQ_ALGO_SKINNY_WS | ((ksplit | (mode << 8) | (4 << 12)) << 8))


def test_skinny_ws_properties_and_workspace_reuse(capi):
    n, k, g = 4096, 16384, 128
    d = linear(n, k, g, seed=12)
    x = to_dev(orc.synth_x(16, k, seed=13))
    ws = capi.workspace(16, n, k, x.device)
    y1 = capi.gemm_ws(x, d["w_dev"], d["zs_dev"], n, k, g, ws=ws)
    # the call leaves the counters zero, so the same workspace serves the next call; results are bit-reproducible
    assert torch.count_nonzero(ws[:65536]).item() == 0
    for _ in range(3):
        assert torch.equal(y1, capi.gemm_ws(x, d["w_dev"], d["zs_dev"], n, k, g, ws=ws))
    y2 = capi.gemm_ws(x * 2, d["w_dev"], d["zs_dev"], n, k, g, ws=ws)
    normal = y1.abs() >= 2.0 ** -13
    assert torch.equal(y2[normal], (y1 * 2)[normal])
    e = torch.zeros((16, k), dtype=torch.float16, device=DEV)
    cols = [(977 * i + 5) % k for i in range(16)]
    for i, c in enumerate(cols):
        e[i, c] = 1.0
    ye = capi.gemm_ws(e, d["w_dev"], d["zs_dev"], n, k, g, ws=ws).cpu().numpy()
    for i, c in enumerate(cols):
        assert np.array_equal(ye[i].view(np.int16), d["w_hat"][:, c].view(np.int16))
    # a smaller problem right after a larger one on the same workspace
    check_gemm_ws(capi, 9, 200, 1536, 64, capi.SQ_ALGO_AUTO)
    # outside 5..32 the call falls through to the workspace-free kernels
    check_gemm_ws(capi, 1, 256, 1024, 128, capi.SQ_ALGO_AUTO)
    check_gemm_ws(capi, 100, 256, 1024, 128, capi.SQ_ALGO_AUTO)


def test_workspace_check_and_reset(capi):
    """The debug check reports a workspace whose counters are not zero (what a launch that died midway or two
    racing streams would leave), the reset kernel repairs it, and a call on the repaired workspace is right."""
    m, n, k, g = 16, 264, 2048, 128
    ws = torch.zeros(capi.lib().sq_w4a16_workspace_bytes(m, n, k), dtype=torch.uint8, device=DEV)
    assert capi.workspace_is_clean(ws)
    d = linear(n, k, g, 3)
    x = to_dev(orc.synth_x(m, k, seed=4))
    good = capi.gemm_ws(x, d["w_dev"], d["zs_dev"], n, k, g, algo=capi.SQ_ALGO_SKINNY_WS | (4 << 8), ws=ws)
    torch.cuda.synchronize()
    assert capi.workspace_is_clean(ws)            # every call leaves the counters zero
    ws[8] = 1                                     # simulate a stale counter
    assert not capi.workspace_is_clean(ws)
    capi.workspace_reset(ws, 65536)
    assert capi.workspace_is_clean(ws)
    again = capi.gemm_ws(x, d["w_dev"], d["zs_dev"], n, k, g, algo=capi.SQ_ALGO_SKINNY_WS | (4 << 8), ws=ws)
    assert torch.equal(good, again)
    L = capi.lib()
    assert L.sq_workspace_check(None, 64, None) == capi.SQ_ERR_NULL_POINTER
    assert L.sq_workspace_reset(ws.data_ptr() + 4, 64, None) == capi.SQ_ERR_MISALIGNED


def test_skinny_ws_rejects_small_workspace(capi):
    d = linear(256, 1024, 128, seed=0)
    x = to_dev(orc.synth_x(16, 1024))
    tiny = torch.zeros(1024, dtype=torch.uint8, device=DEV)
    with pytest.raises(capi.SqError) as ei:
        capi.gemm_ws(x, d["w_dev"], d["zs_dev"], 256, 1024, 128, algo=capi.SQ_ALGO_SKINNY_WS, ws=tiny)
    assert ei.value.code == capi.SQ_ERR_WORKSPACE
    # where the dispatcher picks a workspace-free kernel the workspace is not looked at
    capi.gemm_ws(x, d["w_dev"], d["zs_dev"], 256, 1024, 128, ws=tiny)


@pytest.mark.parametrize("n,k", [(16384, 4096), (4096, 16384), (4096, 4096)])
@pytest.mark.parametrize("m", [8, 16, 32])
def test_quant_extension_decode_batches_use_workspace_path(n, k, m):
    # gemm_awq_ut on decode batches of the fc1 / fc2 shapes goes through sq_w4a16_gemm_ws with the
    # extension's own cached workspace; also replayed from a HIP graph (several replays, same bits).
    import quant
    g = 128
    d = linear(n, k, g, seed=21)
    x = to_dev(orc.synth_x(m, k, seed=22)).reshape(1, m, k)
    y_ref = orc.gemm_ref(x.reshape(m, k).cpu().numpy(), d["w_hat"])
    y = quant.gemm_awq_ut(x, d["w_dev"], d["zs_dev"], m, n, k, g)
    assert y.shape == (1, m, n)
    err = np.max(np.abs(y.float().cpu().numpy().reshape(m, n) - y_ref))
    assert err <= TOL * np.max(np.abs(y_ref))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        y_warm = quant.gemm_awq_ut(x, d["w_dev"], d["zs_dev"], m, n, k, g)  # creates this stream's workspace
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            y_graph = quant.gemm_awq_ut(x, d["w_dev"], d["zs_dev"], m, n, k, g)
    assert torch.equal(y_warm, y)
    for _ in range(3):
        y_graph.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_graph, y)


# ------------------------------------------------------------------ fused epilogue: act(x W^T + bias) + residual
def fused_ref(x, w_hat, bias, residual, act):
    y = orc.gemm_ref(x, w_hat).astype(np.float64)
    if bias is not None:
        y = y + bias.astype(np.float64)[None, :]
    if act == 1:
        y = np.maximum(y, 0.0)
    elif act == 2:
        y = y / (1.0 + np.exp(-y))
    if residual is not None:
        y = y + residual.astype(np.float64)
    return y


FUSED_CASES = [  # (m, n, k, g, algo name, tune) -- one per kernel family and tile variant
    (1, 256, 1024, 128, "GEMV", 0), (3, 136, 640, 32, "GEMV_FIXUP", 0), (8, 200, 1536, 64, "GEMV_FIXUP", 2 | (4 << 4)),
    (5, 256, 1024, 128, "GEMV", 2 | (2 << 4)), (17, 136, 640, 32, "SKINNY", 0), (32, 256, 1024, 128, "SKINNY", 0),
    (9, 520, 1056, 32, "SKINNY_WS", 1), (16, 264, 2048, 128, "SKINNY_WS", 4), (32, 256, 1024, 128, "SKINNY_WS", 2),
    (70, 264, 704, 64, "GEMM", 1), (70, 264, 704, 64, "GEMM", 2), (300, 520, 1056, 32, "GEMM", 4),
    (300, 520, 1056, 32, "GEMM", 8), (300, 520, 1056, 32, "GEMM", 9), (300, 520, 1056, 32, "GEMM", 10),
]


@pytest.mark.parametrize("m,n,k,g,algo_name,tune", FUSED_CASES)
@pytest.mark.parametrize("use_bias,use_res,act", [(True, False, 0), (False, True, 0), (True, True, 1), (False, False, 1),
                                                  (True, True, 2)])
def test_fused_epilogue_every_kernel(capi, m, n, k, g, algo_name, tune, use_bias, use_res, act):
    d = linear(n, k, g, seed=31)
    rng = np.random.default_rng(32)
    x = orc.synth_x(m, k, seed=33)
    bias = rng.normal(0, 2.0, size=n).astype(np.float16) if use_bias else None
    res = rng.normal(0, 2.0, size=(m, n)).astype(np.float16) if use_res else None
    y_ref = fused_ref(x, d["w_hat"], bias, res, act)
    algo = getattr(capi, "SQ_ALGO_" + algo_name) | (tune << 8)
    y = capi.gemm_fused(to_dev(x), d["w_dev"], d["zs_dev"], n, k, g, bias=None if bias is None else to_dev(bias),
                        residual=None if res is None else to_dev(res), act=act, algo=algo)
    torch.cuda.synchronize()
    y = y.float().cpu().numpy()
    scale = np.max(np.abs(orc.gemm_ref(x, d["w_hat"])))
    assert np.max(np.abs(y - y_ref)) <= TOL * scale
    if act == 1 and not use_res:
        assert y.min() >= 0.0


def test_fused_epilogue_is_exactly_the_unfused_sum_in_fp32(capi):
    # With bias = 0 and residual = 0 the fused call returns the same bits as the plain one; with a
    # one-hot activation the result is fp16(W_hat[n, c] + bias[n] + residual) rounded once.
    n, k, g = 4096, 4096, 128
    d = linear(n, k, g, seed=7)
    x = to_dev(orc.synth_x(4, k, seed=8))
    zb = torch.zeros(n, dtype=torch.float16, device=DEV)
    zr = torch.zeros((4, n), dtype=torch.float16, device=DEV)
    assert torch.equal(capi.gemm_fused(x, d["w_dev"], d["zs_dev"], n, k, g, bias=zb, residual=zr),
                       capi.gemm(x, d["w_dev"], d["zs_dev"], n, k, g))
    e = torch.zeros((1, k), dtype=torch.float16, device=DEV)
    e[0, 77] = 1.0
    rng = np.random.default_rng(3)
    bias = rng.normal(0, 1, size=n).astype(np.float16)
    res = rng.normal(0, 1, size=(1, n)).astype(np.float16)
    # (exact-W_hat arithmetic mode: the default mode applies the scale in fp32 and is not W_hat to the bit)
    y = capi.gemm_fused(e, d["w_dev"], d["zs_dev"], n, k, g, bias=to_dev(bias), residual=to_dev(res),
                        algo=capi.SQ_ALGO_GEMV).cpu().numpy()
    want = (d["w_hat"][:, 77].astype(np.float32) + bias.astype(np.float32) + res[0].astype(np.float32)).astype(np.float16)
    assert np.array_equal(y[0].view(np.int16), want.view(np.int16))


@pytest.mark.parametrize("m", [1, 2, 4, 8, 16, 24, 32, 40, 100, 300])
@pytest.mark.parametrize("n,k,g", [(512, 1024, 128), (264, 704, 64)])
def test_gated_mlp_front_half(capi, m, n, k, g):
    """silu(x W_gate^T) * (x W_up^T) through sq_w4a16_gemm_silu_dot against the oracle, within this
    suite's bar relative to the largest output (every decode, streaming and tiled kernel of the
    automatic dispatch takes a turn over these token counts); the scratch tensor holds the up projection."""
    gate = linear(n, k, g, seed=51)
    up = linear(n, k, g, seed=52)
    x = orc.synth_x(m, k, seed=53)
    want = orc.silu_dot_ref(x, gate["w_hat"], up["w_hat"])
    y, up_out = capi.gemm_silu_dot(to_dev(x), gate["w_dev"], gate["zs_dev"], up["w_dev"], up["zs_dev"], n, k, g)
    torch.cuda.synchronize()
    got = y.float().cpu().numpy().astype(np.float64)
    assert np.max(np.abs(got - want)) <= TOL * np.max(np.abs(want))
    up_ref = orc.gemm_ref(x, up["w_hat"])
    assert np.max(np.abs(up_out.float().cpu().numpy() - up_ref)) <= TOL * np.max(np.abs(up_ref))


def test_gated_mlp_rejections(capi):
    n, k, g = 256, 1024, 128
    d = linear(n, k, g, seed=0)
    x = to_dev(orc.synth_x(2, k))
    y = torch.empty((2, n), dtype=torch.float16, device=DEV)
    L = capi.lib()
    p = lambda t: t.data_ptr()
    args = (p(x), p(d["w_dev"]), p(d["zs_dev"]), p(d["w_dev"]), p(d["zs_dev"]))
    assert L.sq_w4a16_gemm_silu_dot(*args, p(y), None, 2, n, k, g, capi.SQ_LAYOUT_L1, None, 0, None) == capi.SQ_ERR_NULL_POINTER
    assert L.sq_w4a16_gemm_silu_dot(*args, p(y), p(y), 2, n, k, g, capi.SQ_LAYOUT_L1, None, 0, None) == capi.SQ_ERR_BAD_SHAPE
    assert L.sq_w4a16_gemm_silu_dot(*args, p(y), p(y) + 2, 2, n, k, g, capi.SQ_LAYOUT_L1, None, 0, None) == capi.SQ_ERR_MISALIGNED
    assert L.sq_w4a16_gemm_silu_dot(*args, p(y), p(x), 2, n, k, 48, capi.SQ_LAYOUT_L1, None, 0, None) == capi.SQ_ERR_BAD_GROUP
    assert L.sq_w4a16_gemm_silu_dot(*args, p(y), None, 0, n, k, g, capi.SQ_LAYOUT_L1, None, 0, None) == capi.SQ_OK


@pytest.mark.parametrize("m", [1, 8, 128])
def test_quant_extension_gated_mlp(m):
    """gemm_awq_silu_dot_ut with the call shapes, the data recipe and the tolerance of the reference's kernel
    test (nn.Linear weights through the packer, x ~ N(0, 0.5), two weights or one packed weight with 2N
    outputs, allclose at atol = rtol = 2e-2; quantization/nvidia/script/gemm_awq_test.py:50-56,66-72,92-105),
    in both layouts; the expected value is the oracle's on the dequantised weights."""
    import quant
    from sqamd import quant_funcs as qf
    torch.manual_seed(7)
    n, k, g = 256, 1024, 128
    lin1 = torch.nn.Linear(k, n, bias=False, device=DEV, dtype=torch.float16)
    lin2 = torch.nn.Linear(k, n, bias=False, device=DEV, dtype=torch.float16)
    qw1, zs1 = qf.quant_muxi(lin1.weight.data, k, n, n_bit=4, group_size=g)
    qw2, zs2 = qf.quant_muxi(lin2.weight.data, k, n, n_bit=4, group_size=g)
    w_hat1 = orc.dequant_l1(qw1.cpu().numpy(), zs1.cpu().numpy(), g)
    w_hat2 = orc.dequant_l1(qw2.cpu().numpy(), zs2.cpu().numpy(), g)
    xd = torch.empty((1, m, k), dtype=torch.float16, device=DEV).normal_(mean=0.0, std=0.5)
    want = orc.silu_dot_ref(xd.cpu().numpy().reshape(m, k), w_hat1, w_hat2)

    def check(out):
        assert tuple(out.shape) == (1, m, n) and out.dtype == torch.float16
        got = out.float().cpu().numpy().reshape(m, n).astype(np.float64)
        assert np.all(np.abs(got - want) <= 2e-2 + 2e-2 * np.abs(want))
        assert np.max(np.abs(got - want)) <= TOL * np.max(np.abs(want))

    check(quant.gemm_awq_silu_dot_ut(xd, qw1, qw2, zs1, zs2, None, None, m, n, k, g))
    w13 = torch.cat((lin1.weight.data, lin2.weight.data), dim=0).contiguous()
    qw13, zs13 = qf.quant_muxi(w13, k, 2 * n, n_bit=4, group_size=g)
    assert torch.equal(qw13, torch.cat((qw1, qw2), dim=0))
    check(quant.gemm_awq_silu_dot_ut(xd, None, None, None, None, qw13, zs13, m, n, k, g))
    qw13_l2, zs13_l2, _ = qf.quant_lmdeploy(w13, k, 2 * n, group_size=g, n_bit=4)
    check(quant.gemm_awq_silu_dot_ut(xd, None, None, None, None, qw13_l2, zs13_l2, m, n, k, g))
    with pytest.raises(ValueError):
        quant.gemm_awq_silu_dot_ut(xd, qw1, None, zs1, None, None, None, m, n, k, g)
    quant.clear_repack_cache()


@pytest.mark.parametrize("m,n,k,g", [(300, 520, 1056, 32), (70, 264, 1024, 128), (24, 256, 8192, 128), (8, 256, 16384, 128),
                                     (2048, 512, 1024, 128)])
def test_fused_epilogue_operands_at_odd_addresses(capi, m, n, k, g):
    """bias and residual only need 2-byte alignment: the tiled kernels' tile store and the split-K decode
    kernels' four-column tail fall back from their wide loads, same results as with aligned operands."""
    d = linear(n, k, g, seed=71)
    rng = np.random.default_rng(72)
    x = to_dev(orc.synth_x(m, k, seed=73))
    bias = rng.normal(0, 2.0, size=n).astype(np.float16)
    res = rng.normal(0, 2.0, size=(m, n)).astype(np.float16)
    bias_buf = torch.zeros(n + 8, dtype=torch.float16, device=DEV)
    res_buf = torch.zeros(m * n + 8, dtype=torch.float16, device=DEV)
    outs = []
    for off in (0, 1, 4):  # 16-byte, 2-byte and 8-byte aligned
        b = bias_buf[off:off + n]
        r = res_buf[off:off + m * n].view(m, n)
        b.copy_(to_dev(bias))
        r.copy_(to_dev(res))
        assert b.data_ptr() % 16 == 2 * off
        y = capi.gemm_fused(x, d["w_dev"], d["zs_dev"], n, k, g, bias=b, residual=r, act=capi.SQ_ACT_RELU)
        torch.cuda.synchronize()
        outs.append(y.clone())
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    want = fused_ref(x.cpu().numpy(), d["w_hat"], bias, res, 1)
    assert np.max(np.abs(outs[0].float().cpu().numpy() - want)) <= TOL * np.max(np.abs(orc.gemm_ref(x.cpu().numpy(), d["w_hat"])))


def test_fused_rejects_bad_activation(capi):
    d = linear(256, 1024, 128, seed=0)
    x = to_dev(orc.synth_x(2, 1024))
    with pytest.raises(capi.SqError) as ei:
        capi.gemm_fused(x, d["w_dev"], d["zs_dev"], 256, 1024, 128, act=7)
    assert ei.value.code == capi.SQ_ERR_BAD_ALGO


@pytest.mark.parametrize("m", [1, 8, 16, 200])
def test_quant_extension_fused_variants(m):
    import quant
    from sqamd.qlinear import WALinear
    n, k, g = 512, 2048, 128
    d = linear(n, k, g, seed=41)
    rng = np.random.default_rng(42)
    x = to_dev(orc.synth_x(m, k, seed=43)).reshape(1, m, k)
    r = to_dev(rng.normal(0, 2.0, size=(1, m, n)).astype(np.float16))
    b = to_dev(rng.normal(0, 2.0, size=(1, n)).astype(np.float16))
    plain = quant.gemm_awq_ut(x, d["w_dev"], d["zs_dev"], m, n, k, g).float()
    y = quant.gemm_awq_residual_ut(x, d["w_dev"], d["zs_dev"], r, m, n, k, g)
    assert torch.allclose(y.float(), plain + r.float(), atol=2e-2, rtol=2e-2)  # the reference test's own tolerance
    lin = WALinear(k, n, w_bit=4, group_size=g, bias=True, dev=DEV)
    lin.weight, lin.zeros_scales, lin.bias = d["w_dev"], d["zs_dev"], b
    y2 = lin(x.reshape(m, k), residual=r.reshape(m, n), act="relu")
    want = torch.relu(plain.reshape(m, n) + b.float()) + r.reshape(m, n).float()
    assert y2.shape == (m, n)
    assert torch.allclose(y2.float(), want, atol=2e-2, rtol=2e-2)
    assert torch.allclose(lin(x).float(), plain + b.float(), atol=2e-2, rtol=2e-2)
    with pytest.raises((RuntimeError, ValueError)):
        quant.gemm_awq_fused_ut(x, d["w_dev"], d["zs_dev"], None, None, "gelu", n, g)
    with pytest.raises((RuntimeError, ValueError)):
        quant.gemm_awq_residual_ut(x, d["w_dev"], d["zs_dev"], r[:, :, :8].contiguous(), m, n, k, g)


# ------------------------------------------------------------------ the reference's own kernel-test grids
REF_DIMS = [(4096, 4096), (5120, 5120), (11008, 4096), (13696, 5120)]  # (in, out), gemm_awq_test.py "Dim"


@pytest.mark.parametrize("k,n", REF_DIMS)
def test_reference_grid_uint8_layout(k, n):
    """quantization/muxi/script/gemm_awq_test.py:26-34,80-109: batch 1, sequence lengths 1..512, group 128,
    x ~ N(0, 0.5), allclose(atol = rtol = 2e-2) against x @ W_hat^T (seeded here)."""
    import quant
    from sqamd import quant_funcs as qf
    torch.manual_seed(k + n)
    g = 128
    lin = torch.nn.Linear(k, n, bias=False, device=DEV, dtype=torch.float16)
    qweight, zeros_scales = qf.quant_muxi(lin.weight.data, k, n, n_bit=4, group_size=g)
    w_fp16 = qf.dequant_to_fp16(lin.weight.data, 4, g).float()
    for seq in (1, 2, 4, 8, 16, 32, 64, 128, 256, 512):
        x = torch.empty((1, seq, k), dtype=torch.float16, device=DEV).normal_(mean=0.0, std=0.5)
        out = quant.gemm_awq_ut(x, qweight, zeros_scales, seq, n, k, g)
        ref = torch.matmul(x.float(), w_fp16.t())
        assert torch.allclose(ref, out.float(), atol=2e-2, rtol=2e-2), (k, n, seq)


@pytest.mark.parametrize("k,n", REF_DIMS)
def test_reference_grid_int32_layout(k, n):
    """quantization/nvidia/script/gemm_awq_test.py:33-38,89-114: sequence lengths 1 and 128, batch sizes
    1..64, group 128, weights in the tensor-core tile layout produced by the converter chain."""
    import quant
    from sqamd import quant_funcs as qf
    torch.manual_seed(k * 3 + n)
    g = 128
    lin = torch.nn.Linear(k, n, bias=False, device=DEV, dtype=torch.float16)
    qweight, zeros_scales, _ = qf.quant_lmdeploy(lin.weight.data, k, n, group_size=g)
    assert qweight.dtype == torch.int32 and tuple(qweight.shape) == (k, n // 8)
    w_fp16 = qf.dequant_to_fp16(lin.weight.data, 4, g).float()
    for seq in (1, 128):
        for bs in (1, 2, 4, 8, 16, 32, 48, 64):
            x = torch.empty((bs, seq, k), dtype=torch.float16, device=DEV).normal_(mean=0.0, std=0.5)
            out = quant.gemm_awq_ut(x, qweight, zeros_scales, bs * seq, n, k, g)
            ref = torch.matmul(x.float(), w_fp16.t())
            assert tuple(out.shape) == (bs, seq, n)
            assert torch.allclose(ref, out.float(), atol=2e-2, rtol=2e-2), (k, n, bs, seq)
    quant.clear_repack_cache()


# ------------------------------------------------------------------ 33..512 tokens through the dispatcher
@pytest.mark.parametrize("n,k,g", [(520, 1056, 32), (4096, 4096, 128), (16384, 4096, 128), (4096, 16384, 128)])
@pytest.mark.parametrize("m", [33, 48, 64, 65, 100, 128, 129, 200, 512])
def test_mid_size_batches_auto_dispatch(capi, n, k, g, m):
    # with a workspace (token blocks through the split-K kernel where the GEMM grid would be tiny) ...
    check_gemm_ws(capi, m, n, k, g, capi.SQ_ALGO_AUTO)
    # ... and without one
    check_gemm(capi, m, n, k, g, capi.SQ_ALGO_AUTO)


def test_mid_size_batch_fused_epilogue_blocks(capi):
    # bias / ReLU / residual reach every 32-token block of a blocked launch
    m, n, k, g = 100, 4096, 16384, 128
    d = linear(n, k, g, seed=51)
    rng = np.random.default_rng(52)
    x = orc.synth_x(m, k, seed=53)
    bias = rng.normal(0, 2.0, size=n).astype(np.float16)
    res = rng.normal(0, 2.0, size=(m, n)).astype(np.float16)
    y = capi.gemm_fused(to_dev(x), d["w_dev"], d["zs_dev"], n, k, g, bias=to_dev(bias), residual=to_dev(res), act=1)
    y_ref = fused_ref(x, d["w_hat"], bias, res, 1)
    scale = np.max(np.abs(orc.gemm_ref(x, d["w_hat"])))
    assert np.max(np.abs(y.float().cpu().numpy() - y_ref)) <= TOL * scale


@pytest.mark.parametrize("mi", [1, 2, 4])
@pytest.mark.parametrize("ksplit", [2, 4, 8])
def test_gemm_split_k_every_tile_height(capi, mi, ksplit):
    # K split over workgroups in the tiled GEMM (partial tiles through the workspace), incl. ragged N, M and
    # K ranges that do not divide evenly; bit-reproducible across calls on one workspace
    for (m, n, k, g) in [(70, 264, 2112, 64), (200, 520, 4096, 128), (129, 4096, 4096, 128)]:
        algo = capi.SQ_ALGO_GEMM | ((mi | (ksplit << 8)) << 8)
        d = linear(n, k, g, seed=61)
        x = to_dev(orc.synth_x(m, k, seed=62))
        ws = torch.zeros(64 * 1024 * 1024, dtype=torch.uint8, device=DEV)
        y1 = capi.gemm_ws(x, d["w_dev"], d["zs_dev"], n, k, g, algo=algo, ws=ws)
        y_ref = orc.gemm_ref(x.cpu().numpy(), d["w_hat"])
        assert np.max(np.abs(y1.float().cpu().numpy() - y_ref)) <= TOL * np.max(np.abs(y_ref))
        assert torch.count_nonzero(ws[:65536]).item() == 0
        assert torch.equal(y1, capi.gemm_ws(x, d["w_dev"], d["zs_dev"], n, k, g, algo=algo, ws=ws))


@pytest.mark.parametrize("mi", [1, 2, 4])
@pytest.mark.parametrize("ksplit", [1, 2, 4, 8])
def test_gemm_operands_through_lds(capi, mi, ksplit):
    # the tiled kernel whose weights, activations and zeros/scales all reach LDS by direct loads (group sizes 32, 64,
    # 128; K a multiple of 256): parity against the oracle on ragged M and N, K = 256 x odd, K ranges of the split that
    # are padded; bit-identical to the register-staged kernel at the same tile height and split; counters left clean
    lds = 0x80
    for (m, n, k, g) in [(33, 264, 768, 128), (70, 520, 1280, 128), (129, 4096, 4096, 128), (200, 264, 2816, 128),
                         (300, 1000, 11008, 128), (70, 520, 1280, 64), (129, 1000, 2816, 64), (300, 264, 768, 64),
                         (70, 520, 1280, 32), (129, 1000, 2816, 32), (300, 264, 768, 32)]:
        d = linear(n, k, g, seed=71)
        x = to_dev(orc.synth_x(m, k, seed=72))
        ws = torch.zeros(64 * 1024 * 1024, dtype=torch.uint8, device=DEV)
        tune = mi | (ksplit << 8)
        y_lds = capi.gemm_ws(x, d["w_dev"], d["zs_dev"], n, k, g, algo=capi.SQ_ALGO_GEMM | ((tune | lds) << 8), ws=ws)
        y_ref = orc.gemm_ref(x.cpu().numpy(), d["w_hat"])
        assert np.max(np.abs(y_lds.float().cpu().numpy() - y_ref)) <= TOL * np.max(np.abs(y_ref)), (m, n, k)
        assert torch.count_nonzero(ws[:65536]).item() == 0
        if ksplit == 1:  # the split ranges of the two kernels differ (whole groups of four steps here)
            y_reg = capi.gemm_ws(x, d["w_dev"], d["zs_dev"], n, k, g, algo=capi.SQ_ALGO_GEMM | (tune << 8), ws=ws)
            assert torch.equal(y_lds, y_reg), (m, n, k)
        assert torch.equal(y_lds, capi.gemm_ws(x, d["w_dev"], d["zs_dev"], n, k, g,
                                               algo=capi.SQ_ALGO_GEMM | ((tune | lds) << 8), ws=ws))


def test_gemm_lds_request_falls_back_where_it_does_not_apply(capi):
    # a K that is no multiple of 256 runs the register-staged kernel under the same request
    for (m, n, k, g) in [(70, 264, 704, 64), (100, 520, 1056, 32), (65, 264, 640, 128)]:
        check_gemm(capi, m, n, k, g, capi.SQ_ALGO_GEMM | ((2 | 0x80) << 8))


@pytest.mark.parametrize("m", [33, 64, 100, 256, 1000, 2048])
def test_gemm_lds_fused_epilogue(capi, m):
    # bias, ReLU and residual through the automatic choice at group size 128 (the LDS kernel, K split for small m)
    n, k, g = 1000, 2816, 128
    d = linear(n, k, g, seed=81)
    rng = np.random.default_rng(82)
    x = orc.synth_x(m, k, seed=83)
    bias = rng.normal(0, 2.0, size=n).astype(np.float16)
    res = rng.normal(0, 2.0, size=(m, n)).astype(np.float16)
    y = capi.gemm_fused(to_dev(x), d["w_dev"], d["zs_dev"], n, k, g, bias=to_dev(bias), residual=to_dev(res), act=1)
    y_ref = fused_ref(x, d["w_hat"], bias, res, 1)
    scale = np.max(np.abs(orc.gemm_ref(x, d["w_hat"])))
    assert np.max(np.abs(y.float().cpu().numpy() - y_ref)) <= TOL * scale


def test_mfma_probe_reports_one_instruction_per_32_cycles(capi):
    data = torch.randn(5120, device=DEV).half()
    ticks = capi.mfma_probe(data, 4, 2000)
    torch.cuda.synchronize()
    per = ticks.double().median().item() / (2000 * 16)
    assert 31.0 <= per <= 40.0, per
    with pytest.raises(capi.SqError):
        capi.mfma_probe(data, 0, 10)


def test_read_probe_runs_on_every_reference_shape(capi):
    out = torch.zeros(4096, dtype=torch.int32, device=DEV)
    for n, k in ((4096, 4096), (16384, 4096), (4096, 16384), (11008, 4096), (200, 1056)):
        g = 128 if k % 128 == 0 else 32
        w = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device=DEV)
        zs = torch.zeros((n, 2 * (k // g)), dtype=torch.float16, device=DEV)
        rc = capi.probes().sq_read_probe(w.data_ptr(), zs.data_ptr(), out.data_ptr(), n, k, g, None)
        assert rc == 0
    torch.cuda.synchronize()
    assert capi.probes().sq_read_probe(None, None, out.data_ptr(), 4096, 4096, 128, None) == capi.SQ_ERR_NULL_POINTER


def test_measured_kernel_choice_is_recorded_and_used(capi):
    """sq_w4a16_autotune times every kernel that can serve a shape and records the fastest for SQ_ALGO_AUTO: the
    recorded word is one sq_w4a16_gemm_ex accepts, the automatic path then gives that kernel's result bit for bit
    and stays within the bar of the oracle; clearing forgets the choice."""
    g = 128
    capi.autotune_clear()
    for m, n, k in ((8, 1024, 8192), (32, 2048, 2048), (96, 1536, 4096)):
        d = orc.synth_linear(n, k, g, seed=m + n)
        w, zs = to_dev(d["w_l1"]), to_dev(d["zs_l1"])
        x = to_dev(orc.synth_x(m, k, seed=m))
        ws = capi.workspace(m, n, k, DEV)
        y_tuned = torch.empty((m, n), dtype=torch.float16, device=DEV)
        word, t_best, t_auto = capi.autotune(x, w, zs, n, k, g, ws=ws, reps=5, out=y_tuned)
        assert 0 < t_best <= t_auto
        y_ref = orc.gemm_ref(orc.synth_x(m, k, seed=m), orc.dequant_l1(d["w_l1"], d["zs_l1"], g))
        assert np.max(np.abs(y_tuned.float().cpu().numpy() - y_ref)) <= TOL * np.max(np.abs(y_ref))
        y_auto = capi.gemm_ws(x, w, zs, n, k, g, ws=ws)
        torch.cuda.synchronize()
        assert torch.equal(y_auto, y_tuned)
        if word:
            y_ex = capi.gemm_ws(x, w, zs, n, k, g, algo=word, ws=ws)
            torch.cuda.synchronize()
            assert torch.equal(y_ex, y_tuned)
    capi.autotune_clear()
    assert capi.autotune_clear() == 0


# ------------------------------------------------------------------ seeded random shapes through the built-in choice
@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_shapes_fused_auto_dispatch(capi, seed):
    """Eighty seeded random (M, N, K, group, bias, residual, activation) cases per seed through SQ_ALGO_AUTO, each
    with and without a workspace (so that every kernel family the rule table can pick is reached at shapes nobody
    tuned), against the oracle's fp32 result and the fp32 epilogue formula."""
    rng = np.random.default_rng(seed)
    for c in range(80):
        g = int(rng.choice([32, 64, 128]))
        if rng.random() < 0.7:
            k = max(g, 128) * int(rng.choice([1, 2, 3, 4, 5, 8, 11, 16, 32, 43]))
        else:
            k = g * int(rng.integers(1, 40))
        k = max((k + 31) // 32 * 32, g)
        n = int(rng.choice([8, 16, 24, 40, 64, 72, 128, 136, 256, 264, 520, 1024, 1032, 2048, 4096]))
        m = int(rng.choice([1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 24, 31, 32, 33, 48, 64, 65, 100, 128, 129, 200, 257,
                            512, 700]))
        if n * k > 4096 * 8192:
            k = 1024
        d = orc.synth_linear(n, k, g, seed=1000 * seed + c)
        w_hat = orc.dequant_l1(d["w_l1"], d["zs_l1"], g)
        x = orc.synth_x(m, k, seed=1000 * seed + c + 500)
        use_b, use_r, act = bool(rng.integers(0, 2)), bool(rng.integers(0, 2)), int(rng.integers(0, 3))
        bias = (rng.standard_normal(n) * 2).astype(np.float16) if use_b else None
        res = (rng.standard_normal((m, n)) * 2).astype(np.float16) if use_r else None
        z = orc.gemm_ref(x, w_hat) + (bias.astype(np.float32) if use_b else 0)
        if act == capi.SQ_ACT_RELU:
            z = np.maximum(z, 0)
        elif act == capi.SQ_ACT_SILU:
            z = z / (1 + np.exp(-z))
        y_ref = z + (res.astype(np.float32) if use_r else 0)
        xd, wd, zd = to_dev(x), to_dev(d["w_l1"]), to_dev(d["zs_l1"])
        bd = to_dev(bias) if use_b else None
        rd = to_dev(res) if use_r else None
        for use_ws in (False, True):
            y = capi.gemm_fused(xd, wd, zd, n, k, g, bias=bd, residual=rd, act=act, use_workspace=use_ws)
            torch.cuda.synchronize()
            y = y.float().cpu().numpy()
            what = (seed, c, m, n, k, g, use_b, use_r, act, use_ws)
            assert np.all(np.isfinite(y)), what
            assert np.max(np.abs(y - y_ref)) <= TOL * max(np.max(np.abs(y_ref)), 1e-6), what


@pytest.mark.parametrize("m,n,k,g", [(32, 13824, 5120, 128), (17, 13824, 5120, 128), (24, 5120, 13824, 128),
                                     (32, 8192, 4352, 64), (20, 8192, 4352, 32)])
def test_large_weights_17_to_32_tokens_auto_dispatch(capi, m, n, k, g):
    """Large weights whose K is no multiple of 4096 at 17..32 tokens, which the automatic choice serves with the tiled
    GEMM's 32-row tiles and a K split through the workspace: every output element against the oracle with bias,
    ReLU and residual in the store, and against the split-K decode kernel asked for by name on the same operands."""
    d = orc.synth_linear(n, k, g, seed=n + k + m)
    w_hat = orc.dequant_l1(d["w_l1"], d["zs_l1"], g)
    x = orc.synth_x(m, k, seed=m + 3)
    rng = np.random.default_rng(m + n)
    bias = (rng.standard_normal(n) * 2).astype(np.float16)
    res = (rng.standard_normal((m, n)) * 2).astype(np.float16)
    y_ref = np.maximum(orc.gemm_ref(x, w_hat) + bias.astype(np.float32), 0) + res.astype(np.float32)
    xd, wd, zd, bd, rd = to_dev(x), to_dev(d["w_l1"]), to_dev(d["zs_l1"]), to_dev(bias), to_dev(res)
    scale = np.max(np.abs(y_ref))
    for use_ws in (True, False):
        y = capi.gemm_fused(xd, wd, zd, n, k, g, bias=bd, residual=rd, act=capi.SQ_ACT_RELU, use_workspace=use_ws)
        torch.cuda.synchronize()
        y = y.float().cpu().numpy()
        assert np.all(np.isfinite(y))
        assert np.max(np.abs(y - y_ref)) <= TOL * scale, (m, n, k, g, use_ws)
    y_named = capi.gemm_fused(xd, wd, zd, n, k, g, bias=bd, residual=rd, act=capi.SQ_ACT_RELU,
                              algo=capi.SQ_ALGO_SKINNY_WS, use_workspace=True)
    torch.cuda.synchronize()
    assert np.max(np.abs(y_named.float().cpu().numpy() - y_ref)) <= TOL * scale
