"""GPU parity at the full sizes of the benchmark configurations, against the CPU oracle.

The HIP path runs the whole problem through the product dispatch; the oracle checks it on sampled
token rows (all N columns of each), which keeps the fp32 reference matmul to seconds on the host:
  * prefill: M in {2048, 4096} on the five prefill shapes (4096x4096, 4096->16384, 16384->4096,
    4096->11008, 11008->4096), group 128, through the C ABI and through quant.gemm_awq_ut, the
    int32 tensor-core layout included (weights packed by the oracle, not by the package);
  * the gated MLP front half at the Llama-7B size (two 11008 x 4096 weights) at 1, 8 and 2048 tokens;
  * LUT attention at batch 8, 16 heads, head dim 64, 4096 tokens, 25 % density, non-causal, on
    sampled (batch, head) pairs;
  * one full-width OPT-6.7B decoder layer (hidden 4096, FFN 16384, 32 heads, batch 8, 640-row cache)
    against the composition of the oracle's LayerNorm, dequant, GEMM and decode attention;
  * the 32-layer decode harness: eager and HIP-graph replays generate the same tokens.
Bars as everywhere: dequant bit-exact, max|Y - Y_ref| <= 1e-2 * max|Y_ref|."""
import numpy as np
import pytest
import torch

import lut_attention_oracle as att
import w4a16_oracle as orc

pytestmark = pytest.mark.gpu
TOL = 1e-2
DEV = "cuda:0"
PREFILL_SHAPES = [(4096, 4096), (16384, 4096), (4096, 16384), (11008, 4096), (4096, 11008)]  # (N, K)


@pytest.fixture(scope="module")
def capi(built_lib):
    from sqamd import capi as c
    c.lib()
    return c


def to_dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def sample_rows(m, count, seed):
    """Token rows to check: the corners of the 256-row output tiles plus random ones."""
    fixed = [r for r in (0, 1, 31, 32, 127, 128, 255, 256, 257, m // 2 - 1, m // 2, m - 257, m - 256, m - 2, m - 1) if 0 <= r < m]
    rng = np.random.default_rng(seed)
    rows = sorted(set(fixed) | set(rng.choice(m, size=count, replace=False).tolist()))
    return np.array(rows[:max(count, len(fixed))])


def rel_err(y, y_ref):
    y = np.asarray(y, dtype=np.float64)
    assert np.all(np.isfinite(y))
    return np.max(np.abs(y - y_ref)) / np.max(np.abs(y_ref))


@pytest.mark.parametrize("n,k", PREFILL_SHAPES)
def test_prefill_full_size_against_oracle(capi, n, k):
    import quant
    g = 128
    d = orc.synth_linear(n, k, g, seed=n // 64 + k)
    w_hat = orc.dequant_l1(d["w_l1"], d["zs_l1"], g)
    w, zs = to_dev(d["w_l1"]), to_dev(d["zs_l1"])
    deq = quant.dequant(w, zs, n, k, g)
    assert np.array_equal(deq.cpu().numpy().view(np.int16), w_hat.view(np.int16)), "dequant is not bit-exact"
    del deq
    for m in (2048, 4096):
        x = orc.synth_x(m, k, seed=m + n)
        rows = sample_rows(m, 64, seed=m)
        y_ref = orc.gemm_ref(x[rows], w_hat)
        xd = to_dev(x)
        print("prefill parity n=%d k=%d m=%d" % (n, k, m), flush=True)
        y_abi = capi.gemm(xd, w, zs, n, k, g)                       # sq_w4a16_gemm_ex, automatic dispatch
        y_ext = quant.gemm_awq_ut(xd.view(1, m, k), w, zs, m, n, k, g)  # the extension's call path
        torch.cuda.synchronize()
        idx = torch.from_numpy(rows).to(DEV)
        e1 = rel_err(y_abi[idx].float().cpu().numpy(), y_ref)
        e2 = rel_err(y_ext.view(m, n)[idx].float().cpu().numpy(), y_ref)
        assert e1 <= TOL and e2 <= TOL, "n=%d k=%d m=%d: %.3e %.3e" % (n, k, m, e1, e2)
        assert e1 < 5e-3 and e2 < 5e-3
        # the rows that were not sampled: finite, and the two call paths agree on the whole output
        assert torch.isfinite(y_abi).all()
        assert torch.equal(y_abi, y_ext.view(m, n))


@pytest.mark.parametrize("m", [1, 8, 2048])
def test_gated_mlp_llama_size_against_oracle(capi, m):
    """silu(x W_gate^T) * (x W_up^T) at the Llama-7B MLP size (two 11008 x 4096 weights, group 128): the fused
    entry point and the extension's packed call shape against the oracle on sampled token rows, with bias-free
    weights packed by the oracle; the scratch tensor holds the plain up projection."""
    import quant
    n, k, g = 11008, 4096, 128
    gate = orc.synth_linear(n, k, g, seed=5)
    up = orc.synth_linear(n, k, g, seed=6)
    wg_hat = orc.dequant_l1(gate["w_l1"], gate["zs_l1"], g)
    wu_hat = orc.dequant_l1(up["w_l1"], up["zs_l1"], g)
    x = orc.synth_x(m, k, seed=m)
    rows = sample_rows(m, 32, seed=m) if m > 64 else np.arange(m)
    want = orc.silu_dot_ref(x[rows], wg_hat, wu_hat)
    xd = to_dev(x)
    wg, zg, wu, zu = (to_dev(a) for a in (gate["w_l1"], gate["zs_l1"], up["w_l1"], up["zs_l1"]))
    print("gated mlp parity m=%d" % m, flush=True)
    y, up_out = capi.gemm_silu_dot(xd, wg, zg, wu, zu, n, k, g)
    w13 = torch.cat((wg, wu), dim=0).contiguous()
    zs13 = torch.cat((zg, zu), dim=0).contiguous()
    y_ext = quant.gemm_awq_silu_dot_ut(xd.view(1, m, k), None, None, None, None, w13, zs13, m, n, k, g)
    torch.cuda.synchronize()
    idx = torch.from_numpy(rows).to(DEV)
    assert rel_err(y[idx].float().cpu().numpy(), want) <= TOL
    assert rel_err(up_out[idx].float().cpu().numpy(), orc.gemm_ref(x[rows], wu_hat)) <= TOL
    assert torch.isfinite(y).all()
    assert torch.equal(y, y_ext.view(m, n))


@pytest.mark.parametrize("n,k", [(4096, 4096), (4096, 11008)])
def test_prefill_full_size_int32_layout_against_oracle(n, k):
    """The tensor-core layout at the reference's own test sizes (quantization/nvidia/script/
    gemm_awq_test.py:33-38 with M = 2048): weight and zeros_scales packed by the oracle's restatement
    of the converter chain, product through quant.gemm_awq_ut (repacked once behind the call)."""
    import quant
    g, m = 128, 2048
    d = orc.synth_linear(n, k, g, seed=7 + n // 64 + k)
    w_hat = orc.dequant_l1(d["w_l1"], d["zs_l1"], g)
    w2 = orc.pack_l2(d["q"])
    zs2 = orc.transpose_merge_zeros_scales(d["z"].astype(np.float16), d["s"], k, n, g)
    assert np.array_equal(orc.dequant_l2(w2, zs2, g, k, n).view(np.int16), w_hat.view(np.int16))
    w2d, zs2d = to_dev(w2.view(np.int32)), to_dev(zs2)
    assert np.array_equal(quant.dequant(w2d, zs2d, n, k, g).cpu().numpy().view(np.int16), w_hat.view(np.int16))
    x = orc.synth_x(m, k, seed=3)
    rows = sample_rows(m, 64, seed=5)
    y_ref = orc.gemm_ref(x[rows], w_hat)
    quant.clear_repack_cache()
    y = quant.gemm_awq_ut(to_dev(x).view(1, m, k), w2d, zs2d, m, n, k, g)
    torch.cuda.synchronize()
    err = rel_err(y.view(m, n)[torch.from_numpy(rows).to(DEV)].float().cpu().numpy(), y_ref)
    assert err < 5e-3, "n=%d k=%d: %.3e" % (n, k, err)
    quant.clear_repack_cache()


def test_int32_layout_repack_cache_follows_zeros_scales():
    """The repack cache behind gemm_awq_ut holds the converted zeros_scales too: a call with the same
    weight and other (or modified) zeros_scales must not be served the stale conversion."""
    import quant
    n, k, g, m = 256, 512, 128, 6
    d = orc.synth_linear(n, k, g, seed=11)
    w2d = to_dev(orc.pack_l2(d["q"]).view(np.int32))
    x = orc.synth_x(m, k, seed=12)
    xd = to_dev(x).view(1, m, k)
    quant.clear_repack_cache()
    rng = np.random.default_rng(13)

    def zs_l2(z, s):
        return to_dev(orc.transpose_merge_zeros_scales(z.astype(np.float16), s, k, n, g))

    def ref(z, s):
        return orc.gemm_ref(x, orc.dequant_l1(d["w_l1"], orc.zeros_scales_l1(z, s), g))

    za, sa = d["z"], d["s"]
    zsa = zs_l2(za, sa)
    ya = quant.gemm_awq_ut(xd, w2d, zsa, m, n, k, g)
    assert rel_err(ya.view(m, n).float().cpu().numpy(), ref(za, sa)) < 5e-3
    # another zeros_scales tensor with the same weight
    zb = rng.integers(0, 16, size=za.shape, dtype=np.uint8)
    sb = (sa.astype(np.float32) * 1.5).astype(np.float16)
    zsb = zs_l2(zb, sb)
    yb = quant.gemm_awq_ut(xd, w2d, zsb, m, n, k, g)
    assert rel_err(yb.view(m, n).float().cpu().numpy(), ref(zb, sb)) < 5e-3
    # the same zeros_scales tensor modified in place
    zc = rng.integers(0, 16, size=za.shape, dtype=np.uint8)
    zsb.copy_(zs_l2(zc, sb))
    yc = quant.gemm_awq_ut(xd, w2d, zsb, m, n, k, g)
    assert rel_err(yc.view(m, n).float().cpu().numpy(), ref(zc, sb)) < 5e-3
    # a cache hit from another stream is ordered behind the conversion
    quant.clear_repack_cache()
    side = torch.cuda.Stream()
    y0 = quant.gemm_awq_ut(xd, w2d, zsa, m, n, k, g)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        y1 = quant.gemm_awq_ut(xd, w2d, zsa, m, n, k, g)
    torch.cuda.synchronize()
    assert torch.equal(y0, y1) and quant.repack_cache_size() == 1
    quant.clear_repack_cache()


def test_lut_attention_bert_large_4096_against_oracle(capi):
    """Batch 8, 16 heads, head dim 64, 4096 tokens, 64x64 blocks at 25 % density with the diagonal kept,
    non-causal, scale 1/8: the whole problem on the GPU, the float64 oracle on sampled (batch, head)."""
    z, h, s, d = 8, 16, 4096, 64
    gen = torch.Generator(device=DEV)
    gen.manual_seed(40)
    q = torch.randn((z, h, s, d), device=DEV, generator=gen).half()
    k = torch.randn((z, h, s, d), device=DEV, generator=gen).half()
    v = torch.randn((z, h, s, d), device=DEV, generator=gen).half()
    lut = att.layout_to_lut(att.synth_layout(h, s // 64, 0.25, False, seed=41))
    out = capi.lut_attention(q, k, v, torch.from_numpy(lut).to(DEV), 0.125, False)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
    for zi, hi in [(0, 0), (3, 7), (7, 15), (5, 2)]:
        sl = (slice(zi, zi + 1), slice(hi, hi + 1))
        ref = att.attention_ref(q[sl].cpu().numpy(), k[sl].cpu().numpy(), v[sl].cpu().numpy(), lut[hi:hi + 1], 0.125, False)
        err = rel_err(out[sl].float().cpu().numpy(), ref)
        assert err <= TOL, "z=%d h=%d: %.3e" % (zi, hi, err)


def _oracle_linear(lin, x, g=128, act=None, residual=None):
    """fp16(act(x W_hat^T + bias) + residual) of a WALinear's buffers through the oracle (float64 tail)."""
    w = lin.weight.cpu().numpy()
    zs = lin.zeros_scales.cpu().numpy()
    y = orc.gemm_ref(x, orc.dequant_l1(w, zs, g)).astype(np.float64)
    if lin.bias is not None:
        y = y + lin.bias.float().cpu().numpy().reshape(1, -1)
    if act == "relu":
        y = np.maximum(y, 0.0)
    if residual is not None:
        y = y + residual.astype(np.float64)
    return y.astype(np.float16)


def test_full_width_decoder_layer_against_oracle_composition(capi):
    """One OPT-6.7B decoder layer (hidden 4096, 32 heads, FFN 16384, group 128, scales |N(0,0.02)|+1e-3),
    batch 8, one decode step over a 640-row cache (639 valid rows + the appended one): LayerNorm, one-launch
    q/k/v, decode attention with append, out_proj + residual, LayerNorm, fc1 + ReLU, fc2 + residual --
    against the same chain through the oracle, every intermediate rounded to fp16 where the kernels do."""
    from sqamd import opt_decode
    hidden, heads, ffn, b, rows = 4096, 32, 16384, 8, 640
    hd = hidden // heads
    gen = torch.Generator(device=DEV)
    gen.manual_seed(50)
    layer = opt_decode.DecoderLayer(hidden, heads, ffn, 128, DEV, gen, scale_std=0.02, scale_min=1e-3)
    layer.ln1.weight.data = (1.0 + 0.1 * torch.randn(hidden, device=DEV, generator=gen)).half()
    layer.ln1.bias.data = (0.1 * torch.randn(hidden, device=DEV, generator=gen)).half()
    layer.ln2.weight.data = (1.0 + 0.1 * torch.randn(hidden, device=DEV, generator=gen)).half()
    layer.ln2.bias.data = (0.1 * torch.randn(hidden, device=DEV, generator=gen)).half()
    x = torch.randn((b, 1, hidden), device=DEV, generator=gen).half()
    kc = torch.randn((b, heads, rows, hd), device=DEV, generator=gen).half()
    vc = torch.randn((b, heads, rows, hd), device=DEV, generator=gen).half()
    kc[:, :, rows - 1] = float("nan")  # the row the step appends
    vc[:, :, rows - 1] = float("nan")
    k0, v0 = kc.cpu().numpy(), vc.cpu().numpy()
    pos = torch.tensor([rows - 1], device=DEV)

    # oracle chain (before fusing q/k/v, from the three separate modules)
    xn = x.cpu().numpy().reshape(b, hidden)
    f16 = lambda a: np.asarray(a).astype(np.float16)
    h1 = f16(orc.layernorm_ref(xn, layer.ln1.weight.detach().cpu().numpy(), layer.ln1.bias.detach().cpu().numpy(), layer.ln1.eps))
    qo, ko, vo = (_oracle_linear(p, h1).reshape(b, heads, hd) for p in (layer.q_proj, layer.k_proj, layer.v_proj))
    k0[:, :, rows - 1] = ko
    v0[:, :, rows - 1] = vo
    a = f16(att.decode_attention_ref(qo, k0, v0, 1.0 / np.sqrt(hd))).reshape(b, hidden)
    x2 = _oracle_linear(layer.out_proj, a, residual=xn)
    h2 = f16(orc.layernorm_ref(x2, layer.ln2.weight.detach().cpu().numpy(), layer.ln2.bias.detach().cpu().numpy(), layer.ln2.eps))
    f = _oracle_linear(layer.fc1, h2, act="relu")
    want = _oracle_linear(layer.fc2, f, residual=x2).astype(np.float64)

    layer.fuse_qkv()
    with torch.no_grad():
        got = layer(x, kc, vc, pos)
    torch.cuda.synchronize()
    err = rel_err(got.float().cpu().numpy().reshape(b, hidden), want)
    assert err <= TOL, "decoder layer: %.3e" % err
    assert np.array_equal(kc[:, :, rows - 1].cpu().numpy(), ko) or \
        rel_err(kc[:, :, rows - 1].float().cpu().numpy(), ko.astype(np.float64)) < 5e-3
    assert rel_err(vc[:, :, rows - 1].float().cpu().numpy(), vo.astype(np.float64)) < 5e-3
    assert torch.equal(kc[:, :, :rows - 1].cpu(), torch.from_numpy(k0[:, :, :rows - 1]))


def test_opt67_decode_eager_and_graph_generate_the_same_tokens():
    """The 32-layer end-to-end harness (batch 8): the decode step replayed as a HIP graph generates
    exactly the tokens of the same step launched eagerly."""
    from sqamd import opt_decode
    eager = opt_decode.run_e2e(batch=8, prompt=64, new_tokens=12, use_graph=False, return_tokens=True)
    graph = opt_decode.run_e2e(batch=8, prompt=64, new_tokens=12, use_graph=True, return_tokens=True)
    assert eager["tokens_checksum"] == graph["tokens_checksum"]
    assert torch.equal(eager["tokens"], graph["tokens"])
    assert eager["tokens"].shape == (12, 8, 1)
