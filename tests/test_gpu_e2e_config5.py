"""The end-to-end harness of BASELINE configuration 5 at its full width and prompt length against the oracle:
a two-layer OPT-6.7B-shaped decoder (hidden 4096, 32 heads, FFN 16384, vocab 50272, group 128), batch 8, prompt
512, then greedy decode steps; and the same prefill with every layer's attention through the LUT kernel as the
reference's OPT attention runs it (test/nvidia/module/opt/modeling_opt_ours.py:435-438).
Bars: logits within 1e-2 * max|ref| of the oracle composition (every intermediate rounded to fp16 where the
kernels store fp16); the token the device picks is a maximum of the oracle's logits up to that tolerance;
attention outputs within 1e-2 * max|ref| of the masked dense oracle."""
import numpy as np
import pytest
import torch

import lut_attention_oracle as att
import w4a16_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 1e-2


@pytest.fixture(scope="module")
def capi(built_lib):
    from sqamd import capi as c
    c.lib()
    return c


def rel_err(y, y_ref):
    y = np.asarray(y, dtype=np.float64)
    assert np.all(np.isfinite(y))
    return float(np.max(np.abs(y - y_ref)) / max(np.max(np.abs(y_ref)), 1e-30))


f16 = lambda a: np.asarray(a).astype(np.float16)


class OracleLinear:
    """fp16(act(x W_hat^T + bias) + residual) from a WALinear's buffers; the weight is dequantised once."""

    def __init__(self, lin, g=128):
        self.w_hat = orc.dequant_l1(lin.weight.cpu().numpy(), lin.zeros_scales.cpu().numpy(), g)
        self.bias = None if lin.bias is None else lin.bias.float().cpu().numpy().reshape(1, -1).astype(np.float64)

    def __call__(self, x, act=None, residual=None):
        y = orc.gemm_ref(x, self.w_hat).astype(np.float64)
        if self.bias is not None:
            y = y + self.bias
        if act == "relu":
            y = np.maximum(y, 0.0)
        if residual is not None:
            y = y + residual.astype(np.float64)
        return f16(y)


class OracleLayer:
    def __init__(self, layer):
        self.q, self.k, self.v = OracleLinear(layer.q_proj), OracleLinear(layer.k_proj), OracleLinear(layer.v_proj)
        self.out, self.fc1, self.fc2 = OracleLinear(layer.out_proj), OracleLinear(layer.fc1), OracleLinear(layer.fc2)
        ln = lambda m: (m.weight.detach().cpu().numpy(), m.bias.detach().cpu().numpy(), m.eps)
        self.ln1, self.ln2 = ln(layer.ln1), ln(layer.ln2)
        self.heads, self.hd = layer.heads, layer.hd
        self.kc = self.vc = None  # fp16 [B, heads, L, hd]

    def _tail(self, x, a):
        x2 = self.out(a, residual=x)
        h2 = f16(orc.layernorm_ref(x2, *self.ln2))
        return self.fc2(self.fc1(h2, act="relu"), residual=x2)

    def prefill(self, x, b, t):
        """x fp16 [b * t, hidden] -> fp16 [b * t, hidden]; dense causal attention over the prompt."""
        h1 = f16(orc.layernorm_ref(x, *self.ln1))
        split = lambda y: y.reshape(b, t, self.heads, self.hd).transpose(0, 2, 1, 3)
        q, k, v = split(self.q(h1)), split(self.k(h1)), split(self.v(h1))
        self.kc, self.vc = np.ascontiguousarray(k), np.ascontiguousarray(v)
        nb = (t + 63) // 64
        lut = att.layout_to_lut(np.tril(np.ones((self.heads, nb, nb), dtype=bool)))
        a = f16(att.attention_ref(q, k, v, lut, 1.0 / np.sqrt(self.hd), True))
        return self._tail(x, a.transpose(0, 2, 1, 3).reshape(b * t, self.heads * self.hd))

    def decode(self, x, b):
        """x fp16 [b, hidden]: one new token per sequence; appends to the oracle's own cache."""
        h1 = f16(orc.layernorm_ref(x, *self.ln1))
        split = lambda y: y.reshape(b, self.heads, self.hd)
        q, k, v = split(self.q(h1)), split(self.k(h1)), split(self.v(h1))
        self.kc = np.concatenate([self.kc, k[:, :, None]], axis=2)
        self.vc = np.concatenate([self.vc, v[:, :, None]], axis=2)
        a = f16(att.decode_attention_ref(q, self.kc, self.vc, 1.0 / np.sqrt(self.hd)))
        return self._tail(x, a.reshape(b, self.heads * self.hd))


def _model(layers=2, seed=3):
    from sqamd import opt_decode
    model = opt_decode.OPTDecoder(layers=layers, dev=DEV, seed=seed)
    gen = torch.Generator(device=DEV)
    gen.manual_seed(seed + 100)
    for m in [model.final_ln] + [ln for layer in model.layers for ln in (layer.ln1, layer.ln2)]:
        m.weight.data = (1.0 + 0.1 * torch.randn(model.hidden, device=DEV, generator=gen)).half()
        m.bias.data = (0.1 * torch.randn(model.hidden, device=DEV, generator=gen)).half()
    return model


def test_config5_prompt_and_decode_steps_against_oracle(capi):
    """Batch 8, prompt 512, three greedy decode steps on a two-layer full-width model: the logits of the prefill
    and of every step against the oracle composition through the fp16 lm_head."""
    b, t, steps = 8, 512, 3
    model = _model()
    oracle_layers = [OracleLayer(layer) for layer in model.layers]  # from the separate q, k, v modules
    for layer in model.layers:
        layer.fuse_qkv()
    gen = torch.Generator(device=DEV)
    gen.manual_seed(11)
    ids = torch.randint(0, 50272, (b, t), device=DEV, generator=gen)
    cache = model.new_cache(b, t + steps + 1)
    embed, pos = model.embed.cpu().numpy(), model.pos.cpu().numpy()
    lm_head = model.lm_head.float().cpu().numpy().astype(np.float64)
    fln = (model.final_ln.weight.detach().cpu().numpy(), model.final_ln.bias.detach().cpu().numpy(), model.final_ln.eps)

    def oracle_logits(x_last):
        return f16(orc.layernorm_ref(x_last, *fln)).astype(np.float64) @ lm_head.T

    def check(logits_dev, ref, what):
        got = logits_dev.float().cpu().numpy().reshape(b, -1)
        assert rel_err(got, ref) <= TOL, what
        tok = got.argmax(-1)
        bound = TOL * np.max(np.abs(ref))
        for j in range(b):  # the device's choice is a maximum of the oracle's logits up to the tolerance
            assert ref[j, tok[j]] >= ref[j].max() - 2 * bound, (what, j)
        return torch.from_numpy(tok).to(DEV).view(b, 1)

    logits = model(ids, cache, 0)
    torch.cuda.synchronize()
    idn = ids.cpu().numpy()
    x = (embed[idn] + pos[np.arange(t) + 2][None]).astype(np.float16).reshape(b * t, -1)  # fp16 add, as on the device
    for ol in oracle_layers:
        x = ol.prefill(x, b, t)
    tok = check(logits, oracle_logits(x.reshape(b, t, -1)[:, -1]), "prefill")
    # the cache the device wrote against the oracle's keys and values
    for (kc, vc), ol in zip(cache, oracle_layers):
        assert rel_err(kc[:, :, :t].float().cpu().numpy(), ol.kc.astype(np.float64)) <= TOL
        assert rel_err(vc[:, :, :t].float().cpu().numpy(), ol.vc.astype(np.float64)) <= TOL

    pos_t = torch.tensor([t], device=DEV, dtype=torch.long)
    for s in range(steps):
        logits = model(tok, cache, pos_t, pos_ids=pos_t + 2)
        torch.cuda.synchronize()
        x = (embed[tok.cpu().numpy().reshape(b)] + pos[t + s + 2][None]).astype(np.float16)
        for ol in oracle_layers:
            x = ol.decode(x, b)
        tok = check(logits, oracle_logits(x), "decode step %d" % s)
        pos_t += 1


def test_two_layer_prefill_through_the_lut_kernel(capi):
    """The prefill of the same model with every layer's attention through sparse_attention(q, k, v, scaling, lut,
    LT=True): causal per-head tables of block density 0.26 at D = 128.  The attention output of each layer on
    sampled (sequence, head) pairs against the masked dense oracle fed with the q, k, v the device produced; the
    prompt's logits stay finite and differ from the dense prefill's (the mask is really applied)."""
    b, t = 8, 512
    model = _model(seed=5)
    for layer in model.layers:
        layer.fuse_qkv()
        layer.capture = {}
    gen = torch.Generator(device=DEV)
    gen.manual_seed(12)
    ids = torch.randint(0, 50272, (b, t), device=DEV, generator=gen)
    cache = model.new_cache(b, t + 1)
    dense = model(ids, cache, 0).clone()
    model.set_prefill_lut(t, 0.26, seed=7)
    sparse = model(ids, cache, 0)
    torch.cuda.synchronize()
    assert torch.isfinite(sparse).all()
    assert (sparse.float() - dense.float()).abs().max().item() > 1e-3 * dense.float().abs().max().item()
    rng = np.random.default_rng(0)
    for layer in model.layers:
        cap, lut = layer.capture, layer.lut.cpu().numpy()
        assert lut.shape[0] == model.heads and lut.shape[1] == t // 64
        for _ in range(3):
            z, h = int(rng.integers(b)), int(rng.integers(model.heads))
            pick = lambda name: cap[name][z:z + 1, h:h + 1].float().cpu().numpy()
            ref = att.attention_ref(pick("q"), pick("k"), pick("v"), lut[h:h + 1], 1.0 / np.sqrt(layer.hd), True)
            assert rel_err(pick("a"), ref) <= TOL, (z, h)
