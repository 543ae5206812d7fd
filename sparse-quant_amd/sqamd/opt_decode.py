"""Random-init OPT-6.7B-shaped decoder with W4A16 linears: the end-to-end harness.

This is the shape generator of the end-to-end benchmark configuration, not a model port: 32
pre-LN decoder layers, hidden 4096, 32 heads (head dim 128), FFN 16384 with ReLU,
vocab 50272, learned positions with OPT's +2 offset, fp16 lm_head; q/k/v/out/fc1/fc2
are `WALinear` modules (layout L1, group 128) with random packed weights -- the same
six linears per layer, in the same order and with the same [1, tokens, K] call shape
the reference feeds to gemm_awq_ut (test/nvidia/module/opt/modeling_opt_ours.py:
158-164, 505-506, 598-611).  Decode attention is dense (the reference's decode path is dense
too): the decode step appends to the preallocated fp16 KV cache and attends in one kernel
(sq_decode_attention) that reads the position from the device, so the step is a fixed
kernel sequence that can be captured in a HIP graph.  Prefill attention is dense causal by
default; a layer that has been given a look-up table (`DecoderLayer.lut`, per head) runs its
prefill through sparse_attention(q, k, v, scaling, lut, LT=True) as the reference's OPT
attention does (test/nvidia/module/opt/modeling_opt_ours.py:435-438).
"""
import math
import time

import torch
from torch import nn

from . import capi, lut_layout
from .block_sparse_attention_lut import sparse_attention
from .qlinear import WALinear


# Scales of the end-to-end harness: |N(0, 0.004)| + 2e-4.  The single-linear benchmark distribution
# (|N(0, 0.02)| + 1e-3) makes every layer multiply the hidden state's magnitude, and 32 random layers
# in a row then overflow fp16; the smaller scales keep the random-init model finite.  Bandwidth and
# kernel choice do not depend on the values.
E2E_SCALE_STD, E2E_SCALE_MIN = 0.004, 2e-4


def _random_walinear(in_f, out_f, g, dev, gen, scale_std=E2E_SCALE_STD, scale_min=E2E_SCALE_MIN):
    lin = WALinear(in_f, out_f, w_bit=4, group_size=g, bias=True, dev=dev, layout="l1")
    lin.weight = torch.randint(0, 256, (out_f, in_f // 2), dtype=torch.uint8, device=dev, generator=gen)
    z = torch.randint(0, 16, (out_f, in_f // g), device=dev, generator=gen).half() + 64
    s = (torch.randn((out_f, in_f // g), device=dev, generator=gen).abs() * scale_std + scale_min).half()
    lin.zeros_scales = torch.stack([z, s], dim=-1).reshape(out_f, 2 * (in_f // g)).contiguous()
    lin.bias = (torch.randn((1, out_f), device=dev, generator=gen) * 0.01).half()
    return lin


def _layernorm(ln, x):
    """nn.LayerNorm parameters through the one-launch kernel (torch's takes as long as a decode GEMV)."""
    return capi.layernorm(x.contiguous(), ln.weight, ln.bias, ln.eps)


class DecoderLayer(nn.Module):
    def __init__(self, hidden, heads, ffn, g, dev, gen, scale_std=E2E_SCALE_STD, scale_min=E2E_SCALE_MIN):
        super().__init__()
        self.heads, self.hd = heads, hidden // heads
        self.ln1 = nn.LayerNorm(hidden, device=dev, dtype=torch.float16)
        self.ln2 = nn.LayerNorm(hidden, device=dev, dtype=torch.float16)
        self.q_proj = _random_walinear(hidden, hidden, g, dev, gen, scale_std, scale_min)
        self.k_proj = _random_walinear(hidden, hidden, g, dev, gen, scale_std, scale_min)
        self.v_proj = _random_walinear(hidden, hidden, g, dev, gen, scale_std, scale_min)
        self.out_proj = _random_walinear(hidden, hidden, g, dev, gen, scale_std, scale_min)
        self.fc1 = _random_walinear(hidden, ffn, g, dev, gen, scale_std, scale_min)
        self.fc2 = _random_walinear(ffn, hidden, g, dev, gen, scale_std, scale_min)
        self.qkv_proj = None
        self.fuse_ln = True  # LayerNorm inside the q/k/v and fc1 launches
        self.lut = None      # int [heads, ceil(T / 64), nnz]: prefill attention through the LUT kernel
        self.capture = None  # a dict: the prefill's q, k, v and attention output are left in it (tests)

    def forward(self, x, kc, vc, pos0):
        """x [B, T, H]; kc, vc [B, heads, Lmax, hd]; writes cache rows pos0 .. pos0+T-1."""
        b, t, hdim = x.shape
        if self.qkv_proj is not None:
            # the first LayerNorm rides in the q/k/v launch (inside the kernel at decode batch sizes)
            flat = x.reshape(1, b * t, hdim)  # the reference flattens to [1, bs*seq, K] as well
            if self.fuse_ln:
                qkv = self.qkv_proj(flat, pre_ln=self.ln1)
            else:
                qkv = self.qkv_proj(_layernorm(self.ln1, x).reshape(1, b * t, hdim))
            qkv = qkv.view(b, t, 3, self.heads, self.hd)
            q, k, v = (qkv[:, :, j].transpose(1, 2) for j in range(3))
        else:
            flat = _layernorm(self.ln1, x).reshape(1, b * t, hdim)
            q = self.q_proj(flat).view(b, t, self.heads, self.hd).transpose(1, 2)
            k = self.k_proj(flat).view(b, t, self.heads, self.hd).transpose(1, 2)
            v = self.v_proj(flat).view(b, t, self.heads, self.hd).transpose(1, 2)
        if isinstance(pos0, int):
            kc[:, :, pos0:pos0 + t] = k
            vc[:, :, pos0:pos0 + t] = v
            if self.lut is not None and pos0 == 0 and t > 1:
                a = sparse_attention(q, k, v, 1.0 / math.sqrt(self.hd), self.lut, LT=True)
            else:
                a = nn.functional.scaled_dot_product_attention(q, kc[:, :, :pos0 + t], vc[:, :, :pos0 + t],
                                                               is_causal=(t > 1))
            if self.capture is not None:
                self.capture.update(q=q.detach().clone(), k=k.detach().clone(), v=v.detach().clone(), a=a.detach().clone())
            a = a.transpose(1, 2).reshape(1, b * t, hdim)
        else:
            # graph-captured decode step: the position lives in a device tensor; one kernel appends the
            # new key/value rows to the cache and attends over rows 0 .. pos0, output already [b, 1, hidden]
            a = capi.decode_attention(q, kc, vc, pos0, 1.0 / math.sqrt(self.hd), k_new=k, v_new=v).view(1, b * t, hdim)
        # bias, ReLU and the two residual adds ride in the kernels' stores
        x = self.out_proj(a, residual=x.reshape(1, b * t, hdim)).view(b, t, hdim)
        if self.fuse_ln:
            h = self.fc1(x.reshape(1, b * t, hdim), act="relu", pre_ln=self.ln2)  # the second LayerNorm rides in fc1
        else:
            h = self.fc1(_layernorm(self.ln2, x).reshape(1, b * t, hdim), act="relu")
        return self.fc2(h, residual=x.reshape(1, b * t, hdim)).view(b, t, hdim)

    def fuse_qkv(self):
        """Serve q, k and v with one launch: layout L1 is row-major in N, so the three weights
        (and their zeros_scales and biases) concatenate along the output dimension."""
        ps = (self.q_proj, self.k_proj, self.v_proj)
        fused = WALinear(ps[0].in_features, 3 * ps[0].out_features, group_size=ps[0].group_size, bias=True,
                         dev=ps[0].weight.device)
        fused.weight = torch.cat([p.weight for p in ps], 0).contiguous()
        fused.zeros_scales = torch.cat([p.zeros_scales for p in ps], 0).contiguous()
        fused.bias = torch.cat([p.bias for p in ps], 1).contiguous()
        self.qkv_proj = fused
        self.q_proj = self.k_proj = self.v_proj = None


class OPTDecoder(nn.Module):
    def __init__(self, layers=32, hidden=4096, heads=32, ffn=16384, vocab=50272, max_pos=2048, group=128,
                 dev="cuda", seed=0, scale_std=E2E_SCALE_STD, scale_min=E2E_SCALE_MIN):
        super().__init__()
        gen = torch.Generator(device=dev)
        gen.manual_seed(seed)
        self.hidden, self.heads = hidden, heads
        self.embed = (torch.randn((vocab, hidden), device=dev, generator=gen) * 0.02).half()
        self.pos = (torch.randn((max_pos + 2, hidden), device=dev, generator=gen) * 0.02).half()
        self.layers = nn.ModuleList([DecoderLayer(hidden, heads, ffn, group, dev, gen, scale_std, scale_min)
                                     for _ in range(layers)])
        self.final_ln = nn.LayerNorm(hidden, device=dev, dtype=torch.float16)
        self.lm_head = (torch.randn((vocab, hidden), device=dev, generator=gen) * 0.02).half()

    def set_prefill_lut(self, tokens, density, seed=0):
        """Give every layer a causal look-up table of the given block density for prompts of `tokens` tokens
        (diagonal block always kept, the others drawn from a seed, a table per layer and head), or none
        (density None): the reference loads such tables from a file (`--lut_path`,
        test/eval_compress_opt_support_3090.sh:35: density 26 %)."""
        nb = (tokens + 63) // 64
        for idx, layer in enumerate(self.layers):
            if density is None:
                layer.lut = None
                continue
            layout = lut_layout.synth_layout(self.heads, nb, density, causal=True, seed=seed + idx)
            layer.lut = lut_layout.layout2lut_single_density(layout[None])[0].to(self.embed.device)

    def new_cache(self, batch, max_len):
        hd = self.hidden // self.heads
        shape = (batch, self.heads, max_len, hd)
        dev = self.embed.device
        return [(torch.zeros(shape, dtype=torch.float16, device=dev), torch.zeros(shape, dtype=torch.float16, device=dev))
                for _ in self.layers]

    @torch.no_grad()
    def forward(self, ids, cache, pos0, pos_ids=None):
        b, t = ids.shape
        if pos_ids is None:
            pos_ids = torch.arange(pos0, pos0 + t, device=ids.device) + 2
        x = self.embed[ids] + self.pos[pos_ids]
        for layer, (kc, vc) in zip(self.layers, cache):
            x = layer(x, kc, vc, pos0)
        x = _layernorm(self.final_ln, x[:, -1:])
        return torch.matmul(x, self.lm_head.t())  # [B, 1, vocab]

    @torch.no_grad()
    def greedy_step(self, tok, cache, pos_t, history=None, step_t=None):
        """One greedy decode step for up to 8 sequences with nothing but library launches, so that a HIP graph
        holds the whole of it: tok int64 [B, 1] is read at the start and replaced by the chosen tokens at the
        end, pos_t int64 [1] (the cache row the new keys and values go to) is advanced, and with history int64
        [T, B] and step_t int64 [1] the chosen tokens are also written to history[step_t].  Embeddings, final
        LayerNorm, fp16 lm_head and argmax are what forward() computes with torch ops (the embeddings bit for bit;
        the logits with fp32 sums in another order).  Returns the logits [B, vocab]."""
        b = tok.shape[0]
        if getattr(self, "_parts", None) is None:
            self._parts = capi.f16_gemv_parts(self.lm_head.shape[0], self.lm_head.device)
        x = capi.embed_rows(self.embed, self.pos, tok.view(-1), pos_t, 2).view(b, 1, self.hidden)
        for layer, (kc, vc) in zip(self.layers, cache):
            x = layer(x, kc, vc, pos_t)
        x = _layernorm(self.final_ln, x.view(b, self.hidden))
        logits = capi.f16_gemv(x, self.lm_head, parts=self._parts)
        capi.greedy_feedback(self._parts, b, tok.view(-1), pos=pos_t, history=history, step=step_t)
        return logits


@torch.no_grad()
def run_e2e(batch=8, prompt=512, new_tokens=128, layers=32, use_graph=True, seed=0, fuse_qkv=True,
            return_tokens=False, lut_density=0.26, scale_std=E2E_SCALE_STD, scale_min=E2E_SCALE_MIN, fused_ends=True):
    """Greedy generation on random token ids; returns timing and throughput figures."""
    dev = "cuda"
    model = OPTDecoder(layers=layers, dev=dev, seed=seed, scale_std=scale_std, scale_min=scale_min)
    if fuse_qkv:
        for layer in model.layers:
            layer.fuse_qkv()
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed + 1)
    ids = torch.randint(0, 50272, (batch, prompt), device=dev, generator=gen)
    max_len = prompt + new_tokens
    cache = model.new_cache(batch, max_len)

    model(ids, cache, 0)  # untimed first pass: code objects, library handles and workspaces come into being here
    torch.cuda.synchronize()
    # The same prefill with the attention of every layer through the LUT kernel (causal tables of the
    # reference's OPT density); the dense pass that follows rewrites the cache, decode starts from that one.
    prefill_lut_s = None
    if lut_density is not None and prompt >= 128:
        model.set_prefill_lut(prompt, lut_density, seed=seed)
        model(ids, cache, 0)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        model(ids, cache, 0)
        torch.cuda.synchronize()
        prefill_lut_s = time.perf_counter() - t0
        model.set_prefill_lut(prompt, None)
    t0 = time.perf_counter()
    logits = model(ids, cache, 0)
    nxt = logits.argmax(-1)
    torch.cuda.synchronize()
    prefill_s = time.perf_counter() - t0

    # One decode step with device-side position so that it can be replayed as a graph.  fused_ends: embeddings,
    # lm_head, argmax and the feedback of the chosen token are library launches inside the step (greedy_step);
    # otherwise they are torch ops, three of them between two replays.
    pos_t = torch.tensor([prompt], device=dev, dtype=torch.long)
    tok = nxt.clone()
    out_tok = torch.empty_like(tok)
    fused_ends = fused_ends and batch <= 8
    history = torch.zeros((new_tokens, batch), dtype=torch.long, device=dev) if fused_ends else None
    step_t = torch.zeros(1, dtype=torch.long, device=dev) if fused_ends else None
    first_tok = tok.clone()

    def step():
        if fused_ends:
            model.greedy_step(tok, cache, pos_t, history, step_t)
        else:
            lg = model(tok, cache, pos_t, pos_ids=pos_t + 2)
            out_tok.copy_(lg.argmax(-1))

    def rewind():
        # the warm-up and the capture run a step each: put token, position and step counter back
        tok.copy_(first_tok)
        pos_t.fill_(prompt)
        if step_t is not None:
            step_t.zero_()

    graph = None
    if use_graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()  # warm-up outside capture
            rewind()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):  # same stream as the warm-up: per-stream workspaces exist
            step()
        rewind()
    generated = [tok.clone()]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(new_tokens - 1):
        if graph is not None:
            graph.replay()
        else:
            step()
        if not fused_ends:
            tok.copy_(out_tok)
            pos_t += 1
            generated.append(tok.clone())
    torch.cuda.synchronize()
    decode_s = time.perf_counter() - t0
    steps = new_tokens - 1
    if fused_ends:
        generated += [history[i].view(batch, 1).clone() for i in range(steps)]
    extra = {"tokens": torch.stack(generated).cpu()} if return_tokens else {}
    # Algorithmic bytes of one decode step: every packed weight with its zeros/scales and the batch's
    # activations (N*K/2 + (K/g)*N*4 + M*K*2 + M*N*2 per linear, q/k/v as one linear), the valid K/V cache
    # rows read once (average over the timed steps), the fp16 lm_head.
    hidden, ffn, g, vocab = model.hidden, model.layers[0].fc1.out_features, 128, model.lm_head.shape[0]
    lin = lambda n, k: n * k // 2 + (k // g) * n * 4 + batch * k * 2 + batch * n * 2
    rows_avg = prompt + (steps + 1) / 2.0
    per_layer = lin(3 * hidden, hidden) + lin(hidden, hidden) + lin(ffn, hidden) + lin(hidden, ffn) + \
        2 * batch * hidden * rows_avg * 2
    step_bytes = layers * per_layer + vocab * hidden * 2
    step_s = decode_s / steps
    return {
        **extra,
        "weights": "random packed int4, zeros U{0..15}, scales |N(0,%g)|+%g%s" % (
            scale_std, scale_min,
            " (smaller than the single-linear benchmark's |N(0,0.02)|+1e-3 so that 32 random layers stay finite in fp16)"
            if scale_std < 0.02 else " (the single-linear benchmark's distribution)"),
        "batch": batch, "prompt": prompt, "new_tokens": new_tokens, "layers": layers,
        "launch": "hip-graph replay" if graph is not None else "eager",
        "fused": "bias+relu+residual in the GEMM store" + ("; q/k/v one launch" if fuse_qkv else "") +
                 "; both LayerNorms inside the q/k/v and fc1 kernels at decode; decode attention appends K/V in the same "
                 "launch" + ("; embeddings, fp16 lm_head + argmax, token feedback as three launches inside the step"
                             if fused_ends else ""),
        "prefill_ms": round(prefill_s * 1e3, 2),
        "prefill_attention": "dense causal (torch SDPA)",
        "prefill_lut_ms": None if prefill_lut_s is None else round(prefill_lut_s * 1e3, 2),
        "prefill_lut_attention": None if prefill_lut_s is None else
        "sparse_attention(q, k, v, scaling, lut, LT=True) in every layer: causal per-head tables, block density %.2f, "
        "D = 128 (sq_lut_attention_fwd)" % lut_density,
        "prefill_tok_per_s": round(batch * prompt / prefill_s, 1),
        "decode_ms_per_step": round(decode_s * 1e3 / steps, 4),
        "decode_tok_per_s": round(batch * steps / decode_s, 1),
        "roofline": {"bound": "hbm", "bytes_per_step": int(step_bytes), "achieved": round(step_bytes / step_s / 1e9, 1),
                     "peak": 8000.0, "unit": "GB/s", "frac": round(step_bytes / step_s / 1e9 / 8000.0, 4),
                     "what": "int4 weights + zeros/scales + activations of the %d x 4 linears, K/V cache rows read once "
                             "(%.0f rows on average), fp16 lm_head; per decode step" % (layers, rows_avg)},
        "parity": "covered by tests/test_gpu_full_size.py: one full-width decoder layer against the oracle composition, "
                  "eager and HIP-graph decode steps generate identical tokens; tests/test_gpu_step_ends.py: the step "
                  "with library launches at its ends generates the tokens of the step with torch ops there",
        "tokens_checksum": int(torch.stack(generated).sum().item()),
        "logits_finite": bool(torch.isfinite(logits).all().item()),
    }


if __name__ == "__main__":
    import json
    import sys
    print(json.dumps(run_e2e(use_graph="--no-graph" not in sys.argv)))
