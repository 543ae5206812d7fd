"""LUT block-sparse attention: host-side mirror of the reference's `playground` kernel module.

Same entry point and argument meaning as
sparse-attention/nvidia/playground/kernels/block_sparse_attention_lut.py:246-309
(`sparse_attention(q, k, v, sm_scale, lut, LT, BLOCK_M, BLOCK_N, attention_mask,
attention_dropout)`): prefill (q_len == kv_len) runs the HIP kernel behind
sq_lut_attention_fwd; decode (q_len < kv_len, q_len == 1) is dense attention over
the whole KV cache, the same quantity the reference computes with two matmuls and a softmax,
here in one kernel behind sq_decode_attention.
"""
import torch

from . import capi


def sparse_attention_prefill(q, k, v, sm_scale, lut, LT=True, BLOCK_M=64, BLOCK_N=64):
    """q, k, v fp16 [Z, H, N_CTX, L]; lut integer [H, ceil(N_CTX/64), nnz] -> fp16 [Z, H, N_CTX, L]."""
    assert q.dtype == torch.float16 and k.dtype == torch.float16 and v.dtype == torch.float16
    assert q.shape[-1] == k.shape[-1] == v.shape[-1]
    if BLOCK_M != 64 or BLOCK_N != 64:
        raise ValueError("the LUT attention kernel is built for 64 x 64 blocks")
    if lut.dtype not in (torch.int32, torch.int64):
        raise TypeError("lut must be int32 or int64")
    if not q.is_cuda:
        raise RuntimeError("sparse_attention_prefill needs device tensors; there is no host path")
    return capi.lut_attention(q.contiguous(), k.contiguous(), v.contiguous(), lut.contiguous().to(q.device),
                              sm_scale, LT)


def sparse_attention(q, k, v, sm_scale, lut, LT=True, BLOCK_M=64, BLOCK_N=64, attention_mask=None,
                     attention_dropout=0.0):
    bsz, num_heads, q_len, _ = q.shape
    kv_len = k.size(2)
    if q_len < kv_len:  # decode: dense over the cache, one kernel
        assert q_len == 1
        if attention_mask is not None and attention_mask.size() != (bsz, 1, q_len, kv_len):
            raise ValueError("Attention mask should be of size %s, but is %s"
                             % ((bsz, 1, q_len, kv_len), tuple(attention_mask.size())))
        if attention_dropout != 0.0:
            raise ValueError("decode attention is inference only (the reference applies dropout with training=False)")
        if not q.is_cuda:
            raise RuntimeError("sparse_attention needs device tensors; there is no host path")
        if k.stride(-1) != 1 or k.stride(2) != k.size(3) or v.stride() != k.stride():
            k, v = k.contiguous(), v.contiguous()
        if attention_mask is not None:
            attention_mask = attention_mask.to(torch.float16).contiguous()
        out = capi.decode_attention(q.contiguous(), k, v, kv_len, sm_scale, mask=attention_mask)
        return out.view(bsz, num_heads, 1, -1)
    return sparse_attention_prefill(q, k, v, sm_scale, lut, LT, BLOCK_M, BLOCK_N)
