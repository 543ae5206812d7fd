"""LUT block-sparse attention: host-side mirror of the reference's `playground` kernel module.

Same entry point and argument meaning as
sparse-attention/nvidia/playground/kernels/block_sparse_attention_lut.py:246-309
(`sparse_attention(q, k, v, sm_scale, lut, LT, BLOCK_M, BLOCK_N, attention_mask,
attention_dropout)`): prefill (q_len == kv_len) runs the HIP kernel behind
sq_lut_attention_fwd; decode (q_len < kv_len, q_len == 1) is dense attention over
the whole KV cache in torch, exactly as the reference does it.
"""
import torch
from torch import nn

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
    if q_len < kv_len:  # decode: dense over the cache
        assert q_len == 1
        w = torch.matmul(q, k.transpose(2, 3)) * sm_scale
        if attention_mask is not None:
            if attention_mask.size() != (bsz, 1, q_len, kv_len):
                raise ValueError("Attention mask should be of size %s, but is %s"
                                 % ((bsz, 1, q_len, kv_len), tuple(attention_mask.size())))
            w = w + attention_mask
        w = nn.functional.softmax(w, dim=-1, dtype=torch.float32).to(q.dtype)
        w = nn.functional.dropout(w, p=attention_dropout, training=False)
        return torch.matmul(w, v)
    return sparse_attention_prefill(q, k, v, sm_scale, lut, LT, BLOCK_M, BLOCK_N)
