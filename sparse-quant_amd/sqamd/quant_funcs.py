"""Host-side packers: fp16 weight -> packed int4 weight + zeros_scales.

Mirror of the reference's Python packers (same names, same arguments, same
tensors out), written with vectorised torch ops so they run on the device the
weight lives on:

    quant_muxi      test/muxi/utils/quant_funcs.py:75-83   (layout L1, uint8 [N, K*b/8])
    quant_lmdeploy  test/nvidia/utils/quant_dequant_nvidia.py:5-32 (layout L2, int32 [K, N/8])
    quantize_tensor test/muxi/utils/quant_funcs.py:96-114  (round-to-nearest groups)

The layout-L2 chain calls the three converter kernels of the `quant` extension,
exactly like the reference does, so it needs a GPU; the L1 path is pure torch.

Like the reference, the quantiser computes in the dtype of the weight it is given
(fp16 for the models the reference packs), so scales, zeros and codes of an fp16
weight are bit-identical to the reference's; pass `compute_dtype=torch.float32` to
quantise an fp16 weight in fp32 instead.
"""
import torch


def quantize_tensor(w, n_bit, q_group_size):
    """Asymmetric round-to-nearest quantisation per group of `q_group_size` along K.

    Returns (q, scales, zeros) with q in [0, 2^b - 1] shaped like w, and scales /
    zeros shaped [N, K/g].  s = clamp(max - min, 1e-5) / (2^b - 1),
    z = clamp(-round(min / s), 0, 2^b - 1), q = clamp(round(w / s) + z, 0, 2^b - 1).
    """
    shape = w.shape
    if q_group_size > 0:
        assert shape[-1] % q_group_size == 0
        w = w.reshape(-1, q_group_size)
    assert w.dim() == 2
    hi = w.amax(dim=1, keepdim=True)
    lo = w.amin(dim=1, keepdim=True)
    qmax = 2 ** n_bit - 1
    scales = (hi - lo).clamp(min=1e-5) / qmax
    zeros = (-torch.round(lo / scales)).clamp_(0, qmax)
    q = torch.clamp(torch.round(w / scales) + zeros, 0, qmax)
    return q.reshape(shape), scales.reshape(shape[0], -1), zeros.reshape(shape[0], -1)


def interleave_k(q):
    """[.., k0..k7, ..] -> [.., k0,k2,k4,k6,k1,k3,k5,k7, ..] for every run of 8 along K."""
    n, k = q.shape
    return q.reshape(n, k // 8, 4, 2).transpose(2, 3).reshape(n, k)


def write_4bit_tensor(q):
    """uint8 [N, K/2]: byte j = q[2j+1] << 4 | q[2j] (first of the pair in the low nibble)."""
    q = q.to(torch.uint8)
    return (q[:, 1::2] << 4) | q[:, 0::2]


def write_2bit_tensor(q):
    """uint8 [N, K/4]: of each 4 values (a,b,c,d) the byte is a<<4 | b<<6 | c | d<<2."""
    q = q.to(torch.uint8).reshape(q.shape[0], -1, 4)
    return (q[..., 0] << 4) | (q[..., 1] << 6) | q[..., 2] | (q[..., 3] << 2)


def merge_zeros_scales(zeros, scales):
    """[N, K/g] zeros (integers) and scales -> fp16 [N, 2K/g] of pairs (zero + 64, scale)."""
    z = zeros.half() + 64
    s = scales.half()
    return torch.stack([z, s], dim=-1).reshape(z.shape[0], -1).contiguous()


def _as(weight, compute_dtype):
    return weight if compute_dtype is None else weight.to(compute_dtype)


def quant_muxi(weight, input_features, output_features, n_bit=4, group_size=64, compute_dtype=None):
    """fp16 weight [N, K] -> (qweight uint8 [N, K*n_bit/8], zeros_scales fp16 [N, 2K/g]) in layout L1.

    The K-interleave permutes within runs of 8, i.e. inside a group, so zeros and
    scales are the same as those of the un-permuted weight.
    """
    assert weight.shape == (output_features, input_features)
    q, scales, zeros = quantize_tensor(_as(weight, compute_dtype), n_bit, group_size)
    q = interleave_k(q)
    if n_bit == 4:
        qweight = write_4bit_tensor(q)
    elif n_bit == 2:
        qweight = write_2bit_tensor(q)
    else:
        raise ValueError("n_bit must be 2 or 4")
    return qweight.contiguous(), merge_zeros_scales(zeros, scales)


def dequant_to_fp16(weight, n_bit=4, group_size=64, compute_dtype=None):
    """The fake-quantised weight: fp16((q - z) * s) with fp16 zeros and scales.

    (reference: quantization/muxi/script/quant_dequant_muxi.py:73-85 applied to
    the un-permuted quantisation.)
    """
    q, scales, zeros = quantize_tensor(_as(weight, compute_dtype), n_bit, group_size)
    z = zeros.half().repeat_interleave(group_size, dim=1)
    s = scales.half().repeat_interleave(group_size, dim=1)
    return (q.half() - z) * s


def quant_lmdeploy(weight, input_features, output_features, group_size=128, n_bit=4, compute_dtype=None):
    """fp16 weight [N, K] -> (qweight int32 [K, N/8], zeros_scales fp16 [K/g, 2N], w_fp16 [N, K]) in
    layout L2; w_fp16 = (q - z) * s in the compute dtype is the fake-quantised weight the reference
    returns as its third value (test/nvidia/utils/quant_dequant_nvidia.py:32,70-71).

    Same three-step chain as the reference: "ours" bytes (even k in the high
    nibble) -> AWQ order -> tensor-core tile order, plus the transposed merge of
    zeros and scales; every step is a kernel of the `quant` extension.  n_bit = 2 quantises to
    four levels and passes the words through convert_4bit_to_2bit as the reference does (:29-30),
    which returns int32 [K, N/16].
    """
    import quant

    if n_bit not in (2, 4):
        raise ValueError("n_bit must be 2 or 4")
    w = _as(weight, compute_dtype)
    q, scales, zeros = quantize_tensor(w, n_bit, group_size)
    g = group_size
    w_fp16 = ((q.reshape(-1, g) - zeros.reshape(-1, 1)) * scales.reshape(-1, 1)).reshape(q.shape)
    q = q.to(torch.uint8)
    ours = ((q[:, 0::2] << 4) | q[:, 1::2]).contiguous()
    dev = weight.device
    zeros_scales = torch.empty((input_features // group_size, output_features * 2), dtype=torch.float16, device=dev)
    quant.transpose_merge_zeros_scales(zeros.half().contiguous(), scales.half().contiguous(), zeros_scales,
                                       input_features, output_features, group_size)
    awq = torch.empty((input_features, output_features // 2), dtype=torch.uint8, device=dev)
    quant.convert_ours_to_awq(ours, awq, input_features, output_features)
    qweight = torch.empty((input_features, output_features // 8), dtype=torch.int32, device=dev)
    quant.convert_awq_to_lmdeploy(awq, qweight, input_features, output_features)
    if n_bit == 2:
        qweight = convert_4bit_to_2bit(qweight)
    return qweight, zeros_scales, w_fp16


def convert_4bit_to_2bit(qweight_4bit):
    """int32 [K, N/8] -> int32 [K, N/16], bit for bit what the reference's function of this name
    returns (test/nvidia/utils/quant_dequant_nvidia.py:34-43).  Its shifts bind tighter than its
    `&`, so the eight masks per word add up to a constant: a pair of words (a, b) becomes
    (a & 0xFFFF0000) + (b & 0x0000FFFF), not a 2-bit compaction of both."""
    import quant

    return quant.convert_4bit_to_2bit(qweight_4bit.contiguous())


def convert_2bit_to_4bit(qweight_2bit):
    """int32 [K, N/16] -> int32 [K, N/8] (:45-54 of the same file): every stored word w yields the
    pair (w & 0x33333333, w & 0x33333333).  uint8 input is the L1 expansion instead."""
    import quant

    return quant.convert_2bit_to_4bit(qweight_2bit.contiguous())
