"""CPU oracle for the W4A16 quantized-linear path.  TEST INFRASTRUCTURE ONLY.

This file restates, in numpy, the algorithm of the reference's `quant`
extension and of the Python packers around it.  It is the checker the parity
tests, the smoke test and the `cpu_baseline` leg of the benchmark compare the
HIP kernels against; nothing in the product path may import it.

Notation: q = unsigned int4 weight in [0,15], z = integer zero point in
[0,15] stored as fp16 (z + 64), s = fp16 scale, g = group size along K.
    W_hat[n,k] = fp16_rn((q[n,k] - z[n,k//g]) * s[n,k//g])
    Y[m,n]     = sum_k X[m,k] * W_hat[n,k]          (fp32 accumulate)

Pinning status of every function (what, other than this file, fixes it):
  unpack_u32_magic      exhaustive closed form 64 + ((w >> 4*pi(i)) & 15)
  pack_l1 / unpack_l1   byte formula of the reference packer + round trip +
                        hand-written 8-nibble vector
  zeros_scales_l1       interleave formula; round trip through split
  dequant_l1            IEEE fp16 arithmetic vs exact rational arithmetic
                        (fractions) on every (q,z) pair and many scales; C
                        restatement (w4a16_oracle.c) agrees bit for bit
  pack_ours, ours_to_awq, awq_to_lmdeploy
                        brute-force 10-d nibble permutation vs independent
                        closed-form index map; bijectivity
  transpose_merge_zeros_scales   index formula; round trip
  gemm_ref              textbook matmul; float64 cross-check; one-hot rows
  rtn_quantize          closed form on hand-computed vectors
  silu_dot_ref          scipy's logistic function; closed forms (silu(0) = 0, silu(a) - silu(-a) = a,
                        large |a| limits); x W^T through gemm_ref
  convert_2bit_to_4bit  exhaustive over the 256 byte values
  convert_4bit_to_2bit_l2 / convert_2bit_to_4bit_l2
                        closed-form masks vs the sixteen terms of each loop evaluated
                        one by one with Python's operator precedence; one-hot words
                        (which of the 64 input bits survive, and where); hand vector
No function here is "parity unpinned".
"""
import numpy as np

# ---------------------------------------------------------------------------
# int4 -> fp16 unpack
# ---------------------------------------------------------------------------

# Output order of the magic-number unpack relative to nibble positions X0..X7
# (X0 = least significant nibble): [X0, X4, X1, X5, X2, X6, X3, X7].
MAGIC_ORDER = (0, 4, 1, 5, 2, 6, 3, 7)


def unpack_u32_magic(words):
    """uint32[...] -> float16[..., 8] holding 64 + nibble, order MAGIC_ORDER.

    Follows quantization/muxi/backend/utils.cuh:81-134 (same routine as
    quantization/nvidia/kernel/gemm_s4_f16/common.h:114-153): low nibbles are
    OR-ed with 0x0540 and shifted left by 4, high nibbles are OR-ed with
    0x5400; both give the fp16 bit pattern of 64 + nibble because ulp(64) in
    fp16 is 1/16.
    """
    w = np.asarray(words, dtype=np.uint32)
    top = w >> np.uint32(8)
    h0 = ((w & np.uint32(0x000F000F)) | np.uint32(0x05400540)) << np.uint32(4)
    h1 = (w & np.uint32(0x00F000F0)) | np.uint32(0x54005400)
    h2 = ((top & np.uint32(0x000F000F)) | np.uint32(0x05400540)) << np.uint32(4)
    h3 = (top & np.uint32(0x00F000F0)) | np.uint32(0x54005400)
    packed = np.stack([h0, h1, h2, h3], axis=-1).astype(np.uint32)
    return np.ascontiguousarray(packed).view(np.float16).reshape(w.shape + (8,))


# ---------------------------------------------------------------------------
# Layout L1 (wave64 back-ends): uint8 [N, K/2], fp16 zeros_scales [N, 2K/g]
# ---------------------------------------------------------------------------

def pack_l1(q):
    """q uint8 [N,K] (natural k order) -> uint8 [N,K/2] in layout L1.

    Follows test/muxi/utils/quant_funcs.py:75-83,116-127: every run of 8
    consecutive k is reordered to [k0,k2,k4,k6,k1,k3,k5,k7] and then written
    two per byte with the first of the pair in the low nibble.
    """
    q = np.asarray(q, dtype=np.uint8)
    n, k = q.shape
    assert k % 8 == 0
    r = q.reshape(n, k // 8, 4, 2).transpose(0, 1, 3, 2).reshape(n, k // 2, 2)
    return (r[..., 0] | (r[..., 1] << 4)).astype(np.uint8)


def unpack_l1(w):
    """uint8 [N,K/2] layout L1 -> q uint8 [N,K] in natural k order."""
    w = np.asarray(w, dtype=np.uint8)
    n, kh = w.shape
    nib = np.stack([w & 0xF, w >> 4], axis=-1).reshape(n, kh // 4, 2, 4)
    return nib.transpose(0, 1, 3, 2).reshape(n, kh * 2).astype(np.uint8)


def zeros_scales_l1(z, s):
    """z [N,K/g] integer zero points, s [N,K/g] scales -> fp16 [N, 2K/g].

    Pairs (z + 64, s) interleaved along the last axis
    (test/muxi/utils/quant_funcs.py:158-172).
    """
    z16 = (np.asarray(z).astype(np.float16) + np.float16(64)).astype(np.float16)
    s16 = np.asarray(s).astype(np.float16)
    out = np.empty((z16.shape[0], 2 * z16.shape[1]), dtype=np.float16)
    out[:, 0::2] = z16
    out[:, 1::2] = s16
    return out


def split_zeros_scales_l1(zs):
    """fp16 [N,2K/g] -> (z64 fp16 [N,K/g], s fp16 [N,K/g])."""
    zs = np.asarray(zs, dtype=np.float16)
    return zs[:, 0::2], zs[:, 1::2]


def dequant_l1(w, zs, g):
    """L1 weight + zeros_scales -> W_hat fp16 [N,K], natural k order.

    Follows quantization/tianshu/backend/w4a16_gemm.cuh:1060-1154: unpack to
    64+q, subtract the stored zero (64+z) in fp16 (exact), multiply by the
    scale in fp16 (one round-to-nearest); group index k // g
    (quantization/muxi/backend/w4a16_gemm.cuh:52).
    """
    w = np.ascontiguousarray(w, dtype=np.uint8)
    n, kh = w.shape
    k = kh * 2
    h = unpack_u32_magic(w.view(np.uint32)).reshape(n, k)
    z64, s = split_zeros_scales_l1(zs)
    z64 = np.repeat(z64, g, axis=1)
    s = np.repeat(s, g, axis=1)
    return ((h - z64).astype(np.float16) * s).astype(np.float16)


# ---------------------------------------------------------------------------
# Layout L2 (tensor-core back-end): int32 [K, N/8], fp16 zeros_scales [K/g, 2N]
# ---------------------------------------------------------------------------

def pack_ours(q):
    """q uint8 [N,K] -> uint8 [N,K/2], even k in the HIGH nibble.

    Follows test/nvidia/utils/quant_dequant_nvidia.py:79-88.
    """
    q = np.asarray(q, dtype=np.uint8)
    return ((q[:, 0::2] << 4) | q[:, 1::2]).astype(np.uint8)


def ours_to_awq(src, in_features, out_features):
    """uint8 [N,K/2] ("ours") -> uint32 [K, N/8].

    Follows quantization/nvidia/kernel/gemm_s4_f16/format.cu:151-201: word
    (k, c) holds out-features 8c + [0,2,4,6,1,3,5,7] from its least
    significant nibble up.
    """
    src = np.asarray(src, dtype=np.uint8).reshape(out_features, in_features // 2)
    q = np.empty((out_features, in_features), dtype=np.uint32)
    q[:, 0::2] = src >> 4
    q[:, 1::2] = src & 0xF
    qt = q.T.reshape(in_features, out_features // 8, 8)  # [k, c, j]
    order = (0, 2, 4, 6, 1, 3, 5, 7)
    word = np.zeros((in_features, out_features // 8), dtype=np.uint32)
    for pos, j in enumerate(order):
        word |= qt[:, :, j] << np.uint32(4 * pos)
    return word


def _nibbles(words):
    w = np.asarray(words, dtype=np.uint32).reshape(-1)
    sh = (np.arange(8, dtype=np.uint32) * 4)[None, :]
    return ((w[:, None] >> sh) & 0xF).astype(np.uint8).reshape(-1)


def _from_nibbles(nib):
    nib = np.asarray(nib, dtype=np.uint32).reshape(-1, 8)
    sh = (np.arange(8, dtype=np.uint32) * 4)[None, :]
    return (nib << sh).sum(axis=1, dtype=np.uint64).astype(np.uint32)


def awq_to_lmdeploy(src, in_features, out_features):
    """uint32 [K,N/8] (AWQ order) -> uint32 [K,N/8] storage in tile order.

    Brute-force statement of format.cu:24-57,66-71: the flat nibble array is
    viewed with shape (K/32,2,2,4,2, N/32,2,2,2,4) and element `indices` is
    written to the offset obtained by reading the axes in the order
    (0,5,9,8,3,1,6,4,2,7).
    """
    k, m = in_features, out_features
    assert k % 32 == 0 and m % 32 == 0
    shape = (k // 32, 2, 2, 4, 2, m // 32, 2, 2, 2, 4)
    order = (0, 5, 9, 8, 3, 1, 6, 4, 2, 7)
    nib = _nibbles(src).reshape(shape)
    out = np.ascontiguousarray(nib.transpose(order)).reshape(-1)
    return _from_nibbles(out).reshape(k, m // 8)


def lmdeploy_nibble_offset(n, k, out_features):
    """Closed form: flat nibble offset of element (n,k) in the L2 weight."""
    kk, nn = k % 32, n % 32
    lane = (nn % 8) * 4 + (kk % 8) // 2
    u32 = (kk // 16) * 2 + (nn // 16)
    nib = (kk % 2) * 4 + ((kk // 8) % 2) * 2 + ((nn // 8) % 2)
    tile = (k // 32) * (out_features // 32) + n // 32
    return (((tile * 32 + lane) * 4 + u32) * 8) + nib


def pack_l2(q):
    """q uint8 [N,K] -> int32 [K,N/8] in layout L2 (full producer chain)."""
    n, k = q.shape
    w = awq_to_lmdeploy(ours_to_awq(pack_ours(q), k, n), k, n)
    return w.view(np.int32)


def unpack_l2(w, in_features, out_features):
    """int32 [K,N/8] layout L2 -> q uint8 [N,K] (via the closed-form map)."""
    nib = _nibbles(np.asarray(w).view(np.uint32))
    nn, kk = np.meshgrid(np.arange(out_features), np.arange(in_features), indexing="ij")
    return nib[lmdeploy_nibble_offset(nn, kk, out_features)]


def transpose_merge_zeros_scales(zeros, scales, in_features, out_features, g):
    """zeros,scales fp16 [N,K/g] (zeros WITHOUT the +64) -> fp16 [K/g, 2N].

    Follows format.cu:206-239: element (n, j) goes to half2 index j*N + n as
    (zero + 64, scale).
    """
    z = np.asarray(zeros, dtype=np.float16).reshape(out_features, in_features // g)
    s = np.asarray(scales, dtype=np.float16).reshape(out_features, in_features // g)
    out = np.empty((in_features // g, out_features, 2), dtype=np.float16)
    out[:, :, 0] = (z + np.float16(64)).astype(np.float16).T
    out[:, :, 1] = s.T
    return out.reshape(in_features // g, 2 * out_features)


def dequant_l2(w, zs, g, in_features, out_features):
    """L2 weight + zeros_scales -> W_hat fp16 [N,K]."""
    q = unpack_l2(w, in_features, out_features)
    zs = np.asarray(zs, dtype=np.float16).reshape(in_features // g, out_features, 2)
    z64 = np.repeat(zs[:, :, 0].T, g, axis=1)
    s = np.repeat(zs[:, :, 1].T, g, axis=1)
    h = (q.astype(np.float16) + np.float16(64)).astype(np.float16)
    return ((h - z64).astype(np.float16) * s).astype(np.float16)


# ---------------------------------------------------------------------------
# The linear itself
# ---------------------------------------------------------------------------

def gemm_ref(x, w_hat):
    """X fp16 [M,K], W_hat fp16 [N,K] -> Y fp32 [M,N] (fp32 accumulate).

    The reference's own check is `x @ W_hat.T` (quantization/muxi/script/
    gemm_awq_test.py:44-45,100).
    """
    return np.asarray(x, dtype=np.float32) @ np.asarray(w_hat, dtype=np.float32).T


def gemm_l1(x, w, zs, g):
    """Full path for layout L1: returns (Y fp32, Y fp16)."""
    y = gemm_ref(x, dequant_l1(w, zs, g))
    return y, y.astype(np.float16)


def gemm_l2(x, w, zs, g, in_features, out_features):
    y = gemm_ref(x, dequant_l2(w, zs, g, in_features, out_features))
    return y, y.astype(np.float16)


def silu_dot_ref(x, w_hat_gate, w_hat_up):
    """silu(X W_gate_hat^T) * (X W_up_hat^T) in float64, [M, N].

    The expected value of the fused gated-MLP variant as the reference's kernel test computes it
    (quantization/nvidia/script/gemm_awq_test.py:50-56: matmul, matmul, silu(first) * second),
    which that test accepts within atol = rtol = 2e-2 (:105).
    """
    a = np.asarray(x, dtype=np.float64) @ np.asarray(w_hat_gate, dtype=np.float64).T
    b = np.asarray(x, dtype=np.float64) @ np.asarray(w_hat_up, dtype=np.float64).T
    return a / (1.0 + np.exp(-a)) * b


# ---------------------------------------------------------------------------
# Either side of the path: quantizer and 2-bit expansion
# ---------------------------------------------------------------------------

def rtn_quantize(w, n_bit, g, dtype=np.float32):
    """Round-to-nearest asymmetric group quantization.

    Follows test/muxi/utils/quant_funcs.py:96-114: per group of g along the
    last axis, s = clamp(max - min, 1e-5) / (2^b - 1), z = clamp(-round(min /
    s), 0, 2^b - 1), q = clamp(round(w / s) + z, 0, 2^b - 1); rounding is
    half-to-even.  Every operation is rounded to `dtype`: the reference computes in
    the dtype of the weight it is handed (np.float16 for the fp16 models it packs).
    Returns (q uint8 [N,K], s [N,K/g], z [N,K/g]) with s, z in `dtype`.
    """
    ft = np.dtype(dtype).type
    w = np.asarray(w, dtype=dtype)
    n, k = w.shape
    wg = w.reshape(-1, g)
    hi = wg.max(axis=1, keepdims=True)
    lo = wg.min(axis=1, keepdims=True)
    qmax = ft(2 ** n_bit - 1)
    s = np.maximum(hi - lo, ft(1e-5)) / qmax
    z = np.clip(-np.rint(lo / s), 0, qmax)
    q = np.clip(np.rint(wg / s) + z, 0, qmax)
    return (q.reshape(n, k).astype(np.uint8), s.reshape(n, k // g), z.reshape(n, k // g))


def pack_2bit_l1(q2):
    """q2 uint8 [N,K] with values in [0,3] -> uint8 [N,K/4].

    Follows test/muxi/utils/quant_funcs.py:129-140: of each 4 values
    (a,b,c,d) the byte is a<<4 | b<<6 | c | d<<2.
    """
    r = np.asarray(q2, dtype=np.uint8).reshape(q2.shape[0], -1, 4)
    return ((r[..., 0] << 4) | (r[..., 1] << 6) | r[..., 2] | (r[..., 3] << 2)).astype(np.uint8)


def convert_2bit_to_4bit_l1(w2):
    """uint8 [N,K/4] 2-bit packed -> uint8 [N,K/2] 4-bit packed.

    Follows test/muxi/module/qlinear/qlinear.py:93-103: byte b yields the two
    bytes ((b & 0xC0) >> 2) + ((b & 0x30) >> 4) and ((b & 0x0C) << 2) + (b & 3).
    """
    b = np.asarray(w2, dtype=np.uint8)
    first = ((b & 0xC0) >> 2) + ((b & 0x30) >> 4)
    second = ((b & 0x0C) << 2) + (b & 0x03)
    return np.stack([first, second], axis=-1).reshape(b.shape[0], b.shape[1] * 2).astype(np.uint8)


def convert_4bit_to_2bit_l2(w4):
    """int32 [K, N/8] -> int32 [K, N/16], the tensor-core layout's 2-bit storage.

    Follows test/nvidia/utils/quant_dequant_nvidia.py:34-43 as Python evaluates it: the words are
    taken in pairs (a, b) in row-major order, and each of the eight loop trips adds
    `a & (0x30000000 >> 4*(i-1)) << 2*i` and `b & (0x30000000 >> 4*(i-1)) >> 16 - 2*i`.  `<<` and
    `>>` bind tighter than `&`, so the shifts apply to the mask, not to the masked word: the masks
    of a are 0xC0000000, 0x30000000, ... 0x00030000 (together 0xFFFF0000), those of b are 0xC000,
    0x3000, ... 0x3 (together 0x0000FFFF), and the sum is (a & 0xFFFF0000) + (b & 0x0000FFFF).
    """
    w = np.ascontiguousarray(w4).view(np.uint32)
    pairs = w.reshape(-1, 2)
    out = (pairs[:, 0] & np.uint32(0xFFFF0000)) + (pairs[:, 1] & np.uint32(0x0000FFFF))
    return out.astype(np.uint32).view(np.int32).reshape(w.shape[0], w.shape[1] // 2)


def convert_2bit_to_4bit_l2(w2):
    """int32 [K, N/16] -> int32 [K, N/8].

    Follows test/nvidia/utils/quant_dequant_nvidia.py:45-54 as Python evaluates it: for a stored
    word w the first output word sums `w & (0xC0000000 >> 2*(i-1)) >> 2*i`, whose masks are
    0x30000000, 0x03000000, ... 0x3, the second sums `w & (0x0000C000 >> 2*(i-1)) << 16 - 2*i`
    with the same eight masks: both are w & 0x33333333.
    """
    w = np.ascontiguousarray(w2).view(np.uint32)
    m = (w & np.uint32(0x33333333)).reshape(-1)
    out = np.stack([m, m], axis=1)
    return out.view(np.int32).reshape(w.shape[0], w.shape[1] * 2)


# ---------------------------------------------------------------------------
# Synthetic inputs of the benchmark configurations
# ---------------------------------------------------------------------------

def synth_linear(n, k, g, seed=0):
    """Seeded synthetic quantized linear: q,z ~ U{0..15}, s = |N(0,.02)|+1e-3.

    Returns dict with q, z, s (fp16) and both packed layouts' L1 tensors.
    """
    rng = np.random.default_rng(seed)
    q = rng.integers(0, 16, size=(n, k), dtype=np.uint8)
    z = rng.integers(0, 16, size=(n, k // g), dtype=np.uint8)
    s = (np.abs(rng.normal(0.0, 0.02, size=(n, k // g))) + 1e-3).astype(np.float16)
    return {"q": q, "z": z, "s": s, "w_l1": pack_l1(q), "zs_l1": zeros_scales_l1(z, s)}


def synth_x(m, k, seed=1):
    rng = np.random.default_rng(seed)
    return rng.normal(0.0, 1.0, size=(m, k)).astype(np.float16)


def layernorm_ref(x, gamma=None, beta=None, eps=1e-5):
    """LayerNorm over the last axis in float64: (x - mean) / sqrt(biased var + eps) * gamma + beta,
    what nn.LayerNorm computes at the call sites test/nvidia/module/opt/modeling_opt_ours.py:561-562,
    603-604.  Pinned by closed forms in tests/test_oracle.py (constant rows, +-1 rows, shift
    invariance, a row whose statistics are known by hand)."""
    x = np.asarray(x, dtype=np.float64)
    mean = x.mean(axis=-1, keepdims=True)
    var = ((x - mean) ** 2).mean(axis=-1, keepdims=True)
    y = (x - mean) / np.sqrt(var + eps)
    if gamma is not None:
        y = y * np.asarray(gamma, dtype=np.float64)
    if beta is not None:
        y = y + np.asarray(beta, dtype=np.float64)
    return y
