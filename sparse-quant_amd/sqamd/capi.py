"""ctypes binding of the C ABI in include/sq_w4a16.h (libsq_w4a16.so).

This is the thinnest possible host side: torch tensors are used only for device
memory and streams; every call forwards raw pointers.  The library must already
be built (python -m sqamd.build); loading fails loudly otherwise.
"""
import ctypes
import os

import torch  # noqa: F401  (loads torch's HIP runtime first so that one runtime is shared)

PKG_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(PKG_ROOT, "libsq_w4a16.so")

SQ_OK = 0
SQ_ERR_NULL_POINTER, SQ_ERR_BAD_SHAPE, SQ_ERR_BAD_GROUP, SQ_ERR_BAD_LAYOUT = 1, 2, 3, 4
SQ_ERR_BAD_ALGO, SQ_ERR_MISALIGNED, SQ_ERR_LAUNCH, SQ_ERR_WORKSPACE = 5, 6, 7, 8
SQ_LAYOUT_L1, SQ_LAYOUT_L2 = 1, 2
SQ_ALGO_AUTO, SQ_ALGO_GEMV, SQ_ALGO_GEMV_FIXUP, SQ_ALGO_SKINNY, SQ_ALGO_GEMM = 0, 1, 2, 3, 4

_vp, _i = ctypes.c_void_p, ctypes.c_int

# name -> (restype, argtypes); mirrors include/sq_w4a16.h one to one.
SIGNATURES = {
    "sq_version": (_i, []),
    "sq_strerror": (ctypes.c_char_p, [_i]),
    "sq_w4a16_gemm": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "sq_w4a16_gemm_ex": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp]),
    "sq_w4a16_gemm_ws": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp, ctypes.c_size_t, _vp]),
    "sq_w4a16_gemm_static_ws": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp]),
    "sq_w4a16_gemm_fused": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, ctypes.c_size_t, _vp]),
    "sq_w4a16_gemm_silu_dot": (_i, [_vp] * 7 + [_i] * 5 + [_vp, ctypes.c_size_t, _vp]),
    "sq_w4a16_workspace_bytes": (ctypes.c_size_t, [_i, _i, _i]),
    "sq_w4a16_autotune": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, ctypes.c_size_t, _i, ctypes.c_size_t,
                               ctypes.c_size_t, _i, _vp, ctypes.POINTER(_i), ctypes.POINTER(ctypes.c_float),
                               ctypes.POINTER(ctypes.c_float)]),
    "sq_w4a16_autotune_clear": (_i, []),
    "sq_workspace_reset": (_i, [_vp, ctypes.c_size_t, _vp]),
    "sq_workspace_check": (_i, [_vp, ctypes.c_size_t, _vp]),
    "sq_w4a16_dequant": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "sq_transpose_merge_zeros_scales": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "sq_convert_ours_to_awq": (_i, [_vp, _vp, _i, _i, _vp]),
    "sq_convert_awq_to_lmdeploy": (_i, [_vp, _vp, _i, _i, _vp]),
    "sq_repack_l2_to_l1": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "sq_convert_2bit_to_4bit": (_i, [_vp, _vp, _i, _i, _vp]),
    "sq_l2_convert_4bit_to_2bit": (_i, [_vp, _vp, _i, _i, _vp]),
    "sq_l2_convert_2bit_to_4bit": (_i, [_vp, _vp, _i, _i, _vp]),
    "sq_decode_attention": (_i, [_vp] * 7 + [_i] * 4 + [ctypes.c_long] * 7 + [_i, _vp, ctypes.c_float, _vp, ctypes.c_size_t,
                                 _vp]),
    "sq_decode_attention_workspace_bytes": (ctypes.c_size_t, [_i, _i, _i]),
    "sq_layernorm": (_i, [_vp, _vp, _vp, _vp, _i, _i, ctypes.c_float, _vp]),
    "sq_w4a16_ln_fusable": (_i, [_i, _i, _i, _i, _i]),
    "sq_w4a16_gemm_ln_fused": (_i, [_vp, _vp, _vp, ctypes.c_float, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i,
                                    _vp, ctypes.c_size_t, _vp]),
    "sq_lut_attention_fwd": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, ctypes.c_float, _i, _vp]),
    "sq_embed_rows": (_i, [_vp, _vp, _vp, _vp, ctypes.c_longlong, _vp, _i, _i, ctypes.c_longlong, ctypes.c_longlong, _vp]),
    "sq_f16_gemv_parts": (_i, [_i]),
    "sq_f16_gemv": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "sq_greedy_feedback": (_i, [_vp, _vp, _i, _i, _vp, _vp, _vp, _vp, ctypes.c_longlong, _vp]),
}

# include/sq_probes.h (libsq_probes.so): diagnostic kernels used by the benchmark only.
PROBES_PATH = os.path.join(PKG_ROOT, "libsq_probes.so")
PROBE_SIGNATURES = {
    "sq_clock_probe": (_i, [_vp, _i, _vp]),
    "sq_mfma_probe": (_i, [_vp, _vp, _i, _i, _vp]),
    "sq_read_probe": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
}



class LinearDesc(ctypes.Structure):
    """sq_linear_desc of include/sq_w4a16.h."""
    _fields_ = [("x", _vp), ("w", _vp), ("zs", _vp), ("bias", _vp), ("residual", _vp), ("y", _vp),
                ("N", _i), ("K", _i), ("group_size", _i), ("act", _i), ("depends", _i)]


SIGNATURES["sq_w4a16_gemv_sequence"] = (_i, [ctypes.POINTER(LinearDesc), _i, _i, _i, _i, _vp, ctypes.c_size_t, _vp])
SQ_SEQ_AUTO, SQ_SEQ_ONE_LAUNCH = 0, 1
SIGNATURES["sq_w4a16_gemv_sequence_workspace_bytes"] = (ctypes.c_size_t, [ctypes.POINTER(LinearDesc), _i, _i])
SIGNATURES["sq_w4a16_gemv_sequence_tune"] = (_i, [ctypes.c_uint, _i])
SIGNATURES["sq_w4a16_gemv_sequence_status"] = (_i, [ctypes.POINTER(LinearDesc), _i, _i, _vp, ctypes.c_size_t, _i, _vp])
SQ_ERR_SEQ_TIMEOUT = 10
SQ_SEQUENCE_MAX = 8

_lib = None
_probes = None


class SqError(RuntimeError):
    def __init__(self, code, what):
        self.code = code
        super().__init__("%s: %s (code %d)" % (what, strerror(code), code))


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libsq_w4a16.so is missing at %s: run `python -m sqamd.build` first; there is no "
                               "fallback path" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def probes():
    """The loaded diagnostic library; raises if it has not been built."""
    global _probes
    if _probes is None:
        if not os.path.exists(PROBES_PATH):
            raise RuntimeError("libsq_probes.so is missing at %s: run `python -m sqamd.build` first" % PROBES_PATH)
        handle = ctypes.CDLL(PROBES_PATH)
        for name, (res, args) in PROBE_SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _probes = handle
    return _probes


def strerror(code):
    return lib().sq_strerror(int(code)).decode()


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream(stream=None):
    if stream is None:
        stream = torch.cuda.current_stream()
    return ctypes.c_void_p(stream.cuda_stream)


def _check(code, what):
    if code != SQ_OK:
        raise SqError(code, what)


def gemm(x, w, zs, n, k, group_size, layout=SQ_LAYOUT_L1, algo=SQ_ALGO_AUTO, out=None, stream=None):
    """x fp16 [M,K] -> y fp16 [M,N] through sq_w4a16_gemm_ex."""
    m = x.numel() // k
    if out is None:
        out = torch.empty((m, n), dtype=torch.float16, device=x.device)
    _check(lib().sq_w4a16_gemm_ex(_ptr(x), _ptr(w), _ptr(zs), _ptr(out), m, n, k, group_size, layout, algo,
                                  _stream(stream)), "sq_w4a16_gemm_ex")
    return out


SQ_ALGO_SKINNY_WS = 5
SQ_ALGO_STREAM = 6
_workspaces = {}
_retired = []  # outgrown workspaces: a captured HIP graph may still hold their address


def _cached_workspace(key, need, device):
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < need:
        if ws is not None:
            _retired.append(ws)
        ws = torch.zeros(need, dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def workspace(m, n, k, device, stream=None):
    """A zero-initialised workspace tensor, cached per (device, stream) and grown on demand."""
    need = lib().sq_w4a16_workspace_bytes(m, n, k)
    key = (str(device), (stream or torch.cuda.current_stream()).cuda_stream)
    return _cached_workspace(key, max(need, 1 << 20), device)


def workspace_reset(ws, nbytes=None, stream=None):
    """Clear the first nbytes (default: all) of a workspace tensor with the library's fill kernel."""
    n = ws.numel() if nbytes is None else int(nbytes)
    _check(lib().sq_workspace_reset(_ptr(ws), n - n % 4, _stream(stream)), "sq_workspace_reset")


def workspace_is_clean(ws, nbytes=65536, stream=None):
    """Debugging aid (synchronises): True if the counter region of a workspace is all zero."""
    rc = lib().sq_workspace_check(_ptr(ws), min(int(nbytes), ws.numel()) // 4 * 4, _stream(stream))
    if rc not in (SQ_OK, SQ_ERR_WORKSPACE):
        raise SqError(rc, "sq_workspace_check")
    return rc == SQ_OK


def gemm_ws(x, w, zs, n, k, group_size, algo=SQ_ALGO_AUTO, out=None, stream=None, ws=None):
    """x fp16 [M,K] -> y fp16 [M,N] through sq_w4a16_gemm_ws (workspace-backed split-K for 5 <= M <= 32)."""
    m = x.numel() // k
    if out is None:
        out = torch.empty((m, n), dtype=torch.float16, device=x.device)
    if ws is None:
        ws = workspace(max(m, 1), n, k, x.device, stream)
    _check(lib().sq_w4a16_gemm_ws(_ptr(x), _ptr(w), _ptr(zs), _ptr(out), m, n, k, group_size, SQ_LAYOUT_L1, algo,
                                  _ptr(ws), ws.numel(), _stream(stream)), "sq_w4a16_gemm_ws")
    return out


def autotune(x, w, zs, n, k, group_size, ws=None, reps=20, out=None, stream=None):
    """Time every kernel that can serve this shape (sq_w4a16_autotune; synchronises) and record the fastest for
    SQ_ALGO_AUTO.  w uint8 [N, K/2] or a pool [copies, N, K/2] with zs [copies, N, 2K/g] (timed in rotation, i.e.
    from HBM when the pool exceeds the last-level cache).  Returns (kernel word or 0, best us, built-in us)."""
    m = x.numel() // k
    if out is None:
        out = torch.empty((m, n), dtype=torch.float16, device=x.device)
    copies = w.shape[0] if w.dim() == 3 else 1
    best, t_best, t_auto = ctypes.c_int(0), ctypes.c_float(0), ctypes.c_float(0)
    _check(lib().sq_w4a16_autotune(_ptr(x), _ptr(w), _ptr(zs), _ptr(out), m, n, k, group_size, SQ_LAYOUT_L1, _ptr(ws),
                                   0 if ws is None else ws.numel(), copies, n * k // 2, n * (k // group_size) * 4,
                                   int(reps), _stream(stream), ctypes.byref(best), ctypes.byref(t_best),
                                   ctypes.byref(t_auto)), "sq_w4a16_autotune")
    return best.value, t_best.value, t_auto.value


def autotune_clear():
    return lib().sq_w4a16_autotune_clear()


SQ_ERR_STATIC_WS = 9
SQ_STATIC_WS_BYTES = 16 * 1024 * 1024 + 64 * 1024


def gemm_static_ws(x, w, zs, n, k, group_size, algo=SQ_ALGO_AUTO, out=None, stream=None):
    """x fp16 [M,K] -> y fp16 [M,N] through sq_w4a16_gemm_static_ws (workspace inside the library)."""
    m = x.numel() // k
    if out is None:
        out = torch.empty((m, n), dtype=torch.float16, device=x.device)
    _check(lib().sq_w4a16_gemm_static_ws(_ptr(x), _ptr(w), _ptr(zs), _ptr(out), m, n, k, group_size, SQ_LAYOUT_L1, algo,
                                         _stream(stream)), "sq_w4a16_gemm_static_ws")
    return out


SQ_ACT_NONE, SQ_ACT_RELU, SQ_ACT_SILU = 0, 1, 2


def gemm_fused(x, w, zs, n, k, group_size, bias=None, residual=None, act=SQ_ACT_NONE, algo=SQ_ALGO_AUTO, out=None,
               stream=None, ws=None, use_workspace=True):
    """y = act(x W_hat^T + bias) + residual through sq_w4a16_gemm_fused."""
    m = x.numel() // k
    if out is None:
        out = torch.empty((m, n), dtype=torch.float16, device=x.device)
    if ws is None and use_workspace and 2 < m <= 1024:
        ws = workspace(m, n, k, x.device, stream)
    _check(lib().sq_w4a16_gemm_fused(_ptr(x), _ptr(w), _ptr(zs), _ptr(bias), _ptr(residual), _ptr(out), m, n, k,
                                     group_size, SQ_LAYOUT_L1, act, algo, _ptr(ws), 0 if ws is None else ws.numel(),
                                     _stream(stream)), "sq_w4a16_gemm_fused")
    return out


def gemm_silu_dot(x, w_gate, zs_gate, w_up, zs_up, n, k, group_size, out=None, stream=None, ws=None, use_workspace=True,
                  up_out=None):
    """y = silu(x W_gate_hat^T) * (x W_up_hat^T) through sq_w4a16_gemm_silu_dot; returns (y, up projection)."""
    m = x.numel() // k
    if out is None:
        out = torch.empty((m, n), dtype=torch.float16, device=x.device)
    up = up_out if up_out is not None else torch.empty((m, n), dtype=torch.float16, device=x.device)
    if ws is None and use_workspace and 2 < m <= 1024:
        ws = workspace(m, n, k, x.device, stream)
    _check(lib().sq_w4a16_gemm_silu_dot(_ptr(x), _ptr(w_gate), _ptr(zs_gate), _ptr(w_up), _ptr(zs_up), _ptr(out), _ptr(up),
                                        m, n, k, group_size, SQ_LAYOUT_L1, _ptr(ws), 0 if ws is None else ws.numel(),
                                        _stream(stream)), "sq_w4a16_gemm_silu_dot")
    return out, up


def gemm_ln_fused(x, ln_gamma, ln_beta, ln_eps, w, zs, n, k, group_size, bias=None, residual=None, act=SQ_ACT_NONE,
                  out=None, stream=None, ws=None):
    """y = act(LayerNorm(x) W_hat^T + bias) + residual through sq_w4a16_gemm_ln_fused (the normalisation inside the
    linear's kernel where sq_w4a16_ln_fusable says so, the LayerNorm kernel into a scratch tensor otherwise)."""
    m = x.numel() // k
    if out is None:
        out = torch.empty((m, n), dtype=torch.float16, device=x.device)
    scratch = None
    if not lib().sq_w4a16_ln_fusable(m, n, k, group_size, SQ_LAYOUT_L1):
        scratch = torch.empty((m, k), dtype=torch.float16, device=x.device)
        if ws is None and 2 < m <= 1024:
            ws = workspace(m, n, k, x.device, stream)
    _check(lib().sq_w4a16_gemm_ln_fused(_ptr(x), _ptr(ln_gamma), _ptr(ln_beta), float(ln_eps), _ptr(scratch), _ptr(w),
                                        _ptr(zs), _ptr(bias), _ptr(residual), _ptr(out), m, n, k, group_size, SQ_LAYOUT_L1,
                                        act, _ptr(ws), 0 if ws is None else ws.numel(), _stream(stream)),
           "sq_w4a16_gemm_ln_fused")
    return out


class LinearSequence:
    """Up to SQ_SEQUENCE_MAX decode linears bound once, launched with one call (sq_w4a16_gemv_sequence).

    linears: list of dicts with keys x, w, zs, y (tensors), n, k, group_size and optionally bias,
    residual, act, depends.  The descriptor array and the workspace are kept; `run()` only launches."""

    def __init__(self, linears, m, device, workspace=True, mode=SQ_SEQ_AUTO):
        self.count = len(linears)
        self.m = int(m)
        self.mode = int(mode)
        self.descs = (LinearDesc * max(self.count, 1))()
        self.keep = list(linears)
        for d, l in zip(self.descs, linears):
            d.x, d.w, d.zs, d.y = l["x"].data_ptr(), l["w"].data_ptr(), l["zs"].data_ptr(), l["y"].data_ptr()
            d.bias = l["bias"].data_ptr() if l.get("bias") is not None else None
            d.residual = l["residual"].data_ptr() if l.get("residual") is not None else None
            d.N, d.K, d.group_size = int(l["n"]), int(l["k"]), int(l["group_size"])
            d.act, d.depends = int(l.get("act", SQ_ACT_NONE)), int(bool(l.get("depends", False)))
        self.ws = torch.zeros(lib().sq_w4a16_gemv_sequence_workspace_bytes(self.descs, self.count, self.m),
                              dtype=torch.uint8, device=device) if workspace else None
        self._fn = lib().sq_w4a16_gemv_sequence

    def run(self, stream=None):
        _check(self._fn(self.descs, self.count, self.m, SQ_LAYOUT_L1, self.mode, _ptr(self.ws),
                        0 if self.ws is None else self.ws.numel(), _stream(stream)), "sq_w4a16_gemv_sequence")

    def error_flag(self, clear=False, stream=None):
        """1 if a wait of the one-launch kernel for another workgroup's output ever ran out of polls since the
        word was last cleared, else 0 (synchronises; sq_w4a16_gemv_sequence_status)."""
        if self.ws is None:
            return 0
        rc = lib().sq_w4a16_gemv_sequence_status(self.descs, self.count, self.m, _ptr(self.ws), self.ws.numel(),
                                                 int(bool(clear)), _stream(stream))
        if rc not in (SQ_OK, SQ_ERR_SEQ_TIMEOUT):
            raise SqError(rc, "sq_w4a16_gemv_sequence_status")
        return int(rc == SQ_ERR_SEQ_TIMEOUT)


def sequence_tune(spin_limit=1 << 16, loads_in_flight=0):
    """Process-wide tuning of the one-launch sequence kernel: polls allowed per wait, loads a wave keeps in flight."""
    _check(lib().sq_w4a16_gemv_sequence_tune(int(spin_limit), int(loads_in_flight)), "sq_w4a16_gemv_sequence_tune")


def dequant(w, zs, n, k, group_size, layout=SQ_LAYOUT_L1, stream=None):
    out = torch.empty((n, k), dtype=torch.float16, device=w.device)
    _check(lib().sq_w4a16_dequant(_ptr(w), _ptr(zs), _ptr(out), n, k, group_size, layout, _stream(stream)),
           "sq_w4a16_dequant")
    return out


def transpose_merge_zeros_scales(zeros, scales, in_features, out_features, group_size, stream=None):
    zs = torch.empty((in_features // group_size, 2 * out_features), dtype=torch.float16, device=zeros.device)
    _check(lib().sq_transpose_merge_zeros_scales(_ptr(zeros), _ptr(scales), _ptr(zs), in_features, out_features,
                                                 group_size, _stream(stream)), "sq_transpose_merge_zeros_scales")
    return zs


def convert_ours_to_awq(src, in_features, out_features, stream=None):
    dst = torch.empty((in_features, out_features // 2), dtype=torch.uint8, device=src.device)
    _check(lib().sq_convert_ours_to_awq(_ptr(src), _ptr(dst), in_features, out_features, _stream(stream)),
           "sq_convert_ours_to_awq")
    return dst


def convert_awq_to_lmdeploy(src, in_features, out_features, stream=None):
    dst = torch.empty((in_features, out_features // 8), dtype=torch.int32, device=src.device)
    _check(lib().sq_convert_awq_to_lmdeploy(_ptr(src), _ptr(dst), in_features, out_features, _stream(stream)),
           "sq_convert_awq_to_lmdeploy")
    return dst


def repack_l2_to_l1(w_l2, zs_l2, n, k, group_size, stream=None):
    w1 = torch.empty((n, k // 2), dtype=torch.uint8, device=w_l2.device)
    zs1 = torch.empty((n, 2 * (k // group_size)), dtype=torch.float16, device=w_l2.device)
    _check(lib().sq_repack_l2_to_l1(_ptr(w_l2), _ptr(zs_l2), _ptr(w1), _ptr(zs1), n, k, group_size,
                                    _stream(stream)), "sq_repack_l2_to_l1")
    return w1, zs1


def convert_2bit_to_4bit(w2, stream=None):
    n, k4 = w2.shape
    out = torch.empty((n, k4 * 2), dtype=torch.uint8, device=w2.device)
    _check(lib().sq_convert_2bit_to_4bit(_ptr(w2), _ptr(out), n, k4 * 4, _stream(stream)),
           "sq_convert_2bit_to_4bit")
    return out


def l2_convert_4bit_to_2bit(w4, stream=None):
    """int32 [K, N/8] -> int32 [K, N/16]."""
    k, n8 = w4.shape
    out = torch.empty((k, n8 // 2), dtype=torch.int32, device=w4.device)
    _check(lib().sq_l2_convert_4bit_to_2bit(_ptr(w4), _ptr(out), k, n8 * 8, _stream(stream)),
           "sq_l2_convert_4bit_to_2bit")
    return out


def l2_convert_2bit_to_4bit(w2, stream=None):
    """int32 [K, N/16] -> int32 [K, N/8]."""
    k, n16 = w2.shape
    out = torch.empty((k, n16 * 2), dtype=torch.int32, device=w2.device)
    _check(lib().sq_l2_convert_2bit_to_4bit(_ptr(w2), _ptr(out), k, n16 * 16, _stream(stream)),
           "sq_l2_convert_2bit_to_4bit")
    return out


def lut_attention(q, k, v, lut, sm_scale, causal, stream=None):
    """q, k, v fp16 [Z,H,S,D] contiguous; lut int32/int64 [H, ceil(S/64), nnz] -> out fp16 [Z,H,S,D]."""
    z, h, s, d = q.shape
    out = torch.empty_like(q)
    _check(lib().sq_lut_attention_fwd(_ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lut), lut.element_size(), z, h, s, d,
                                      lut.shape[-1], float(sm_scale), int(bool(causal)), _stream(stream)),
           "sq_lut_attention_fwd")
    return out


def decode_attention(q, k_cache, v_cache, cache_len, sm_scale, k_new=None, v_new=None, mask=None, out=None,
                     stream=None, ws=None, use_workspace=True):
    """Dense decode attention over an fp16 KV cache, optionally appending the new row.

    q [B,H,1,D] or [B,H,D] (any batch/head strides, D contiguous); k_cache, v_cache [B,H,Lmax,D] with
    contiguous rows (a slice cache[:, :, :L] of a bigger buffer is fine); k_new, v_new like q or None;
    cache_len: int, or an int64 device tensor of one element (read by the kernel); mask None or fp16
    [B,1,1,L] / [B,L] additive.  With fewer than 256 (batch, head) pairs a zeroed workspace (cached per
    device and stream unless `ws` is given) lets several workgroups share a head.  Returns out fp16
    [B, 1, H*D]."""
    b, h = q.shape[0], q.shape[1]
    d = q.shape[-1]
    q3 = q.reshape(b, h, d) if q.dim() == 4 else q
    if q3.stride(-1) != 1 or k_cache.stride(-1) != 1 or k_cache.stride(2) != d or v_cache.stride() != k_cache.stride():
        raise ValueError("decode_attention needs D-contiguous q and caches with contiguous rows")
    lmax = k_cache.shape[2]
    kn = vn = None
    n_bs = n_hs = 0
    if k_new is not None:
        kn = k_new.reshape(b, h, d) if k_new.dim() == 4 else k_new
        vn = v_new.reshape(b, h, d) if v_new.dim() == 4 else v_new
        if kn.stride(-1) != 1 or vn.stride() != kn.stride():
            raise ValueError("k_new and v_new must be D-contiguous with equal strides")
        n_bs, n_hs = kn.stride(0), kn.stride(1)
    m_bs = 0
    if mask is not None:
        mask = mask.reshape(b, -1)
        if mask.dtype != torch.float16 or mask.stride(-1) != 1:
            raise ValueError("mask must be fp16 with contiguous rows")
        m_bs = mask.stride(0)
    if out is None:
        out = torch.empty((b, 1, h * d), dtype=torch.float16, device=q.device)
    if torch.is_tensor(cache_len):
        if cache_len.dtype != torch.int64 or not cache_len.is_cuda:
            raise TypeError("a device-side cache_len must be an int64 device tensor")
        len_host, len_dev = 0, _ptr(cache_len)
    else:
        len_host, len_dev = int(cache_len), None
    if ws is None and use_workspace and b * h < 256:
        need = lib().sq_decode_attention_workspace_bytes(b, h, d)
        key = ("attn", str(q.device), (stream or torch.cuda.current_stream()).cuda_stream)
        ws = _cached_workspace(key, need, q.device)
    _check(lib().sq_decode_attention(_ptr(q3), _ptr(kn) if kn is not None else None,
                                     _ptr(vn) if vn is not None else None, _ptr(k_cache), _ptr(v_cache),
                                     _ptr(mask) if mask is not None else None, _ptr(out), b, h, d, lmax,
                                     q3.stride(0), q3.stride(1), n_bs, n_hs, k_cache.stride(0), k_cache.stride(1), m_bs,
                                     len_host, len_dev, float(sm_scale), _ptr(ws), 0 if ws is None else ws.numel(),
                                     _stream(stream)), "sq_decode_attention")
    return out


def embed_rows(embed, pos_table, tok, pos, pos_offset=0, out=None, stream=None):
    """out[r] = embed[tok[r]] + pos_table[pos[0] + pos_offset] through sq_embed_rows; tok int64 [rows], pos int64 [1]."""
    rows, hidden = tok.numel(), embed.shape[1]
    if out is None:
        out = torch.empty((rows, hidden), dtype=torch.float16, device=embed.device)
    _check(lib().sq_embed_rows(_ptr(embed), _ptr(pos_table), _ptr(tok), _ptr(pos), int(pos_offset), _ptr(out), rows, hidden,
                               embed.shape[0], pos_table.shape[0], _stream(stream)), "sq_embed_rows")
    return out


def f16_gemv(x, w, out=None, parts=None, stream=None):
    """y [M, N] = x [M, K] w[N, K]^T in fp16 through sq_f16_gemv (M <= 8).  parts: None, or a (values, rows) pair of
    float32 / int32 tensors [8, sq_f16_gemv_parts(N)] that receive every workgroup's best candidate per token."""
    n, k = w.shape
    m = x.numel() // k
    if out is None:
        out = torch.empty((m, n), dtype=torch.float16, device=x.device)
    pv, pi = parts if parts is not None else (None, None)
    _check(lib().sq_f16_gemv(_ptr(x), _ptr(w), _ptr(out), _ptr(pv), _ptr(pi), m, n, k, _stream(stream)), "sq_f16_gemv")
    return out


def f16_gemv_parts(n, device):
    """The (values, rows) pair sq_f16_gemv fills for a weight of n rows."""
    p = lib().sq_f16_gemv_parts(n)
    return (torch.empty((8, p), dtype=torch.float32, device=device), torch.empty((8, p), dtype=torch.int32, device=device))


def greedy_feedback(parts, m, tok, pos=None, history=None, step=None, stream=None):
    """tok[i] = argmax of token i from the candidates of f16_gemv; optional history[step] = tok, pos += 1, step += 1
    (all int64 on the device) through sq_greedy_feedback."""
    pv, pi = parts
    _check(lib().sq_greedy_feedback(_ptr(pv), _ptr(pi), pv.shape[1], m, _ptr(tok), _ptr(pos), _ptr(history), _ptr(step),
                                    0 if history is None else history.shape[0], _stream(stream)), "sq_greedy_feedback")
    return tok


def layernorm(x, gamma, beta, eps=1e-5, out=None, stream=None):
    """LayerNorm over the last dimension of a contiguous fp16 tensor; gamma / beta fp16 [cols] or None."""
    cols = x.shape[-1]
    if out is None:
        out = torch.empty_like(x)
    _check(lib().sq_layernorm(_ptr(x), _ptr(gamma), _ptr(beta), _ptr(out), x.numel() // cols, cols, float(eps),
                              _stream(stream)), "sq_layernorm")
    return out


def mfma_probe(data, workgroups, iters, stream=None):
    """Launch the matrix-instruction loop; returns the int64 tensor of per-workgroup shader ticks."""
    out = torch.zeros(workgroups + 1, dtype=torch.int64, device=data.device)
    _check(probes().sq_mfma_probe(_ptr(data), _ptr(out), int(workgroups), int(iters), _stream(stream)), "sq_mfma_probe")
    return out[:workgroups]


def clock_probe(spins=400000, stream=None):
    """Launch the clock probe on `stream`; returns the uint64[3] result tensor (read it after a sync):
    shader ticks, 100 MHz ticks, dummy."""
    dev = torch.device("cuda", torch.cuda.current_device())
    out = torch.zeros(3, dtype=torch.int64, device=dev)
    _check(probes().sq_clock_probe(_ptr(out), int(spins), _stream(stream)), "sq_clock_probe")
    return out
