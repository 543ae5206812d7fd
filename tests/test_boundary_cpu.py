"""CPU-only checks of the drop-in boundary: the C-ABI library loads and exports
every symbol include/sq_w4a16.h declares, argument errors are reported before any
launch, and the `quant` extension mirrors the reference's validation."""
import ctypes
import os
import re
import sys

import numpy as np
import pytest
import torch

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(REPO, "include", "sq_w4a16.h")


PROBES_HEADER = os.path.join(REPO, "include", "sq_probes.h")


def declared_functions(header=HEADER):
    text = open(header).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sq_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_expected_entry_points():
    names = declared_functions()
    for must in ("sq_w4a16_gemm", "sq_w4a16_dequant", "sq_transpose_merge_zeros_scales",
                 "sq_convert_ours_to_awq", "sq_convert_awq_to_lmdeploy", "sq_strerror"):
        assert must in names


def test_library_exports_every_declared_symbol(built_lib):
    lib = ctypes.CDLL(built_lib)
    for name in declared_functions():
        assert hasattr(lib, name), "libsq_w4a16.so does not export %s" % name


def test_ctypes_binding_covers_header(built_lib):
    from sqamd import capi
    assert sorted(capi.SIGNATURES) == declared_functions()
    assert capi.lib().sq_version() >= 100
    assert capi.strerror(0) == "ok"
    for code in range(1, 9):
        assert capi.strerror(code) not in ("ok", "unknown error code")
    assert capi.strerror(999) == "unknown error code"


def test_probe_library_exports_its_header(built_lib):
    from sqamd import capi
    names = declared_functions(PROBES_HEADER)
    assert names == sorted(capi.PROBE_SIGNATURES) and len(names) == 3
    lib = capi.probes()
    for name in names:
        assert hasattr(lib, name)
    assert not set(names) & set(declared_functions()), "diagnostics do not belong to the product header"
    assert lib.sq_read_probe(None, None, None, 64, 128, 64, None) == 1
    assert lib.sq_clock_probe(None, 10, None) == 1


def test_argument_errors_come_before_any_launch(built_lib):
    # No GPU is needed: every call below must be rejected by validation alone.
    from sqamd import capi
    L = capi.lib()
    buf = np.zeros(64, dtype=np.uint8)
    p = ctypes.c_void_p(buf.ctypes.data - (buf.ctypes.data % 16) + 16)
    odd = ctypes.c_void_p(p.value + 2)
    gemm = L.sq_w4a16_gemm
    assert gemm(None, p, p, p, 1, 64, 128, 64, 1, None) == capi.SQ_ERR_NULL_POINTER
    assert gemm(p, p, p, None, 1, 64, 128, 64, 1, None) == capi.SQ_ERR_NULL_POINTER
    assert gemm(p, p, p, p, 1, 64, 128, 48, 1, None) == capi.SQ_ERR_BAD_GROUP
    assert gemm(p, p, p, p, 1, 64, 128, 64, 9, None) == capi.SQ_ERR_BAD_LAYOUT
    assert gemm(p, p, p, p, 1, 60, 128, 64, 1, None) == capi.SQ_ERR_BAD_SHAPE      # N % 8
    assert gemm(p, p, p, p, 1, 64, 100, 64, 1, None) == capi.SQ_ERR_BAD_SHAPE      # K % 32
    assert gemm(p, p, p, p, 1, 64, 96, 64, 1, None) == capi.SQ_ERR_BAD_SHAPE       # K % g
    assert gemm(p, p, p, p, -1, 64, 128, 64, 1, None) == capi.SQ_ERR_BAD_SHAPE
    assert gemm(p, p, p, p, 1, 0, 128, 64, 1, None) == capi.SQ_ERR_BAD_SHAPE
    assert gemm(odd, p, p, p, 1, 64, 128, 64, 1, None) == capi.SQ_ERR_MISALIGNED
    assert gemm(p, p, p, p, 0, 64, 128, 64, 1, None) == capi.SQ_OK                 # empty input: nothing launched
    assert L.sq_w4a16_gemm_ex(p, p, p, p, 1, 64, 128, 64, 1, 77, None) == capi.SQ_ERR_BAD_ALGO
    assert L.sq_w4a16_gemm_ex(p, p, p, p, 9, 64, 128, 64, 1, capi.SQ_ALGO_GEMV, None) == capi.SQ_ERR_BAD_ALGO
    assert L.sq_w4a16_gemm_ex(p, p, p, p, 65, 64, 128, 64, 1, capi.SQ_ALGO_SKINNY, None) == capi.SQ_ERR_BAD_ALGO
    assert L.sq_w4a16_dequant(p, p, None, 64, 128, 64, 1, None) == capi.SQ_ERR_NULL_POINTER
    assert L.sq_w4a16_dequant(p, p, p, 64, 128, 64, 2, None) == capi.SQ_ERR_BAD_GROUP  # L2 needs g == 128
    assert L.sq_w4a16_dequant(p, p, p, 48, 128, 128, 2, None) == capi.SQ_ERR_BAD_SHAPE  # L2 needs N % 32
    assert L.sq_transpose_merge_zeros_scales(p, p, p, 128, 64, 0, None) == capi.SQ_ERR_BAD_GROUP
    assert L.sq_transpose_merge_zeros_scales(p, None, p, 128, 64, 64, None) == capi.SQ_ERR_NULL_POINTER
    assert L.sq_convert_ours_to_awq(p, p, 128, 60, None) == capi.SQ_ERR_BAD_SHAPE
    assert L.sq_convert_awq_to_lmdeploy(p, p, 100, 64, None) == capi.SQ_ERR_BAD_SHAPE
    assert L.sq_convert_awq_to_lmdeploy(p, p, 128, 64, None) == capi.SQ_ERR_BAD_SHAPE  # in place
    assert L.sq_repack_l2_to_l1(p, p, p, p, 64, 128, 64, None) == capi.SQ_ERR_BAD_GROUP
    assert L.sq_convert_2bit_to_4bit(p, None, 8, 64, None) == capi.SQ_ERR_NULL_POINTER
    assert L.sq_convert_2bit_to_4bit(p, p, 8, 62, None) == capi.SQ_ERR_BAD_SHAPE
    for fn in (L.sq_l2_convert_4bit_to_2bit, L.sq_l2_convert_2bit_to_4bit):
        assert fn(p, None, 8, 64, None) == capi.SQ_ERR_NULL_POINTER
        assert fn(p, p, 8, 24, None) == capi.SQ_ERR_BAD_SHAPE
        assert fn(p, p, 0, 64, None) == capi.SQ_ERR_BAD_SHAPE


def _ext():
    ext = [f for f in os.listdir(os.path.join(REPO, "sparse-quant_amd")) if f.startswith("quant.") and f.endswith(".so")]
    if not ext:
        pytest.skip("quant extension not built (python -m sqamd.build)")
    import quant
    return quant


def test_host_side_queries_need_no_gpu(built_lib):
    # Workspace sizes and the LayerNorm-fusion query are host arithmetic: what a binding may call at load time.
    from sqamd import capi
    L = capi.lib()
    counters = 65536
    # decode batches: counters + 8 K ranges x 64-row blocks x (4 row tiles x token tiles x 4 x 64 lanes) floats
    assert L.sq_w4a16_workspace_bytes(1, 4096, 4096) == counters + 8 * 64 * (4 * 1 * 4 * 64) * 4
    assert L.sq_w4a16_workspace_bytes(32, 16384, 4096) == counters + 8 * 256 * (4 * 2 * 4 * 64) * 4
    # beyond 32 tokens: the larger of that and the tiled kernel's K split (64-row x 256-column tiles, four parts)
    assert L.sq_w4a16_workspace_bytes(64, 16384, 4096) == counters + 4 * 64 * 64 * 256 * 4
    # a grid that fills the chip splits nothing: only the decode kernels' share remains
    assert L.sq_w4a16_workspace_bytes(2048, 16384, 4096) == L.sq_w4a16_workspace_bytes(32, 16384, 4096)
    assert L.sq_w4a16_workspace_bytes(0, 4096, 4096) == 0
    sizes = [L.sq_w4a16_workspace_bytes(m, 4096, 16384) for m in (1, 16, 17, 32, 33, 64, 512, 1024)]
    assert all(b >= counters for b in sizes) and sizes[0] <= sizes[1] <= sizes[2] == sizes[3]
    fus = L.sq_w4a16_ln_fusable
    assert fus(8, 16384, 4096, 128, capi.SQ_LAYOUT_L1) == 1 and fus(1, 12288, 4096, 128, capi.SQ_LAYOUT_L1) == 1
    for bad in ((9, 16384, 4096, 128, capi.SQ_LAYOUT_L1), (8, 16384, 2048, 128, capi.SQ_LAYOUT_L1),
                (8, 16384, 8192, 128, capi.SQ_LAYOUT_L1), (8, 16384, 4096, 64, capi.SQ_LAYOUT_L1),
                (8, 16384, 4096, 128, capi.SQ_LAYOUT_L2), (0, 16384, 4096, 128, capi.SQ_LAYOUT_L1)):
        assert fus(*bad) == 0, bad


def test_quant_module_surface():
    quant = _ext()
    for name in ("gemm_awq_ut", "dequant", "transpose_merge_zeros_scales", "convert_ours_to_awq",
                 "convert_awq_to_lmdeploy"):
        assert callable(getattr(quant, name))
    assert os.path.dirname(quant.__file__) == os.path.join(REPO, "sparse-quant_amd")


def test_quant_rejects_bad_tensors_before_launch():
    quant = _ext()
    x = torch.zeros(1, 1, 128, dtype=torch.float16)
    w = torch.zeros(64, 64, dtype=torch.uint8)
    zs = torch.zeros(64, 4, dtype=torch.float16)
    # host tensors: the reference's CHECK_DEVICE
    with pytest.raises(RuntimeError, match="must be on CUDA"):
        quant.gemm_awq_ut(x, w, zs, 1, 64, 128, 64)
    with pytest.raises(RuntimeError, match="must be on CUDA"):
        quant.dequant(w, zs, 64, 128, 64)
    with pytest.raises(RuntimeError, match="must be on CUDA"):
        quant.transpose_merge_zeros_scales(zs, zs, zs, 128, 64, 64)
    with pytest.raises(RuntimeError, match="must be on CUDA"):
        quant.convert_ours_to_awq(w, w, 128, 64)
    with pytest.raises(RuntimeError, match="must be on CUDA"):
        quant.convert_awq_to_lmdeploy(w, w.view(torch.int32), 128, 64)


def test_host_packers_match_oracle():
    import w4a16_oracle as orc
    from sqamd import quant_funcs as qf
    rng = np.random.default_rng(0)
    w = rng.normal(0, 0.05, size=(32, 256)).astype(np.float32)
    for g in (64, 128):
        qw, zs = qf.quant_muxi(torch.from_numpy(w), 256, 32, n_bit=4, group_size=g)
        q, s, z = orc.rtn_quantize(w, 4, g)
        assert qw.dtype == torch.uint8 and tuple(qw.shape) == (32, 128)
        assert np.array_equal(qw.numpy(), orc.pack_l1(q))
        assert np.array_equal(zs.numpy().view(np.uint16), orc.zeros_scales_l1(z, s).view(np.uint16))
        # the fake-quantised weight equals the oracle's dequantisation of the packed tensors
        deq = qf.dequant_to_fp16(torch.from_numpy(w), 4, g).numpy()
        assert np.array_equal(deq.view(np.uint16), orc.dequant_l1(qw.numpy(), zs.numpy(), g).view(np.uint16))
    # an fp16 weight is quantised in fp16, like the reference does: bit-equal to the oracle's fp16 restatement,
    # and in fp32 on request
    wh = w.astype(np.float16)
    for g in (64, 128):
        qw, zs = qf.quant_muxi(torch.from_numpy(wh), 256, 32, n_bit=4, group_size=g)
        q, s, z = orc.rtn_quantize(wh, 4, g, dtype=np.float16)
        assert np.array_equal(qw.numpy(), orc.pack_l1(q))
        assert np.array_equal(zs.numpy().view(np.uint16), orc.zeros_scales_l1(z, s).view(np.uint16))
        qw32, zs32 = qf.quant_muxi(torch.from_numpy(wh), 256, 32, n_bit=4, group_size=g, compute_dtype=torch.float32)
        q, s, z = orc.rtn_quantize(wh.astype(np.float32), 4, g)
        assert np.array_equal(qw32.numpy(), orc.pack_l1(q))
        assert np.array_equal(zs32.numpy().view(np.uint16), orc.zeros_scales_l1(z, s).view(np.uint16))
    # 2-bit packing, then expansion to 4-bit nibbles
    qw2, zs2 = qf.quant_muxi(torch.from_numpy(w), 256, 32, n_bit=2, group_size=64)
    q2, s2, z2 = orc.rtn_quantize(w, 2, 64)
    q2i = q2.reshape(32, 32, 4, 2).transpose(0, 1, 3, 2).reshape(32, 256)
    assert np.array_equal(qw2.numpy(), orc.pack_2bit_l1(q2i))
    assert np.array_equal(orc.convert_2bit_to_4bit_l1(qw2.numpy()), orc.pack_l1(q2))
