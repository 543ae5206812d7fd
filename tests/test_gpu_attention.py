"""GPU parity of the LUT block-sparse attention kernel (through the C ABI) against the
float64 dense-masked oracle.  Bar: max|out - ref| <= 1e-2 * max|ref| (fp16 in/out, fp16
probabilities into the matrix core, fp32 softmax state), same bar as the linear path."""
import numpy as np
import pytest
import torch

import lut_attention_oracle as att

pytestmark = pytest.mark.gpu
TOL = 1e-2


@pytest.fixture(scope="module")
def capi(built_lib):
    from sqamd import capi as c
    c.lib()
    return c


def run_case(capi, z, h, s, d, density, causal, seed=0, lut_dtype=torch.int64, scale=None):
    rng = np.random.default_rng(seed)
    q = rng.normal(size=(z, h, s, d)).astype(np.float16)
    k = rng.normal(size=(z, h, s, d)).astype(np.float16)
    v = rng.normal(size=(z, h, s, d)).astype(np.float16)
    nb = (s + 63) // 64
    lut = att.layout_to_lut(att.synth_layout(h, nb, density, causal, seed=seed + 1))
    scale = scale if scale is not None else 1.0 / np.sqrt(d)
    ref = att.attention_ref(q, k, v, lut, scale, causal)
    out = capi.lut_attention(torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(),
                             torch.from_numpy(lut).to(lut_dtype).cuda(), scale, causal)
    torch.cuda.synchronize()
    out = out.float().cpu().numpy().astype(np.float64)
    assert np.all(np.isfinite(out))
    err = np.max(np.abs(out - ref))
    assert err <= TOL * np.max(np.abs(ref)), "z=%d h=%d s=%d d=%d causal=%s: err %.3e" % (z, h, s, d, causal, err)
    return out, ref


@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("s,density", [(64, 1.0), (128, 0.5), (512, 0.25), (200, 0.5), (1000, 0.3)])
def test_attention_parity(capi, d, causal, s, density):
    run_case(capi, 2, 3, s, d, density, causal, seed=s + d)


def test_attention_bert_large_shape(capi):
    # batch 8 x 16 heads x 512 x 64, ~25 % density, non-causal (the benchmark's BERT-large configuration)
    run_case(capi, 8, 16, 512, 64, 0.25, False, seed=5)


def test_attention_long_sequence_causal_int32_lut(capi):
    run_case(capi, 1, 4, 4096, 128, 0.26, True, seed=6, lut_dtype=torch.int32)


def test_attention_properties(capi):
    z, h, s, d = 1, 2, 256, 64
    rng = np.random.default_rng(9)
    q = torch.from_numpy(rng.normal(size=(z, h, s, d)).astype(np.float16)).cuda()
    k = torch.from_numpy(rng.normal(size=(z, h, s, d)).astype(np.float16)).cuda()
    lay = att.synth_layout(h, 4, 0.5, True, seed=2)
    lut = torch.from_numpy(att.layout_to_lut(lay)).cuda()
    # constant V comes back unchanged (softmax weights sum to one)
    vc = torch.arange(d, dtype=torch.float16).repeat(z, h, s, 1).cuda()
    out = capi.lut_attention(q, k, vc, lut, 0.125, True)
    assert torch.allclose(out.float(), vc.float(), atol=0.05)
    # causal: query 0 sees only key 0 -> returns that V row exactly
    v = torch.from_numpy(rng.normal(size=(z, h, s, d)).astype(np.float16)).cuda()
    out = capi.lut_attention(q, k, v, lut, 0.125, True)
    assert torch.equal(out[:, :, 0], v[:, :, 0])
    # a LUT padded with repeated entries, and one with more columns than blocks, give the same result
    lut_np = att.layout_to_lut(lay)
    padded = np.concatenate([lut_np, np.repeat(lut_np[:, :, -1:], 3, axis=2)], axis=2)
    out2 = capi.lut_attention(q, k, v, torch.from_numpy(padded).cuda(), 0.125, True)
    assert torch.equal(out, out2)
    # determinism
    assert torch.equal(out, capi.lut_attention(q, k, v, lut, 0.125, True))


def test_sparse_attention_module_api(capi):
    from sqamd.block_sparse_attention_lut import sparse_attention
    rng = np.random.default_rng(11)
    z, h, s, d = 2, 4, 192, 128
    q = torch.from_numpy(rng.normal(size=(z, h, s, d)).astype(np.float16)).cuda()
    k = torch.from_numpy(rng.normal(size=(z, h, s, d)).astype(np.float16)).cuda()
    v = torch.from_numpy(rng.normal(size=(z, h, s, d)).astype(np.float16)).cuda()
    lut = torch.from_numpy(att.layout_to_lut(att.synth_layout(h, 3, 0.7, True, seed=4))).cuda()
    out = sparse_attention(q, k, v, d ** -0.5, lut, True, 64, 64)
    ref = att.attention_ref(q.cpu().numpy(), k.cpu().numpy(), v.cpu().numpy(), lut.cpu().numpy(), d ** -0.5, True)
    assert np.max(np.abs(out.float().cpu().numpy() - ref)) <= TOL * np.max(np.abs(ref))
    # decode step: one query against the whole cache is dense, as in the reference
    q1 = q[:, :, -1:, :]
    o1 = sparse_attention(q1, k, v, d ** -0.5, lut, True, 64, 64)
    w = torch.softmax((q1.float() @ k.float().transpose(2, 3)) * d ** -0.5, dim=-1)
    assert torch.allclose(o1.float(), w @ v.float(), atol=2e-2, rtol=2e-2)
    with pytest.raises(ValueError):
        sparse_attention(q, k, v, 1.0, lut, True, 32, 64)


def test_attention_argument_errors(capi):
    L = capi.lib()
    import ctypes
    p = ctypes.c_void_p(4096)
    assert L.sq_lut_attention_fwd(p, p, p, p, p, 8, 1, 1, 64, 96, 1, 1.0, 0, None) == capi.SQ_ERR_BAD_SHAPE   # D
    assert L.sq_lut_attention_fwd(p, p, p, p, p, 2, 1, 1, 64, 64, 1, 1.0, 0, None) == capi.SQ_ERR_BAD_LAYOUT  # lut width
    assert L.sq_lut_attention_fwd(p, p, None, p, p, 8, 1, 1, 64, 64, 1, 1.0, 0, None) == capi.SQ_ERR_NULL_POINTER
    assert L.sq_lut_attention_fwd(p, p, p, p, p, 8, 1, 1, 0, 64, 1, 1.0, 0, None) == capi.SQ_ERR_BAD_SHAPE


@pytest.mark.parametrize("d", [64, 128])
def test_block_named_again_after_a_different_one_is_attended_twice(capi, d):
    """Only an entry equal to its predecessor is padding: rows such as [1, 3, 1, 0] visit block 1 twice
    (its keys carry double weight), [2, 2, 0, 0] visits 2 and 0 once each, entries beyond the sequence
    select nothing -- the oracle weighs every key block by its number of visits."""
    rng = np.random.default_rng(31)
    z, h, s = 2, 2, 250
    q = rng.normal(size=(z, h, s, d)).astype(np.float16)
    k = rng.normal(size=(z, h, s, d)).astype(np.float16)
    v = rng.normal(size=(z, h, s, d)).astype(np.float16)
    lut = np.array([[[0, 1, 0, 1], [1, 3, 1, 0], [2, 2, 0, 0], [3, 0, 3, 0]],
                    [[2, 0, 2, 2], [1, 1, 1, 1], [0, 9, 0, 2], [3, 2, 1, 0]]], dtype=np.int64)
    assert att.lut_to_counts(lut, 4).max() == 2
    ref = att.attention_ref(q, k, v, lut, 0.11, False)
    out = capi.lut_attention(torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(),
                             torch.from_numpy(lut).cuda(), 0.11, False)
    torch.cuda.synchronize()
    out = out.float().cpu().numpy().astype(np.float64)
    assert np.max(np.abs(out - ref)) <= TOL * np.max(np.abs(ref))


def test_query_rows_without_a_visible_key_are_nan(capi):
    # causal, query block 0 of head 0 is pointed at key block 1 only: nothing is visible -> NaN, like the
    # reference's running sums; every other row is unaffected
    rng = np.random.default_rng(32)
    z, h, s, d = 1, 2, 128, 64
    q = rng.normal(size=(z, h, s, d)).astype(np.float16)
    lut = np.array([[[1], [1]], [[0], [1]]], dtype=np.int64)
    with np.errstate(invalid="ignore"):
        ref = att.attention_ref(q, q, q, lut, 0.125, True)
    qt = torch.from_numpy(q).cuda()
    out = capi.lut_attention(qt, qt, qt, torch.from_numpy(lut).cuda(), 0.125, True).float().cpu().numpy()
    assert np.all(np.isnan(out[0, 0, :64])) and np.all(np.isnan(ref[0, 0, :64]))
    ok = np.isfinite(ref)
    assert np.array_equal(ok, np.isfinite(out))
    assert np.max(np.abs(out[ok] - ref[ok])) <= TOL * np.max(np.abs(ref[ok]))
