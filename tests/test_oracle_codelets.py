"""Pins for the CPU checker's codelet-level functions.

Each check is chosen so that a plausible slip in the restatement (a dropped
term, a transposed operand, a wrong stride) fails it: closed forms and data
formulas taken from the reference's own kernel tests, invariants of the
mathematics, and brute force in fp64 on small inputs.
"""
import numpy as np
import pytest
import torch

from .conftest import rel_fro


# ---- gemm: src/kernel/cblas.cc:28-121 ---------------------------------------

@pytest.mark.parametrize("ta,tb", [(0, 0), (1, 0), (0, 1), (1, 1)])
@pytest.mark.parametrize("m,n,k,batch", [(1, 1, 1, 1), (7, 5, 3, 2),
                                         (13, 11, 64, 3), (64, 19, 37, 2),
                                         (33, 14, 128, 1)])
@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (0.125, 1.0), (-2.0, 0.5)])
def test_gemm_matches_einsum(oracle, ta, tb, m, n, k, batch, alpha, beta):
    rng = np.random.default_rng(42)
    # column-major op(A) is m-by-k: stored as [batch, k, m] (C order) when not
    # transposed (element (i,l) at i + l*m), [batch, m, k] when transposed.
    A = rng.standard_normal((batch, m, k) if ta else (batch, k, m)).astype(np.float32)
    B = rng.standard_normal((batch, k, n) if tb else (batch, n, k)).astype(np.float32)
    C = rng.standard_normal((batch, n, m)).astype(np.float32)
    opA = A if ta else A.transpose(0, 2, 1)       # -> [batch, m, k]
    opB = B if tb else B.transpose(0, 2, 1)       # -> [batch, k, n]
    want = alpha * np.einsum("bik,bkj->bji", opA.astype(np.float64),
                             opB.astype(np.float64)) + beta * C
    got = C.copy()
    oracle.gemm(ta, tb, m, n, k, batch, alpha, A, B, beta, got)
    assert rel_fro(got, want) < 1e-5


def test_gemm_beta_zero_overwrites_nan(oracle):
    A = np.ones((1, 4, 3), np.float32)
    B = np.ones((1, 2, 4), np.float32)
    C = np.full((1, 2, 3), np.nan, np.float32)
    oracle.gemm(0, 0, 3, 2, 4, 1, 1.0, A, B, 0.0, C)
    assert np.array_equal(C, np.full((1, 2, 3), 4.0, np.float32))


def test_gemm_attention_shapes_match_layer_einsums(oracle):
    # tests/layer/test_sdpa.py:173,179 (reference python tests): the two GEMMs of the layer are
    # einsum("hsbn,htbn->stbn") for scores and ("hsbn,stbn->htbn") for values.
    rng = np.random.default_rng(1)
    head, kseq, qseq, batch = 16, 9, 7, 3
    K = rng.standard_normal((batch, kseq, head)).astype(np.float32)
    Q = rng.standard_normal((batch, qseq, head)).astype(np.float32)
    V = rng.standard_normal((batch, kseq, head)).astype(np.float32)
    S = np.zeros((batch, qseq, kseq), np.float32)
    oracle.gemm(1, 0, kseq, qseq, head, batch, 0.25, K, Q, 0.0, S)
    assert rel_fro(S, 0.25 * np.einsum("bsh,bth->bts", K, Q)) < 1e-6
    Y = np.zeros((batch, qseq, head), np.float32)
    oracle.gemm(0, 0, head, qseq, kseq, batch, 1.0, V, S, 0.0, Y)
    assert rel_fro(Y, np.einsum("bsh,bts->bth", V, S)) < 1e-6


# ---- mask_scalar: src/kernel/mask_scalar/cpu.cc:21-49 ----------------------

def test_mask_scalar_all_false_sets_everything(oracle):
    # tests/kernel/mask_scalar.cc:69-100
    nrows, ncols = 12, 5
    data = np.arange(nrows * ncols, dtype=np.float32)
    mask = np.zeros(nrows, np.uint8)
    oracle.mask_scalar(nrows, ncols, mask, -3.5, data)
    assert np.all(data == -3.5)


def test_mask_scalar_rows_across_all_columns(oracle):
    rng = np.random.default_rng(3)
    nrows, ncols = 37, 4
    data = rng.standard_normal((ncols, nrows)).astype(np.float32)
    mask = (rng.random(nrows) < 0.5)
    want = np.where(mask[None, :], data, -np.inf)
    got = data.copy()
    oracle.mask_scalar(nrows, ncols, mask.astype(np.uint8), -np.inf, got)
    assert np.array_equal(got, want.astype(np.float32))


# ---- maxsumexp: src/kernel/maxsumexp/cpu.cc:22-128 -------------------------

def _maxsumexp_ref64(m, n, k, src, init):
    """fp64 statement of tests/kernel/maxsumexp.cc:64-148."""
    src = np.asarray(src, np.float64).reshape(n, k, m)
    out = np.asarray(init, np.float64).reshape(n, m, 2).copy()
    for j in range(n):
        for i in range(m):
            f = src[j, :, i]
            vis = f[~np.isinf(f)]
            if vis.size == 0:
                continue
            mx = vis.max()
            sm = np.exp(vis - mx).sum()
            if out[j, i, 1] == 0.0:
                out[j, i] = (mx, sm)
            else:
                mo, so = out[j, i]
                top = max(mo, mx)
                out[j, i] = (top, so * np.exp(mo - top) + sm * np.exp(mx - top))
    return out.reshape(-1)


@pytest.mark.parametrize("m,n,k", [(1, 9, 10), (8, 9, 1), (8, 1, 10),
                                   (4, 7, 8), (1, 33, 257)])
def test_maxsumexp_preset_data_of_reference_test(oracle, m, n, k):
    # tests/kernel/maxsumexp.cc:176-189: src[i]=2i+1-size, init[i]=5*size-2i
    size, dsize = m * n * k, 2 * m * n
    src = (2 * np.arange(size) + 1 - size).astype(np.float32)
    init = (5 * dsize - 2 * np.arange(dsize)).astype(np.float32)
    got = init.copy()
    oracle.maxsumexp(m, n, k, src, got)
    want = _maxsumexp_ref64(m, n, k, src, init)
    # tolerance of the reference test for fp32: 3.1e-3 (:226); we are far inside
    assert rel_fro(got, want) < 1e-6


def test_maxsumexp_random_data_of_reference_test(oracle):
    # tests/kernel/maxsumexp.cc:191-200: uniform[0,1) from a seeded generator
    rng = np.random.default_rng(42)
    m, n, k = 3, 11, 129
    src = rng.random(m * n * k).astype(np.float32)
    init = rng.random(2 * m * n).astype(np.float32)
    got = init.copy()
    oracle.maxsumexp(m, n, k, src, got)
    assert rel_fro(got, _maxsumexp_ref64(m, n, k, src, init)) < 1e-6


def test_maxsumexp_equals_logsumexp_of_fibre(oracle):
    from scipy.special import logsumexp as sp_lse
    rng = np.random.default_rng(7)
    n, k = 50, 300
    src = (5 * rng.standard_normal((n, k))).astype(np.float32)
    stats = np.zeros(2 * n, np.float32)
    oracle.maxsumexp(1, n, k, src, stats)
    lse = np.empty(n, np.float32)
    oracle.logsumexp(n, stats, lse)
    assert np.allclose(lse, sp_lse(src.astype(np.float64), axis=1), rtol=1e-6)
    assert np.array_equal(stats[0::2], src.max(axis=1))


def test_maxsumexp_split_fibre_equals_whole(oracle):
    rng = np.random.default_rng(8)
    n, k = 17, 96
    src = (3 * rng.standard_normal((n, k))).astype(np.float32)
    whole = np.zeros(2 * n, np.float32)
    oracle.maxsumexp(1, n, k, src, whole)
    parts = np.zeros(2 * n, np.float32)
    for lo, hi in [(0, 32), (32, 33), (33, 96)]:
        oracle.maxsumexp(1, n, hi - lo, np.ascontiguousarray(src[:, lo:hi]), parts)
    assert np.array_equal(whole[0::2], parts[0::2])
    assert np.allclose(whole[1::2], parts[1::2], rtol=2e-6)
    # the same merge through accumulate_maxsumexp (src/kernel/accumulate_maxsumexp/cpu.cc:22-63)
    a = np.zeros(2 * n, np.float32)
    b = np.zeros(2 * n, np.float32)
    oracle.maxsumexp(1, n, 40, np.ascontiguousarray(src[:, :40]), a)
    oracle.maxsumexp(1, n, 56, np.ascontiguousarray(src[:, 40:]), b)
    oracle.accumulate_maxsumexp(n, a, b)
    assert np.array_equal(whole[0::2], b[0::2])
    assert np.allclose(whole[1::2], b[1::2], rtol=2e-6)


def test_maxsumexp_masked_entries(oracle):
    # -inf entries (from the mask) are skipped; a fully masked fibre writes nothing
    src = np.array([[0.5, -np.inf, 1.5, -np.inf],
                    [-np.inf, -np.inf, -np.inf, -np.inf],
                    [-np.inf, 2.0, -np.inf, 1.0]], np.float32)
    stats = np.zeros(6, np.float32)
    stats[2:4] = (7.0, 0.0)     # sum 0 == uninitialised: must stay as it is
    oracle.maxsumexp(1, 3, 4, src, stats)
    assert stats[0] == 1.5 and np.isclose(stats[1], 1 + np.exp(-1.0))
    assert stats[2] == 7.0 and stats[3] == 0.0
    assert stats[4] == 2.0 and np.isclose(stats[5], 1 + np.exp(-1.0))


# ---- softmax_inplace: src/kernel/softmax_inplace/cpu.cc:22-70 -------------

@pytest.mark.parametrize("m,n,k", [(1, 9, 10), (8, 9, 1), (8, 1, 10), (4, 7, 8)])
def test_softmax_inplace_closed_form_of_reference_test(oracle, m, n, k):
    # tests/kernel/softmax_inplace.cc:68-108
    i0, i1, i2 = np.meshgrid(np.arange(m), np.arange(n), np.arange(k), indexing="ij")
    dst = np.zeros(m * n * k, np.float32)
    dst[((i1 * k + i2) * m + i0).ravel()] = ((i0 + i1 + i2) / 100.0).ravel()
    stats = np.zeros(2 * m * n, np.float32)
    j0, j1 = np.meshgrid(np.arange(m), np.arange(n), indexing="ij")
    stats[(2 * (j1 * m + j0)).ravel()] = ((j0 + j1 + k - 1) / 100.0).ravel()
    stats[(2 * (j1 * m + j0) + 1).ravel()] = ((j0 + j1 + 1) / 100.0).ravel()
    oracle.softmax_inplace(m, n, k, stats, 1.0, dst)
    want = np.exp((i2 - k + 1) / 100.0) * 100.0 / (i0 + i1 + 1)
    got = dst[((i1 * k + i2) * m + i0).ravel()].reshape(want.shape)
    assert np.all(np.abs(got - want) / want < 100 * np.finfo(np.float32).eps)


def test_softmax_inplace_inf_to_zero_and_alpha(oracle):
    dst = np.array([0.0, -np.inf, 1.0], np.float32)
    stats = np.array([1.0, 2.0], np.float32)
    oracle.softmax_inplace(1, 1, 3, stats, 3.0, dst)
    assert dst[1] == 0.0
    assert np.allclose(dst[[0, 2]], [3 * np.exp(-1.0) / 2, 1.5])


# ---- accumulate_attn_output: src/kernel/accumulate_attn_output/cpu.cc:38-115

def _preset_accumulate(head, seq, batch):
    # tests/kernel/accumulate_attn_output.cc:98-128
    lin = np.arange(seq * batch)
    base = -3.0 + 0.25 * (lin % 17)
    d_on = ((lin + 1) % 3) != 0
    s_on = ((lin + 2) % 4) != 0
    dst_lse = np.where(d_on, base, -np.inf).astype(np.float32)
    src_lse = np.where(s_on, base + 0.5, -np.inf).astype(np.float32)
    h = np.arange(head)[None, :]
    dst = np.where(d_on[:, None], 0.1 * ((lin[:, None] + h) % 11) - 1.0, 0.0)
    src = np.where(s_on[:, None], 0.2 * ((lin[:, None] + h + 3) % 13) - 0.5, 0.0)
    return src_lse, src.astype(np.float32), dst_lse, dst.astype(np.float32)


def _accumulate_ref64(src_lse, src, dst_lse, dst):
    sl, dl = src_lse.astype(np.float64), dst_lse.astype(np.float64)
    new = np.logaddexp(sl, dl)
    with np.errstate(invalid="ignore"):
        wd = np.where(np.isneginf(dl), 0.0, np.exp(dl - new))
        ws = np.where(np.isneginf(sl), 0.0, np.exp(sl - new))
    out = wd[:, None] * dst.astype(np.float64) + ws[:, None] * src.astype(np.float64)
    return new, out


@pytest.mark.parametrize("head,seq,batch", [(8, 5, 3), (64, 33, 2), (128, 7, 4), (5, 9, 1)])
def test_accumulate_attn_output_preset_fp32(oracle, head, seq, batch):
    src_lse, src, dst_lse, dst = _preset_accumulate(head, seq, batch)
    want_lse, want = _accumulate_ref64(src_lse, src, dst_lse, dst)
    oracle.accumulate_attn_output("fp32", head, seq, batch, src_lse, src, dst_lse, dst)
    fin = np.isfinite(want_lse)
    assert np.array_equal(np.isneginf(dst_lse), ~fin)
    assert np.max(np.abs(dst_lse[fin] - want_lse[fin])) < 1e-5     # :176-184
    assert np.max(np.abs(dst - want)) < 1e-5


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
def test_accumulate_attn_output_preset_16bit(oracle, dtype):
    head, seq, batch = 64, 19, 3
    src_lse, src, dst_lse, dst = _preset_accumulate(head, seq, batch)
    to16 = oracle.f32_to_bf16 if dtype == "bf16" else oracle.f32_to_fp16
    to32 = oracle.bf16_to_f32 if dtype == "bf16" else oracle.fp16_to_f32
    s16, d16 = to16(src), to16(dst)
    want_lse, want = _accumulate_ref64(src_lse, to32(s16), dst_lse, to32(d16))
    oracle.accumulate_attn_output(dtype, head, seq, batch, src_lse, s16, dst_lse, d16)
    assert np.max(np.abs(to32(d16) - want)) < 5e-3 * max(1.0, np.abs(want).max())


def test_accumulate_attn_output_identity_and_untouched_rows(oracle):
    head, n = 4, 3
    dst_lse = np.array([-np.inf, 0.3, -np.inf], np.float32)
    dst = np.arange(12, dtype=np.float32).reshape(3, 4)
    src_lse = np.array([-np.inf, -np.inf, 1.0], np.float32)
    src = 100 + np.arange(12, dtype=np.float32).reshape(3, 4)
    keep = dst.copy()
    oracle.accumulate_attn_output("fp32", head, n, 1, src_lse, src, dst_lse, dst)
    assert np.array_equal(dst[0], keep[0])          # both sides empty: untouched
    assert np.array_equal(dst[1], keep[1]) and dst_lse[1] == np.float32(0.3)
    assert np.array_equal(dst[2], src[2]) and dst_lse[2] == 1.0   # empty dst: takes src


# ---- 16-bit storage: include/nntile/base_types.hh:506-581 ------------------

def test_bf16_round_to_nearest_even_matches_torch(oracle):
    rng = np.random.default_rng(5)
    x = np.concatenate([rng.standard_normal(10000).astype(np.float32) * 100,
                        np.array([0.0, -0.0, np.inf, -np.inf, 1.00390625, 1.01171875],
                                 np.float32)])
    got = oracle.bf16_to_f32(oracle.f32_to_bf16(x))
    want = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
    assert np.array_equal(got, want)
    got = oracle.fp16_to_f32(oracle.f32_to_fp16(x))
    want = torch.from_numpy(x).to(torch.float16).float().numpy()
    assert np.array_equal(got, want)
