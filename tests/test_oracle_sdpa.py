"""Pins for the CPU checker's attention composition
(gemm -> mask_scalar -> maxsumexp -> softmax_inplace -> gemm, + logsumexp)."""
import numpy as np
import pytest
import torch

from nntile_amd import synth
from .conftest import rel_fro


def _preset(seq, head, batch):
    # tests/kernel/flash_sdpa_fwd_cudnn.cc:211-219 (reference kernel test data)
    i = np.arange(batch * seq * head)
    k = ((i % 20 - 10) * 0.1).astype(np.float32).reshape(batch, seq, head)
    return k, (k * np.float32(0.8)), (k * np.float32(1.2))


def _uniform(seq, head, batch, seed=42):
    rng = np.random.default_rng(seed)
    return tuple(rng.uniform(-0.5, 0.5, (batch, seq, head)).astype(np.float32)
                 for _ in range(3))


def _additive(mask_bool):
    return np.where(mask_bool, 0.0, -np.inf).astype(np.float32)


@pytest.mark.parametrize("seq,head,batch", [(32, 32, 1), (64, 64, 2), (128, 64, 3), (96, 128, 2)])
@pytest.mark.parametrize("data", ["preset", "uniform"])
@pytest.mark.parametrize("causal", [True, False])
def test_vanilla_matches_fp64_bruteforce(oracle, seq, head, batch, data, causal):
    # shapes/cases of tests/kernel/flash_sdpa_fwd_cudnn.cc:565-588, tolerance fp32 1e-4 (:296)
    K, Q, V = _preset(seq, head, batch) if data == "preset" else _uniform(seq, head, batch)
    mask = synth.causal_mask(seq, seq) if causal else np.ones((seq, seq), bool)
    Y, lse = oracle.sdpa_vanilla(K, Q, V, mask)
    A64, lse64 = oracle.sdpa_bruteforce_f64(K, Q, V, _additive(mask))
    assert rel_fro(Y, A64) < 1e-5
    assert rel_fro(lse, lse64) < 1e-5


def test_bruteforce_and_vanilla_match_torch_sdpa(oracle):
    # independent second opinion: textbook SDPA (wrappers/python/tests/layer/test_sdpa.py:167-189)
    K, Q, V = _uniform(80, 64, 4, seed=3)
    mask = synth.causal_mask(80, 80)
    want = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(Q).double(), torch.from_numpy(K).double(), torch.from_numpy(V).double(),
        attn_mask=torch.from_numpy(mask)).numpy()
    s = np.einsum("bqh,bkh->bqk", Q.astype(np.float64), K.astype(np.float64)) / 8.0
    s = np.where(mask[None], s, -np.inf)
    want_lse = torch.logsumexp(torch.from_numpy(s), dim=-1).numpy()
    A64, lse64 = oracle.sdpa_bruteforce_f64(K, Q, V, _additive(mask))
    assert rel_fro(A64, want) < 1e-12 and rel_fro(lse64, want_lse) < 1e-12
    Y, lse = oracle.sdpa_vanilla(K, Q, V, mask)
    assert rel_fro(Y, want) < 1e-5 and rel_fro(lse, want_lse) < 1e-5


def test_identical_keys_give_mean_of_values(oracle):
    # no mask + identical K rows => uniform softmax => O = mean(V), lse = s + log(n)
    rng = np.random.default_rng(0)
    seq, head = 48, 32
    K = np.tile(rng.standard_normal((1, 1, head)).astype(np.float32), (1, seq, 1))
    Q = rng.standard_normal((1, seq, head)).astype(np.float32)
    V = rng.standard_normal((1, seq, head)).astype(np.float32)
    Y, lse = oracle.sdpa_vanilla(K, Q, V, None)
    assert np.allclose(Y, np.broadcast_to(V.mean(axis=1, keepdims=True), Y.shape), atol=1e-6)
    s = (Q[0] @ K[0, 0]) / np.sqrt(np.float32(head))
    assert np.allclose(lse[0], s + np.log(seq), rtol=1e-5, atol=1e-5)


def test_scale_is_applied_before_mask_and_value_of_scale(oracle):
    # scale = 1/sqrt(head) (layer/sdpa.py:149); with one visible key lse == scale*<q,k>
    rng = np.random.default_rng(2)
    head = 64
    K = rng.standard_normal((1, 4, head)).astype(np.float32)
    Q = rng.standard_normal((1, 4, head)).astype(np.float32)
    V = rng.standard_normal((1, 4, head)).astype(np.float32)
    mask = np.eye(4, dtype=bool)
    Y, lse = oracle.sdpa_vanilla(K, Q, V, mask)
    assert np.allclose(lse[0], np.einsum("qh,qh->q", Q[0], K[0]) / 8.0, rtol=1e-6)
    assert np.allclose(Y[0], V[0], rtol=1e-6)


def test_mask_orientation_key_by_query(oracle):
    # mask is [k_seq, q_seq] Fortran == [q_seq, k_seq] C: row = query.  A mask
    # that lets query 0 see every key and every other query only key 0
    # distinguishes the two orientations.
    rng = np.random.default_rng(4)
    K, Q, V = (rng.standard_normal((1, 6, 16)).astype(np.float32) for _ in range(3))
    mask = np.zeros((6, 6), bool)
    mask[0, :] = True
    mask[:, 0] = True
    Y, _ = oracle.sdpa_vanilla(K, Q, V, mask)
    assert np.allclose(Y[0, 1:], np.broadcast_to(V[0, 0], (5, 16)), atol=1e-6)
    assert not np.allclose(Y[0, 0], V[0, 0], atol=1e-3)


def test_fully_masked_query_gives_zero_and_minus_inf(oracle):
    rng = np.random.default_rng(6)
    K, Q, V = (rng.standard_normal((2, 8, 16)).astype(np.float32) for _ in range(3))
    mask = synth.causal_mask(8, 8, offset=-1)      # query 0 sees nothing
    Y, lse = oracle.sdpa_vanilla(K, Q, V, mask)
    assert np.all(Y[:, 0] == 0.0) and np.all(np.isneginf(lse[:, 0]))
    assert np.all(np.isfinite(lse[:, 1:]))


@pytest.mark.parametrize("k_tile", [1, 7, 16, 64])
def test_key_tiling_does_not_change_result(oracle, k_tile):
    # tensor-level accumulation over key tiles (src/tensor/maxsumexp.cc:80-107,
    # src/tensor/gemm.cc:378-408) == single tile; mirrors tests/tensor/flash_sdpa_fwd_cudnn.cc
    K, Q, V = _uniform(64, 32, 3, seed=9)
    mask = np.abs(np.arange(64)[:, None] - np.arange(64)[None, :]) <= 32   # tests/tile/...:57-86 window
    one, lse_one = oracle.sdpa_vanilla(K, Q, V, mask)
    many, lse_many = oracle.sdpa_vanilla(K, Q, V, mask, k_tile=k_tile)
    assert rel_fro(many, one) < 2e-6 and rel_fro(lse_many, lse_one) < 2e-6


def test_gqa_repeat_equals_explicit_repeat(oracle):
    # model/llama_attention.py:579-580 repeats K/V along kv_group; layout
    # [head, seq, n_batch, kv_group, n_head_kv]
    rng = np.random.default_rng(11)
    head, q_seq, k_seq, n_batch, group, n_kv = 16, 5, 23, 3, 4, 2
    Q = rng.standard_normal((n_kv, group, n_batch, q_seq, head)).astype(np.float32)
    K = rng.standard_normal((n_kv, n_batch, k_seq, head)).astype(np.float32)
    V = rng.standard_normal((n_kv, n_batch, k_seq, head)).astype(np.float32)
    mask = synth.causal_mask(q_seq, k_seq, offset=k_seq - q_seq)     # layer/sdpa.py:516-531
    Krep = np.repeat(K[:, None], group, axis=1).reshape(-1, k_seq, head)
    Vrep = np.repeat(V[:, None], group, axis=1).reshape(-1, k_seq, head)
    want, want_lse = oracle.sdpa_vanilla(Krep, Q.reshape(-1, q_seq, head), Vrep, mask)
    got, got_lse = oracle.sdpa_vanilla(K.reshape(-1, k_seq, head), Q.reshape(-1, q_seq, head),
                                       V.reshape(-1, k_seq, head), mask,
                                       n_batch=n_batch, kv_repeat=group)
    assert np.array_equal(got, want) and np.array_equal(got_lse, want_lse)
    A64, lse64 = oracle.sdpa_bruteforce_f64(Krep, Q.reshape(-1, q_seq, head), Vrep, _additive(mask))
    assert rel_fro(got, A64) < 1e-5 and rel_fro(got_lse, lse64) < 1e-5


def test_merge_of_key_splits_equals_unsplit(oracle):
    # the flash path's hand-off: per-key-tile partial (lse, O) merged with
    # accumulate_attn_output == attention over all keys
    K, Q, V = _uniform(96, 32, 2, seed=13)
    mask = synth.causal_mask(96, 96)
    want, want_lse = oracle.sdpa_vanilla(K, Q, V, mask)
    run = np.zeros_like(want)
    run_lse = np.full(want_lse.shape, -np.inf, np.float32)
    for lo in range(0, 96, 32):
        part, part_lse = oracle.sdpa_vanilla(K[:, lo:lo + 32], Q, V[:, lo:lo + 32],
                                             mask[:, lo:lo + 32])
        oracle.accumulate_attn_output("fp32", 32, 96, 2, part_lse, part, run_lse, run)
    assert rel_fro(run, want) < 1e-6 and rel_fro(run_lse, want_lse) < 1e-6
