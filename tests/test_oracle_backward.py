"""Pins of the backward checker (CPU only).  Neither restatement is trusted
because it was typed in: both are compared with finite differences of the
forward checker, with each other, and with torch's autograd on CPU (a second
opinion that is not the reference), on shapes small enough for fp64 brute
force; a dropped term, a wrong sign or a transposed operand fails them."""
import numpy as np
import pytest
import torch

from nntile_amd import synth


def _data(seed, batch, q_seq, k_seq, head, scale=1.0):
    rng = np.random.default_rng(seed)
    mk = lambda *s: (scale * rng.standard_normal(s)).astype(np.float32)
    return mk(batch, k_seq, head), mk(batch, q_seq, head), mk(batch, k_seq, head), mk(batch, q_seq, head)


def _forward64(oracle, K, Q, V, add):
    A, lse = oracle.sdpa_bruteforce_f64(K, Q, V, add)
    return A, lse


@pytest.mark.parametrize("causal", [False, True])
def test_flash_form_matches_finite_differences(oracle, causal):
    batch, q_seq, k_seq, head = 2, 5, 7, 4
    K, Q, V, G = _data(1, batch, q_seq, k_seq, head)
    mask = synth.causal_mask(q_seq, k_seq, k_seq - q_seq) if causal else np.ones((q_seq, k_seq), bool)
    add = np.where(mask, 0, -np.inf).astype(np.float32)
    A, lse = _forward64(oracle, K, Q, V, add)
    dK, dQ, dV = oracle.sdpa_bwd_flash_f64(K, Q, V, A, G, lse, add)

    def loss(Kx, Qx, Vx):
        # the forward brute force takes fp32 inputs: difference quotients of
        # it with steps that fp32 represents exactly enough
        Ax, _ = oracle.sdpa_bruteforce_f64(Kx, Qx, Vx, add)
        return float((Ax * G).sum())

    eps = 2.0 ** -7
    for name, X, dX in (("K", K, dK), ("Q", Q, dQ), ("V", V, dV)):
        rng = np.random.default_rng(7)
        for _ in range(12):
            idx = tuple(int(rng.integers(0, n)) for n in X.shape)
            Xp, Xm = X.copy(), X.copy()
            Xp[idx] = np.float32(X[idx] + eps)
            Xm[idx] = np.float32(X[idx] - eps)
            step = float(Xp[idx]) - float(Xm[idx])
            args_p = {"K": (Xp, Q, V), "Q": (K, Xp, V), "V": (K, Q, Xp)}[name]
            args_m = {"K": (Xm, Q, V), "Q": (K, Xm, V), "V": (K, Q, Xm)}[name]
            fd = (loss(*args_p) - loss(*args_m)) / step
            assert abs(fd - dX[idx]) < 2e-3 * max(1.0, abs(dX[idx])), (name, idx, fd, dX[idx])


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(2, 16, 16, 8), (3, 9, 33, 16), (1, 40, 24, 64)])
def test_flash_form_matches_torch_autograd(oracle, shape, causal):
    batch, q_seq, k_seq, head = shape
    K, Q, V, G = _data(2, batch, q_seq, k_seq, head)
    mask = synth.causal_mask(q_seq, k_seq, max(k_seq - q_seq, 0)) if causal \
        else np.ones((q_seq, k_seq), bool)
    add = np.where(mask, 0, -np.inf).astype(np.float32)
    A, lse = _forward64(oracle, K, Q, V, add)
    dK, dQ, dV = oracle.sdpa_bwd_flash_f64(K, Q, V, A, G, lse, add)
    tq, tk, tv = (torch.tensor(x, dtype=torch.float64, requires_grad=True) for x in (Q, K, V))
    out = torch.nn.functional.scaled_dot_product_attention(
        tq, tk, tv, attn_mask=torch.tensor(mask))
    out.backward(torch.tensor(G, dtype=torch.float64))
    for got, want in ((dQ, tq.grad), (dK, tk.grad), (dV, tv.grad)):
        assert np.allclose(got, want.numpy(), rtol=1e-9, atol=1e-10)


@pytest.mark.parametrize("causal", [False, True])
def test_vanilla_composition_matches_flash_form(oracle, causal):
    batch, q_seq, k_seq, head = 3, 24, 24, 16
    K, Q, V, G = _data(3, batch, q_seq, k_seq, head)
    mask = synth.causal_mask(q_seq, k_seq) if causal else None
    add = None if mask is None else np.where(mask, 0, -np.inf).astype(np.float32)
    A, lse = _forward64(oracle, K, Q, V, add)
    want = oracle.sdpa_bwd_flash_f64(K, Q, V, A, G, lse, add)
    got = oracle.sdpa_bwd_vanilla(K, Q, V, G, mask)
    for g, w in zip(got, want):
        assert np.linalg.norm(g - w) <= 1e-5 * np.linalg.norm(w)


def test_flash_form_takes_a_and_lse_as_given(oracle):
    """A and lse are inputs, not recomputed (tests/kernel/flash_sdpa_bwd_cudnn.cc
    feeds values that do not belong to K, Q, V): doubling exp(-lse) doubles P."""
    batch, q_seq, k_seq, head = 1, 6, 6, 8
    K, Q, V, G = _data(4, batch, q_seq, k_seq, head)
    A = np.zeros((batch, q_seq, head))          # D = 0: dS = P dP
    lse = np.zeros((batch, q_seq))
    dK0, dQ0, dV0 = oracle.sdpa_bwd_flash_f64(K, Q, V, A, G, lse)
    dK1, dQ1, dV1 = oracle.sdpa_bwd_flash_f64(K, Q, V, A, G, lse - np.log(2.0))
    for a, b in ((dK0, dK1), (dQ0, dQ1), (dV0, dV1)):
        assert np.allclose(2 * a, b, rtol=1e-12)


def test_flash_form_grouped_queries(oracle):
    n_batch, group, n_kv, q_seq, k_seq, head = 2, 3, 2, 5, 9, 8
    batch = n_batch * group * n_kv
    rng = np.random.default_rng(5)
    Q = rng.standard_normal((batch, q_seq, head)).astype(np.float32)
    G = rng.standard_normal((batch, q_seq, head)).astype(np.float32)
    K = rng.standard_normal((n_batch * n_kv, k_seq, head)).astype(np.float32)
    V = rng.standard_normal((n_batch * n_kv, k_seq, head)).astype(np.float32)
    # repeat K/V per query batch entry and compare with the grouped call
    kv_of = [(b % n_batch) + n_batch * ((b // n_batch) // group) for b in range(batch)]
    Kr, Vr = K[kv_of], V[kv_of]
    A, lse = oracle.sdpa_bruteforce_f64(Kr, Q, Vr, None)
    dKr, dQr, dVr = oracle.sdpa_bwd_flash_f64(Kr, Q, Vr, A, G, lse)
    dK, dQ, dV = oracle.sdpa_bwd_flash_f64(K, Q, V, A, G, lse, kv_repeat=group, n_batch=n_batch)
    assert np.allclose(dQ, dQr)
    for kv in range(n_batch * n_kv):
        sel = [b for b in range(batch) if kv_of[b] == kv]
        assert np.allclose(dK[kv], dKr[sel].sum(axis=0))
        assert np.allclose(dV[kv], dVr[sel].sum(axis=0))
