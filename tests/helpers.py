"""Shared builders for the parity tests: seeded inputs in the three tile
dtypes, the oracle's answer on the same (rounded) values, and the error
metric."""
import numpy as np
import torch

from nntile_amd import synth

TOL = {"fp32": 1e-4, "bf16": 1e-2, "fp16": 1e-3}   # tests/kernel/flash_sdpa_fwd_cudnn.cc:286-301
TORCH_DT = {"fp32": torch.float32, "bf16": torch.bfloat16, "fp16": torch.float16}


def rounded(x, dtype):
    """fp32 array -> (torch CPU tensor in the tile dtype, the same values as fp32)."""
    t = torch.from_numpy(np.ascontiguousarray(x, np.float32)).to(TORCH_DT[dtype])
    return t, t.float().numpy()


def make_qkv(seed, batch, q_seq, k_seq, head, dtype, kv_batch=None, scale=1.0):
    kv_batch = batch if kv_batch is None else kv_batch
    q = scale * synth.randn(seed, 0, batch * q_seq * head).reshape(batch, q_seq, head)
    k = scale * synth.randn(seed, 1, kv_batch * k_seq * head).reshape(kv_batch, k_seq, head)
    v = scale * synth.randn(seed, 2, kv_batch * k_seq * head).reshape(kv_batch, k_seq, head)
    (Q, qf), (K, kf), (V, vf) = rounded(q, dtype), rounded(k, dtype), rounded(v, dtype)
    return (Q, K, V), (qf, kf, vf)


def additive_mask(mask_bool, dtype):
    m = np.where(mask_bool, 0.0, -np.inf).astype(np.float32)
    return torch.from_numpy(m).to(TORCH_DT[dtype])


def fresh_outputs(batch, q_seq, head, dtype, device="cuda", poison=True):
    """lse = -inf; A poisoned with NaN: rows with lse = -inf must not be read."""
    lse = torch.full((batch, q_seq), float("-inf"), dtype=torch.float32, device=device)
    fill = float("nan") if poison else 0.0
    A = torch.full((batch, q_seq, head), fill, dtype=TORCH_DT[dtype], device=device)
    return lse, A


def to_np(t):
    return t.detach().float().cpu().numpy()


def rel_fro(a, b):
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    inf_a, inf_b = np.isneginf(a), np.isneginf(b)
    assert np.array_equal(inf_a, inf_b), "-inf pattern differs"
    a, b = a[~inf_a], b[~inf_b]
    assert np.all(np.isfinite(a)), "non-finite values in the result"
    denom = np.linalg.norm(b)
    return float(np.linalg.norm(a - b) / (denom if denom > 0 else 1.0))


# Per-row bounds beside the whole-tensor metric: one wrong query row out of
# 131072 moves the relative Frobenius error of a full-size output by 3e-3 and
# would pass the tolerance above.  A row's own relative error is looser than
# the tensor's: the rounding of the probabilities to the tile type does not
# average out over a row whose softmax sits on a few keys (worst rows seen on
# the benchmark shapes: 8e-3 for bf16).  The logsumexp is accumulated in fp32
# from unrounded terms in every kernel and gets a tight bound, relative to
# max(1, |logsumexp|).
ROW_TOL = {"fp32": 1e-4, "bf16": 2.5e-2, "fp16": 3e-3}
LSE_TOL = {"fp32": 1e-5, "bf16": 1e-4, "fp16": 1e-4}


def row_errors(a, b, lse_a, lse_b):
    """(largest relative error of a query row of the output, largest
    difference of a logsumexp value relative to max(1, |value|)); rows whose
    logsumexp is -inf in the reference must be -inf in the result and are
    left out."""
    a = np.asarray(a, np.float64).reshape(-1, np.shape(a)[-1])
    b = np.asarray(b, np.float64).reshape(-1, np.shape(b)[-1])
    la = np.asarray(lse_a, np.float64).ravel()
    lb = np.asarray(lse_b, np.float64).ravel()
    dead = np.isneginf(lb)
    assert np.array_equal(np.isneginf(la), dead), "-inf pattern of logsumexp differs"
    live = ~dead
    assert np.all(np.isfinite(a[live])) and np.all(np.isfinite(la[live])), "non-finite values"
    num = np.linalg.norm(a[live] - b[live], axis=1)
    den = np.maximum(np.linalg.norm(b[live], axis=1), 1e-30)
    dl = np.abs(la[live] - lb[live]) / np.maximum(1.0, np.abs(lb[live]))
    return float((num / den).max(initial=0.0)), float(dl.max(initial=0.0))


def check_rows(a, b, lse_a, lse_b, dtype, what=""):
    row, lse = row_errors(a, b, lse_a, lse_b)
    print("row check %s: worst row %.3e (bound %.0e), worst logsumexp %.3e (bound %.0e)"
          % (what, row, ROW_TOL[dtype], lse, LSE_TOL[dtype]), flush=True)
    assert row < ROW_TOL[dtype], "a query row is off by %.3e" % row
    assert lse < LSE_TOL[dtype], "a logsumexp value is off by %.3e" % lse
