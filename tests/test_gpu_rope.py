"""GPU parity of the rotary embedding kernels against the CPU checker,
through the C ABI.  Tolerance: the reference's own acceptance interval
(tests/kernel/rope.cc:57,95-137): every value within ref (1 +- eps) +- eps with
eps = 2 x the type's epsilon (fp32 2^-23, fp16 2^-10, bf16 2^-7)."""
import numpy as np
import pytest
import torch

from nntile_amd import hip_sdpa, synth
from . import helpers as H
from .test_oracle_rope import reference_case, within_reference_interval

pytestmark = pytest.mark.gpu

EPS = {"fp32": 2.0 ** -23, "fp16": 2.0 ** -10, "bf16": 2.0 ** -7}


def _tile(x, dtype):
    t, f = H.rounded(x, dtype)
    return t.cuda(), f


def _run(sin, cos, src, dtype, backward=False, inplace=False):
    S, sf = _tile(sin, dtype)
    C, cf = _tile(cos, dtype)
    X, xf = _tile(src, dtype)
    D = X if inplace else torch.full_like(X, float("nan"))
    hip_sdpa.rope(S, C, X, D, backward=backward)
    torch.cuda.synchronize()
    return H.to_np(D), sf, cf, xf


@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("m,n", [(0, 5), (1, 10), (10, 100)])
def test_reference_kernel_test_cases(oracle, dtype, m, n):
    print("case rope reference", dtype, m, n, flush=True)
    sin, cos, src = reference_case(m, n)
    got, sf, cf, xf = _run(sin, cos, src, dtype)
    if m == 0:
        return
    assert within_reference_interval(got, sf, cf, xf, 2 * EPS[dtype])


@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("backward", [False, True])
@pytest.mark.parametrize("shape", [
    (64, 1024, 2, 8),       # Llama: head 128, seq 1024, batch 2 | 8 heads: sin is [64, 1024, 2]
    (32, 333, 1, 5),        # m a multiple of 4, odd sizes
    (5, 77, 1, 3),          # m odd: one pair per thread
    (2, 3, 1, 1),
])
def test_against_checker(oracle, dtype, backward, shape):
    print("case rope", dtype, backward, shape, flush=True)
    half, seq, batch, n = shape
    m = half * seq * batch
    ang = synth.randn(70, 0, m).astype(np.float64) * 2.0
    sin, cos = np.sin(ang).astype(np.float32), np.cos(ang).astype(np.float32)
    src = synth.randn(71, 0, 2 * m * n)
    got, sf, cf, xf = _run(sin, cos, src, dtype, backward=backward)
    want = oracle.rope(sf, cf, xf, backward=backward)
    assert np.all(np.isfinite(got))
    err = np.abs(got.reshape(-1) - want.reshape(-1))
    assert np.all(err <= 2 * EPS[dtype] * (np.abs(want.reshape(-1)) + 1.0))
    # in place gives the same bits
    again, _, _, _ = _run(sin, cos, src, dtype, backward=backward, inplace=True)
    assert np.array_equal(again, got)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_unaligned_addresses_and_round_trip(oracle, dtype):
    """Tensors that start one element into an allocation take the
    pair-per-thread kernel; backward(forward(x)) returns x for unit (sin, cos)
    up to the two roundings."""
    m, n = 64 * 50, 6
    ang = synth.randn(72, 0, m).astype(np.float64)
    sin, cos = np.sin(ang).astype(np.float32), np.cos(ang).astype(np.float32)
    src = synth.randn(73, 0, 2 * m * n)
    S, sf = _tile(np.concatenate([[0.0], sin]), dtype)
    C, cf = _tile(np.concatenate([[0.0], cos]), dtype)
    X, xf = _tile(np.concatenate([[0.0], src]), dtype)
    Y = torch.zeros_like(X)
    Z = torch.zeros_like(X)
    hip_sdpa.rope(S[1:], C[1:], X[1:], Y[1:])
    hip_sdpa.rope(S[1:], C[1:], Y[1:], Z[1:], backward=True)
    torch.cuda.synchronize()
    want = oracle.rope(sf[1:], cf[1:], xf[1:])
    got = H.to_np(Y)[1:]
    assert np.all(np.abs(got - want) <= 2 * EPS[dtype] * (np.abs(want) + 1.0))
    assert H.to_np(Y)[0] == 0.0 and H.to_np(Z)[0] == 0.0
    back = H.to_np(Z)[1:]
    assert np.all(np.abs(back - xf[1:]) <= 6 * EPS[dtype] * (np.abs(xf[1:]) + 1.0))


def test_errors():
    x = torch.zeros(8, device="cuda")
    s = torch.zeros(2, device="cuda")
    fn = hip_sdpa.lib().nntile_hip_rope_fp32
    assert fn(None, -1, 1, s.data_ptr(), s.data_ptr(), x.data_ptr(), x.data_ptr()) == hip_sdpa.EINVAL
    assert fn(None, 2, 2, None, s.data_ptr(), x.data_ptr(), x.data_ptr()) == hip_sdpa.EINVAL
    assert fn(None, 0, 7, None, None, None, None) == hip_sdpa.OK
    with pytest.raises(hip_sdpa.SdpaError):
        hip_sdpa.rope(s, s, x[:6], x[:6])       # 6 is not a multiple of 2 m = 4
