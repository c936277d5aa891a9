"""The CPU checker of the rotary embedding, pinned without running the
reference: a rotation is a complex multiplication (numpy's complex product is
the independent routine), special angles have exact answers, the backward is
the transposed map, and the reference's own test loop
(tests/kernel/rope.cc:84-137) accepts the checker's output on its data."""
import numpy as np
import pytest

from oracle import cpu_oracle as O


def _rand(shape, seed):
    return np.random.default_rng(seed).standard_normal(shape).astype(np.float32)


@pytest.mark.parametrize("m,n", [(1, 1), (1, 10), (10, 100), (64, 7), (6, 5)])
def test_forward_is_a_complex_product_broadcast_over_n(m, n):
    ang = np.random.default_rng(1).uniform(-np.pi, np.pi, m)
    s, c = np.sin(ang).astype(np.float32), np.cos(ang).astype(np.float32)
    x = _rand(2 * m * n, 2)
    got = O.rope(s, c, x)
    z = x.astype(np.float64).reshape(n, m, 2)
    w = (z[..., 0] + 1j * z[..., 1]) * (c.astype(np.float64) + 1j * s.astype(np.float64))[None, :]
    want = np.stack([w.real, w.imag], axis=-1).reshape(-1)
    assert np.max(np.abs(got - want)) < 1e-6
    # a checker that took sin/cos per column j instead of per position i fails here
    if m > 1 and n > 1 and m != n:
        wrong = (z[..., 0] + 1j * z[..., 1]) * np.resize(c + 1j * s, (m, n)).T
        assert np.max(np.abs(got.reshape(n, m, 2)[..., 0] - wrong.real)) > 1e-3


def test_special_angles_are_exact():
    x = _rand(2 * 4 * 3, 3)
    zero, one = np.zeros(4, np.float32), np.ones(4, np.float32)
    assert np.array_equal(O.rope(zero, one, x), x)                      # angle 0
    q = O.rope(one, zero, x).reshape(-1, 2)                             # angle pi/2: (a, b) -> (-b, a)
    assert np.array_equal(q[:, 0], -x.reshape(-1, 2)[:, 1])
    assert np.array_equal(q[:, 1], x.reshape(-1, 2)[:, 0])
    h = O.rope(zero, -one, x)                                           # angle pi: -x
    assert np.array_equal(h, -x)


@pytest.mark.parametrize("m,n", [(10, 100), (5, 3)])
def test_norm_is_kept_and_angles_add(m, n):
    rng = np.random.default_rng(4)
    a1, a2 = rng.uniform(-3, 3, m), rng.uniform(-3, 3, m)
    f = lambda a, x: O.rope(np.sin(a).astype(np.float32), np.cos(a).astype(np.float32), x)
    x = _rand(2 * m * n, 5)
    y = f(a1, x)
    assert np.allclose(np.sum(y.reshape(-1, 2) ** 2, 1), np.sum(x.reshape(-1, 2) ** 2, 1), rtol=1e-5)
    assert np.allclose(f(a2, y), f(a1 + a2, x), atol=2e-6)


@pytest.mark.parametrize("m,n", [(10, 100), (3, 4)])
def test_backward_is_the_transposed_map(m, n):
    # for ANY sin, cos (not only unit ones): <rope(x), y> = <x, rope_backward(y)>
    s, c = _rand(m, 6), _rand(m, 7)
    x, y = _rand(2 * m * n, 8), _rand(2 * m * n, 9)
    lhs = np.dot(O.rope(s, c, x).astype(np.float64), y.astype(np.float64))
    rhs = np.dot(x.astype(np.float64), O.rope(s, c, y, backward=True).astype(np.float64))
    assert abs(lhs - rhs) < 1e-4 * max(1.0, abs(lhs))
    # and with unit sin, cos it undoes the forward
    ang = np.random.default_rng(10).uniform(-3, 3, m)
    su, cu = np.sin(ang).astype(np.float32), np.cos(ang).astype(np.float32)
    assert np.allclose(O.rope(su, cu, O.rope(su, cu, x), backward=True), x, atol=2e-6)


def reference_case(m, n, dtype=np.float32):
    """Data of tests/kernel/rope.cc:69-83."""
    total = 2 * m * n
    i = np.arange(total, dtype=np.float64)
    src = ((2 * i + 1 - total) / 1000.0).astype(dtype)
    k = np.arange(m, dtype=np.float64)
    sin = ((2 * k + 1 - m) / max(m, 1)).astype(dtype)
    cos = np.sqrt(1 - sin.astype(dtype) * sin.astype(dtype)).astype(dtype)
    return sin, cos, src


def within_reference_interval(got, sin, cos, src, eps):
    """The acceptance interval of tests/kernel/rope.cc:95-137: each value
    within ref * (1 +- eps) +- eps of the value computed in the tile's
    representation type."""
    m = sin.size
    v = src.astype(np.float64).reshape(-1, m, 2)
    c, s = cos.astype(np.float64), sin.astype(np.float64)
    ref = np.stack([c * v[..., 0] - s * v[..., 1], s * v[..., 0] + c * v[..., 1]], -1).reshape(-1)
    lo = np.where(ref < 0, ref * (1 + eps) - eps, ref * (1 - eps) - eps)
    hi = np.where(ref < 0, ref * (1 - eps) + eps, ref * (1 + eps) + eps)
    g = np.asarray(got, np.float64).reshape(-1)
    return bool(np.all((g >= lo) & (g <= hi)))


@pytest.mark.parametrize("m,n", [(0, 5), (1, 10), (10, 100)])
def test_reference_test_data(m, n):
    sin, cos, src = reference_case(m, n)
    got = O.rope(sin, cos, src)
    assert got.shape == src.shape
    if m:
        assert within_reference_interval(got, sin, cos, src, 2 * np.finfo(np.float32).eps)
