"""The CPU checker of the scaled transpose: brute force over the reference's
index formula on small shapes, the involution, and the reference's own test
data and bound (tests/kernel/transpose.cc:66-92)."""
import numpy as np
import pytest

from oracle import cpu_oracle as O


def reference_case(m, n):
    # tests/kernel/transpose.cc:72-78: src(i0, i1) = (i0 + 2 i1 + 1) / 20
    i0, i1 = np.meshgrid(np.arange(m), np.arange(n), indexing="ij")
    src = np.empty(m * n, np.float32)
    src[(i1 * m + i0).ravel()] = ((i0 + 2 * i1 + 1) / 20.0).astype(np.float32).ravel()
    return src


@pytest.mark.parametrize("m,n", [(1, 9), (8, 9), (8, 1), (4, 7), (65, 3)])
def test_index_formula_by_brute_force(m, n):
    src = np.random.default_rng(3).standard_normal(m * n).astype(np.float32)
    got = O.transpose(m, n, -2.0, src)
    for i in range(m):
        for j in range(n):
            assert got[i * n + j] == np.float32(-2.0) * src[i + j * m]


@pytest.mark.parametrize("m,n", [(8, 9), (130, 67)])
def test_twice_is_the_identity_and_reference_data(m, n):
    src = reference_case(m, n)
    back = O.transpose(n, m, 0.5, O.transpose(m, n, 2.0, src))
    assert np.array_equal(back, src)
    got = O.transpose(m, n, -2.0, src)
    ref = -2.0 * src.astype(np.float64).reshape(n, m).T.reshape(-1)
    assert np.all(np.abs(got / ref - 1) <= 10 * np.finfo(np.float32).eps)
