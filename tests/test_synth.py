"""The seeded generator behind every synthetic input: slices of a stream do
not depend on what precedes them, and its torch evaluation (which the
benchmark runs on the GPU) yields the numpy values."""
import numpy as np

from nntile_amd import synth


def test_slices_of_a_stream_are_position_independent():
    whole = synth.randn(44, 1, 5000)
    assert np.array_equal(whole[1234:2345], synth.randn(44, 1, 1111, offset=1234))
    assert not np.array_equal(whole[:100], synth.randn(44, 2, 100))
    assert not np.array_equal(whole[:100], synth.randn(45, 1, 100))
    # N(0,1): moments of a long draw
    x = synth.randn(7, 0, 1 << 20).astype(np.float64)
    assert abs(x.mean()) < 5e-3 and abs(x.std() - 1.0) < 5e-3 and abs((x ** 3).mean()) < 2e-2


def test_torch_evaluation_matches_numpy():
    for seed, stream, n, off, chunk in [(44, 0, 70000, 0, 1 << 24), (45, 12, 4097, 99999, 1000),
                                        (1, 7, 33, 2 ** 33, 1 << 24)]:
        a = synth.randn(seed, stream, n, off)
        b = synth.randn_torch(seed, stream, n, "cpu", off, chunk).numpy()
        # the uniform variates are bit-identical; log / sqrt / cos of two
        # libraries may differ in the last place
        assert np.allclose(a, b, rtol=1e-6, atol=1e-7)
        assert (a != b).mean() < 1e-3
