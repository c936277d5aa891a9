"""The committed fixture tests/golden/sdpa_preset.npz (written by
tests/golden/make_golden.py: float64 numpy on the input formulas of the
reference's own kernel and tile tests) against the CPU checker, and against
the HIP path through the C ABI."""
import importlib.util
import os

import numpy as np
import pytest
import torch

from . import helpers as H

HERE = os.path.dirname(os.path.abspath(__file__))
_spec = importlib.util.spec_from_file_location("make_golden",
                                               os.path.join(HERE, "golden", "make_golden.py"))
G = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(G)

CASES = {
    "preset_causal": lambda: G.preset_kernel_test(64, 32, 2),
    "preset_full": lambda: G.preset_kernel_test(64, 32, 2),
    "preset_window": lambda: G.preset_tile_test(96, 64, 1),
    "hidden_rows": lambda: G.preset_kernel_test(64, 32, 2),
}


@pytest.fixture(scope="module")
def golden():
    return np.load(os.path.join(HERE, "golden", "sdpa_preset.npz"), allow_pickle=False)


def _inputs(name):
    return tuple(G.round_bf16(x) for x in CASES[name]())


def test_fixture_is_what_the_generator_writes(golden):
    for name in CASES:
        q, k, v = (x.astype(np.float64) for x in _inputs(name))
        a, lse = G.attention(q, k, v, golden[name + "_visible"])
        assert np.array_equal(a.astype(np.float32), golden[name + "_A"])
        assert np.array_equal(lse.astype(np.float32), golden[name + "_lse"])


@pytest.mark.parametrize("name", sorted(CASES))
def test_checker_matches_fixture(oracle, golden, name):
    q, k, v = _inputs(name)
    vis = golden[name + "_visible"]
    got, got_lse = oracle.sdpa_vanilla(k, q, v, vis)
    assert H.rel_fro(got, golden[name + "_A"]) < 2e-6
    assert H.rel_fro(got_lse, golden[name + "_lse"]) < 2e-6
    got, got_lse = oracle.sdpa_bruteforce_f64(k, q, v, np.where(vis, 0, -np.inf).astype(np.float32))
    assert H.rel_fro(got, golden[name + "_A"]) < 2e-7
    assert H.rel_fro(got_lse, golden[name + "_lse"]) < 2e-7


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("mode", ["additive", "bool"])
@pytest.mark.parametrize("name", sorted(CASES))
def test_hip_matches_fixture(golden, name, mode, dtype):
    from nntile_amd import hip_sdpa
    q, k, v = _inputs(name)          # bf16-representable, so exact in fp16 and fp32 too
    vis = golden[name + "_visible"]
    Q, K, V = (torch.from_numpy(x).to(H.TORCH_DT[dtype]).cuda() for x in (q, k, v))
    assert all(np.array_equal(H.to_np(t), x) for t, x in ((Q, q), (K, k), (V, v)))
    lse, A = H.fresh_outputs(q.shape[0], q.shape[1], q.shape[2], dtype)
    if mode == "additive":
        hip_sdpa.flash_sdpa_fwd(K, Q, H.additive_mask(vis, dtype).cuda(), lse, V, A)
    else:
        hip_sdpa.sdpa_fwd_tile(K, Q, torch.from_numpy(vis).cuda(), lse, V, A, hip_sdpa.MASK_BOOL)
    torch.cuda.synchronize()
    want, want_lse = golden[name + "_A"], golden[name + "_lse"]
    hidden = np.isneginf(want_lse)
    got = H.to_np(A)
    # rows with no visible key are left as they were (here: the NaN poison)
    assert np.all(np.isnan(got[hidden]))
    got[hidden] = 0.0
    assert H.rel_fro(got, want) < H.TOL[dtype]
    assert H.rel_fro(H.to_np(lse), want_lse) < H.TOL[dtype]
