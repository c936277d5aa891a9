"""The StarPU-shaped bodies of the whole-grid calls
(nntile_hip_sdpa_fwd_grid_codelet_*, nntile_hip_sdpa_bwd_grid_codelet_*), run
as a HIP worker would run them - look-alike variable interfaces tile after
tile, the geometry in cl_args - against the direct calls of the same C ABI:
same bits.  A task whose arguments do not fit is a no-op."""
import pytest
import torch

from nntile_amd import hip_sdpa
from . import helpers as H

pytestmark = pytest.mark.gpu


def _tiles(x, step):
    return [x[:, s:s + step].contiguous().cuda() for s in range(0, x.shape[1], step)]


def _bits(t):
    return t.view(torch.int16 if t.element_size() == 2 else torch.int32)


@pytest.mark.parametrize("dtype,head", [("bf16", 128), ("fp16", 64), ("fp32", 64)])
@pytest.mark.parametrize("n_slabs,batch,q_seq,k_seq,q_tile,k_tile,causal", [
    (1, 4, 512, 512, 128, 128, True),
    (3, 2, 320, 320, 128, 128, True),        # several slabs, ragged last tiles
    (2, 5, 96, 200, 96, 64, False),          # rectangular, no mask
])
def test_forward_body(dtype, head, n_slabs, batch, q_seq, k_seq, q_tile, k_tile, causal):
    print("case", dtype, head, n_slabs, batch, q_seq, k_seq, q_tile, k_tile, causal, flush=True)
    offset = k_seq - q_seq
    mode = hip_sdpa.MASK_CAUSAL if causal else hip_sdpa.MASK_NONE
    Kt, Vt, Qt = [], [], []
    for s in range(n_slabs):
        (Q, K, V), _ = H.make_qkv(200 + s, batch, q_seq, k_seq, head, dtype)
        Kt += _tiles(K, k_tile)
        Vt += _tiles(V, k_tile)
        Qt += _tiles(Q, q_tile)
    direct = [H.fresh_outputs(batch, t.shape[1], head, dtype) for t in Qt]
    body = [H.fresh_outputs(batch, t.shape[1], head, dtype) for t in Qt]
    untouched = [H.fresh_outputs(batch, t.shape[1], head, dtype, poison=False) for t in Qt]
    hip_sdpa.sdpa_fwd_grid(Kt, Qt, [o[0] for o in direct], Vt, [o[1] for o in direct], q_seq, k_seq,
                           q_tile, k_tile, mode, causal_offset=offset, n_slabs=n_slabs)
    hip_sdpa.sdpa_fwd_grid_codelet(Kt, Qt, [o[0] for o in body], Vt, [o[1] for o in body], q_seq,
                                   k_seq, q_tile, k_tile, mode, causal_offset=offset,
                                   n_slabs=n_slabs)
    # a tile count that contradicts the sequence length: reported, nothing runs
    hip_sdpa.sdpa_fwd_grid_codelet(Kt, Qt, [o[0] for o in untouched], Vt, [o[1] for o in untouched],
                                   q_seq, k_seq, q_tile, k_tile, mode, causal_offset=offset,
                                   n_slabs=n_slabs, n_q_tiles=len(Qt) // n_slabs - 1)
    torch.cuda.synchronize()
    for d, b, u in zip(direct, body, untouched):
        assert torch.equal(d[0], b[0]) and torch.equal(_bits(d[1]), _bits(b[1]))
        assert bool(torch.isneginf(u[0]).all()) and bool((u[1] == 0).all())
    # overwrite mode through the body: the running pair need not be initialised
    body2 = [(torch.full_like(o[0], 7.0), torch.full_like(o[1], float("nan"))) for o in body]
    hip_sdpa.sdpa_fwd_grid_codelet(Kt, Qt, [o[0] for o in body2], Vt, [o[1] for o in body2], q_seq,
                                   k_seq, q_tile, k_tile, mode, causal_offset=offset,
                                   n_slabs=n_slabs, flags=hip_sdpa.OVERWRITE)
    torch.cuda.synchronize()
    for d, b in zip(direct, body2):
        assert torch.allclose(d[0], b[0], rtol=1e-5, atol=1e-5)
        assert torch.allclose(d[1].float(), b[1].float(), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("dtype,head", [("bf16", 128), ("fp16", 64)])
@pytest.mark.parametrize("n_slabs,batch,seq,tile,causal", [(1, 4, 512, 128, True), (2, 2, 384, 128, True),
                                                           (2, 3, 256, 256, False)])
def test_backward_body(dtype, head, n_slabs, batch, seq, tile, causal):
    print("case", dtype, head, n_slabs, batch, seq, tile, causal, flush=True)
    mode = hip_sdpa.MASK_CAUSAL if causal else hip_sdpa.MASK_NONE
    Kt, Vt, Qt, Gt = [], [], [], []
    for s in range(n_slabs):
        (Q, K, V), _ = H.make_qkv(300 + s, batch, seq, seq, head, dtype)
        (G, _, _), _ = H.make_qkv(400 + s, batch, seq, seq, head, dtype)
        Kt += _tiles(K, tile)
        Vt += _tiles(V, tile)
        Qt += _tiles(Q, tile)
        Gt += _tiles(G, tile)
    At = [torch.zeros_like(q) for q in Qt]
    Lt = [torch.full((batch, q.shape[1]), float("-inf"), device="cuda") for q in Qt]
    hip_sdpa.sdpa_fwd_grid(Kt, Qt, Lt, Vt, At, seq, seq, tile, tile, mode, flags=hip_sdpa.OVERWRITE,
                           n_slabs=n_slabs)
    ws = torch.empty(4 * n_slabs * seq * batch, dtype=torch.uint8, device="cuda")
    grads = lambda: ([torch.zeros_like(k) for k in Kt], [torch.zeros_like(q) for q in Qt],
                     [torch.zeros_like(v) for v in Vt])
    dK0, dQ0, dV0 = grads()
    dK1, dQ1, dV1 = grads()
    hip_sdpa.sdpa_bwd_grid(Kt, Qt, Vt, At, Gt, Lt, dK0, dQ0, dV0, seq, seq, tile, tile, mode,
                           workspace=ws, n_slabs=n_slabs)
    hip_sdpa.sdpa_bwd_grid_codelet(Kt, Qt, Vt, At, Gt, Lt, dK1, dQ1, dV1, seq, seq, tile, tile, mode,
                                   ws, n_slabs=n_slabs)
    torch.cuda.synchronize()
    for a, b in zip(dK0 + dQ0 + dV0, dK1 + dQ1 + dV1):
        assert torch.equal(_bits(a), _bits(b))
    assert any(bool((t != 0).any()) for t in dQ1)
    # a scratch buffer that is too small: reported, nothing added
    dK2, dQ2, dV2 = grads()
    hip_sdpa.sdpa_bwd_grid_codelet(Kt, Qt, Vt, At, Gt, Lt, dK2, dQ2, dV2, seq, seq, tile, tile, mode,
                                   ws[:16], n_slabs=n_slabs)
    torch.cuda.synchronize()
    assert all(bool((t == 0).all()) for t in dK2 + dQ2 + dV2)
