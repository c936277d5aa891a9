"""The entry points enqueue kernels and nothing else (no allocation, no
synchronisation, no memset nodes), so a caller can capture them in a HIP
graph.  Each graph is replayed several times with eager work and
synchronisations in between, and every replay is compared with the eager
result."""
import pytest
import torch

from nntile_amd import hip_sdpa
from . import helpers as H

pytestmark = pytest.mark.gpu


def _randn(shape, dtype, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return torch.randn(shape, generator=g, device="cuda").to(dtype)


def _replays(graph, check, disturb):
    for _ in range(3):
        disturb()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        check()


@pytest.mark.parametrize("n_batch", [2, 4])
def test_decode_step_through_the_cache_in_a_graph(n_batch):
    """n_batch 2: 4 units, the merge of the key splits is a launch of its own.
    n_batch 4: 8 units, the merge rides in the main launch and its flags live
    in the workspace - a replay carries the captured call's tag again and
    finds them as the previous replay (or `disturb`) left them."""
    n_kv, group, head, cap, old, new = 2, 4, 128, 1024, 600, 16
    kvb, batch = n_batch * n_kv, n_batch * n_kv * group
    dt = torch.bfloat16
    Kc, Vc = _randn((kvb, cap, head), dt, 1), _randn((kvb, cap, head), dt, 2)
    k_new, v_new = _randn((kvb, new, head), dt, 3), _randn((kvb, new, head), dt, 4)
    Q = _randn((batch, new, head), dt, 5)
    k_seq = old + new
    ws = torch.empty(hip_sdpa.decode_cache_workspace_bytes(k_seq, Q, n_batch, group),
                     dtype=torch.uint8, device="cuda")

    def step(lse, A):
        hip_sdpa.kv_cache_append(k_new, v_new, Kc, Vc, old)
        hip_sdpa.sdpa_fwd_decode_cache(Kc, Vc, k_seq, Q, None, lse, A, hip_sdpa.MASK_CAUSAL, n_batch,
                                       group, ws, causal_offset=old, flags=hip_sdpa.OVERWRITE)

    lse0, A0 = H.fresh_outputs(batch, new, head, "bf16")
    step(lse0, A0)
    torch.cuda.synchronize()
    lse, A = H.fresh_outputs(batch, new, head, "bf16")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(lse, A)

    def disturb():      # what a replay must restore: the appended rows, the outputs, the workspace
        Kc[:, old:k_seq].zero_()
        Vc[:, old:k_seq].zero_()
        A.fill_(float("nan"))
        lse.fill_(float("nan"))
        ws.random_(0, 255)

    def check():
        assert torch.equal(A.view(torch.int16), A0.view(torch.int16)) and torch.equal(lse, lse0)
        assert torch.equal(Kc[:, old:k_seq], k_new) and torch.equal(Vc[:, old:k_seq], v_new)

    _replays(graph, check, disturb)


def test_prefill_and_backward_in_a_graph():
    batch, seq, head, tile = 4, 512, 128, 256
    dt = torch.bfloat16
    Q, K, V, G = (_randn((batch, seq, head), dt, 10 + i) for i in range(4))
    split = lambda t: [t[:, s:s + tile].contiguous() for s in range(0, seq, tile)]
    Qt, Kt, Vt = split(Q), split(K), split(V)
    nbytes = hip_sdpa.sdpa_bwd_workspace_bytes(seq, seq, batch, hip_sdpa.MASK_CAUSAL)
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")

    def step(lse_t, A_t, A, lse, dK, dQ, dV):
        hip_sdpa.sdpa_fwd_grid(Kt, Qt, lse_t, Vt, A_t, seq, seq, tile, tile, hip_sdpa.MASK_CAUSAL,
                               flags=hip_sdpa.OVERWRITE)
        hip_sdpa.sdpa_fwd_tile(K, Q, None, lse, V, A, hip_sdpa.MASK_CAUSAL, flags=hip_sdpa.OVERWRITE)
        hip_sdpa.sdpa_bwd_tile(K, Q, V, A, G, None, lse, dK, dQ, dV, hip_sdpa.MASK_CAUSAL,
                               workspace=ws, flags=hip_sdpa.OVERWRITE)

    def buffers():
        lse_t = [torch.full((batch, tile), float("nan"), device="cuda") for _ in Qt]
        A_t = [torch.full_like(q, float("nan")) for q in Qt]
        A = torch.full_like(Q, float("nan"))
        lse = torch.full((batch, seq), float("nan"), device="cuda")
        return lse_t, A_t, A, lse, torch.full_like(Q, float("nan")), torch.full_like(Q, float("nan")), \
            torch.full_like(Q, float("nan"))

    want = buffers()
    step(*want)
    torch.cuda.synchronize()
    got = buffers()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(*got)

    def flat(b):
        return list(b[0]) + list(b[1]) + list(b[2:])

    def disturb():
        for t in flat(got):
            t.fill_(float("nan"))
        ws.random_(0, 255)

    def check():
        for g, w in zip(flat(got), flat(want)):
            gi = g.view(torch.int16) if g.dtype == dt else g.view(torch.int32)
            wi = w.view(torch.int16) if w.dtype == dt else w.view(torch.int32)
            assert torch.equal(gi, wi)
        # the grid launch and the single-tile launch agree on the forward
        assert torch.allclose(torch.cat(got[1], dim=1).float(), got[2].float(), rtol=2e-2, atol=2e-2)

    _replays(graph, check, disturb)


def test_reference_call_with_a_mask_tile_and_scratch_in_a_graph():
    """The reference-signature call scans a large mask once per call.  Outside a
    capture the scan rides in the attention launch behind a tag unique to the
    call; a captured call would carry its tag into every replay, so under
    capture the scan is a launch of its own.  Replays after the mask has been
    rewritten in place must follow the new mask, and so must eager calls in
    between (the scratch keeps what the other form left there)."""
    import numpy as np
    batch, seq, head = 3, 1024, 128
    dt = torch.bfloat16
    Q, K, V = (_randn((batch, seq, head), dt, 20 + i) for i in range(3))
    i = np.arange(seq)[:, None]
    j = np.arange(seq)[None, :]
    masks = [np.ascontiguousarray(np.broadcast_to(m, (seq, seq)))
             for m in (j <= i, np.abs(i - j) <= 100, (j <= i) & (i >= 300), j >= 0)]
    as_tile = lambda vis: torch.from_numpy(np.where(vis, 0.0, -np.inf).astype(np.float32)).to(dt).cuda()
    mask = as_tile(masks[0]).clone()
    scratch = torch.full((batch, seq), float("nan"), device="cuda")

    def call(lse, A):
        lse.fill_(float("-inf"))
        A.zero_()
        hip_sdpa.flash_sdpa_fwd(K, Q, mask, lse, V, A, scratch_lse=scratch)

    lse_g, A_g = H.fresh_outputs(batch, seq, head, "bf16")
    call(lse_g, A_g)                      # warm-up, eager
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(lse_g, A_g)
    for vis in masks[1:] + masks[:1]:
        mask.copy_(as_tile(vis))
        # eager, without the scratch: every workgroup scans its own rows
        lse_e, A_e = H.fresh_outputs(batch, seq, head, "bf16")
        lse_e.fill_(float("-inf"))
        A_e.zero_()
        hip_sdpa.flash_sdpa_fwd(K, Q, mask, lse_e, V, A_e)
        # eager with the scratch (the scan rides in the launch), then the replay
        lse_s, A_s = H.fresh_outputs(batch, seq, head, "bf16")
        call(lse_s, A_s)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        rows = torch.from_numpy(vis.any(axis=1)).cuda()
        for lse_x, A_x in ((lse_s, A_s), (lse_g, A_g)):
            assert torch.equal(lse_x, lse_e)
            assert torch.equal(A_x[:, rows].view(torch.int16), A_e[:, rows].view(torch.int16))
