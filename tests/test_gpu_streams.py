"""Calls on different streams are independent: the tile pairs of different
query tiles, each on its own stream (what StarPU workers with one stream each
would do), give the bits of the same calls issued on one stream."""
import pytest
import torch

from nntile_amd import hip_sdpa
from . import helpers as H

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
def test_query_tiles_on_their_own_streams(dtype):
    batch, seq, head, tile = 8, 1024, 64, 256
    dt = H.TORCH_DT[dtype]
    g = torch.Generator(device="cuda").manual_seed(5)
    Q, K, V = (torch.randn((batch, seq, head), generator=g, device="cuda").to(dt) for _ in range(3))
    split = lambda t: [t[:, s:s + tile].contiguous() for s in range(0, seq, tile)]
    Qt, Kt, Vt = split(Q), split(K), split(V)
    nt = seq // tile

    def run(streams):
        outs = [H.fresh_outputs(batch, tile, head, dtype, poison=False) for _ in range(nt)]
        main = torch.cuda.current_stream()
        for st in streams:
            st.wait_stream(main)
        for qi in range(nt):
            st = streams[qi % len(streams)] if streams else None
            for ki in range(qi + 1):
                hip_sdpa.sdpa_fwd_tile(Kt[ki], Qt[qi], None, outs[qi][0], Vt[ki], outs[qi][1],
                                       hip_sdpa.MASK_CAUSAL, q_pos0=qi * tile, k_pos0=ki * tile,
                                       stream=st)
        for st in streams:
            main.wait_stream(st)
        torch.cuda.synchronize()
        return outs

    one = run([])
    many = run([torch.cuda.Stream() for _ in range(4)])
    for (l1, a1), (l2, a2) in zip(one, many):
        assert torch.equal(l1, l2)
        assert torch.equal(a1.view(torch.int32 if dtype == "fp32" else torch.int16),
                           a2.view(torch.int32 if dtype == "fp32" else torch.int16))
        assert bool(torch.isfinite(l1).all())
