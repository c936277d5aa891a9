"""A seeded sweep of random shapes, modes and flags through the forward entry
points (tile, tile in key pieces, grid, decode, tile and decode on a cache) and
the backward tile entry point, against the CPU checker with the whole-tensor
and the per-row bounds.  The cases are drawn from a counter-based generator,
so every run tests the same list; a failing case prints its parameters.

What the fixed lists of the other test files do not vary together: odd
sequence lengths against every head size and type, grouped heads with ragged
key tiles, causal offsets that hide whole query rows (negative) or nothing,
random masks with rows that see no key, overwrite against merge into a fresh
pair, and positions of the pair inside a larger sequence."""
import os

import numpy as np
import pytest
import torch

from nntile_amd import hip_sdpa, synth
from . import helpers as H

pytestmark = pytest.mark.gpu

# (the environment variables widen the sweep for a one-off run; the cases of
# the default run are a prefix of it)
N_FORWARD = int(os.environ.get("NNTILE_SWEEP_FORWARD", "160"))
N_BACKWARD = int(os.environ.get("NNTILE_SWEEP_BACKWARD", "48"))
BWD_TOL = {"bf16": 1e-2, "fp16": 2e-3}


def _uniform(seed, stream, n):
    """n doubles in [0, 1) that depend on (seed, stream) only."""
    return np.random.Generator(np.random.PCG64([seed, stream])).random(n)


class Draw:
    """Choices of case number `case`, the same in every run."""

    def __init__(self, seed, case):
        self.u = _uniform(seed, case, 64)
        self.i = 0

    def below(self, n):
        v = int(self.u[self.i] * n)
        self.i += 1
        return min(v, n - 1)

    def pick(self, options):
        return options[self.below(len(options))]

    def between(self, lo, hi):
        return lo + self.below(hi - lo + 1)


def _visibility(kind, q_seq, k_seq, offset, d, seed):
    """[q, k] bool: True where the key is visible."""
    if kind == "none":
        return np.ones((q_seq, k_seq), bool)
    if kind == "causal":
        return synth.causal_mask(q_seq, k_seq, offset)
    p = d.pick([0.05, 0.5, 0.9])
    vis = _uniform(seed, 900, q_seq * k_seq).reshape(q_seq, k_seq) < p
    # some rows see nothing, some blocks are uniform
    if q_seq > 3:
        vis[d.below(q_seq)] = False
    if k_seq > 70:
        vis[:, : 64] = True
    return vis


def _check_forward(got_A, got_lse, want_A, want_lse, vis, dtype, overwrite, what):
    rows = vis.any(axis=1)
    gA, gl = H.to_np(got_A), H.to_np(got_lse)
    # rows without a visible key: lse = -inf; A untouched (merge) or zero (overwrite)
    assert np.all(np.isneginf(gl[:, ~rows])), what
    if overwrite:
        assert np.all(gA[:, ~rows] == 0), what
    if rows.any():
        assert H.rel_fro(gA[:, rows], want_A[:, rows]) < H.TOL[dtype], what
        assert H.rel_fro(gl[:, rows], want_lse[:, rows]) < H.TOL[dtype], what
        H.check_rows(gA[:, rows], want_A[:, rows], gl[:, rows], want_lse[:, rows], dtype, what)


def _forward_case(case):
    d = Draw(4242, case)
    entry = d.pick(["tile", "tile", "pieces", "grid", "decode", "tile_cache", "decode_cache"])
    dtype = d.pick(["bf16", "fp16", "fp32"])
    head = d.pick([32, 64, 128])
    n_batch, group, n_kv = d.between(1, 3), d.pick([1, 1, 2, 4]), d.between(1, 2)
    q_seq, k_seq = d.between(1, 300), d.between(1, 400)
    kind = d.pick(["causal", "causal", "none", "additive", "bool"])
    overwrite = d.pick([True, False])
    if entry in ("decode", "decode_cache"):
        dtype = d.pick(["bf16", "fp16"])
        head = d.pick([64, 128])
        q_seq = d.between(1, 64 // group)
        k_seq = d.between(1, 1500)
    if entry == "grid" and kind in ("additive", "bool"):
        kind = "causal"         # the grid entry point takes analytic masks only
    # new tokens are the last keys, shifted by up to +-20 (negative: the first
    # query rows see nothing)
    offset = k_seq - q_seq + d.between(-20, 20) if kind == "causal" else 0
    return dict(case=case, entry=entry, dtype=dtype, head=head, n_batch=n_batch, group=group,
                n_kv=n_kv, q_seq=q_seq, k_seq=k_seq, kind=kind, overwrite=overwrite, offset=offset,
                draw=d)


@pytest.mark.parametrize("case", range(N_FORWARD))
def test_forward_random_case(oracle, case):
    c = _forward_case(case)
    d = c.pop("draw")
    print("case", c, flush=True)
    dtype, head, n_batch, group, n_kv = c["dtype"], c["head"], c["n_batch"], c["group"], c["n_kv"]
    q_seq, k_seq, kind, overwrite, offset, entry = (c["q_seq"], c["k_seq"], c["kind"],
                                                    c["overwrite"], c["offset"], c["entry"])
    batch, kvb = n_batch * group * n_kv, n_batch * n_kv
    seed = 7000 + case
    (Q, K, V), (qf, kf, vf) = H.make_qkv(seed, batch, q_seq, k_seq, head, dtype, kv_batch=kvb)
    vis = _visibility(kind, q_seq, k_seq, offset, d, seed)
    want_A, want_lse = oracle.sdpa_vanilla(kf, qf, vf, None if kind == "none" else vis,
                                           n_batch=n_batch, kv_repeat=group)
    mode = {"causal": hip_sdpa.MASK_CAUSAL, "none": hip_sdpa.MASK_NONE,
            "additive": hip_sdpa.MASK_ADDITIVE, "bool": hip_sdpa.MASK_BOOL}[kind]
    m = None
    if kind == "additive":
        m = H.additive_mask(vis, dtype).cuda()
    elif kind == "bool":
        m = torch.from_numpy(vis.copy()).cuda()
    Kd, Qd, Vd = K.cuda(), Q.cuda(), V.cuda()
    lse, A = H.fresh_outputs(batch, q_seq, head, dtype)
    flags = hip_sdpa.OVERWRITE if overwrite else 0
    # positions: the pair sits somewhere inside a longer sequence
    pos = d.pick([0, 0, 1000, 123457])
    kw = dict(q_pos0=pos, k_pos0=pos, causal_offset=offset)

    if entry == "tile":
        hip_sdpa.sdpa_fwd_tile(Kd, Qd, m, lse, Vd, A, mode, n_batch, group, flags=flags, **kw)
    elif entry == "pieces":
        # key pieces in a shuffled order, merged into the running pair; only
        # the first may overwrite
        cuts = sorted({0, k_seq} | {d.below(k_seq + 1) for _ in range(3)})
        pieces = [(lo, hi) for lo, hi in zip(cuts[:-1], cuts[1:]) if hi > lo]
        order = [pieces[i] for i in np.argsort(_uniform(seed, 901, len(pieces)))]
        for n, (lo, hi) in enumerate(order):
            mp = None if m is None else m[:, lo:hi].contiguous()
            hip_sdpa.sdpa_fwd_tile(Kd[:, lo:hi].contiguous(), Qd, mp, lse, Vd[:, lo:hi].contiguous(), A,
                                   mode, n_batch, group, q_pos0=pos, k_pos0=pos + lo,
                                   causal_offset=offset, flags=flags if n == 0 else 0)
        if overwrite and len(order) > 1:
            # rows hidden in the first piece were written as empty and later
            # pieces merged into them: the zero-row rule no longer applies
            overwrite = bool(vis.any(axis=1).all())
    elif entry == "grid":
        q_tile, k_tile = d.pick([64, 100, 128, 300]), d.pick([64, 96, 128, 400])
        Kt = [Kd[:, s:s + k_tile].contiguous() for s in range(0, k_seq, k_tile)]
        Vt = [Vd[:, s:s + k_tile].contiguous() for s in range(0, k_seq, k_tile)]
        Qt = [Qd[:, s:s + q_tile].contiguous() for s in range(0, q_seq, q_tile)]
        outs = [H.fresh_outputs(batch, q.shape[1], head, dtype) for q in Qt]
        hip_sdpa.sdpa_fwd_grid(Kt, Qt, [o[0] for o in outs], Vt, [o[1] for o in outs], q_seq, k_seq,
                               q_tile, k_tile, mode, n_batch, group, flags=flags, **kw)
        torch.cuda.synchronize()
        A = torch.cat([o[1] for o in outs], dim=1)
        lse = torch.cat([o[0] for o in outs], dim=1)
    elif entry == "decode":
        ws = torch.empty(hip_sdpa.decode_workspace_bytes(Kd, Qd, n_batch, group), dtype=torch.uint8,
                         device="cuda")
        hip_sdpa.sdpa_fwd_decode(Kd, Qd, m, lse, Vd, A, mode, n_batch, group, ws, flags=flags, **kw)
    else:
        # caches with room behind the filled rows, poisoned there
        cap = k_seq + d.between(0, 70)
        Kc = torch.full((kvb, cap, head), float("nan"), dtype=H.TORCH_DT[dtype], device="cuda")
        Vc = torch.full_like(Kc, float("nan"))
        Kc[:, :k_seq], Vc[:, :k_seq] = Kd, Vd
        if entry == "tile_cache":
            hip_sdpa.sdpa_fwd_tile_cache(Kc, Vc, k_seq, Qd, m, lse, A, mode, n_batch, group,
                                         flags=flags, **kw)
        else:
            ws = torch.empty(hip_sdpa.decode_cache_workspace_bytes(k_seq, Qd, n_batch, group),
                             dtype=torch.uint8, device="cuda")
            hip_sdpa.sdpa_fwd_decode_cache(Kc, Vc, k_seq, Qd, m, lse, A, mode, n_batch, group, ws,
                                           flags=flags, **kw)
    torch.cuda.synchronize()
    _check_forward(A, lse, want_A, want_lse, vis, dtype, overwrite, str(c))
    # the inputs are unchanged
    assert torch.equal(Qd.cpu().view(torch.uint8), Q.view(torch.uint8))
    assert torch.equal(Kd.cpu().view(torch.uint8), K.view(torch.uint8))


@pytest.mark.parametrize("case", range(N_BACKWARD))
def test_backward_random_case(oracle, case):
    d = Draw(4343, case)
    dtype = d.pick(["bf16", "fp16"])
    head = d.pick([32, 64, 128])
    n_batch, group, n_kv = d.between(1, 2), d.pick([1, 1, 2, 4]), d.between(1, 2)
    q_seq, k_seq = d.between(1, 260), d.between(1, 330)
    kind = d.pick(["causal", "none", "additive", "bool"])
    overwrite = d.pick([True, False])
    offset = max(k_seq - q_seq, 0) + d.between(0, 10) if kind == "causal" else 0
    c = dict(case=case, dtype=dtype, head=head, n_batch=n_batch, group=group, n_kv=n_kv,
             q_seq=q_seq, k_seq=k_seq, kind=kind, overwrite=overwrite, offset=offset)
    print("case bwd", c, flush=True)
    batch, kvb = n_batch * group * n_kv, n_batch * n_kv
    seed = 8000 + case
    (Q, K, V), (qf, kf, vf) = H.make_qkv(seed, batch, q_seq, k_seq, head, dtype, kv_batch=kvb)
    G, gf = H.rounded(synth.randn(seed, 5, batch * q_seq * head).reshape(batch, q_seq, head), dtype)
    if kind == "none":
        vis = np.ones((q_seq, k_seq), bool)
    elif kind == "causal":
        vis = synth.causal_mask(q_seq, k_seq, offset)
    else:
        vis = _uniform(seed, 900, q_seq * k_seq).reshape(q_seq, k_seq) < d.pick([0.3, 0.8])
        vis[:, 0] = True            # every query sees a key: A and lse are defined
    add = np.where(vis, 0, -np.inf).astype(np.float32)
    # A and lse of a forward pass over the same inputs (query slab b reads
    # key/value slab (b % n_batch) + n_batch * (b / (n_batch * group)))
    kv_of = [(b % n_batch) + n_batch * ((b // n_batch) // group) for b in range(batch)]
    A64, lse64 = oracle.sdpa_bruteforce_f64(kf[kv_of], qf, vf[kv_of], add)
    A, af = H.rounded(np.ascontiguousarray(A64, dtype=np.float32), dtype)
    lse = lse64.astype(np.float32)
    wKs, wQ, wVs = oracle.sdpa_bwd_flash_f64(kf, qf, vf, af, gf, lse, add, kv_repeat=group,
                                             n_batch=n_batch)
    m = None
    mode = {"causal": hip_sdpa.MASK_CAUSAL, "none": hip_sdpa.MASK_NONE,
            "additive": hip_sdpa.MASK_ADDITIVE, "bool": hip_sdpa.MASK_BOOL}[kind]
    if kind == "additive":
        m = H.additive_mask(vis, dtype).cuda()
    elif kind == "bool":
        m = torch.from_numpy(vis.copy()).cuda()
    dt = H.TORCH_DT[dtype]
    if overwrite:
        dK = torch.full(K.shape, float("nan"), dtype=dt, device="cuda")
        dQ = torch.full(Q.shape, float("nan"), dtype=dt, device="cuda")
        dV = torch.full(V.shape, float("nan"), dtype=dt, device="cuda")
    else:
        dK, dQ, dV = (torch.zeros(x.shape, dtype=dt, device="cuda") for x in (K, Q, V))
    hip_sdpa.sdpa_bwd_tile(K.cuda(), Q.cuda(), V.cuda(), A.cuda(), G.cuda(), m,
                           torch.from_numpy(lse).cuda(), dK, dQ, dV, mode, n_batch, group,
                           causal_offset=offset, flags=hip_sdpa.OVERWRITE if overwrite else 0)
    torch.cuda.synchronize()
    for got, want, name in ((dK, wKs, "dK"), (dQ, wQ, "dQ"), (dV, wVs, "dV")):
        err = H.rel_fro(H.to_np(got), want)
        assert err < BWD_TOL[dtype], (name, err, c)
