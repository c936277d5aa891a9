"""GPU parity of the key/value-cache entry points, through the C ABI: append
is bit-exact against the checker's cache, decode-from-cache equals the decode
over dense copies of the filled rows bit for bit and the checker within the
tolerance, and the reference's own test shape (prefill, then decode chunk by
chunk == rows of one pass over the whole sequence,
wrappers/python/tests/model/test_llama_attention.py:320-345)."""
import numpy as np
import pytest
import torch

from nntile_amd import hip_sdpa, synth
from nntile_amd.kv_cache import KVCache
from . import helpers as H

pytestmark = pytest.mark.gpu


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16 if t.element_size() == 2 else torch.int32).numpy()


@pytest.mark.parametrize("dtype", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("head,entries,cap,chunks", [
    (128, 16, 64, (17, 1, 1, 16, 29)),      # 16-byte pieces
    (64, 3, 40, (40,)),                     # fills the cache in one go
    (6, 5, 19, (3, 1, 7)),                  # 4-byte pieces for 16-bit types
    (5, 4, 9, (2, 3, 1)),                   # odd row bytes: element copies
    (128, 1, 300, (1, 1, 1, 250))])
def test_append_matches_checker_bit_for_bit(oracle, dtype, head, entries, cap, chunks):
    print("case", dtype, head, entries, cap, chunks, flush=True)
    dt = H.TORCH_DT[dtype]
    k_cache = torch.full((entries, cap, head), 7.0, dtype=dt, device="cuda")
    v_cache = torch.full((entries, cap, head), -3.0, dtype=dt, device="cuda")
    ref = oracle.KVCache(cap, 1)
    filled = 0
    for c, rows in enumerate(chunks):
        k, _ = H.rounded(synth.randn(31 + c, 0, entries * rows * head).reshape(entries, rows, head), dtype)
        v, _ = H.rounded(synth.randn(31 + c, 1, entries * rows * head).reshape(entries, rows, head), dtype)
        hip_sdpa.kv_cache_append(k.cuda(), v.cuda(), k_cache, v_cache, filled)
        # the checker works in the reference's axis order [head, seq, entries]
        ref.append(_bits(k).transpose(2, 1, 0), _bits(v).transpose(2, 1, 0))
        filled += rows
        torch.cuda.synchronize()
        assert np.array_equal(_bits(k_cache[:, :filled]), ref.k_partial.transpose(2, 1, 0))
        assert np.array_equal(_bits(v_cache[:, :filled]), ref.v_partial.transpose(2, 1, 0))
        # rows behind the filled ones keep what they held
        assert bool((k_cache[:, filled:] == 7.0).all()) and bool((v_cache[:, filled:] == -3.0).all())


def test_append_beyond_capacity_raises_and_writes_nothing():
    k_cache = torch.zeros((2, 8, 64), dtype=torch.bfloat16, device="cuda")
    v_cache = torch.zeros_like(k_cache)
    new = torch.ones((2, 3, 64), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(hip_sdpa.SdpaError):
        hip_sdpa.kv_cache_append(new, new, k_cache, v_cache, 6)
    torch.cuda.synchronize()
    assert not bool(k_cache.any()) and not bool(v_cache.any())
    cache = KVCache(4)
    cache.append(new, new)
    with pytest.raises(hip_sdpa.SdpaError):
        cache.append(new, new)
    assert len(cache) == 3


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("q_seq,k_seq,cap,n_batch,group,n_kv,head", [
    (16, 512, 1024, 2, 4, 2, 128), (1, 300, 301, 3, 4, 2, 128), (16, 1000, 4096, 1, 4, 1, 64),
    (5, 77, 77, 2, 8, 3, 128), (64, 200, 333, 2, 1, 2, 64)])
@pytest.mark.parametrize("mode", ["causal", "bool", "none"])
def test_decode_from_cache(oracle, dtype, q_seq, k_seq, cap, n_batch, group, n_kv, head, mode):
    print("case", dtype, q_seq, k_seq, cap, n_batch, group, n_kv, head, mode, flush=True)
    batch, kvb = n_batch * group * n_kv, n_batch * n_kv
    (Q, K, V), f32 = H.make_qkv(23, batch, q_seq, k_seq, head, dtype, kv_batch=kvb)
    offset = k_seq - q_seq
    mask = None if mode == "none" else synth.causal_mask(q_seq, k_seq, offset)
    qf, kf, vf = f32
    want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, mask, n_batch=n_batch, kv_repeat=group)
    Qd = Q.cuda()
    # rows behind the filled ones hold NaN: they must never be read into a result
    Kc = torch.full((kvb, cap, head), float("nan"), dtype=H.TORCH_DT[dtype], device="cuda")
    Vc = torch.full_like(Kc, float("nan"))
    Kc[:, :k_seq] = K.cuda()
    Vc[:, :k_seq] = V.cuda()
    m, mm = {"causal": (None, hip_sdpa.MASK_CAUSAL), "none": (None, hip_sdpa.MASK_NONE),
             "bool": (None if mask is None else torch.from_numpy(mask).cuda(), hip_sdpa.MASK_BOOL)}[mode]
    ws = torch.empty(hip_sdpa.decode_cache_workspace_bytes(k_seq, Qd, n_batch, group),
                     dtype=torch.uint8, device="cuda")
    lse, A = H.fresh_outputs(batch, q_seq, head, dtype)
    hip_sdpa.sdpa_fwd_decode_cache(Kc, Vc, k_seq, Qd, m, lse, A, mm, n_batch, group, ws,
                                   causal_offset=offset)
    torch.cuda.synchronize()
    assert H.rel_fro(H.to_np(A), want) < H.TOL[dtype]
    assert H.rel_fro(H.to_np(lse), want_lse) < H.TOL[dtype]
    # the same call over dense copies of the filled rows: identical bits
    lse2, A2 = H.fresh_outputs(batch, q_seq, head, dtype)
    hip_sdpa.sdpa_fwd_decode(K.cuda(), Qd, m, lse2, V.cuda(), A2, mm, n_batch, group, ws,
                             causal_offset=offset)
    torch.cuda.synchronize()
    assert np.array_equal(_bits(A), _bits(A2))
    assert np.array_equal(_bits(lse), _bits(lse2))


@pytest.mark.parametrize("dtype", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("head,group", [(128, 4), (64, 1), (32, 2)])
def test_prefill_then_decode_chunks_equal_the_full_pass(oracle, dtype, head, group):
    """Prefill with the causal tile entry, keys and values appended to the
    cache; then chunks of 1, 1, 5, 16 and 40 new tokens through the cache."""
    n_batch, n_kv, prefill = 2, 2, 150
    chunks = (1, 1, 5, 16, 40)          # short 16-bit chunks: decode kernel; the rest: tile kernel
    total = prefill + sum(chunks)
    batch, kvb = n_batch * group * n_kv, n_batch * n_kv
    (Q, K, V), (qf, kf, vf) = H.make_qkv(29, batch, total, total, head, dtype, kv_batch=kvb)
    want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, synth.causal_mask(total, total),
                                         n_batch=n_batch, kv_repeat=group)
    Qd, Kd, Vd = Q.cuda(), K.cuda(), V.cuda()
    cache = KVCache(max_cache_size=total + 7)
    got, got_lse = [], []
    # prefill: the dense causal pass, then the cache takes its keys and values
    Qp, Kp, Vp = (t[:, :prefill].contiguous() for t in (Qd, Kd, Vd))
    lse, A = H.fresh_outputs(batch, prefill, head, dtype)
    hip_sdpa.sdpa_fwd_tile(Kp, Qp, None, lse, Vp, A, hip_sdpa.MASK_CAUSAL, n_batch=n_batch,
                           kv_group=group)
    cache.append(Kp, Vp)
    got.append(H.to_np(A))
    got_lse.append(H.to_np(lse))
    pos = prefill
    for rows in chunks:
        cache.append(Kd[:, pos:pos + rows].contiguous(), Vd[:, pos:pos + rows].contiguous())
        assert len(cache) == pos + rows
        lse, A = H.fresh_outputs(batch, rows, head, dtype)
        cache.attend(Qd[:, pos:pos + rows].contiguous(), lse, A, n_batch, group)
        got.append(H.to_np(A))
        got_lse.append(H.to_np(lse))
        pos += rows
    torch.cuda.synchronize()
    assert H.rel_fro(np.concatenate(got, axis=1), want) < H.TOL[dtype]
    assert H.rel_fro(np.concatenate(got_lse, axis=1), want_lse) < H.TOL[dtype]


def test_full_size_decode_step_through_the_cache():
    """The GQA decode configuration (8 x 8 key/value heads, group 4, head 128,
    8192 cached tokens + 16 new): append into a cache of 16384 rows, attend,
    and compare bit for bit with the decode over dense tensors."""
    n_batch, n_kv, group, head, old, new, cap = 8, 8, 4, 128, 8192, 16, 16384
    kvb, batch = n_batch * n_kv, n_batch * n_kv * group
    g = torch.Generator(device="cuda").manual_seed(77)
    K = torch.randn((kvb, old + new, head), generator=g, device="cuda").bfloat16()
    V = torch.randn((kvb, old + new, head), generator=g, device="cuda").bfloat16()
    Q = torch.randn((batch, new, head), generator=g, device="cuda").bfloat16()
    cache = KVCache(cap)
    cache.append(K[:, :old].contiguous(), V[:, :old].contiguous())
    cache.append(K[:, old:].contiguous(), V[:, old:].contiguous())
    assert len(cache) == old + new
    assert torch.equal(cache.k_partial, K) and torch.equal(cache.v_partial, V)
    lse, A = H.fresh_outputs(batch, new, head, "bf16")
    cache.attend(Q, lse, A, n_batch, group)
    ws = torch.empty(hip_sdpa.decode_workspace_bytes(K, Q, n_batch, group), dtype=torch.uint8,
                     device="cuda")
    lse2, A2 = H.fresh_outputs(batch, new, head, "bf16")
    hip_sdpa.sdpa_fwd_decode(K, Q, None, lse2, V, A2, hip_sdpa.MASK_CAUSAL, n_batch, group, ws,
                             causal_offset=old, flags=hip_sdpa.OVERWRITE)
    torch.cuda.synchronize()
    assert torch.equal(A.view(torch.int16), A2.view(torch.int16))
    assert torch.equal(lse, lse2)
    assert bool(torch.isfinite(lse).all())


@pytest.mark.parametrize("q_full,k_full", [(64, 64), (40, 64), (64, 40), (30, 30)])
def test_mask_slice_equals_the_checker(oracle, q_full, k_full):
    """KVCache.mask_slice == Sdpa._prepare_mask_for_kv_cache as the checker
    restates it, also when the mask is smaller than the cache on either axis."""
    rng = np.random.default_rng(q_full * 100 + k_full)
    mask = rng.random((q_full, k_full)) < 0.6                      # [queries, keys]
    cache = KVCache(64)
    z = torch.zeros((2, 1, 64), dtype=torch.bfloat16, device="cuda")
    for filled, q_seq in ((1, 1), (17, 16), (18, 1), (48, 30), (64, 16)):
        while len(cache) < filled:
            cache.append(z, z)
        got = cache.mask_slice(torch.from_numpy(mask).cuda(), q_seq).cpu().numpy()
        want = oracle.prepare_mask_for_kv_cache(mask.T, filled, q_seq).T
        assert np.array_equal(got, want), (filled, q_seq)


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
def test_attend_with_a_mask_given_as_values(oracle, dtype):
    """A bool mask that is not causal (a window plus the first key), sliced
    for the cached keys, chunks of 3 and 37 tokens."""
    head, n_batch, n_kv, group, prefill = 128, 2, 2, 4, 60
    chunks = (3, 37)
    total = prefill + sum(chunks)
    batch, kvb = n_batch * group * n_kv, n_batch * n_kv
    (Q, K, V), (qf, kf, vf) = H.make_qkv(37, batch, total, total, head, dtype, kv_batch=kvb)
    i = np.arange(total)
    full = (np.abs(i[:, None] - i[None, :]) <= 20) & (i[None, :] <= i[:, None])
    full[:, 0] = True                                              # [queries, keys]
    want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, full, n_batch=n_batch, kv_repeat=group)
    Qd, Kd, Vd = Q.cuda(), K.cuda(), V.cuda()
    mask_d = torch.from_numpy(full).cuda()
    cache = KVCache(total)
    cache.append(Kd[:, :prefill].contiguous(), Vd[:, :prefill].contiguous())
    pos = prefill
    for rows in chunks:
        cache.append(Kd[:, pos:pos + rows].contiguous(), Vd[:, pos:pos + rows].contiguous())
        lse, A = H.fresh_outputs(batch, rows, head, dtype)
        cache.attend(Qd[:, pos:pos + rows].contiguous(), lse, A, n_batch, group, mask=mask_d)
        torch.cuda.synchronize()
        assert H.rel_fro(H.to_np(A), want[:, pos:pos + rows]) < H.TOL[dtype]
        assert H.rel_fro(H.to_np(lse), want_lse[:, pos:pos + rows]) < H.TOL[dtype]
        pos += rows


@pytest.mark.parametrize("dtype", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("q_seq,k_seq,cap,n_batch,group,n_kv,head,mode", [
    (100, 300, 512, 2, 4, 2, 128, "causal"), (1, 77, 80, 3, 2, 2, 64, "causal"),
    (130, 130, 131, 1, 1, 3, 32, "causal"), (70, 200, 333, 2, 2, 1, 64, "bool"),
    (33, 1000, 1000, 1, 8, 1, 128, "none")])
def test_tile_entry_reading_the_cache(oracle, dtype, q_seq, k_seq, cap, n_batch, group, n_kv, head, mode):
    """The tile kernel over a cache whose unfilled rows hold NaN == the checker
    within the tolerance and == the same call over dense copies bit for bit."""
    print("case", dtype, q_seq, k_seq, cap, n_batch, group, n_kv, head, mode, flush=True)
    batch, kvb = n_batch * group * n_kv, n_batch * n_kv
    (Q, K, V), (qf, kf, vf) = H.make_qkv(41, batch, q_seq, k_seq, head, dtype, kv_batch=kvb)
    offset = k_seq - q_seq
    mask = None if mode == "none" else synth.causal_mask(q_seq, k_seq, offset)
    want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, mask, n_batch=n_batch, kv_repeat=group)
    Qd = Q.cuda()
    Kc = torch.full((kvb, cap, head), float("nan"), dtype=H.TORCH_DT[dtype], device="cuda")
    Vc = torch.full_like(Kc, float("nan"))
    Kc[:, :k_seq] = K.cuda()
    Vc[:, :k_seq] = V.cuda()
    m, mm = {"causal": (None, hip_sdpa.MASK_CAUSAL), "none": (None, hip_sdpa.MASK_NONE),
             "bool": (None if mask is None else torch.from_numpy(mask).cuda(), hip_sdpa.MASK_BOOL)}[mode]
    lse, A = H.fresh_outputs(batch, q_seq, head, dtype)
    hip_sdpa.sdpa_fwd_tile_cache(Kc, Vc, k_seq, Qd, m, lse, A, mm, n_batch, group,
                                 causal_offset=offset)
    lse2, A2 = H.fresh_outputs(batch, q_seq, head, dtype)
    hip_sdpa.sdpa_fwd_tile(K.cuda(), Qd, m, lse2, V.cuda(), A2, mm, n_batch=n_batch, kv_group=group,
                           causal_offset=offset)
    torch.cuda.synchronize()
    assert H.rel_fro(H.to_np(A), want) < H.TOL[dtype]
    assert H.rel_fro(H.to_np(lse), want_lse) < H.TOL[dtype]
    assert torch.equal(A.view(torch.int32 if dtype == "fp32" else torch.int16),
                       A2.view(torch.int32 if dtype == "fp32" else torch.int16))
    assert torch.equal(lse, lse2)
