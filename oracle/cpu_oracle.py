"""ctypes front-end of the CPU checker (test infrastructure only).

Only tests, the smoke check and the benchmark's CPU-baseline leg load this
module; the shipped library never does.  Arrays follow the NNTile tile layout:
Fortran order, which in numpy C-order terms is ``[batch, seq, head]`` for
K/Q/V/Y, ``[batch, seq]`` for logsumexp and ``[q_seq, k_seq]`` for the mask
(element (k, q) of the reference's ``[k_seq, q_seq]`` mask sits at
``k + q*k_seq``).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libnntile_cpu_oracle.so")
_lib = None

_i64 = ctypes.c_int64
_f32 = ctypes.c_float
_ptr = ctypes.c_void_p


def build(force=False):
    """Compile the checker with the Makefile beside this file."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-C", _HERE, "libnntile_cpu_oracle.so"])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.nntile_oracle_gemm_f32.argtypes = [
            ctypes.c_int, ctypes.c_int, _i64, _i64, _i64, _i64, _f32, _ptr,
            _ptr, _f32, _ptr]
        _lib.nntile_oracle_mask_scalar_f32.argtypes = [_i64, _i64, _ptr, _f32,
                                                       _ptr]
        _lib.nntile_oracle_maxsumexp_f32.argtypes = [_i64, _i64, _i64, _ptr,
                                                     _ptr]
        _lib.nntile_oracle_softmax_inplace_f32.argtypes = [
            _i64, _i64, _i64, _ptr, _f32, _ptr]
        _lib.nntile_oracle_logsumexp_f32.argtypes = [_i64, _ptr, _ptr]
        _lib.nntile_oracle_accumulate_maxsumexp_f32.argtypes = [_i64, _ptr,
                                                                _ptr]
        for name in ("fp32", "bf16", "fp16"):
            getattr(_lib, "nntile_oracle_accumulate_attn_output_" + name
                    ).argtypes = [_i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr]
        for name in ("f32_to_bf16", "bf16_to_f32", "f32_to_fp16",
                     "fp16_to_f32"):
            getattr(_lib, "nntile_oracle_" + name).argtypes = [_i64, _ptr,
                                                               _ptr]
        _lib.nntile_oracle_sdpa_vanilla_f32.argtypes = [
            _i64, _i64, _i64, _i64, _i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr,
            _ptr, _ptr, ctypes.c_int]
        _lib.nntile_oracle_sdpa_vanilla_f32.restype = ctypes.c_int
        _lib.nntile_oracle_sdpa_bruteforce_f64.argtypes = [
            _i64, _i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr]
        _lib.nntile_oracle_max_threads.restype = ctypes.c_int
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(_ptr)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def max_threads():
    return int(lib().nntile_oracle_max_threads())


# ---- 16-bit storage helpers (round to nearest even) -----------------------

def f32_to_bf16(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().nntile_oracle_f32_to_bf16(x.size, _p(x), _p(out))
    return out


def bf16_to_f32(x):
    x = _c(x, np.uint16)
    out = np.empty(x.shape, np.float32)
    lib().nntile_oracle_bf16_to_f32(x.size, _p(x), _p(out))
    return out


def f32_to_fp16(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().nntile_oracle_f32_to_fp16(x.size, _p(x), _p(out))
    return out


def fp16_to_f32(x):
    x = _c(x, np.uint16)
    out = np.empty(x.shape, np.float32)
    lib().nntile_oracle_fp16_to_f32(x.size, _p(x), _p(out))
    return out


# ---- codelet-level restatements -------------------------------------------

def gemm(transA, transB, m, n, k, batch, alpha, A, B, beta, C):
    """Batched column-major GEMM on flat fp32 buffers, C updated in place."""
    lib().nntile_oracle_gemm_f32(int(transA), int(transB), m, n, k, batch,
                                 alpha, _p(A), _p(B), beta, _p(C))


def mask_scalar(nrows, ncols, mask, val, data):
    lib().nntile_oracle_mask_scalar_f32(nrows, ncols, _p(mask), val, _p(data))


def maxsumexp(m, n, k, src, dst):
    lib().nntile_oracle_maxsumexp_f32(m, n, k, _p(src), _p(dst))


def softmax_inplace(m, n, k, stats, alpha, dst):
    lib().nntile_oracle_softmax_inplace_f32(m, n, k, _p(stats), alpha, _p(dst))


def logsumexp(nelems, stats, out):
    lib().nntile_oracle_logsumexp_f32(nelems, _p(stats), _p(out))


def accumulate_maxsumexp(nelems, src, dst):
    lib().nntile_oracle_accumulate_maxsumexp_f32(nelems, _p(src), _p(dst))


def accumulate_attn_output(dtype, head, seq, batch, src_lse, src_attn,
                           dst_lse, dst_attn):
    """dtype in {'fp32','bf16','fp16'}; 16-bit values are uint16 storage."""
    fn = getattr(lib(), "nntile_oracle_accumulate_attn_output_" + dtype)
    fn(head, seq, batch, _p(src_lse), _p(src_attn), _p(dst_lse), _p(dst_attn))


# ---- the composition --------------------------------------------------------

def sdpa_vanilla(K, Q, V, mask=None, k_tile=0, n_batch=None, kv_repeat=1,
                 nthreads=0):
    """gemm -> mask_scalar -> maxsumexp -> softmax_inplace -> gemm on fp32.

    K, V: [kv_batch, k_seq, head]; Q: [batch, q_seq, head] (C-order views of
    the Fortran tiles); mask: bool [q_seq, k_seq] C-order (= Fortran
    [k_seq, q_seq]) or None.  Query batch entry b reads K/V entry
    ``nb + n_batch*hkv`` with ``b = nb + n_batch*(g + kv_repeat*hkv)``.
    Returns (Y [batch, q_seq, head] fp32, lse [batch, q_seq] fp32).
    """
    K = _c(K, np.float32)
    Q = _c(Q, np.float32)
    V = _c(V, np.float32)
    batch, q_seq, head = Q.shape
    kv_batch, k_seq, _ = K.shape
    assert V.shape == K.shape and K.shape[2] == head
    if n_batch is None:
        if kv_repeat != 1:
            raise ValueError("n_batch is required when kv_repeat > 1")
        n_batch = batch
    assert kv_batch * kv_repeat == batch and batch % (n_batch * kv_repeat) == 0
    m = None
    if mask is not None:
        m = _c(mask, np.uint8)
        assert m.shape == (q_seq, k_seq)
    Y = np.empty((batch, q_seq, head), np.float32)
    lse = np.empty((batch, q_seq), np.float32)
    rc = lib().nntile_oracle_sdpa_vanilla_f32(
        head, q_seq, k_seq, batch, n_batch, kv_repeat, k_tile, _p(K), _p(Q),
        _p(m), _p(V), _p(Y), _p(lse), nthreads)
    if rc != 0:
        raise ValueError("bad sizes for sdpa_vanilla")
    return Y, lse


def sdpa_bruteforce_f64(K, Q, V, add_mask=None):
    """fp64 brute force with an additive [q_seq, k_seq] fp32 mask."""
    K = _c(K, np.float32)
    Q = _c(Q, np.float32)
    V = _c(V, np.float32)
    batch, q_seq, head = Q.shape
    k_seq = K.shape[1]
    m = None if add_mask is None else _c(add_mask, np.float32)
    A = np.empty((batch, q_seq, head), np.float64)
    lse = np.empty((batch, q_seq), np.float64)
    lib().nntile_oracle_sdpa_bruteforce_f64(q_seq, k_seq, head, batch, _p(K),
                                            _p(Q), _p(m), _p(V), _p(A),
                                            _p(lse))
    return A, lse


# ---- backward (numpy; test infrastructure like everything above) -------------

def sdpa_bwd_vanilla(K, Q, V, dY, mask=None):
    """Gradients of the forward composition, step by step as the reference's
    `Sdpa._backward_vanilla` (wrappers/python/nntile/layer/sdpa.py:595-698)
    takes them, in fp32:

        attn.grad  = V^T dY                                   (gemm, :606-618)
        v.grad    += dY attn^T                                (gemm, :623-635)
        s[q]       = sum_h y[h,q] dY[h,q]                     (sumprod_slice, :640-648)
        attn.grad  = (attn.grad - s[q]) * attn                (add_slice_inplace, multiply_inplace, :649-653)
        attn.grad  = 0 where the mask hides (k, q)            (mask_scalar, :656-660)
        k.grad    += scale Q attn.grad^T                      (gemm, :667-679)
        q.grad    += scale K attn.grad                        (gemm, :686-698)

    with attn = softmax over keys of scale K^T Q (+ mask), y = V attn as the
    forward pass left them.  K, Q, V, dY: [batch, seq, head] (C-order views of
    the Fortran tiles), mask: bool [q_seq, k_seq] or None.  Returns
    (dK, dQ, dV) as the increments that are added to the .grad tensors."""
    K = _c(K, np.float32)
    Q = _c(Q, np.float32)
    V = _c(V, np.float32)
    dY = _c(dY, np.float32)
    head = Q.shape[2]
    scale = np.float32(1.0) / np.sqrt(np.float32(head))
    # forward quantities, as the forward composition produces them
    scores = np.einsum("bkh,bqh->bkq", K, Q).astype(np.float32) * scale
    if mask is not None:
        scores = np.where(np.asarray(mask, bool).T[None], scores, np.float32(-np.inf))
    mx = scores.max(axis=1, keepdims=True)
    mx = np.where(np.isfinite(mx), mx, np.float32(0))
    e = np.exp(scores - mx, dtype=np.float32)
    sm = e.sum(axis=1, keepdims=True)
    attn = np.where(sm > 0, e / np.where(sm > 0, sm, 1), 0).astype(np.float32)
    y = np.einsum("bkh,bkq->bqh", V, attn).astype(np.float32)
    # backward steps
    dattn = np.einsum("bkh,bqh->bkq", V, dY).astype(np.float32)
    dV = np.einsum("bqh,bkq->bkh", dY, attn).astype(np.float32)
    s = np.einsum("bqh,bqh->bq", y, dY).astype(np.float32)
    dattn = (dattn - s[:, None, :]) * attn
    if mask is not None:
        dattn = np.where(np.asarray(mask, bool).T[None], dattn, np.float32(0))
    dK = scale * np.einsum("bqh,bkq->bkh", Q, dattn).astype(np.float32)
    dQ = scale * np.einsum("bkh,bkq->bqh", K, dattn).astype(np.float32)
    return dK.astype(np.float32), dQ.astype(np.float32), dV


def sdpa_bwd_flash_f64(K, Q, V, A, dA, lse, add_mask=None, kv_repeat=1, n_batch=None):
    """The flash form in fp64, with the forward output A and the logsumexp
    taken as given (they need not belong to K, Q, V), as the reference's test
    of its backward kernel computes it
    (tests/kernel/flash_sdpa_bwd_cudnn.cc:174-262):

        P[q,k]  = exp(scale q.k + mask[q,k] - lse[q])   (0 where the score is -inf)
        dP[q,k] = dA[q,:] . V[k,:]
        D[q]    = dA[q,:] . A[q,:]
        dS      = P (dP - D)
        dV[k,:] = sum_q P[q,k] dA[q,:];  dQ[q,:] = scale sum_k dS[q,k] K[k,:];
        dK[k,:] = scale sum_q dS[q,k] Q[q,:]

    add_mask: additive fp32 [q_seq, k_seq] or None.  With kv_repeat > 1 query
    batch entry b = nb + n_batch*(g + kv_repeat*hkv) reads K/V entry
    nb + n_batch*hkv and dK, dV sum over the group.  Returns (dK, dQ, dV)."""
    K = np.asarray(K, np.float64)
    Q = np.asarray(Q, np.float64)
    V = np.asarray(V, np.float64)
    A = np.asarray(A, np.float64)
    dA = np.asarray(dA, np.float64)
    lse = np.asarray(lse, np.float64)
    batch, q_seq, head = Q.shape
    kv_batch = K.shape[0]
    if n_batch is None:
        n_batch = batch if kv_repeat == 1 else None
    assert n_batch is not None and kv_batch * kv_repeat == batch
    scale = 1.0 / np.sqrt(float(head))
    dK = np.zeros_like(K)
    dV = np.zeros_like(V)
    dQ = np.zeros_like(Q)
    for b in range(batch):
        nb = b % n_batch
        hkv = (b // n_batch) // kv_repeat
        kv = nb + n_batch * hkv
        s = scale * (Q[b] @ K[kv].T)
        if add_mask is not None:
            s = s + np.asarray(add_mask, np.float64)
        with np.errstate(over="ignore", invalid="ignore"):
            p = np.where(np.isneginf(s), 0.0, np.exp(s - lse[b][:, None]))
        dp = dA[b] @ V[kv].T
        d = (dA[b] * A[b]).sum(axis=1)
        ds = p * (dp - d[:, None])
        dV[kv] += p.T @ dA[b]
        dQ[b] = scale * (ds @ K[kv])
        dK[kv] += scale * (ds.T @ Q[b])
    return dK, dQ, dV


def rope(sin, cos, src, backward=False):
    """Rotary embedding of a (2, m, n) tensor (memory order: the pair fastest,
    then the m positions of sin / cos, then n), in fp32 as the reference's
    repr_t (src/kernel/rope/cpu.cc:22-52):

        dst[2i,j]   = cos[i] src[2i,j] - sin[i] src[2i+1,j]
        dst[2i+1,j] = sin[i] src[2i,j] + cos[i] src[2i+1,j]

    backward=True is src/kernel/rope_backward/cpu.cc:22-53 (dy -> dx, written,
    not added): dx[2i] = c dy[2i] + s dy[2i+1], dx[2i+1] = c dy[2i+1] - s dy[2i].
    Returns a float32 array of src's shape (not yet rounded to the tile type)."""
    s = np.asarray(sin, np.float32).ravel()
    c = np.asarray(cos, np.float32).ravel()
    x = np.asarray(src, np.float32)
    m = s.size
    if m == 0 or x.size == 0:
        return np.zeros(x.shape, np.float32)
    v = x.reshape(-1, m, 2)
    a, b = v[..., 0], v[..., 1]
    out = np.empty_like(v)
    if backward:
        out[..., 0] = c * a + s * b
        out[..., 1] = c * b - s * a
    else:
        out[..., 0] = c * a - s * b
        out[..., 1] = s * a + c * b
    return out.reshape(x.shape)


def transpose(m, n, alpha, src):
    """dst[i*n + j] = alpha * src[i + j*m] (src/kernel/transpose/cpu.cc:21-43):
    src is an m x n matrix in Fortran order, dst its transpose in Fortran
    order, the product in fp32.  Returns the flat float32 dst."""
    x = np.asarray(src, np.float32).reshape(n, m)      # x[j, i] = src(i, j)
    return (np.float32(alpha) * np.ascontiguousarray(x.T)).reshape(-1)


# ---- key/value cache of the decode path --------------------------------------

def copy_intersection(src, src_offset, dst, dst_offset):
    """dst <- src where the two overlap, both placed in one global index space
    at their offsets (src/tensor/copy_intersection.cc:84-112; the tile loop
    behind it only distributes the same copy).  Arrays are indexed in the
    reference's axis order (numpy arrays whose axis i is the reference's axis
    i).  dst is changed in place and returned."""
    sl_s, sl_d = [], []
    for n_s, o_s, n_d, o_d in zip(src.shape, src_offset, dst.shape, dst_offset):
        if o_s + n_s <= o_d or o_d + n_d <= o_s:
            return dst
        if o_s < o_d:
            s0, d0 = o_d - o_s, 0
            n = min(n_s - s0, n_d)
        else:
            s0, d0 = 0, o_s - o_d
            n = min(n_d - d0, n_s)
        sl_s.append(slice(s0, s0 + n))
        sl_d.append(slice(d0, d0 + n))
    dst[tuple(sl_d)] = src[tuple(sl_s)]
    return dst


class KVCache:
    """KVCache of wrappers/python/nntile/layer/cache_utils.py:117-225 on numpy
    arrays in the reference's axis order ([head, seq, ...]): zeros of
    max_cache_size rows on the sequence axis, append at the filled size,
    k_partial / v_partial copy the filled part out."""

    def __init__(self, max_cache_size, seq_size_dim):
        self.max_cache_size, self.seq_size_dim = max_cache_size, seq_size_dim
        self.k = self.v = None
        self.k_cache_size = self.v_cache_size = 0

    def __len__(self):
        return self.k_cache_size

    def _zeros_like_cache(self, t):
        shape = list(t.shape)
        shape[self.seq_size_dim] = self.max_cache_size
        return np.zeros(shape, t.dtype)

    def append(self, k_partial, v_partial):
        assert k_partial.shape[self.seq_size_dim] == v_partial.shape[self.seq_size_dim]
        if self.k is None:
            self.k = self._zeros_like_cache(k_partial)
        off = [0] * k_partial.ndim
        off[self.seq_size_dim] = self.k_cache_size
        copy_intersection(k_partial, off, self.k, [0] * self.k.ndim)
        self.k_cache_size += k_partial.shape[self.seq_size_dim]
        if self.v is None:
            self.v = self._zeros_like_cache(v_partial)
        off = [0] * v_partial.ndim
        off[self.seq_size_dim] = self.v_cache_size
        copy_intersection(v_partial, off, self.v, [0] * self.v.ndim)
        self.v_cache_size += v_partial.shape[self.seq_size_dim]

    def _partial(self, full, size):
        shape = list(full.shape)
        shape[self.seq_size_dim] = size
        out = np.empty(shape, full.dtype)
        return copy_intersection(full, [0] * full.ndim, out, [0] * out.ndim)

    @property
    def k_partial(self):
        return self._partial(self.k, self.k_cache_size)

    @property
    def v_partial(self):
        return self._partial(self.v, self.v_cache_size)


def prepare_mask_for_kv_cache(mask, k_seq, q_seq):
    """The bool mask slice that goes with cached keys
    (wrappers/python/nntile/layer/sdpa.py:489-531).  mask: bool in the
    reference's axis order [keys, queries] (True = visible).  A mask that
    already has shape (k_seq, q_seq) is used as it is; otherwise ones of that
    shape, overwritten by the mask placed at [0, 0] against a destination
    placed at [0, k_seq - q_seq]: query column j takes the mask column of the
    token at position j + k_seq - q_seq."""
    mask = np.asarray(mask, bool)
    if mask.shape == (k_seq, q_seq):
        return mask
    out = np.ones((k_seq, q_seq), bool)
    return copy_intersection(mask, [0, 0], out, [0, k_seq - q_seq])


# ---- class of a mask tile ------------------------------------------------------

TILE_MIXED, TILE_OPEN, TILE_HIDDEN, TILE_CAUSAL = 0, 1, 2, 3


def mask_tile_class(mask, offset=0):
    """What one (query tile, key tile) task needs from its mask tile.  mask:
    [k_rows, q_cols] in the reference's axis order (the mask argument of
    src/tile/flash_sdpa_fwd_cudnn.cc:161-196), additive float (0 visible, -inf
    hidden) or bool (True visible).  HIDDEN: nothing visible (the task would
    change nothing); OPEN: everything visible; CAUSAL: visible exactly where
    k <= q + offset; MIXED: anything else, additive values other than 0 and
    -inf included.  No counterpart in the reference, which submits every
    pair; the definition is the specification."""
    m = np.asarray(mask)
    if m.dtype == bool:
        visible, other = m, np.zeros(m.shape, bool)
    else:
        m = m.astype(np.float32)
        visible = m == 0
        other = ~visible & ~np.isneginf(m)
    if other.any():
        return TILE_MIXED
    if visible.all():
        return TILE_OPEN
    if not visible.any():
        return TILE_HIDDEN
    k = np.arange(m.shape[0])[:, None]
    q = np.arange(m.shape[1])[None, :]
    return TILE_CAUSAL if np.array_equal(visible, k <= q + offset) else TILE_MIXED
