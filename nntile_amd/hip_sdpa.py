"""ctypes binding of libnntile_hip_sdpa.so plus thin torch-tensor front-ends.

torch is used for device memory and streams only; every computation goes
through the C ABI declared in include/nntile_hip_sdpa.h.  There is no fallback:
if the library is missing, loading fails.

Tensor convention: torch tensors are C-ordered views of NNTile's Fortran
tiles, i.e. K/V ``[kv_batch, k_seq, head]``, Q/A ``[batch, q_seq, head]``,
lse ``[batch, q_seq]`` fp32, mask ``[q_seq, k_seq]``.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libnntile_hip_sdpa.so")

MASK_ADDITIVE, MASK_NONE, MASK_CAUSAL, MASK_BOOL = 0, 1, 2, 3
MAX_TILES = 64
BWD_MAX_TILES = 32
OVERWRITE = 1
FORM_SHARED, FORM_SPLIT = 0x100, 0x200     # fix the workgroup shape (tests, tuning); 16-bit SPLIT: two groups of four wavefronts
FORM_WIDE = 0x4000                         # 16-bit analytic-mask calls: 256-query workgroups
# decode calls (tests, tuning): merge the key splits in a second launch; exchange
# the partials of the in-launch merge through device-scope fences
DECODE_SEPARATE_MERGE, DECODE_FENCED = 0x400, 0x800

OK, EINVAL, EUNSUPPORTED, ELAUNCH, EWORKSPACE = 0, -1, -2, -3, -4
TILE_MIXED, TILE_OPEN, TILE_HIDDEN, TILE_CAUSAL = 0, 1, 2, 3
_ERR = {EINVAL: "invalid argument", EUNSUPPORTED: "unsupported configuration",
        ELAUNCH: "HIP launch failed", EWORKSPACE: "workspace missing or too small"}

_i64 = ctypes.c_int64
_vp = ctypes.c_void_p


class TileArgs(ctypes.Structure):
    _fields_ = [("q_seq", _i64), ("k_seq", _i64), ("head", _i64),
                ("batch", _i64), ("n_batch", _i64), ("kv_group", _i64),
                ("mask_mode", ctypes.c_int32), ("flags", ctypes.c_int32),
                ("q_pos0", _i64), ("k_pos0", _i64), ("causal_offset", _i64),
                ("K", _vp), ("Q", _vp), ("mask", _vp), ("V", _vp),
                ("lse", _vp), ("A", _vp)]


class GridArgs(ctypes.Structure):
    _fields_ = [("q_seq", _i64), ("k_seq", _i64), ("q_tile", _i64),
                ("k_tile", _i64), ("head", _i64), ("batch", _i64),
                ("n_batch", _i64), ("kv_group", _i64),
                ("mask_mode", ctypes.c_int32), ("n_q_tiles", ctypes.c_int32),
                ("n_kv_tiles", ctypes.c_int32), ("flags", ctypes.c_int32),
                ("n_slabs", ctypes.c_int32), ("reserved", ctypes.c_int32),
                ("q_pos0", _i64), ("k_pos0", _i64), ("causal_offset", _i64),
                ("K", _vp * MAX_TILES), ("V", _vp * MAX_TILES),
                ("Q", _vp * MAX_TILES), ("lse", _vp * MAX_TILES),
                ("A", _vp * MAX_TILES)]


class BwdArgs(ctypes.Structure):
    _fields_ = [("q_seq", _i64), ("k_seq", _i64), ("head", _i64),
                ("batch", _i64), ("n_batch", _i64), ("kv_group", _i64),
                ("mask_mode", ctypes.c_int32), ("flags", ctypes.c_int32),
                ("q_pos0", _i64), ("k_pos0", _i64), ("causal_offset", _i64),
                ("K", _vp), ("Q", _vp), ("V", _vp), ("A", _vp), ("dA", _vp),
                ("mask", _vp), ("lse", _vp), ("dK", _vp), ("dQ", _vp),
                ("dV", _vp), ("workspace", _vp),
                ("workspace_bytes", ctypes.c_size_t)]


class BwdGridArgs(ctypes.Structure):
    _fields_ = [("q_seq", _i64), ("k_seq", _i64), ("q_tile", _i64),
                ("k_tile", _i64), ("head", _i64), ("batch", _i64),
                ("n_batch", _i64), ("kv_group", _i64),
                ("mask_mode", ctypes.c_int32), ("n_q_tiles", ctypes.c_int32),
                ("n_kv_tiles", ctypes.c_int32), ("flags", ctypes.c_int32),
                ("n_slabs", ctypes.c_int32), ("reserved", ctypes.c_int32),
                ("q_pos0", _i64), ("k_pos0", _i64), ("causal_offset", _i64),
                ("K", _vp * BWD_MAX_TILES), ("V", _vp * BWD_MAX_TILES),
                ("Q", _vp * BWD_MAX_TILES), ("A", _vp * BWD_MAX_TILES),
                ("dA", _vp * BWD_MAX_TILES), ("lse", _vp * BWD_MAX_TILES),
                ("dK", _vp * BWD_MAX_TILES), ("dQ", _vp * BWD_MAX_TILES),
                ("dV", _vp * BWD_MAX_TILES), ("workspace", _vp),
                ("workspace_bytes", ctypes.c_size_t)]


class VariableInterface(ctypes.Structure):
    _fields_ = [("id", ctypes.c_int), ("ptr", ctypes.c_size_t),
                ("dev_handle", ctypes.c_size_t), ("offset", ctypes.c_size_t),
                ("elemsize", ctypes.c_size_t)]


class FlashClArgs(ctypes.Structure):
    _fields_ = [("owner", _vp), ("seq", _i64), ("head", _i64), ("batch", _i64)]


class GridClArgs(ctypes.Structure):
    """nntile_hip_sdpa_grid_cl_args: the reference's args_t members, then the
    geometry of the tile grid."""
    _fields_ = [("owner", _vp), ("seq", _i64), ("head", _i64), ("batch", _i64),
                ("q_seq", _i64), ("k_seq", _i64), ("q_tile", _i64), ("k_tile", _i64),
                ("n_batch", _i64), ("kv_group", _i64),
                ("q_pos0", _i64), ("k_pos0", _i64), ("causal_offset", _i64),
                ("mask_mode", ctypes.c_int32), ("flags", ctypes.c_int32),
                ("n_q_tiles", ctypes.c_int32), ("n_kv_tiles", ctypes.c_int32),
                ("n_slabs", ctypes.c_int32), ("reserved", ctypes.c_int32)]


STREAM_PROVIDER = ctypes.CFUNCTYPE(_vp)

EXPORTS = (
    ["nntile_hip_flash_sdpa_fwd_" + t for t in ("bf16", "fp16", "fp32")]
    + ["nntile_hip_sdpa_fwd_tile_" + t for t in ("bf16", "fp16", "fp32")]
    + ["nntile_hip_sdpa_fwd_grid_" + t for t in ("bf16", "fp16", "fp32")]
    + ["nntile_hip_sdpa_fwd_decode_" + t for t in ("bf16", "fp16", "fp32")]
    + ["nntile_hip_sdpa_fwd_decode_workspace_bytes", "nntile_hip_sdpa_fwd_decode_workspace_bytes_fp32",
       "nntile_hip_sdpa_fwd_decode_static"]
    + ["nntile_hip_flash_sdpa_bwd_" + t for t in ("bf16", "fp16")]
    + ["nntile_hip_sdpa_bwd_tile_" + t for t in ("bf16", "fp16")]
    + ["nntile_hip_sdpa_bwd_workspace_bytes"]
    + ["nntile_hip_sdpa_bwd_grid_" + t for t in ("bf16", "fp16")]
    + ["nntile_hip_sdpa_bwd_grid_workspace_bytes"]
    + ["nntile_hip_flash_sdpa_bwd_codelet_" + t for t in ("bf16", "fp16")]
    + ["nntile_hip_accumulate_attn_output_" + t for t in ("bf16", "fp16", "fp32")]
    + ["nntile_hip_flash_sdpa_fwd_codelet_" + t for t in ("bf16", "fp16", "fp32")]
    + ["nntile_hip_rope_" + t for t in ("bf16", "fp16", "fp32")]
    + ["nntile_hip_rope_backward_" + t for t in ("bf16", "fp16", "fp32")]
    + ["nntile_hip_transpose_" + t for t in ("bf16", "fp16", "fp32")]
    + ["nntile_hip_kv_cache_append_" + t for t in ("bf16", "fp16", "fp32")]
    + ["nntile_hip_sdpa_fwd_decode_cache_" + t for t in ("bf16", "fp16", "fp32")]
    + ["nntile_hip_sdpa_fwd_decode_append_cache_" + t for t in ("bf16", "fp16", "fp32")]
    + ["nntile_hip_sdpa_fwd_tile_cache_" + t for t in ("bf16", "fp16", "fp32")]
    + ["nntile_hip_mask_tile_class_" + t for t in ("bf16", "fp16", "fp32", "bool")]
    + ["nntile_hip_sdpa_fwd_grid_codelet_" + t for t in ("bf16", "fp16", "fp32")]
    + ["nntile_hip_sdpa_bwd_grid_codelet_" + t for t in ("bf16", "fp16")]
    + ["nntile_hip_debug_decode_spin_limit", "nntile_hip_debug_decode_sync_timeouts",
       "nntile_hip_debug_decode_sync_misplaced"]
    + ["nntile_hip_set_stream_provider", "nntile_hip_sdpa_version"])

_lib = None


def lib():
    """The loaded C-ABI library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libnntile_hip_sdpa.so is missing: run `python -m nntile_amd.build`")
        L = ctypes.CDLL(LIB_PATH)
        for t in ("bf16", "fp16", "fp32"):
            f = getattr(L, "nntile_hip_flash_sdpa_fwd_" + t)
            f.argtypes = [_vp, _i64, _i64, _i64] + [_vp] * 8
            f.restype = ctypes.c_int
            f = getattr(L, "nntile_hip_sdpa_fwd_tile_" + t)
            f.argtypes = [_vp, ctypes.POINTER(TileArgs)]
            f.restype = ctypes.c_int
            f = getattr(L, "nntile_hip_sdpa_fwd_grid_" + t)
            f.argtypes = [_vp, ctypes.POINTER(GridArgs)]
            f.restype = ctypes.c_int
            f = getattr(L, "nntile_hip_accumulate_attn_output_" + t)
            f.argtypes = [_vp, _i64, _i64, _i64, _vp, _vp, _vp, _vp]
            f.restype = ctypes.c_int
            f = getattr(L, "nntile_hip_flash_sdpa_fwd_codelet_" + t)
            f.argtypes = [ctypes.POINTER(_vp), _vp]
            f.restype = None
        for t in ("bf16", "fp16", "fp32"):
            f = getattr(L, "nntile_hip_sdpa_fwd_decode_" + t)
            f.argtypes = [_vp, ctypes.POINTER(TileArgs), _vp, ctypes.c_size_t]
            f.restype = ctypes.c_int
            f = getattr(L, "nntile_hip_sdpa_fwd_decode_cache_" + t)
            f.argtypes = [_vp, ctypes.POINTER(TileArgs), _i64, _vp, ctypes.c_size_t]
            f.restype = ctypes.c_int
        for t in ("bf16", "fp16", "fp32"):
            f = getattr(L, "nntile_hip_sdpa_fwd_decode_append_cache_" + t)
            f.argtypes = [_vp, ctypes.POINTER(TileArgs), _i64, _vp, _vp, _i64, _vp, ctypes.c_size_t]
            f.restype = ctypes.c_int
        for t in ("bf16", "fp16"):
            f = getattr(L, "nntile_hip_flash_sdpa_bwd_" + t)
            f.argtypes = [_vp, _i64, _i64, _i64] + [_vp] * 13
            f.restype = ctypes.c_int
            f = getattr(L, "nntile_hip_flash_sdpa_bwd_codelet_" + t)
            f.argtypes = [ctypes.POINTER(_vp), _vp]
            f.restype = None
            f = getattr(L, "nntile_hip_sdpa_bwd_tile_" + t)
            f.argtypes = [_vp, ctypes.POINTER(BwdArgs)]
            f.restype = ctypes.c_int
            f = getattr(L, "nntile_hip_sdpa_bwd_grid_" + t)
            f.argtypes = [_vp, ctypes.POINTER(BwdGridArgs)]
            f.restype = ctypes.c_int
        for t in ("bf16", "fp16", "fp32"):
            for name in ("nntile_hip_rope_", "nntile_hip_rope_backward_"):
                f = getattr(L, name + t)
                f.argtypes = [_vp, _i64, _i64, _vp, _vp, _vp, _vp]
                f.restype = ctypes.c_int
        for t in ("bf16", "fp16", "fp32"):
            f = getattr(L, "nntile_hip_transpose_" + t)
            f.argtypes = [_vp, _i64, _i64, ctypes.c_float, _vp, _vp]
            f.restype = ctypes.c_int
            f = getattr(L, "nntile_hip_sdpa_fwd_tile_cache_" + t)
            f.argtypes = [_vp, ctypes.POINTER(TileArgs), _i64]
            f.restype = ctypes.c_int
            f = getattr(L, "nntile_hip_kv_cache_append_" + t)
            f.argtypes = [_vp] + [_i64] * 5 + [_vp] * 4
            f.restype = ctypes.c_int
        for t in ("bf16", "fp16", "fp32", "bool"):
            f = getattr(L, "nntile_hip_mask_tile_class_" + t)
            f.argtypes = [_vp, _i64, _i64, _vp, _i64, _vp, ctypes.POINTER(ctypes.c_int32)]
            f.restype = ctypes.c_int
        L.nntile_hip_sdpa_bwd_workspace_bytes.argtypes = [ctypes.POINTER(BwdArgs)]
        L.nntile_hip_sdpa_bwd_workspace_bytes.restype = ctypes.c_size_t
        L.nntile_hip_sdpa_bwd_grid_workspace_bytes.argtypes = [ctypes.POINTER(BwdGridArgs)]
        L.nntile_hip_sdpa_bwd_grid_workspace_bytes.restype = ctypes.c_size_t
        L.nntile_hip_sdpa_fwd_decode_workspace_bytes.argtypes = [ctypes.POINTER(TileArgs)]
        L.nntile_hip_sdpa_fwd_decode_workspace_bytes.restype = ctypes.c_size_t
        L.nntile_hip_sdpa_fwd_decode_workspace_bytes_fp32.argtypes = [ctypes.POINTER(TileArgs)]
        L.nntile_hip_sdpa_fwd_decode_workspace_bytes_fp32.restype = ctypes.c_size_t
        L.nntile_hip_sdpa_fwd_decode_static.argtypes = [_vp, ctypes.c_int32,
                                                        ctypes.POINTER(TileArgs)]
        L.nntile_hip_sdpa_fwd_decode_static.restype = ctypes.c_int
        L.nntile_hip_set_stream_provider.argtypes = [_vp]
        L.nntile_hip_set_stream_provider.restype = None
        L.nntile_hip_sdpa_version.restype = ctypes.c_char_p
        _lib = L
    return _lib


class SdpaError(RuntimeError):
    def __init__(self, code, what):
        super().__init__("%s: %s (code %d)" % (what, _ERR.get(code, "error"), code))
        self.code = code


def _check(code, what):
    if code != OK:
        raise SdpaError(code, what)


def dtype_name(t):
    if t.dtype == torch.bfloat16:
        return "bf16"
    if t.dtype == torch.float16:
        return "fp16"
    if t.dtype == torch.float32:
        return "fp32"
    raise TypeError("unsupported tile dtype %s" % t.dtype)


def _stream(stream):
    if stream is None:
        stream = torch.cuda.current_stream()
    return ctypes.c_void_p(stream.cuda_stream)


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _dev(*tensors):
    for t in tensors:
        if t is not None and not (t.is_cuda and t.is_contiguous()):
            raise ValueError("tiles must be contiguous device tensors")


def flash_sdpa_fwd(K, Q, mask, lse, V, A, scratch_lse=None, scratch_A=None, stream=None):
    """One square tile with an additive mask: the reference kernel call
    (execute_graph) with its argument order K, Q, mask, lse, V, A.
    scratch_lse ([batch, seq] fp32) and scratch_A (like A) are the reference's
    scratch tiles; the call may overwrite them."""
    _dev(K, Q, mask, lse, V, A, scratch_lse, scratch_A)
    batch, seq, head = Q.shape
    if scratch_lse is not None and scratch_lse.numel() * scratch_lse.element_size() < 4 * batch * seq:
        raise ValueError("scratch_lse is smaller than a logsumexp tile")
    fn = getattr(lib(), "nntile_hip_flash_sdpa_fwd_" + dtype_name(Q))
    _check(fn(_stream(stream), seq, head, batch, _ptr(K), _ptr(Q), _ptr(mask),
              _ptr(scratch_lse), _ptr(V), _ptr(scratch_A), _ptr(lse), _ptr(A)), "flash_sdpa_fwd")


def _tile_args(K, Q, mask, lse, V, A, mask_mode, n_batch, kv_group, q_pos0,
               k_pos0, causal_offset, flags=0):
    batch, q_seq, head = Q.shape
    k_seq = K.shape[1]
    a = TileArgs()
    a.q_seq, a.k_seq, a.head, a.batch = q_seq, k_seq, head, batch
    a.n_batch = batch if n_batch is None else n_batch
    a.kv_group = kv_group
    a.mask_mode = mask_mode
    a.flags = flags
    a.q_pos0, a.k_pos0, a.causal_offset = q_pos0, k_pos0, causal_offset
    a.K, a.Q, a.V = K.data_ptr(), Q.data_ptr(), V.data_ptr()
    a.mask = None if mask is None else mask.data_ptr()
    a.lse, a.A = lse.data_ptr(), A.data_ptr()
    return a


def sdpa_fwd_tile(K, Q, mask, lse, V, A, mask_mode, n_batch=None, kv_group=1,
                  q_pos0=0, k_pos0=0, causal_offset=0, flags=0, stream=None):
    _dev(K, Q, mask, lse, V, A)
    a = _tile_args(K, Q, mask, lse, V, A, mask_mode, n_batch, kv_group, q_pos0,
                   k_pos0, causal_offset, flags)
    fn = getattr(lib(), "nntile_hip_sdpa_fwd_tile_" + dtype_name(Q))
    _check(fn(_stream(stream), ctypes.byref(a)), "sdpa_fwd_tile")


def flash_sdpa_bwd(K, Q, V, A, dA, mask, lse, scratch_dQ, dK, dQ, dV, stream=None):
    """One square tile with an additive mask: the reference's backward kernel
    call (execute_graph) with its argument order; the gradients are added to
    dK, dQ, dV.  scratch_dQ is the reference's scratch tile for dQ."""
    _dev(K, Q, V, A, dA, mask, lse, scratch_dQ, dK, dQ, dV)
    batch, seq, head = Q.shape
    fn = getattr(lib(), "nntile_hip_flash_sdpa_bwd_" + dtype_name(Q))
    _check(fn(_stream(stream), seq, head, batch, _ptr(K), _ptr(Q), _ptr(V), _ptr(A),
              _ptr(dA), _ptr(mask), _ptr(lse), None, _ptr(scratch_dQ), None,
              _ptr(dK), _ptr(dQ), _ptr(dV)), "flash_sdpa_bwd")


def sdpa_bwd_workspace_bytes(q_seq, k_seq, batch, mask_mode):
    """Bytes of workspace sdpa_bwd_tile wants for these shapes."""
    a = BwdArgs()
    a.q_seq, a.k_seq, a.batch, a.mask_mode = q_seq, k_seq, batch, mask_mode
    return lib().nntile_hip_sdpa_bwd_workspace_bytes(ctypes.byref(a))


def sdpa_bwd_tile(K, Q, V, A, dA, mask, lse, dK, dQ, dV, mask_mode, n_batch=None,
                  kv_group=1, q_pos0=0, k_pos0=0, causal_offset=0, flags=0,
                  workspace=None, stream=None):
    """Backward of one (query tile, key tile) pair; the gradients are added to
    dK, dQ, dV (written with flags=OVERWRITE)."""
    _dev(K, Q, V, A, dA, mask, lse, dK, dQ, dV, workspace)
    batch, q_seq, head = Q.shape
    k_seq = K.shape[1]
    a = BwdArgs()
    a.q_seq, a.k_seq, a.head, a.batch = q_seq, k_seq, head, batch
    a.n_batch = batch if n_batch is None else n_batch
    a.kv_group = kv_group
    a.mask_mode = mask_mode
    if workspace is None:
        need = lib().nntile_hip_sdpa_bwd_workspace_bytes(ctypes.byref(a))
        workspace = torch.empty(need, dtype=torch.uint8, device=Q.device)
    a.flags = flags
    a.q_pos0, a.k_pos0, a.causal_offset = q_pos0, k_pos0, causal_offset
    a.K, a.Q, a.V, a.A, a.dA = (t.data_ptr() for t in (K, Q, V, A, dA))
    a.mask = None if mask is None else mask.data_ptr()
    a.lse = lse.data_ptr()
    a.dK, a.dQ, a.dV = dK.data_ptr(), dQ.data_ptr(), dV.data_ptr()
    a.workspace = workspace.data_ptr()
    a.workspace_bytes = workspace.numel() * workspace.element_size()
    fn = getattr(lib(), "nntile_hip_sdpa_bwd_tile_" + dtype_name(Q))
    _check(fn(_stream(stream), ctypes.byref(a)), "sdpa_bwd_tile")


def _grid_args(K_tiles, Q_tiles, lse_tiles, V_tiles, A_tiles, q_seq, k_seq, q_tile, k_tile,
               mask_mode, n_batch, kv_group, q_pos0, k_pos0, causal_offset, flags, n_slabs):
    _dev(*K_tiles, *Q_tiles, *lse_tiles, *V_tiles, *A_tiles)
    batch, _, head = Q_tiles[0].shape
    if (len(Q_tiles) > MAX_TILES or len(K_tiles) > MAX_TILES or n_slabs < 1
            or len(Q_tiles) % n_slabs or len(K_tiles) % n_slabs):
        raise SdpaError(EINVAL, "sdpa_fwd_grid")
    a = GridArgs()
    a.q_seq, a.k_seq, a.q_tile, a.k_tile, a.head = q_seq, k_seq, q_tile, k_tile, head
    a.batch = batch
    a.n_batch = batch if n_batch is None else n_batch
    a.kv_group = kv_group
    a.mask_mode = mask_mode
    a.flags = flags
    a.n_slabs = n_slabs
    a.n_q_tiles, a.n_kv_tiles = len(Q_tiles) // n_slabs, len(K_tiles) // n_slabs
    a.q_pos0, a.k_pos0, a.causal_offset = q_pos0, k_pos0, causal_offset
    for i, (k, v) in enumerate(zip(K_tiles, V_tiles)):
        a.K[i], a.V[i] = k.data_ptr(), v.data_ptr()
    for i, (q, l, o) in enumerate(zip(Q_tiles, lse_tiles, A_tiles)):
        a.Q[i], a.lse[i], a.A[i] = q.data_ptr(), l.data_ptr(), o.data_ptr()
    return a


def sdpa_fwd_grid(K_tiles, Q_tiles, lse_tiles, V_tiles, A_tiles, q_seq, k_seq,
                  q_tile, k_tile, mask_mode, n_batch=None, kv_group=1,
                  q_pos0=0, k_pos0=0, causal_offset=0, flags=0, stream=None, n_slabs=1):
    """All key tiles merged into all query tiles in one launch.  Tiles are
    lists of separately allocated tensors [batch, rows, head]; with n_slabs > 1
    the lists hold the tiles of slab 0, then those of slab 1, ... (the tiles
    along the batch axes, `batch` entries each)."""
    a = _grid_args(K_tiles, Q_tiles, lse_tiles, V_tiles, A_tiles, q_seq, k_seq, q_tile, k_tile,
                   mask_mode, n_batch, kv_group, q_pos0, k_pos0, causal_offset, flags, n_slabs)
    fn = getattr(lib(), "nntile_hip_sdpa_fwd_grid_" + dtype_name(Q_tiles[0]))
    _check(fn(_stream(stream), ctypes.byref(a)), "sdpa_fwd_grid")
    return a


def _bwd_grid_args(K_tiles, Q_tiles, V_tiles, A_tiles, dA_tiles, lse_tiles, dK_tiles, dQ_tiles,
                   dV_tiles, q_seq, k_seq, q_tile, k_tile, mask_mode, n_batch, kv_group, q_pos0,
                   k_pos0, causal_offset, flags, workspace, n_slabs=1):
    batch, _, head = Q_tiles[0].shape
    if (len(Q_tiles) > BWD_MAX_TILES or len(K_tiles) > BWD_MAX_TILES or n_slabs < 1
            or len(Q_tiles) % n_slabs or len(K_tiles) % n_slabs):
        raise SdpaError(EINVAL, "sdpa_bwd_grid")
    a = BwdGridArgs()
    a.q_seq, a.k_seq, a.q_tile, a.k_tile, a.head = q_seq, k_seq, q_tile, k_tile, head
    a.batch = batch
    a.n_batch = batch if n_batch is None else n_batch
    a.kv_group = kv_group
    a.mask_mode = mask_mode
    a.flags = flags
    a.n_slabs = n_slabs
    a.n_q_tiles, a.n_kv_tiles = len(Q_tiles) // n_slabs, len(K_tiles) // n_slabs
    a.q_pos0, a.k_pos0, a.causal_offset = q_pos0, k_pos0, causal_offset
    for i, (k, v, dk, dv) in enumerate(zip(K_tiles, V_tiles, dK_tiles, dV_tiles)):
        a.K[i], a.V[i], a.dK[i], a.dV[i] = (t.data_ptr() for t in (k, v, dk, dv))
    for i, ts in enumerate(zip(Q_tiles, A_tiles, dA_tiles, lse_tiles, dQ_tiles)):
        a.Q[i], a.A[i], a.dA[i], a.lse[i], a.dQ[i] = (t.data_ptr() for t in ts)
    a.workspace = workspace.data_ptr()
    a.workspace_bytes = workspace.numel() * workspace.element_size()
    return a


def sdpa_bwd_grid(K_tiles, Q_tiles, V_tiles, A_tiles, dA_tiles, lse_tiles, dK_tiles, dQ_tiles,
                  dV_tiles, q_seq, k_seq, q_tile, k_tile, mask_mode, n_batch=None, kv_group=1,
                  q_pos0=0, k_pos0=0, causal_offset=0, flags=0, workspace=None, stream=None,
                  n_slabs=1):
    """The backward of every (query tile, key tile) pair in one call: dQ of a
    query tile sums over the key tiles, dK and dV of a key tile over the query
    tiles; the gradients are added to dK, dQ, dV (written with
    flags=OVERWRITE).  Tiles are lists of separately allocated tensors
    [batch, rows, head] (lse: [batch, rows]); with n_slabs > 1 the lists hold
    the tiles of slab 0, then those of slab 1, ..."""
    every = (*K_tiles, *Q_tiles, *V_tiles, *A_tiles, *dA_tiles, *lse_tiles, *dK_tiles,
             *dQ_tiles, *dV_tiles)
    _dev(*every, workspace)
    if workspace is None:
        workspace = torch.empty(4 * n_slabs * q_seq * Q_tiles[0].shape[0], dtype=torch.uint8,
                                device=Q_tiles[0].device)
    a = _bwd_grid_args(K_tiles, Q_tiles, V_tiles, A_tiles, dA_tiles, lse_tiles, dK_tiles,
                       dQ_tiles, dV_tiles, q_seq, k_seq, q_tile, k_tile, mask_mode, n_batch,
                       kv_group, q_pos0, k_pos0, causal_offset, flags, workspace, n_slabs)
    fn = getattr(lib(), "nntile_hip_sdpa_bwd_grid_" + dtype_name(Q_tiles[0]))
    _check(fn(_stream(stream), ctypes.byref(a)), "sdpa_bwd_grid")


def plan_bwd_grid(K_tiles, Q_tiles, V_tiles, A_tiles, dA_tiles, lse_tiles, dK_tiles, dQ_tiles,
                  dV_tiles, q_seq, k_seq, q_tile, k_tile, mask_mode, workspace, n_batch=None,
                  kv_group=1, q_pos0=0, k_pos0=0, causal_offset=0, flags=0, n_slabs=1):
    every = (*K_tiles, *Q_tiles, *V_tiles, *A_tiles, *dA_tiles, *lse_tiles, *dK_tiles,
             *dQ_tiles, *dV_tiles, workspace)
    _dev(*every)
    a = _bwd_grid_args(K_tiles, Q_tiles, V_tiles, A_tiles, dA_tiles, lse_tiles, dK_tiles,
                       dQ_tiles, dV_tiles, q_seq, k_seq, q_tile, k_tile, mask_mode, n_batch,
                       kv_group, q_pos0, k_pos0, causal_offset, flags, workspace, n_slabs)
    fn = getattr(lib(), "nntile_hip_sdpa_bwd_grid_" + dtype_name(Q_tiles[0]))
    return Plan(fn, a, "sdpa_bwd_grid", keep=every)


class Plan:
    """A fully prepared call: argument block built once, launched many times.
    NNTile tiles keep their addresses from step to step, so a layer prepares
    its calls once; `launch` costs one foreign call."""

    def __init__(self, fn, args, what, extra=(), keep=()):
        self._fn, self._args, self._what, self._extra = fn, args, what, extra
        self._keep = keep          # tensors whose memory the call refers to

    def launch(self, stream=None):
        rc = self._fn(_stream(stream), ctypes.byref(self._args), *self._extra)
        if rc != OK:
            raise SdpaError(rc, self._what)


class FlashPlan:
    """flash_sdpa_fwd (the reference kernel call, scratch tiles included)
    prepared once; `launch` costs one foreign call."""

    def __init__(self, K, Q, mask, lse, V, A, scratch_lse=None, scratch_A=None):
        _dev(K, Q, mask, lse, V, A, scratch_lse, scratch_A)
        batch, seq, head = Q.shape
        if scratch_lse is not None and scratch_lse.numel() * scratch_lse.element_size() < 4 * batch * seq:
            raise ValueError("scratch_lse is smaller than a logsumexp tile")
        self._fn = getattr(lib(), "nntile_hip_flash_sdpa_fwd_" + dtype_name(Q))
        self._args = (seq, head, batch, _ptr(K), _ptr(Q), _ptr(mask), _ptr(scratch_lse), _ptr(V),
                      _ptr(scratch_A), _ptr(lse), _ptr(A))
        self._keep = (K, Q, mask, lse, V, A, scratch_lse, scratch_A)

    def launch(self, stream=None):
        rc = self._fn(_stream(stream), *self._args)
        if rc != OK:
            raise SdpaError(rc, "flash_sdpa_fwd")


def plan_grid(K_tiles, Q_tiles, lse_tiles, V_tiles, A_tiles, q_seq, k_seq, q_tile, k_tile,
              mask_mode, n_batch=None, kv_group=1, q_pos0=0, k_pos0=0, causal_offset=0, flags=0,
              n_slabs=1):
    a = _grid_args(K_tiles, Q_tiles, lse_tiles, V_tiles, A_tiles, q_seq, k_seq, q_tile, k_tile,
                   mask_mode, n_batch, kv_group, q_pos0, k_pos0, causal_offset, flags, n_slabs)
    fn = getattr(lib(), "nntile_hip_sdpa_fwd_grid_" + dtype_name(Q_tiles[0]))
    return Plan(fn, a, "sdpa_fwd_grid",
                keep=(K_tiles, Q_tiles, lse_tiles, V_tiles, A_tiles))


def plan_tile(K, Q, mask, lse, V, A, mask_mode, n_batch=None, kv_group=1, q_pos0=0, k_pos0=0,
              causal_offset=0, flags=0):
    _dev(K, Q, mask, lse, V, A)
    a = _tile_args(K, Q, mask, lse, V, A, mask_mode, n_batch, kv_group, q_pos0, k_pos0,
                   causal_offset, flags)
    fn = getattr(lib(), "nntile_hip_sdpa_fwd_tile_" + dtype_name(Q))
    return Plan(fn, a, "sdpa_fwd_tile", keep=(K, Q, mask, lse, V, A))


def plan_decode(K, Q, mask, lse, V, A, mask_mode, n_batch, kv_group, workspace, q_pos0=0,
                k_pos0=0, causal_offset=0, flags=0):
    _dev(K, Q, mask, lse, V, A, workspace)
    a = _tile_args(K, Q, mask, lse, V, A, mask_mode, n_batch, kv_group, q_pos0, k_pos0,
                   causal_offset, flags)
    fn = getattr(lib(), "nntile_hip_sdpa_fwd_decode_" + dtype_name(Q))
    nbytes = workspace.numel() * workspace.element_size()
    return Plan(fn, a, "sdpa_fwd_decode", extra=(_ptr(workspace), nbytes),
                keep=(K, Q, mask, lse, V, A, workspace))


def decode_sync_timeouts():
    """Merge workgroups of in-launch decode merges that gave up waiting for a
    split since the library was loaded (diagnostic; blocks)."""
    f = lib().nntile_hip_debug_decode_sync_timeouts
    f.restype = ctypes.c_longlong
    return int(f())


def decode_sync_misplaced():
    """Merge workgroups of in-launch decode merges that found a split of their
    unit on another XCD than their own since the library was loaded (they
    leave their rows untouched; diagnostic; blocks)."""
    f = lib().nntile_hip_debug_decode_sync_misplaced
    f.restype = ctypes.c_longlong
    return int(f())


def decode_spin_limit(ticks):
    """Sets the longest wait of a merge workgroup for a split, in ticks of the
    100 MHz clock; returns the previous value (diagnostic)."""
    f = lib().nntile_hip_debug_decode_spin_limit
    f.argtypes, f.restype = [ctypes.c_ulonglong], ctypes.c_ulonglong
    return int(f(ticks))


def _decode_ws_fn(Q):
    return getattr(lib(), "nntile_hip_sdpa_fwd_decode_workspace_bytes"
                   + ("_fp32" if dtype_name(Q) == "fp32" else ""))


def decode_workspace_bytes(K, Q, n_batch, kv_group):
    a = _tile_args(K, Q, None, Q, K, Q, MASK_NONE, n_batch, kv_group, 0, 0, 0)
    return int(_decode_ws_fn(Q)(ctypes.byref(a)))


def sdpa_fwd_decode(K, Q, mask, lse, V, A, mask_mode, n_batch, kv_group,
                    workspace, q_pos0=0, k_pos0=0, causal_offset=0, flags=0,
                    stream=None):
    """K, V: [n_head_kv*n_batch, k_seq, head]; Q, A:
    [n_head_kv*kv_group*n_batch, q_seq, head]; workspace: a device byte
    tensor of at least decode_workspace_bytes()."""
    _dev(K, Q, mask, lse, V, A, workspace)
    a = _tile_args(K, Q, mask, lse, V, A, mask_mode, n_batch, kv_group, q_pos0,
                   k_pos0, causal_offset, flags)
    fn = getattr(lib(), "nntile_hip_sdpa_fwd_decode_" + dtype_name(Q))
    nbytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    _check(fn(_stream(stream), ctypes.byref(a), _ptr(workspace), nbytes),
           "sdpa_fwd_decode")


DECODE_STATIC_SCRATCH_BYTES = 16 << 20


def sdpa_fwd_decode_static(K, Q, mask, lse, V, A, mask_mode, n_batch, kv_group, q_pos0=0,
                           k_pos0=0, causal_offset=0, flags=0, stream=None):
    """sdpa_fwd_decode with the split partials in the library's own device
    array (at most DECODE_STATIC_SCRATCH_BYTES): no workspace, no allocation."""
    _dev(K, Q, mask, lse, V, A)
    a = _tile_args(K, Q, mask, lse, V, A, mask_mode, n_batch, kv_group, q_pos0,
                   k_pos0, causal_offset, flags)
    code = {"bf16": 0, "fp16": 1}.get(dtype_name(Q), -1)
    _check(lib().nntile_hip_sdpa_fwd_decode_static(_stream(stream), code, ctypes.byref(a)),
           "sdpa_fwd_decode_static")


def kv_cache_append(k_new, v_new, k_cache, v_cache, filled, stream=None):
    """Write k_new, v_new ([entries, rows, head]) behind the `filled` rows of
    k_cache, v_cache ([entries, capacity, head])."""
    _dev(k_new, v_new, k_cache, v_cache)
    entries, rows, head = k_new.shape
    if (tuple(v_new.shape) != (entries, rows, head) or k_cache.shape != v_cache.shape
            or k_cache.shape[0] != entries or k_cache.shape[2] != head):
        raise SdpaError(EINVAL, "kv_cache_append")
    fn = getattr(lib(), "nntile_hip_kv_cache_append_" + dtype_name(k_cache))
    _check(fn(_stream(stream), head, rows, entries, k_cache.shape[1], filled, _ptr(k_new),
              _ptr(v_new), _ptr(k_cache), _ptr(v_cache)), "kv_cache_append")


def plan_kv_cache_append(k_new, v_new, k_cache, v_cache, filled):
    """kv_cache_append prepared once for a fixed position (a benchmark's or a
    graph's step); `launch(stream)` costs one foreign call."""
    _dev(k_new, v_new, k_cache, v_cache)
    entries, rows, head = k_new.shape
    if (tuple(v_new.shape) != (entries, rows, head) or k_cache.shape != v_cache.shape
            or k_cache.shape[0] != entries or k_cache.shape[2] != head):
        raise SdpaError(EINVAL, "kv_cache_append")
    fn = getattr(lib(), "nntile_hip_kv_cache_append_" + dtype_name(k_cache))
    args = (head, rows, entries, k_cache.shape[1], filled, _ptr(k_new), _ptr(v_new),
            _ptr(k_cache), _ptr(v_cache))

    class _Append:
        def launch(self, stream=None):
            _check(fn(_stream(stream), *args), "kv_cache_append")

    plan = _Append()
    plan._keep = (k_new, v_new, k_cache, v_cache)
    return plan


def _cache_args(K_cache, V_cache, k_seq, Q, mask, lse, A, mask_mode, n_batch, kv_group, q_pos0,
                k_pos0, causal_offset, flags):
    a = _tile_args(K_cache, Q, mask, lse, V_cache, A, mask_mode, n_batch, kv_group, q_pos0,
                   k_pos0, causal_offset, flags)
    a.k_seq = k_seq
    return a


def sdpa_fwd_decode_cache(K_cache, V_cache, k_seq, Q, mask, lse, A, mask_mode, n_batch,
                          kv_group, workspace, q_pos0=0, k_pos0=0, causal_offset=0, flags=0,
                          stream=None):
    """sdpa_fwd_decode over the first k_seq rows of every entry of the caches
    ([n_head_kv*n_batch, capacity, head]), read where they lie."""
    _dev(K_cache, V_cache, Q, mask, lse, A, workspace)
    if K_cache.shape != V_cache.shape:
        raise SdpaError(EINVAL, "sdpa_fwd_decode_cache")
    a = _cache_args(K_cache, V_cache, k_seq, Q, mask, lse, A, mask_mode, n_batch, kv_group,
                    q_pos0, k_pos0, causal_offset, flags)
    fn = getattr(lib(), "nntile_hip_sdpa_fwd_decode_cache_" + dtype_name(Q))
    nbytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    _check(fn(_stream(stream), ctypes.byref(a), K_cache.shape[1], _ptr(workspace), nbytes),
           "sdpa_fwd_decode_cache")


def sdpa_fwd_tile_cache(K_cache, V_cache, k_seq, Q, mask, lse, A, mask_mode, n_batch=None,
                        kv_group=1, q_pos0=0, k_pos0=0, causal_offset=0, flags=0, stream=None):
    """sdpa_fwd_tile over the first k_seq rows of every entry of the caches
    ([entries, capacity, head]), read where they lie; any chunk length, fp32
    included."""
    _dev(K_cache, V_cache, Q, mask, lse, A)
    if K_cache.shape != V_cache.shape:
        raise SdpaError(EINVAL, "sdpa_fwd_tile_cache")
    a = _cache_args(K_cache, V_cache, k_seq, Q, mask, lse, A, mask_mode, n_batch, kv_group,
                    q_pos0, k_pos0, causal_offset, flags)
    fn = getattr(lib(), "nntile_hip_sdpa_fwd_tile_cache_" + dtype_name(Q))
    _check(fn(_stream(stream), ctypes.byref(a), K_cache.shape[1]), "sdpa_fwd_tile_cache")


def plan_decode_cache(K_cache, V_cache, k_seq, Q, mask, lse, A, mask_mode, n_batch, kv_group,
                      workspace, q_pos0=0, k_pos0=0, causal_offset=0, flags=0):
    _dev(K_cache, V_cache, Q, mask, lse, A, workspace)
    a = _cache_args(K_cache, V_cache, k_seq, Q, mask, lse, A, mask_mode, n_batch, kv_group,
                    q_pos0, k_pos0, causal_offset, flags)
    fn = getattr(lib(), "nntile_hip_sdpa_fwd_decode_cache_" + dtype_name(Q))
    nbytes = workspace.numel() * workspace.element_size()
    return Plan(fn, a, "sdpa_fwd_decode_cache",
                extra=(K_cache.shape[1], _ptr(workspace), nbytes),
                keep=(K_cache, V_cache, Q, mask, lse, A, workspace))


def _append_cache_call(k_new, v_new, K_cache, V_cache, k_seq, Q, mask, lse, A, mask_mode, n_batch,
                       kv_group, workspace, q_pos0, k_pos0, causal_offset, flags):
    _dev(k_new, v_new, K_cache, V_cache, Q, mask, lse, A, workspace)
    entries, rows, head = k_new.shape
    if (K_cache.shape != V_cache.shape or tuple(v_new.shape) != (entries, rows, head)
            or K_cache.shape[0] != entries or K_cache.shape[2] != head or rows > k_seq
            or k_new.dtype != K_cache.dtype):
        raise SdpaError(EINVAL, "sdpa_fwd_decode_append_cache")
    a = _cache_args(K_cache, V_cache, k_seq, Q, mask, lse, A, mask_mode, n_batch, kv_group,
                    q_pos0, k_pos0, causal_offset, flags)
    fn = getattr(lib(), "nntile_hip_sdpa_fwd_decode_append_cache_" + dtype_name(Q))
    nbytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    extra = (K_cache.shape[1], _ptr(k_new), _ptr(v_new), rows, _ptr(workspace), nbytes)
    return fn, a, extra


def sdpa_fwd_decode_append_cache(k_new, v_new, K_cache, V_cache, k_seq, Q, mask, lse, A, mask_mode,
                                 n_batch, kv_group, workspace, q_pos0=0, k_pos0=0,
                                 causal_offset=0, flags=0, stream=None):
    """kv_cache_append of k_new, v_new ([entries, rows, head]) behind the
    k_seq - rows filled rows of the caches and sdpa_fwd_decode_cache over the
    k_seq rows, in one launch."""
    fn, a, extra = _append_cache_call(k_new, v_new, K_cache, V_cache, k_seq, Q, mask, lse, A,
                                      mask_mode, n_batch, kv_group, workspace, q_pos0, k_pos0,
                                      causal_offset, flags)
    _check(fn(_stream(stream), ctypes.byref(a), *extra), "sdpa_fwd_decode_append_cache")


def plan_decode_append_cache(k_new, v_new, K_cache, V_cache, k_seq, Q, mask, lse, A, mask_mode,
                             n_batch, kv_group, workspace, q_pos0=0, k_pos0=0, causal_offset=0,
                             flags=0):
    fn, a, extra = _append_cache_call(k_new, v_new, K_cache, V_cache, k_seq, Q, mask, lse, A,
                                      mask_mode, n_batch, kv_group, workspace, q_pos0, k_pos0,
                                      causal_offset, flags)
    return Plan(fn, a, "sdpa_fwd_decode_append_cache", extra=extra,
                keep=(k_new, v_new, K_cache, V_cache, Q, mask, lse, A, workspace))


def decode_cache_workspace_bytes(k_seq, Q, n_batch, kv_group):
    a = TileArgs()
    a.batch, a.q_seq, a.head = Q.shape
    a.k_seq, a.n_batch, a.kv_group = k_seq, n_batch, kv_group
    return int(_decode_ws_fn(Q)(ctypes.byref(a)))


def mask_tile_class(mask, offset=0, workspace=None, stream=None):
    """Class (TILE_*) of one mask tile: a [q_cols, k_rows] C-ordered device
    tensor (NNTile's [k_rows, q_cols]), additive in a tile type or bool,
    against the rule `key <= query + offset`.  Blocking."""
    _dev(mask, workspace)
    if mask.dim() != 2 or not mask.is_contiguous():
        raise SdpaError(EINVAL, "mask_tile_class")
    if workspace is None:
        workspace = torch.empty(1, dtype=torch.int32, device=mask.device)
    q_cols, k_rows = mask.shape
    name = "bool" if mask.dtype in (torch.bool, torch.uint8) else dtype_name(mask)
    out = ctypes.c_int32(-1)
    fn = getattr(lib(), "nntile_hip_mask_tile_class_" + name)
    _check(fn(_stream(stream), k_rows, q_cols, _ptr(mask), offset, _ptr(workspace),
              ctypes.byref(out)), "mask_tile_class")
    return out.value


def accumulate_attn_output(src_lse, src_attn, dst_lse, dst_attn, stream=None):
    """dst <- merge(dst, src) row by row; attn tiles [batch, seq, head]."""
    _dev(src_lse, src_attn, dst_lse, dst_attn)
    batch, seq, head = dst_attn.shape
    fn = getattr(lib(), "nntile_hip_accumulate_attn_output_" + dtype_name(dst_attn))
    _check(fn(_stream(stream), head, seq, batch, _ptr(src_lse), _ptr(src_attn),
              _ptr(dst_lse), _ptr(dst_attn)), "accumulate_attn_output")


def rope(sin, cos, src, dst, backward=False, stream=None):
    """Rotary embedding of src (memory order (2, m, n), m = sin.numel()) into
    dst; backward=True applies the transposed rotation (dy -> dx)."""
    _dev(sin, cos, src, dst)
    m = sin.numel()
    if cos.numel() != m or src.numel() != dst.numel() or (m and src.numel() % (2 * m)):
        raise SdpaError(EINVAL, "rope")
    n = src.numel() // (2 * m) if m else 0
    name = "nntile_hip_rope_backward_" if backward else "nntile_hip_rope_"
    fn = getattr(lib(), name + dtype_name(src))
    _check(fn(_stream(stream), m, n, _ptr(sin), _ptr(cos), _ptr(src), _ptr(dst)), "rope")


def transpose(alpha, src, dst, m, n, stream=None):
    """dst = alpha * src^T; src is m x n in Fortran order (memory order of a
    C-ordered [n, m] tensor), dst n x m in Fortran order."""
    _dev(src, dst)
    if src.numel() != m * n or dst.numel() != m * n:
        raise SdpaError(EINVAL, "transpose")
    fn = getattr(lib(), "nntile_hip_transpose_" + dtype_name(src))
    _check(fn(_stream(stream), m, n, float(alpha), _ptr(src), _ptr(dst)), "transpose")


def flash_sdpa_fwd_codelet(K, Q, mask, lse, V, A, scratch_lse=None, scratch_A=None,
                           seq=None, head=None, batch=None):
    """Calls the StarPU-shaped codelet body with look-alike variable
    interfaces, as a StarPU HIP worker would (null stream unless a provider
    was registered)."""
    tensors = [K, Q, mask, lse, V, A, scratch_lse, scratch_A]
    ifs = []
    for t in tensors:
        v = VariableInterface()
        v.id = 2
        v.ptr = 0 if t is None else t.data_ptr()
        v.dev_handle = v.ptr
        v.offset = 0
        v.elemsize = 0 if t is None else t.numel() * t.element_size()
        ifs.append(v)
    bufs = (_vp * 8)(*[ctypes.addressof(v) for v in ifs])
    b, s, h = Q.shape
    args = FlashClArgs(None, s if seq is None else seq, h if head is None else head,
                       b if batch is None else batch)
    fn = getattr(lib(), "nntile_hip_flash_sdpa_fwd_codelet_" + dtype_name(Q))
    fn(bufs, ctypes.addressof(args))


def _interfaces(tensors):
    """Look-alike StarPU variable interfaces of device tensors and the
    buffers[] array that points at them (keep both alive during the call)."""
    ifs = []
    for t in tensors:
        v = VariableInterface()
        v.id = 2
        v.ptr = 0 if t is None else t.data_ptr()
        v.dev_handle = v.ptr
        v.offset = 0
        v.elemsize = 0 if t is None else t.numel() * t.element_size()
        ifs.append(v)
    return ifs, (_vp * len(ifs))(*[ctypes.addressof(v) for v in ifs])


def _grid_cl_args(Q_tiles, K_tiles, q_seq, k_seq, q_tile, k_tile, mask_mode, n_batch, kv_group,
                  q_pos0, k_pos0, causal_offset, flags, n_slabs):
    batch, _, head = Q_tiles[0].shape
    a = GridClArgs()
    a.owner = None
    a.seq, a.head, a.batch = q_tile, head, batch
    a.q_seq, a.k_seq, a.q_tile, a.k_tile = q_seq, k_seq, q_tile, k_tile
    a.n_batch = batch if n_batch is None else n_batch
    a.kv_group = kv_group
    a.q_pos0, a.k_pos0, a.causal_offset = q_pos0, k_pos0, causal_offset
    a.mask_mode, a.flags = mask_mode, flags
    a.n_slabs = n_slabs
    a.n_q_tiles, a.n_kv_tiles = len(Q_tiles) // n_slabs, len(K_tiles) // n_slabs
    return a


def sdpa_fwd_grid_codelet(K_tiles, Q_tiles, lse_tiles, V_tiles, A_tiles, q_seq, k_seq, q_tile,
                          k_tile, mask_mode, n_batch=None, kv_group=1, q_pos0=0, k_pos0=0,
                          causal_offset=0, flags=0, n_slabs=1, n_q_tiles=None):
    """Calls the StarPU-shaped body of the whole-grid forward as a HIP worker
    would: buffers K tiles, V tiles, Q tiles, lse tiles, A tiles (null stream
    unless a provider was registered).  n_q_tiles overrides the tile count in
    the arguments (to provoke the body's error path)."""
    _dev(*K_tiles, *Q_tiles, *lse_tiles, *V_tiles, *A_tiles)
    a = _grid_cl_args(Q_tiles, K_tiles, q_seq, k_seq, q_tile, k_tile, mask_mode, n_batch, kv_group,
                      q_pos0, k_pos0, causal_offset, flags, n_slabs)
    if n_q_tiles is not None:
        a.n_q_tiles = n_q_tiles
    ifs, bufs = _interfaces(list(K_tiles) + list(V_tiles) + list(Q_tiles) + list(lse_tiles)
                            + list(A_tiles))
    fn = getattr(lib(), "nntile_hip_sdpa_fwd_grid_codelet_" + dtype_name(Q_tiles[0]))
    fn.argtypes, fn.restype = [_vp, _vp], None
    fn(bufs, ctypes.addressof(a))


def sdpa_bwd_grid_codelet(K_tiles, Q_tiles, V_tiles, A_tiles, dA_tiles, lse_tiles, dK_tiles,
                          dQ_tiles, dV_tiles, q_seq, k_seq, q_tile, k_tile, mask_mode, workspace,
                          n_batch=None, kv_group=1, q_pos0=0, k_pos0=0, causal_offset=0, flags=0,
                          n_slabs=1):
    """The body of the whole-grid backward: buffers K, V, Q, A, dA, lse tiles
    (read), dK, dQ, dV tiles (read-write), one scratch buffer."""
    groups = [K_tiles, V_tiles, Q_tiles, A_tiles, dA_tiles, lse_tiles, dK_tiles, dQ_tiles, dV_tiles]
    _dev(*[t for g in groups for t in g], workspace)
    a = _grid_cl_args(Q_tiles, K_tiles, q_seq, k_seq, q_tile, k_tile, mask_mode, n_batch, kv_group,
                      q_pos0, k_pos0, causal_offset, flags, n_slabs)
    ifs, bufs = _interfaces([t for g in groups for t in g] + [workspace])
    fn = getattr(lib(), "nntile_hip_sdpa_bwd_grid_codelet_" + dtype_name(Q_tiles[0]))
    fn.argtypes, fn.restype = [_vp, _vp], None
    fn(bufs, ctypes.addressof(a))


def flash_sdpa_bwd_codelet(K, Q, V, A, dA, mask, lse, dK, dQ, dV, scratch_dK=None,
                           scratch_dQ=None, scratch_dV=None):
    """Calls the StarPU-shaped backward codelet body with look-alike variable
    interfaces (13 buffers in the reference's order)."""
    tensors = [K, Q, V, A, dA, mask, lse, dK, dQ, dV, scratch_dK, scratch_dQ, scratch_dV]
    ifs = []
    for t in tensors:
        v = VariableInterface()
        v.id = 2
        v.ptr = 0 if t is None else t.data_ptr()
        v.dev_handle = v.ptr
        v.offset = 0
        v.elemsize = 0 if t is None else t.numel() * t.element_size()
        ifs.append(v)
    bufs = (_vp * 13)(*[ctypes.addressof(v) for v in ifs])
    b, s, h = Q.shape
    args = FlashClArgs(None, s, h, b)
    fn = getattr(lib(), "nntile_hip_flash_sdpa_bwd_codelet_" + dtype_name(Q))
    fn(bufs, ctypes.addressof(args))
