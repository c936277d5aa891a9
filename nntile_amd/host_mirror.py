"""ctypes front-end of libnntile_host.so, the C++ mirror of the NNTile
tile/tensor/codelet layers for the attention path.  Arrays are numpy,
Fortran-ordered, in the reference's axis order [head, seq, batch, group, kv]."""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "host", "libnntile_host.so")
DTYPES = {"bf16": 0, "fp16": 1, "fp32": 2}
OP_TENSOR, OP_TILE, OP_HIP, OP_CLASSIFIED = 0, 1, 2, 3
# the reference's submission literally, one task per tile pair (forward / backward op codes)
OP_PAIRS, OP_PAIRS_BWD = 3, 4
_lib = None


class HostError(RuntimeError):
    """A std::runtime_error thrown by the C++ layer."""


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libnntile_host.so is missing: run `make -C nntile_amd/host`")
        L = ctypes.CDLL(LIB_PATH)
        vp, i64 = ctypes.c_void_p, ctypes.c_int64
        L.nntile_host_tensor_create.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(i64),
                                                ctypes.POINTER(i64), ctypes.c_char_p, ctypes.c_int]
        L.nntile_host_tensor_create.restype = vp
        L.nntile_host_tensor_free.argtypes = [vp]
        L.nntile_host_tensor_from_array.argtypes = [vp, vp, ctypes.c_char_p, ctypes.c_int]
        L.nntile_host_tensor_to_array.argtypes = [vp, vp, ctypes.c_char_p, ctypes.c_int]
        L.nntile_host_tensor_ntiles.argtypes = [vp]
        L.nntile_host_tensor_ntiles.restype = i64
        L.nntile_host_flash_sdpa_fwd.argtypes = [ctypes.c_int, ctypes.c_int, vp, vp, vp, vp, vp, vp,
                                                 ctypes.c_int, i64, ctypes.c_int, ctypes.c_char_p,
                                                 ctypes.c_int]
        L.nntile_host_flash_sdpa_fwd_classified.argtypes = [
            ctypes.c_int, vp, vp, vp, vp, vp, vp, i64, ctypes.POINTER(ctypes.c_int32), i64,
            ctypes.POINTER(i64), ctypes.c_char_p, ctypes.c_int]
        L.nntile_host_mask_rule.argtypes = [i64, i64, i64, i64, ctypes.POINTER(ctypes.c_int32), i64,
                                            i64, ctypes.POINTER(ctypes.c_int32), ctypes.c_char_p,
                                            ctypes.c_int]
        L.nntile_host_check_shapes.argtypes = [ctypes.c_int, ctypes.POINTER(i64), ctypes.c_char_p,
                                               ctypes.c_int]
        L.nntile_host_flash_sdpa_bwd.argtypes = [ctypes.c_int, ctypes.c_int] + [vp] * 10 + [
            ctypes.c_int, i64, ctypes.POINTER(i64), ctypes.c_char_p, ctypes.c_int]
        L.nntile_host_check_shapes_bwd.argtypes = [ctypes.c_int, ctypes.POINTER(i64), ctypes.c_char_p,
                                                   ctypes.c_int]
        L.nntile_host_footprint_bwd.argtypes = [i64, i64, i64]
        L.nntile_host_footprint_bwd.restype = ctypes.c_uint32
        L.nntile_host_tasks_submitted_bwd.argtypes = [ctypes.c_int]
        L.nntile_host_tasks_submitted_bwd.restype = i64
        L.nntile_host_codelet_name_bwd.argtypes = [ctypes.c_int]
        L.nntile_host_codelet_name_bwd.restype = ctypes.c_char_p
        L.nntile_host_footprint.argtypes = [i64, i64, i64]
        L.nntile_host_footprint.restype = ctypes.c_uint32
        L.nntile_host_tasks_submitted.argtypes = [ctypes.c_int]
        L.nntile_host_tasks_submitted.restype = i64
        L.nntile_host_grid_tasks_submitted.argtypes = [ctypes.c_int, ctypes.c_int]
        L.nntile_host_grid_tasks_submitted.restype = i64
        L.nntile_host_grid_codelet_name.argtypes = [ctypes.c_int, ctypes.c_int]
        L.nntile_host_grid_codelet_name.restype = ctypes.c_char_p
        L.nntile_host_codelet_name.argtypes = [ctypes.c_int]
        L.nntile_host_codelet_name.restype = ctypes.c_char_p
        L.nntile_host_mask_cache_stats.argtypes = [ctypes.POINTER(ctypes.c_uint64)] * 2
        L.nntile_host_mask_cache_stats.restype = None
        L.nntile_host_mask_cache_clear.argtypes = []
        L.nntile_host_mask_cache_clear.restype = None
        L.nntile_host_mask_classifications.argtypes = []
        L.nntile_host_mask_classifications.restype = ctypes.c_uint64
        L.nntile_host_mask_declare_constant.argtypes = [ctypes.c_void_p, ctypes.c_int,
                                                        ctypes.c_char_p, ctypes.c_int]
        L.nntile_host_mask_declare_constant.restype = ctypes.c_int
        L.nntile_host_tensor_tile_ptr.argtypes = [ctypes.c_void_p, i64]
        L.nntile_host_tensor_tile_ptr.restype = ctypes.c_void_p
        L.nntile_host_tensor_tile_bytes.argtypes = [ctypes.c_void_p, i64]
        L.nntile_host_tensor_tile_bytes.restype = i64
        L.nntile_host_tensor_mark_written.argtypes = [vp]
        L.nntile_host_tensor_mark_written.restype = None
        L.nntile_host_time_flash_sdpa_fwd.argtypes = [
            ctypes.c_int, ctypes.c_int, vp, vp, vp, vp, vp, vp, ctypes.c_int, ctypes.c_int,
            ctypes.POINTER(ctypes.c_double), ctypes.POINTER(i64), ctypes.c_char_p, ctypes.c_int]
        _lib = L
    return _lib


def _arr(v):
    return (ctypes.c_int64 * len(v))(*v)


def _call(fn, *args):
    err = ctypes.create_string_buffer(256)
    rc = fn(*args, err, 256)
    if rc != 0:
        raise HostError(err.value.decode())


class Tensor:
    """nntile::tensor::Tensor<T>: a grid of separately allocated device tiles."""

    def __init__(self, dtype, shape, basetile):
        self.dtype, self.shape, self.basetile = dtype, tuple(shape), tuple(basetile)
        err = ctypes.create_string_buffer(256)
        self.h = lib().nntile_host_tensor_create(DTYPES[dtype], len(shape), _arr(shape),
                                                 _arr(basetile), err, 256)
        if not self.h:
            raise HostError(err.value.decode())

    def __del__(self):
        if getattr(self, "h", None):
            lib().nntile_host_tensor_free(self.h)
            self.h = None

    @property
    def ntiles(self):
        return int(lib().nntile_host_tensor_ntiles(self.h))

    def from_array(self, a):
        np_dt = np.float32 if self.dtype == "fp32" else np.uint16
        a = np.asfortranarray(a, dtype=np_dt)
        assert a.shape == self.shape
        _call(lib().nntile_host_tensor_from_array, self.h, a.ctypes.data_as(ctypes.c_void_p))
        return self

    def to_array(self):
        np_dt = np.float32 if self.dtype == "fp32" else np.uint16
        out = np.empty(self.shape, dtype=np_dt, order="F")
        _call(lib().nntile_host_tensor_to_array, self.h, out.ctypes.data_as(ctypes.c_void_p))
        return out

    def mark_written(self):
        """What the runtime does when it hands the tiles to a writer: facts
        cached about their contents (the classes of a mask) are dropped."""
        lib().nntile_host_tensor_mark_written(self.h)


def flash_sdpa_fwd(op, K, Q, mask, lse, V, A, mask_mode=0, offset=0, overwrite=False):
    _call(lib().nntile_host_flash_sdpa_fwd, op, DTYPES[Q.dtype], K.h, Q.h,
          None if mask is None else mask.h, lse.h, V.h, A.h, mask_mode, offset, int(overwrite))


def mask_declare_constant(mask):
    """tensor::flash_sdpa_mask_declare_constant: the mask's contents stay as
    they are; its tiles are classified now (blocking) and the calls with the
    reference's signature use the classes from here on."""
    _call(lib().nntile_host_mask_declare_constant, mask.h, 0)


def mask_forget(mask):
    """tensor::flash_sdpa_mask_forget."""
    _call(lib().nntile_host_mask_declare_constant, mask.h, 1)


def mask_classifications():
    """Blocking classifications of a mask since the start of the process."""
    return int(lib().nntile_host_mask_classifications())


def tile_ptr(tensor, i):
    """(device address, bytes) of tile i: for writes the runtime does not see."""
    return (int(lib().nntile_host_tensor_tile_ptr(tensor.h, i)),
            int(lib().nntile_host_tensor_tile_bytes(tensor.h, i)))


def mask_cache_stats():
    """(look-ups that found the mask's classes, look-ups that did not) behind
    the reference-signature tensor operations (OP_TENSOR), since the start of
    the process."""
    hits, misses = ctypes.c_uint64(0), ctypes.c_uint64(0)
    lib().nntile_host_mask_cache_stats(ctypes.byref(hits), ctypes.byref(misses))
    return hits.value, misses.value


def mask_cache_clear():
    lib().nntile_host_mask_cache_clear()


def time_flash_sdpa_fwd(op, K, Q, mask, lse, V, A, steps, warmup):
    """Milliseconds per pass and attention launches per pass of: logsumexp
    filled with -inf, then tensor::flash_sdpa_fwd_cudnn_async (OP_TENSOR) or
    tensor::flash_sdpa_fwd_cudnn_pairs_async (OP_PAIRS); HIP events on the
    mirror's stream."""
    ms, launches = ctypes.c_double(0.0), ctypes.c_int64(0)
    _call(lib().nntile_host_time_flash_sdpa_fwd, op, DTYPES[Q.dtype], K.h, Q.h, mask.h, lse.h,
          V.h, A.h, steps, warmup, ctypes.byref(ms), ctypes.byref(launches))
    return ms.value, launches.value


def mask_rule(k_seq, q_seq, k_tile, q_tile, classes, offset=0):
    """tensor::flash_sdpa_mask_rule: what the classes of a [k_seq, q_seq] mask's
    tiles (linear order of its grid, key tile fastest) say about the whole
    mask: 1 (MASK_NONE), 2 (MASK_CAUSAL with `offset`) or -1."""
    arr = (ctypes.c_int32 * len(classes))(*classes)
    out = ctypes.c_int32(-9)
    _call(lib().nntile_host_mask_rule, k_seq, q_seq, k_tile, q_tile, arr, len(classes), offset,
          ctypes.byref(out))
    return out.value


def flash_sdpa_fwd_classified(K, Q, mask, lse, V, A, offset=0):
    """tensor::flash_sdpa_mask_classes + the tensor::flash_sdpa_fwd_cudnn_async
    overload that takes them: pairs whose mask tile hides everything are not
    submitted, open and causal ones run without reading the mask.  Returns
    (classes per mask tile in the mask grid's linear order, pairs submitted)."""
    n_tiles = mask.ntiles
    classes = (ctypes.c_int32 * n_tiles)()
    n = ctypes.c_int64(0)
    _call(lib().nntile_host_flash_sdpa_fwd_classified, DTYPES[Q.dtype], K.h, Q.h, mask.h, lse.h,
          V.h, A.h, offset, classes, n_tiles, ctypes.byref(n))
    return list(classes), n.value


def flash_sdpa_bwd(op, K, Q, V, A, dA, mask, lse, dK, dQ, dV, mask_mode=0, offset=0):
    """tensor::flash_sdpa_bwd_cudnn (op 0), tile::flash_sdpa_bwd_cudnn (op 1) or
    tensor::flash_sdpa_bwd_hip_async (op 2: analytic mask, mask=None) or the
    tensor-level overload that classifies the mask's tiles first (op 3; offset
    = the causal rule the tiles are compared with): the gradients are added
    to dK, dQ, dV.  Returns the tile pairs ops 2 and 3 launched."""
    n = ctypes.c_int64(0)
    _call(lib().nntile_host_flash_sdpa_bwd, op, DTYPES[Q.dtype],
          *(None if t is None else t.h for t in (K, Q, V, A, dA, mask, lse, dK, dQ, dV)),
          mask_mode, offset, ctypes.byref(n))
    return n.value


def check_shapes_bwd(level, specs):
    """specs: ten (shape, basetile) pairs in the order K, Q, V, A, dA, mask,
    logsumexp, dK, dQ, dV."""
    flat = []
    for shape, base in specs:
        flat += [len(shape)] + list(shape) + list(base)
    _call(lib().nntile_host_check_shapes_bwd, level, _arr(flat))


def check_shapes(level, specs):
    """specs: six (shape, basetile) pairs in the order K, Q, mask, logsumexp, V, A."""
    flat = []
    for shape, base in specs:
        flat += [len(shape)] + list(shape) + list(base)
    _call(lib().nntile_host_check_shapes, level, _arr(flat))


def footprint(seq, head, batch):
    return int(lib().nntile_host_footprint(seq, head, batch))


def footprint_bwd(seq, head, batch):
    return int(lib().nntile_host_footprint_bwd(seq, head, batch))


def tasks_submitted_bwd(dtype):
    return int(lib().nntile_host_tasks_submitted_bwd(DTYPES[dtype]))


def codelet_name_bwd(dtype):
    return lib().nntile_host_codelet_name_bwd(DTYPES[dtype]).decode()


def grid_tasks_submitted(dtype, backward=False):
    """Tasks of the whole-grid codelets (one per group of slabs) so far."""
    return int(lib().nntile_host_grid_tasks_submitted(DTYPES[dtype], int(backward)))


def grid_codelet_name(dtype, backward=False):
    return lib().nntile_host_grid_codelet_name(DTYPES[dtype], int(backward)).decode()


def tasks_submitted(dtype):
    return int(lib().nntile_host_tasks_submitted(DTYPES[dtype]))


def codelet_name(dtype):
    return lib().nntile_host_codelet_name(DTYPES[dtype]).decode()
