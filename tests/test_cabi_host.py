"""CPU-side checks of the C-ABI library: it loads without a GPU, exports every
symbol the header declares, and rejects bad arguments before touching HIP."""
import ctypes
import os
import re

import pytest

from nntile_amd import hip_sdpa as h

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "nntile_hip_sdpa.h")).read()
    declared = set(re.findall(r"\b(nntile_hip_[a-z0-9_]+)\s*\(", header))
    declared -= {"nntile_hip_stream_provider"}
    assert len(declared) >= 20
    L = h.lib()
    for name in sorted(declared):
        assert hasattr(L, name), name
    assert set(h.EXPORTS) == declared
    assert b"gfx950" in L.nntile_hip_sdpa_version()


def test_struct_layouts_match_header():
    assert ctypes.sizeof(h.TileArgs) == 6 * 8 + 8 + 3 * 8 + 6 * 8
    assert ctypes.sizeof(h.GridArgs) == 8 * 8 + 16 + 8 + 3 * 8 + 5 * 64 * 8
    assert h.GridArgs.n_slabs.offset == 8 * 8 + 16 and h.GridArgs.q_pos0.offset == 8 * 8 + 24
    assert ctypes.sizeof(h.BwdGridArgs) == 8 * 8 + 16 + 8 + 3 * 8 + 9 * 32 * 8 + 16
    assert h.BwdGridArgs.n_slabs.offset == 8 * 8 + 16 and h.BwdGridArgs.q_pos0.offset == 8 * 8 + 24
    assert ctypes.sizeof(h.FlashClArgs) == 32
    assert ctypes.sizeof(h.VariableInterface) == 40


def _tile(**kw):
    a = h.TileArgs()
    a.q_seq = a.k_seq = 64
    a.head, a.batch, a.n_batch, a.kv_group = 64, 2, 2, 1
    a.mask_mode = h.MASK_NONE
    a.K = a.Q = a.V = a.lse = a.A = 4096       # never dereferenced on these paths
    for k, v in kw.items():
        setattr(a, k, v)
    return a


@pytest.mark.parametrize("t", ["bf16", "fp16", "fp32"])
def test_bad_arguments_are_rejected_before_launch(t):
    L = h.lib()
    tile = getattr(L, "nntile_hip_sdpa_fwd_tile_" + t)
    assert tile(None, None) == h.EINVAL
    assert tile(None, ctypes.byref(_tile(q_seq=0))) == h.EINVAL
    assert tile(None, ctypes.byref(_tile(K=None))) == h.EINVAL
    assert tile(None, ctypes.byref(_tile(K=4100))) == h.EINVAL            # misaligned
    assert tile(None, ctypes.byref(_tile(mask_mode=7))) == h.EINVAL
    assert tile(None, ctypes.byref(_tile(mask_mode=h.MASK_ADDITIVE))) == h.EINVAL   # mask missing
    assert tile(None, ctypes.byref(_tile(kv_group=3))) == h.EINVAL        # batch % (n_batch*group)
    assert tile(None, ctypes.byref(_tile(head=48))) == h.EUNSUPPORTED
    flash = getattr(L, "nntile_hip_flash_sdpa_fwd_" + t)
    assert flash(None, 64, 64, 2, 4096, 4096, None, None, 4096, None, 4096, 4096) == h.EINVAL
    assert flash(None, -1, 64, 2, 4096, 4096, 4096, None, 4096, None, 4096, 4096) == h.EINVAL
    grid = getattr(L, "nntile_hip_sdpa_fwd_grid_" + t)
    g = h.GridArgs()
    assert grid(None, ctypes.byref(g)) == h.EINVAL
    g.q_seq = g.k_seq = 256
    g.q_tile = g.k_tile = 64
    g.head, g.batch, g.n_batch, g.kv_group = 64, 2, 2, 1
    g.n_q_tiles, g.n_kv_tiles = 4, 3                                        # 3 != ceil(256/64)
    g.mask_mode = h.MASK_CAUSAL
    assert grid(None, ctypes.byref(g)) == h.EINVAL
    g.n_kv_tiles = 4
    g.mask_mode = h.MASK_ADDITIVE
    assert grid(None, ctypes.byref(g)) == h.EUNSUPPORTED
    g.mask_mode = h.MASK_CAUSAL
    assert grid(None, ctypes.byref(g)) == h.EINVAL                         # null tile pointers
    g.n_slabs = 17                                                          # 17 * 4 tiles > 64
    for i in range(64):
        g.K[i] = g.V[i] = g.Q[i] = g.lse[i] = g.A[i] = 4096
    assert grid(None, ctypes.byref(g)) == h.EINVAL
    g.n_slabs = -1
    assert grid(None, ctypes.byref(g)) == h.EINVAL


@pytest.mark.parametrize("t", ["bf16", "fp16"])
def test_backward_grid_argument_checks(t):
    """Refused before anything is launched: a null block, slab counts that
    overflow the tile tables, a workspace that does not grow with the slabs."""
    L = h.lib()
    grid = getattr(L, "nntile_hip_sdpa_bwd_grid_" + t)
    assert grid(None, None) == h.EINVAL
    g = h.BwdGridArgs()
    g.q_seq = g.k_seq = 512
    g.q_tile = g.k_tile = 128
    g.head, g.batch, g.n_batch, g.kv_group = 64, 2, 2, 1
    g.n_q_tiles = g.n_kv_tiles = 4
    g.mask_mode = h.MASK_CAUSAL
    for i in range(h.BWD_MAX_TILES):
        for name in ("K", "V", "Q", "A", "dA", "lse", "dK", "dQ", "dV"):
            getattr(g, name)[i] = 4096
    g.workspace, g.workspace_bytes = 4096, 4 * 512 * 2
    assert L.nntile_hip_sdpa_bwd_grid_workspace_bytes(ctypes.byref(g)) == 4 * 512 * 2
    g.n_slabs = 9                                                           # 9 * 4 tiles > 32
    assert grid(None, ctypes.byref(g)) == h.EINVAL
    g.n_slabs = -1
    assert grid(None, ctypes.byref(g)) == h.EINVAL
    g.n_slabs = 8                                                           # fits, but the workspace is for one slab
    assert L.nntile_hip_sdpa_bwd_grid_workspace_bytes(ctypes.byref(g)) == 8 * 4 * 512 * 2
    assert grid(None, ctypes.byref(g)) == h.EWORKSPACE
    g.n_slabs = 1
    g.q_tile = 96                                                           # not a multiple of 128
    g.n_q_tiles = 6
    assert grid(None, ctypes.byref(g)) == h.EUNSUPPORTED


def test_decode_argument_checks():
    L = h.lib()
    a = _tile(q_seq=16, k_seq=512, head=128, batch=16, n_batch=2, kv_group=4)
    need = L.nntile_hip_sdpa_fwd_decode_workspace_bytes(ctypes.byref(a))
    assert need > 0
    assert L.nntile_hip_sdpa_fwd_decode_bf16(None, ctypes.byref(a), None, 0) == h.EWORKSPACE
    assert L.nntile_hip_sdpa_fwd_decode_bf16(None, ctypes.byref(a), 4096, need - 1) == h.EWORKSPACE
    a.q_seq = 17                                                            # 17*4 rows > 64
    assert L.nntile_hip_sdpa_fwd_decode_bf16(None, ctypes.byref(a), 4096, 1 << 30) == h.EINVAL
    assert L.nntile_hip_sdpa_fwd_decode_workspace_bytes(ctypes.byref(a)) == 0
    a.q_seq, a.head = 16, 32
    assert L.nntile_hip_sdpa_fwd_decode_bf16(None, ctypes.byref(a), 4096, 1 << 30) == h.EUNSUPPORTED


def test_codelet_body_swallows_bad_input(capfd):
    """Errors in the codelet body are printed and the task becomes a no-op
    (src/starpu/flash_sdpa_fwd_cudnn.cc:69-115)."""
    L = h.lib()
    L.nntile_hip_flash_sdpa_fwd_codelet_bf16(None, None)
    bufs = (ctypes.c_void_p * 8)()
    args = h.FlashClArgs(None, 64, 64, 2)
    L.nntile_hip_flash_sdpa_fwd_codelet_bf16(bufs, ctypes.addressof(args))
    err = capfd.readouterr().err
    assert "skipping task" in err


def test_accumulate_zero_sizes_return_silently():
    # src/kernel/accumulate_attn_output/cuda.cu:123-126
    L = h.lib()
    assert L.nntile_hip_accumulate_attn_output_fp32(None, 0, 4, 4, None, None, None, None) == h.OK
    assert L.nntile_hip_accumulate_attn_output_fp32(None, 8, 4, 4, None, None, None, None) == h.EINVAL


def test_starpu_registration_unit_compiles_to_stubs_here():
    """StarPU is not installed in this image: the registration unit reduces
    to two stubs that say so."""
    from nntile_amd import host_mirror as hm
    L = hm.lib()
    assert L.nntile_hip_starpu_available() == 0
    assert L.nntile_hip_starpu_register(None, None, 0) == -1
    assert L.nntile_hip_starpu_register_grid(None, None, 0) == -1


def test_host_library_exports_what_its_header_declares():
    from nntile_amd import host_mirror as hm
    header = open(os.path.join(ROOT, "include", "nntile_hip_starpu.h")).read()
    declared = set(re.findall(r"\b(nntile_hip_[a-z0-9_]+)\s*\(", header))
    assert declared == {"nntile_hip_starpu_available", "nntile_hip_starpu_register",
                        "nntile_hip_starpu_register_grid"}
    L = hm.lib()
    for name in sorted(declared):
        assert hasattr(L, name), name


def test_grid_codelet_bodies_report_and_return_on_bad_arguments(capfd):
    """Error behaviour of the reference body (src/starpu/flash_sdpa_fwd_cudnn.cc:
    69-115): a line on stderr, the task does nothing."""
    L = h.lib()
    for name in ("nntile_hip_sdpa_fwd_grid_codelet_bf16", "nntile_hip_sdpa_bwd_grid_codelet_fp16"):
        fn = getattr(L, name)
        fn.argtypes, fn.restype = [ctypes.c_void_p, ctypes.c_void_p], None
        fn(None, None)
        a = h.GridClArgs()
        a.n_q_tiles, a.n_kv_tiles, a.n_slabs = 40, 40, 2        # 80 tiles an axis
        bufs = (ctypes.c_void_p * 4)()
        fn(bufs, ctypes.addressof(a))
        a.n_q_tiles, a.n_kv_tiles, a.n_slabs = 1, 1, 1
        fn(bufs, ctypes.addressof(a))                            # null buffers
    err = capfd.readouterr().err
    assert err.count("skipping task") == 6
    assert ctypes.sizeof(h.GridClArgs) == 13 * 8 + 6 * 4


def test_starpu_registration_unit_is_valid_against_the_api_it_names(tmp_path):
    """Syntax check of the StarPU branch of the registration unit against a
    declaration-only rendering of the StarPU API it uses (starpu_codelet's
    hip_funcs / hip_flags / where, STARPU_HIP, STARPU_HIP_ASYNC,
    starpu_hip_get_local_stream, struct starpu_variable_interface as published
    in starpu_data_interfaces.h).  Nothing is linked or run: this only keeps the
    guarded code from rotting where StarPU is absent.  The struct layout is
    asserted again, against the real header, wherever StarPU is installed."""
    import shutil
    import subprocess
    gxx = shutil.which("g++")
    if gxx is None:
        pytest.skip("g++ not found")
    (tmp_path / "starpu.h").write_text(
        "#pragma once\n#include <stddef.h>\n#include <stdint.h>\n"
        "#define STARPU_MAXIMPLEMENTATIONS 4\n#define STARPU_HIP (1 << 7)\n"
        "#define STARPU_HIP_ASYNC 1\n#define STARPU_VARIABLE_NBUFFERS (-1)\n"
        "struct starpu_codelet { uint32_t where; void (*hip_funcs[STARPU_MAXIMPLEMENTATIONS])(void **, void *);"
        " char hip_flags[STARPU_MAXIMPLEMENTATIONS]; int nbuffers; };\n"
        "struct starpu_variable_interface { int id; uintptr_t ptr; uintptr_t dev_handle; size_t offset;"
        " size_t elemsize; };\n")
    (tmp_path / "starpu_hip.h").write_text(
        "#pragma once\ntypedef struct ihipStream_t *hipStream_t;\n"
        "extern \"C\" hipStream_t starpu_hip_get_local_stream(void);\n")
    unit = os.path.join(ROOT, "nntile_amd", "host", "starpu_hip_registration.cc")
    r = subprocess.run([gxx, "-std=c++17", "-fsyntax-only", "-Wall", "-Werror", "-I", str(tmp_path), unit],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
