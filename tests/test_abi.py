"""CPU-side checks of the drop-in boundary: the library loads, exports every symbol include/dsgx.h declares, its
structures have the reference's sizes, and argument errors come back as a status and a message (no GPU call is made:
every check below fails in validation, before any launch)."""
import ctypes as C
import os
import re
import subprocess

import numpy as np
import pytest

from dsgx10_amd import abi, lib
from dsgx10_amd.layer import DESC_DTYPE, HostLayer, mat_bytes

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    L = lib.lib()
    hdr = open(os.path.join(ROOT, "include", "dsgx.h")).read()
    declared = set(re.findall(r"DSGX_API\s+[\w\s\*]+?\b(dsgx_\w+)\s*\(", hdr))
    assert declared == set(abi.SYMBOLS), declared ^ set(abi.SYMBOLS)
    for s in declared:
        assert hasattr(L, s), s
    assert b"gfx950" in L.dsgx_version()


def test_struct_sizes_and_mat_bytes():
    L = lib.lib()
    assert C.sizeof(abi.MatDesc) == 64 == DESC_DTYPE.itemsize          # experts.h:64 of the reference
    # FP8 expert of the DeepSeek-shaped layer: 3 matrices = 25,165,824 + 6,144 bytes
    g = L.dsgx_mat_bytes(abi.FMT_FP8, 2048, 4096)
    d = L.dsgx_mat_bytes(abi.FMT_FP8, 4096, 2048)
    assert 2 * g + d == 25165824 + 6144
    # INT4 expert of the GLM-shaped layer: 3 x 7,274,496
    assert L.dsgx_mat_bytes(abi.FMT_INT4, 2048, 6144) == 7274496 == L.dsgx_mat_bytes(abi.FMT_INT4, 6144, 2048)
    assert L.dsgx_mat_bytes(abi.FMT_BF16, 4096, 6144) == 4096 * 6144 * 2
    for f in (abi.FMT_REF_NVFP4, 1, abi.FMT_REF_INT4, abi.FMT_REF_BF16, 7):   # the reference's tilings and unknown tags: 0
        assert L.dsgx_mat_bytes(f, 512, 6144) == 0
    for fmt, N, K in [(abi.FMT_FP8, 200, 256), (abi.FMT_INT4, 24, 1024), (abi.FMT_BF16, 8, 64)]:
        assert L.dsgx_mat_bytes(fmt, N, K) == mat_bytes(fmt, N, K)
    assert L.dsgx_mat_scale_off(abi.FMT_INT4, 24, 1024) == 24 * 512
    assert L.dsgx_mat_zp_off(abi.FMT_INT4, 24, 1024) == 24 * 512 + 24 * 32 * 2


def _layer(fmt=abi.FMT_FP8):
    Lw = abi.LayerW()
    Lw.pool, Lw.desc = 0x1000, 0x2000
    Lw.fmt, Lw.H, Lw.I, Lw.E, Lw.topk = fmt, 4096, 2048, 256, 8
    return Lw


def _decode_rc(Lw, M=1, x=0x3000, idx=0x4000, w=0x5000, ws=0x6000, yr=0x7000, ys=0x8000, cfg=None):
    return lib.lib().dsgx_moe_decode(C.byref(Lw), x, idx, w, M, ws, yr, ys, None, cfg)


def test_decode_argument_errors():
    L = lib.lib()
    assert _decode_rc(_layer(), M=0) == abi.EINVAL and b"M=0" in L.dsgx_last_error()
    assert _decode_rc(_layer(), M=17) == abi.EINVAL
    assert _decode_rc(_layer(), idx=None) == abi.EINVAL and b"idx and w" in L.dsgx_last_error()
    for f in (0, 2, 3):  # the reference's GB10 tilings are refused, never reinterpreted
        assert _decode_rc(_layer(f)) == abi.EFORMAT and b"GB10" in L.dsgx_last_error()
    assert _decode_rc(_layer(1)) == abi.EFORMAT and _decode_rc(_layer(77)) == abi.EFORMAT
    cfg = abi.DecodeCfg(0, 0, 3, 0, None, None, 1.0, 0, 0x1234)
    assert _decode_rc(_layer(), cfg=C.byref(cfg)) == abi.EUNSUPPORTED and b"ring" in L.dsgx_last_error()
    bad = _layer()
    bad.H = 4000
    assert _decode_rc(bad) == abi.EINVAL
    both = _layer()
    both.sh.g = both.sh.bgu = 0x9000
    assert _decode_rc(both) == abi.EINVAL and b"FP8 and a BF16" in L.dsgx_last_error()
    cfg = abi.DecodeCfg(0, 0, 3, 1, None, None, 1.0, 0, None)
    assert _decode_rc(_layer(), ys=None, cfg=C.byref(cfg)) == abi.EINVAL  # ysum needs ys


def test_gemv_and_route_argument_errors():
    L = lib.lib()
    seg = (abi.GemvSeg * 1)(abi.GemvSeg(abi.FMT_FP8, 0x1000, 0x2000, None, 2048, 128, 128, 0x3000, 2048))
    assert L.dsgx_gemv(0x100, 4096, 0, 4096, seg, 1, 0, 1, None) == abi.EINVAL
    assert L.dsgx_gemv(0x100, 4096, 17, 4096, seg, 1, 0, 1, None) == abi.EINVAL
    assert L.dsgx_gemv(0x100, 4096, 1, 4096, seg, 1, 0, 3, None) == abi.EINVAL      # splitk 1, 2 or 4
    assert L.dsgx_gemv(0x100, 4096, 1, 4096, seg, 5, 0, 1, None) == abi.EINVAL      # at most 4 segments
    seg[0].fmt = 0
    assert L.dsgx_gemv(0x100, 4096, 1, 4096, seg, 1, 0, 1, None) == abi.EFORMAT     # a format is never guessed
    seg[0].fmt, seg[0].n = abi.FMT_FP8, 2050
    assert L.dsgx_gemv(0x100, 4096, 1, 4096, seg, 1, 0, 1, None) == abi.EINVAL
    assert L.dsgx_route(0x100, None, 1, 600, 8, 1.0, 0, 0x200, 0x300, None) == abi.EINVAL
    assert L.dsgx_route(0x100, None, 1, 256, 9, 1.0, 0, 0x200, 0x300, None) == abi.EINVAL
    assert L.dsgx_dequant_int4(0x100, 0x200, 0x300, 12, 64, 0x400, 64, None) == abi.EINVAL


def test_host_layer_pool_layout():
    rng = np.random.default_rng(0)
    I, H = 256, 384
    def fp8(N, K):
        return rng.integers(0, 120, (N, K), dtype=np.uint8), rng.random(((N + 127) // 128, K // 128), dtype=np.float32)
    ex = [(fp8(I, H), fp8(I, H), fp8(H, I)) for _ in range(2)]
    hl = HostLayer(abi.FMT_FP8, H, I, 5, 2, ex, emap=[0, 1, 1, 0, 1])
    assert hl.pool.size == 2 * (2 * mat_bytes(abi.FMT_FP8, I, H) + mat_bytes(abi.FMT_FP8, H, I))
    assert np.all(hl.desc["off"] % 256 == 0) and np.all(hl.desc["s2"] == 1.0) and np.all(hl.desc["rsv"] == 0)
    assert hl.desc["off"][3 * 1 + 0] == hl.desc["off"][3 * 2 + 0] != hl.desc["off"][0]
    off = int(hl.desc["off"][3 * 4 + 2])
    codes, scales = ex[1][2]
    assert np.array_equal(hl.pool[off:off + H * I].reshape(H, I), codes)
    so = off + (H * I + 255) // 256 * 256
    assert np.array_equal(hl.pool[so:so + scales.size * 4].view(np.float32).reshape(scales.shape), scales)


def test_cpp_mirror_headers_compile_and_link():
    """the C++ headers that keep the reference's operator signatures compile as plain C++17 and link against the ABI"""
    src = os.path.join(ROOT, "tests", "golden", "mirror_smoke.cpp")
    if not os.path.exists(src):
        pytest.skip("mirror headers not written yet")
    exe = "/tmp/dsgx_mirror_smoke"
    so_dir = os.path.dirname(lib.so_path())
    subprocess.check_call(["g++", "-std=c++17", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), src, "-o", exe,
                           "-L", so_dir, "-ldsgx", "-Wl,-rpath," + so_dir])
    out = subprocess.run([exe], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout + out.stderr
