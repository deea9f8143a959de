"""ctypes binding of the CPU oracle (oracle/liboracle.so). Test infrastructure: only tests/, smoke() and the
cpu_baseline leg of bench.py import this."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_SO = os.path.join(ROOT, "oracle", "liboracle.so")


def build(force=False):
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "-B" if force else "-s"])
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = C.CDLL(build())
        L = _lib
        L.orc_f32_to_bf16.restype = C.c_uint16
        L.orc_f32_to_bf16.argtypes = [C.c_float]
        L.orc_bf16_to_f32.restype = C.c_float
        L.orc_bf16_to_f32.argtypes = [C.c_uint16]
        L.orc_e4m3_to_f32.restype = C.c_float
        L.orc_e4m3_to_f32.argtypes = [C.c_uint8]
        L.orc_f32_to_e4m3.restype = C.c_uint8
        L.orc_f32_to_e4m3.argtypes = [C.c_float]
        L.orc_mix64.restype = C.c_uint64
        L.orc_mix64.argtypes = [C.c_uint64]
        L.orc_normal.restype = C.c_double
        L.orc_normal.argtypes = [C.c_uint64, C.c_uint64, C.c_uint64]
        L.orc_int4_value_bits.restype = C.c_uint16
        L.orc_int4_value_bits.argtypes = [C.c_int, C.c_int, C.c_uint16]
        L.orc_route_sigmoid.restype = C.c_float
        L.orc_route_sigmoid.argtypes = [C.c_float]
        L.orc_route_score.restype = C.c_float
        L.orc_route_score.argtypes = [C.c_float, C.c_int]
        L.orc_union.restype = C.c_int
        L.orc_threads.restype = C.c_int
    return _lib


def _p(a):
    if a is None:
        return None
    assert isinstance(a, np.ndarray) and a.flags["C_CONTIGUOUS"], "contiguous numpy array expected"
    return a.ctypes.data_as(C.c_void_p)


# ---- ctypes mirrors of include/dsgx.h ------------------------------------------------------------------------
from dsgx10_amd.abi import FMT_BF16, FMT_FP8, FMT_INT4, OUT_BF16, OUT_F32, OUT_SWIGLU, LayerW, MatDesc, SharedW  # noqa: E402,F401


# ---- codecs and data ------------------------------------------------------------------------------------------
def f32_to_bf16(f):
    f = np.ascontiguousarray(f, np.float32)
    o = np.empty(f.shape, np.uint16)
    lib().orc_f32_to_bf16_n(_p(f), C.c_size_t(f.size), _p(o))
    return o


def bf16_to_f32(b):
    return (np.asarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_e4m3(f):
    f = np.ascontiguousarray(f, np.float32)
    o = np.empty(f.shape, np.uint8)
    lib().orc_f32_to_e4m3_n(_p(f), C.c_size_t(f.size), _p(o))
    return o


def e4m3_table():
    return np.array([lib().orc_e4m3_to_f32(i) for i in range(256)], np.float32)


def normal_f32(seed, tid, shape, sigma=1.0):
    o = np.empty(shape, np.float32)
    lib().orc_fill_normal_f32(C.c_uint64(seed), C.c_uint64(tid), C.c_size_t(o.size), C.c_double(sigma), _p(o))
    return o


def normal_bf16(seed, tid, shape, sigma=1.0):
    o = np.empty(shape, np.uint16)
    lib().orc_fill_normal_bf16(C.c_uint64(seed), C.c_uint64(tid), C.c_size_t(o.size), C.c_double(sigma), _p(o))
    return o


# ---- formats --------------------------------------------------------------------------------------------------
def int4_dequant(packed, scale, zp):
    N, K = packed.shape[0], packed.shape[1] * 8
    o = np.empty((N, K), np.uint16)
    lib().orc_int4_dequant(_p(packed), _p(scale), _p(zp), N, K, _p(o))
    return o


def int4_quantize_sym(w):
    w = np.ascontiguousarray(w, np.float32)
    N, K = w.shape
    packed = np.empty((N, K // 8), np.uint32)
    scale = np.empty((N, K // 32), np.uint16)
    zp = np.empty((N // 8, K // 32), np.uint32)
    lib().orc_int4_quantize_sym(_p(w), N, K, _p(packed), _p(scale), _p(zp))
    return packed, scale, zp


def int4_random(seed, N, K):
    packed = np.empty((N, K // 8), np.uint32)
    scale = np.empty((N, K // 32), np.uint16)
    zp = np.empty((N // 8, K // 32), np.uint32)
    lib().orc_int4_random(C.c_uint64(seed), N, K, _p(packed), _p(scale), _p(zp))
    return packed, scale, zp


def fp8_quantize(w):
    w = np.ascontiguousarray(w, np.float32)
    N, K = w.shape
    codes = np.empty((N, K), np.uint8)
    scales = np.empty(((N + 127) // 128, K // 128), np.float32)
    lib().orc_fp8_quantize(_p(w), N, K, _p(codes), _p(scales))
    return codes, scales


def fp8_dequant(codes, scales):
    N, K = codes.shape
    o = np.empty((N, K), np.float32)
    lib().orc_fp8_dequant(_p(codes), _p(scales), N, K, _p(o))
    return o


def fp8_random(seed, N, K, scale):
    codes = np.empty((N, K), np.uint8)
    scales = np.empty(((N + 127) // 128, K // 128), np.float32)
    lib().orc_fp8_random(C.c_uint64(seed), N, K, C.c_float(scale), _p(codes), _p(scales))
    return codes, scales


def act_quant(x):
    x = np.ascontiguousarray(x, np.uint16)
    T, K = x.shape
    q = np.empty((T, K), np.uint8)
    s = np.empty((T, K // 128), np.float32)
    lib().orc_act_quant(_p(x), T, K, _p(q), _p(s))
    return q, s


# ---- router ---------------------------------------------------------------------------------------------------
def route(logits, bias, topk, scale, score_fn=0):
    logits = np.ascontiguousarray(logits, np.float32)
    M, E = logits.shape
    idx = np.empty((M, topk), np.int32)
    w = np.empty((M, topk), np.float32)
    b = None if bias is None else np.ascontiguousarray(bias, np.float32)
    lib().orc_route(_p(logits), _p(b), M, E, topk, C.c_float(scale), score_fn, _p(idx), _p(w))
    return idx, w


def union(idx, E):
    idx = np.ascontiguousarray(idx, np.int32)
    u = np.empty(idx.size, np.int32)
    n = lib().orc_union(_p(idx), idx.size, E, _p(u))
    return u[:n].copy()


# ---- GEMV -----------------------------------------------------------------------------------------------------
def gemv(x, fmt, w, s, zp, N, K, out_kind=OUT_BF16, want64=True):
    """x bf16 bits [M][K]. Returns dict(y16, yf, yd, ymag)."""
    x = np.ascontiguousarray(x, np.uint16)
    M = x.shape[0]
    y16 = np.empty((M, N // 2 if out_kind == OUT_SWIGLU else N), np.uint16)
    yf = np.empty((M, N), np.float32)
    yd = np.empty((M, N), np.float64) if want64 else None
    ym = np.empty((M, N), np.float64) if want64 else None
    lib().orc_gemv(_p(x), x.shape[1], M, K, fmt, _p(w), _p(s), _p(zp), N, out_kind, _p(y16), _p(yf), _p(yd), _p(ym))
    return dict(y16=y16, yf=yf, yd=yd, ymag=ym)


# ---- MoE ------------------------------------------------------------------------------------------------------
def moe_up(hl, x, uni, sum_tol=2e-5, want_range=True):
    """hl: a host layer (dsgx10_amd.layer.HostLayer). Returns dict(h32, h64, lo, hi) [US][M][I]."""
    x = np.ascontiguousarray(x, np.uint16)
    M = x.shape[0]
    uni = np.ascontiguousarray(uni, np.int32)
    US = len(uni) + (1 if hl.has_shared else 0)
    shp = (US, M, hl.I)
    h32, h64 = np.empty(shp, np.uint16), np.empty(shp, np.uint16)
    lo = np.empty(shp, np.float32) if want_range else None
    hi = np.empty(shp, np.float32) if want_range else None
    Lw, desc = hl.host_layer_w()
    lib().orc_moe_up(C.byref(Lw), _p(desc), _p(x), M, _p(uni), len(uni), C.c_double(sum_tol), _p(h32), _p(h64), _p(lo), _p(hi))
    return dict(h32=h32, h64=h64, lo=lo, hi=hi)


def moe_down(hl, h, idx, w, uni, ysum=False, ys_in=None):
    h = np.ascontiguousarray(h, np.uint16)
    M = h.shape[1]
    idx = np.ascontiguousarray(idx, np.int32)
    w = np.ascontiguousarray(w, np.float32)
    uni = np.ascontiguousarray(uni, np.int32)
    H = hl.H
    out = {k: np.zeros((M, H), np.float32 if k.endswith("32") else np.float64)
           for k in ("yr32", "ys32", "yr64", "ys64", "yrmag", "ysmag")}
    Lw, desc = hl.host_layer_w()
    ysi = None if ys_in is None else np.ascontiguousarray(ys_in, np.float32)
    lib().orc_moe_down(C.byref(Lw), _p(desc), _p(h), M, _p(idx), _p(w), _p(uni), len(uni), int(ysum), _p(ysi),
                       _p(out["yr32"]), _p(out["ys32"]), _p(out["yr64"]), _p(out["ys64"]), _p(out["yrmag"]), _p(out["ysmag"]))
    return out


def moe_prefill_fp8_row(hl, xrow, idx, w, h_in=None):
    """h_in: bf16 [topk in expert-id order (+ 1, the shared expert's)][I] to start the down projections from"""
    xrow = np.ascontiguousarray(xrow, np.uint16)
    idx = np.ascontiguousarray(idx, np.int32)
    w = np.ascontiguousarray(w, np.float32)
    H, I, topk = hl.H, hl.I, hl.topk
    h = np.empty((topk + 1, I), np.uint16)
    hin = None if h_in is None else np.ascontiguousarray(h_in, np.uint16)
    out = dict(h=h, yr=np.empty(H, np.float32), yr64=np.empty(H, np.float64), yrmag=np.empty(H, np.float64),
               ys=np.zeros(H, np.float32), ys64=np.zeros(H, np.float64), ysmag=np.zeros(H, np.float64))
    Lw, desc = hl.host_layer_w()
    lib().orc_moe_prefill_fp8_row(C.byref(Lw), _p(desc), _p(xrow), _p(idx), _p(w), _p(h), _p(out["yr"]), _p(out["yr64"]),
                                  _p(out["yrmag"]), _p(out["ys"]), _p(out["ys64"]), _p(out["ysmag"]), _p(hin))
    return out


def moe_prefill_b16_row_mfma(hl, xrow, idx, w):
    """one chunk row through the bf16-activation prefill with every sum added as the bf16 MFMA adds it in the kernels' k map:
    dict(h bf16 [topk in expert-id order (+ 1, the shared expert's)][I], yr f32 [H], ys f32 [H])"""
    xrow = np.ascontiguousarray(xrow, np.uint16)
    idx = np.ascontiguousarray(idx, np.int32)
    w = np.ascontiguousarray(w, np.float32)
    out = dict(h=np.empty((hl.topk + (1 if hl.has_shared else 0), hl.I), np.uint16), yr=np.empty(hl.H, np.float32), ys=np.zeros(hl.H, np.float32))
    Lw, desc = hl.host_layer_w()
    lib().orc_moe_prefill_b16_row_mfma(C.byref(Lw), _p(desc), _p(xrow), _p(idx), _p(w), _p(out["h"]), _p(out["yr"]), _p(out["ys"]))
    return out


def moe_prefill_fp8_row_range(hl, xrow, idx, sum_tol):
    """(lo, hi) f32 [topk in expert-id order (+ 1)][I]: the values h may take when the gate and up sums move by
    sum_tol * their sums of |terms|"""
    xrow = np.ascontiguousarray(xrow, np.uint16)
    idx = np.ascontiguousarray(idx, np.int32)
    n = hl.topk + (1 if hl.has_shared else 0)
    lo, hi = np.empty((n, hl.I), np.float32), np.empty((n, hl.I), np.float32)
    Lw, desc = hl.host_layer_w()
    lib().orc_moe_prefill_fp8_row_range(C.byref(Lw), _p(desc), _p(xrow), _p(idx), C.c_double(sum_tol), _p(lo), _p(hi))
    return lo, hi


def moe_prefill_fp8_row_h_perturbed(hl, xrow, idx, sum_eps, seed=0):
    """h bf16 [topk in expert-id order (+ 1)][I] with every gate and up sum moved by sum_eps * r * its sum of |terms|,
    r uniform in [-1, 1) (seeded); sum_eps = 0: the h of the f64 sums"""
    xrow = np.ascontiguousarray(xrow, np.uint16)
    idx = np.ascontiguousarray(idx, np.int32)
    n = hl.topk + (1 if hl.has_shared else 0)
    h = np.empty((n, hl.I), np.uint16)
    Lw, desc = hl.host_layer_w()
    lib().orc_moe_prefill_fp8_row_h_perturbed(C.byref(Lw), _p(desc), _p(xrow), _p(idx), C.c_double(sum_eps), C.c_uint64(seed), _p(h))
    return h


def add_norm(part, part2, res, w, eps, round2=False):
    """(res_out bf16, xn bf16 from f64 statistics, xn bf16 from sequential f32 statistics), each [M][H]"""
    part = np.ascontiguousarray(part, np.float32)
    M, H = part.shape
    p2 = None if part2 is None else np.ascontiguousarray(part2, np.float32)
    res, w = np.ascontiguousarray(res, np.uint16), np.ascontiguousarray(w, np.uint16)
    ro, xn, xn32 = np.empty((M, H), np.uint16), np.empty((M, H), np.uint16), np.empty((M, H), np.uint16)
    lib().orc_add_norm(_p(part), _p(p2), M, H, _p(res), _p(w), C.c_float(eps), int(round2), _p(ro), _p(xn), _p(xn32))
    return ro, xn, xn32


def finalize(R, S):
    R = np.ascontiguousarray(R, np.float32)
    S = np.ascontiguousarray(S, np.float32)
    o = np.empty(R.shape, np.uint16)
    lib().orc_finalize(_p(R), _p(S), C.c_size_t(R.size), _p(o))
    return o


def set_f32_only(on):
    """the timed CPU baseline computes the f32 contract sums only"""
    lib().orc_set_f32_only(int(on))


def threads():
    return lib().orc_threads()


# ---- DeepSeek's MXFP4 x FP8 expert ---------------------------------------------------------------------------------------
def e2m1_table():
    lib().orc_e2m1_value.restype = C.c_float
    return np.array([lib().orc_e2m1_value(i) for i in range(16)], np.float32)


def ue8m0_value(b):
    lib().orc_ue8m0_value.restype = C.c_float
    return lib().orc_ue8m0_value(int(b))


def act_scale_byte(amax):
    return lib().orc_act_scale_byte(C.c_float(amax))


def act_quant_ue8m0(x):
    """x bf16 bits [T][K] -> (e4m3 codes u8 [T][K], ue8m0 bytes u8 [T][K/32])"""
    x = np.ascontiguousarray(x, np.uint16)
    T, K = x.shape
    q, s = np.empty((T, K), np.uint8), np.empty((T, K // 32), np.uint8)
    lib().orc_act_quant_ue8m0(_p(x), T, K, _p(q), _p(s))
    return q, s


def dequant_act_ue8m0(q, s):
    q, s = np.ascontiguousarray(q, np.uint8), np.ascontiguousarray(s, np.uint8)
    T, K = q.shape
    o = np.empty((T, K), np.float32)
    lib().orc_dequant_act_ue8m0(_p(q), _p(s), T, K, _p(o))
    return o


def mxfp4_dequant(w, s):
    """w u8 [N][K/2], s ue8m0 [N][K/32] -> f32 [N][K]"""
    w, s = np.ascontiguousarray(w, np.uint8), np.ascontiguousarray(s, np.uint8)
    N, K = w.shape[0], w.shape[1] * 2
    o = np.empty((N, K), np.float32)
    lib().orc_mxfp4_dequant(_p(w), _p(s), N, K, _p(o))
    return o


def fp8e_dequant(w, s):
    """e4m3 codes u8 [N][K], ue8m0 [N/32][K/32] -> f32 [N][K]"""
    w, s = np.ascontiguousarray(w, np.uint8), np.ascontiguousarray(s, np.uint8)
    N, K = w.shape
    o = np.empty((N, K), np.float32)
    lib().orc_fp8e_dequant(_p(w), _p(s), N, K, _p(o))
    return o


def dsk_up(w1, w3, xd, rw=None, limit=10.0, sum_tol=2e-5, want_range=True):
    """dequantised w1, w3 f32 [I][H], xd f32 [M][H], rw f32 [M] or None (the shared expert) -> dict h32, h64 (bf16 bits), lo, hi"""
    w1, w3, xd = (np.ascontiguousarray(a, np.float32) for a in (w1, w3, xd))
    I, H = w1.shape
    M = xd.shape[0]
    r = None if rw is None else np.ascontiguousarray(rw, np.float32)
    h32, h64 = np.empty((M, I), np.uint16), np.empty((M, I), np.uint16)
    lo, hi = (np.empty((M, I), np.float32), np.empty((M, I), np.float32)) if want_range else (None, None)
    lib().orc_dsk_up(_p(w1), _p(w3), _p(xd), M, H, I, _p(r), C.c_float(limit), C.c_double(sum_tol), _p(h32), _p(h64), _p(lo), _p(hi))
    return dict(h32=h32, h64=h64, lo=lo, hi=hi)


def dsk_down(w2, hpre):
    """dequantised w2 f32 [H][I], hpre bf16 bits [M][I] -> dict hq, hs, out32, out64, mag, outb (bf16 bits)"""
    w2, hpre = np.ascontiguousarray(w2, np.float32), np.ascontiguousarray(hpre, np.uint16)
    H, I = w2.shape
    M = hpre.shape[0]
    o = dict(hq=np.empty((M, I), np.uint8), hs=np.empty((M, I // 32), np.uint8), out32=np.empty((M, H), np.float32),
             out64=np.empty((M, H), np.float64), mag=np.empty((M, H), np.float64), outb=np.empty((M, H), np.uint16))
    lib().orc_dsk_down(_p(w2), _p(hpre), M, H, I, _p(o["hq"]), _p(o["hs"]), _p(o["out32"]), _p(o["out64"]), _p(o["mag"]), _p(o["outb"]))
    return o


def dsk_up_mx(w1, s1, w3, s3, a_fp4, xq, xs, rw=None, limit=10.0):
    """DeepSeek's gate/up with every dot product added as the block-scaled MFMA adds it: weights as stored (e2m1 pairs [I][H/2]
    with ue8m0 [I][H/32], or e4m3 [I][H] with ue8m0 [I/32][H/32]), rows e4m3 [M][H] + ue8m0 [M][H/32] -> h bf16 bits [M][I]"""
    w1, s1, w3, s3, xq, xs = (np.ascontiguousarray(v, np.uint8) for v in (w1, s1, w3, s3, xq, xs))
    M, H = xq.shape
    I = w1.shape[0]
    r = None if rw is None else np.ascontiguousarray(rw, np.float32)
    h = np.empty((M, I), np.uint16)
    lib().orc_dsk_up_mx(_p(w1), _p(s1), _p(w3), _p(s3), int(a_fp4), _p(xq), _p(xs), M, H, I, _p(r), C.c_float(limit), _p(h))
    return h


def dsk_down_mx(w2, s2, a_fp4, hpre):
    """w2 as stored ([H][I/2] e2m1 or [H][I] e4m3), hpre bf16 bits [M][I] -> dict hq, hs (h as the GEMM reads it), outb (bf16 bits [M][H])"""
    w2, s2, hpre = np.ascontiguousarray(w2, np.uint8), np.ascontiguousarray(s2, np.uint8), np.ascontiguousarray(hpre, np.uint16)
    M, I = hpre.shape
    H = w2.shape[0]
    o = dict(hq=np.empty((M, I), np.uint8), hs=np.empty((M, I // 32), np.uint8), outb=np.empty((M, H), np.uint16))
    lib().orc_dsk_down_mx(_p(w2), _p(s2), int(a_fp4), _p(hpre), M, H, I, _p(o["hq"]), _p(o["hs"]), _p(o["outb"]))
    return o


def mfma_fp8_k128(a, b):
    """the oracle's statement of gfx950's v_mfma_f32_16x16x128_f8f6f4 block sum: e4m3 codes a [R][128], b [S][128] in
    register order -> f32 [R][S]"""
    a, b = np.ascontiguousarray(a, np.uint8), np.ascontiguousarray(b, np.uint8)
    lib().orc_mfma_fp8_k128.restype = C.c_float
    out = np.empty((a.shape[0], b.shape[0]), np.float32)
    for i in range(a.shape[0]):
        for j in range(b.shape[0]):
            out[i, j] = lib().orc_mfma_fp8_k128(C.c_void_p(a[i].ctypes.data), C.c_void_p(b[j].ctypes.data))
    return out


def mfma_scaled_k128(a, sa, a_fp4, b, sb, acc=None):
    """the oracle's statement of gfx950's v_mfma_scale_f32_16x16x128_f8f6f4: a [R][64] e2m1 pairs (a_fp4) or [R][128] e4m3 codes,
    b e4m3 [S][128], sa [R][4], sb [S][4] ue8m0 bytes, acc f32 [R][S] (None: zeros), all in k order as stored -> f32 [R][S]"""
    a, b, sa, sb = (np.ascontiguousarray(v, np.uint8) for v in (a, b, sa, sb))
    f = lib().orc_mfma_scaled_k128
    f.restype = C.c_float
    f.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_float]
    out = np.empty((a.shape[0], b.shape[0]), np.float32)
    for i in range(a.shape[0]):
        for j in range(b.shape[0]):
            out[i, j] = f(a[i].ctypes.data, sa[i].ctypes.data, int(a_fp4), b[j].ctypes.data, sb[j].ctypes.data, 0.0 if acc is None else float(acc[i, j]))
    return out


def mfma_bf16_k32(a, b, acc=None):
    """the oracle's statement of gfx950's v_mfma_f32_16x16x32_bf16: a bf16 bits [R][32], b [S][32] in the instruction's k order
    (k = 8 part + i of a lane), acc f32 [R][S] (None: zeros) -> f32 [R][S]"""
    a, b = (np.ascontiguousarray(v, np.uint16) for v in (a, b))
    f = lib().orc_mfma_bf16_k32
    f.restype = C.c_float
    f.argtypes = [C.c_void_p, C.c_void_p, C.c_float]
    out = np.empty((a.shape[0], b.shape[0]), np.float32)
    for i in range(a.shape[0]):
        for j in range(b.shape[0]):
            out[i, j] = f(a[i].ctypes.data, b[j].ctypes.data, 0.0 if acc is None else float(acc[i, j]))
    return out


def dot2_bf16(a, b, c):
    """the oracle's statement of v_dot2_f32_bf16: a, b packed bf16 pairs (uint32 [n]), c f32 [n] -> f32 [n]"""
    a, b, c = np.ascontiguousarray(a, np.uint32), np.ascontiguousarray(b, np.uint32), np.ascontiguousarray(c, np.float32)
    f = lib().orc_dot2_bf16
    f.restype = C.c_float
    f.argtypes = [C.c_uint32, C.c_uint32, C.c_float]
    return np.array([f(int(a[i]), int(b[i]), float(c[i])) for i in range(a.size)], np.float32)


def set_dot_rule(rule, splitk=1):
    """how moe_up / moe_down / gemv add the f32 sum of a dot product: 0 in the contract's order (sequential), 1 as the bf16 MFMA
    adds it in the prefill kernels, 2 as in the MFMA decode kernels (cfg.up = 1), 3 as in the vector-unit decode kernels (cfg.up = 0),
    4 as in the dense GEMV (splitk: the split of K the call asked for, where the kernel honours it: up to 8192 rows).
    Tests that set it put it back to 0."""
    lib().orc_set_dot_rule(int(rule))
    lib().orc_set_gemv_splitk(int(splitk))


def set_dsk_dot_rule(rule):
    """how dsk_up / dsk_down add their f32 sums: 0 in k order, 1 / 3 as DeepSeek's decode kernels add them on the bf16 MFMA (1: the
    MXFP4 experts, 3: the shared expert). Tests that set it put it back to 0."""
    lib().orc_set_dsk_dot_rule(int(rule))


def set_fp8_block_rule(rule):
    """0: a 128-k block's products are added sequentially in f32 (the contract as the reference's CPU stand-in states it);
    1: by the gfx950 matrix unit's rule (orc_mfma_fp8_k128) in the prefill kernels' k map"""
    lib().orc_set_fp8_block_rule(int(rule))
