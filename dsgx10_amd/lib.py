"""Loader of the C ABI (dsgx10_amd/csrc/libdsgx.so) and the Python mirror of the reference's operators for this path
(gx::route, gx::moe_decode, gx::moe_prefill, gx::finalize, glm::gemv, glm::dequant_int4): same names, argument
meaning and error behaviour (the reference dies; these raise DsgxError). torch is used for device memory and
streams only. There is no CPU path: a missing library raises."""
import ctypes as C
import os

from . import abi

_SO = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", os.environ.get("DSGX_LIB", "libdsgx.so"))
_lib = None


class DsgxError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("dsgx status %d: %s" % (code, msg))
        self.code = code


def so_path():
    return _SO


def lib():
    """The loaded C ABI. Raises if the HIP extension has not been built (python -m dsgx10_amd.build)."""
    global _lib
    if _lib is None:
        import torch  # noqa: F401  first: the library must bind to the HIP runtime torch's streams and buffers belong to
        if not os.path.exists(_SO):
            raise RuntimeError("dsgx10_amd: %s is missing; build it with `python -m dsgx10_amd.build` (there is no CPU fallback)" % _SO)
        L = C.CDLL(_SO)
        L.dsgx_last_error.restype = C.c_char_p
        L.dsgx_version.restype = C.c_char_p
        for f in ("dsgx_mat_bytes", "dsgx_mat_scale_off", "dsgx_mat_zp_off"):
            getattr(L, f).restype = C.c_size_t
            getattr(L, f).argtypes = [C.c_uint32, C.c_int, C.c_int]
        for f in ("dsgx_decode_ws_bytes", "dsgx_decode_ws_flag_offset"):
            getattr(L, f).restype = C.c_size_t
            getattr(L, f).argtypes = [C.POINTER(abi.LayerW)]
        L.dsgx_route.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_float, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        L.dsgx_moe_decode.argtypes = [C.POINTER(abi.LayerW), C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p,
                                      C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(abi.DecodeCfg)]
        L.dsgx_moe_decode_noalloc.argtypes = [C.POINTER(abi.LayerW), C.c_void_p, C.c_void_p, C.c_void_p, C.c_int,
                                              C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(abi.DecodeCfg)]
        L.dsgx_decode_status.argtypes = [C.POINTER(abi.LayerW), C.c_void_p, C.c_void_p]
        L.dsgx_dsk_moe.argtypes = [C.POINTER(abi.LayerW), C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                   C.c_void_p, C.c_void_p, C.POINTER(abi.DskCfg)]
        L.dsgx_finalize.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]
        L.dsgx_add_norm.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_float,
                                    C.c_void_p, C.c_int, C.c_void_p]
        L.dsgx_gemv.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.POINTER(abi.GemvSeg), C.c_int, C.c_int, C.c_int, C.c_void_p]
        for f in ("dsgx_dequant_int4", "dsgx_probe_dequant_int4"):
            getattr(L, f).argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_size_t, C.c_void_p]
        L.dsgx_widen_fp8.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_size_t, C.c_void_p]
        L.dsgx_act_quant.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        L.dsgx_stream_read.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p]
        L.dsgx_stream_read_cfg.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_int, C.c_int, C.c_void_p]
        L.dsgx_stream_copy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]
        L.dsgx_probe_mfma_fp8.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p]
        L.dsgx_dsk_ws_bytes.restype = C.c_size_t
        L.dsgx_dsk_ws_bytes.argtypes = [C.c_int, C.c_int]
        L.dsgx_dsk_moe_stacked.argtypes = [C.POINTER(abi.DskWeights), C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                           C.c_void_p, C.POINTER(abi.DskCfg), C.c_void_p, C.c_void_p]
        L.dsgx_dsk_prefill_ws_bytes.restype = C.c_size_t
        L.dsgx_dsk_prefill_ws_bytes.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
        L.dsgx_dsk_moe_prefill.argtypes = [C.POINTER(abi.DskWeights), C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                           C.c_void_p, C.POINTER(abi.DskPrefillCfg)]
        L.dsgx_dsk_prefill_view_get.argtypes = [C.POINTER(abi.DskWeights), C.c_void_p, C.c_int, C.POINTER(abi.DskPrefillView)]
        L.dsgx_probe_mfma_scaled.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        L.dsgx_probe_mfma_bf16.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        L.dsgx_probe_dot2_bf16.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p]
        L.dsgx_add_norm_gemv.argtypes = [C.POINTER(abi.NormIn), C.c_int, C.c_int, C.POINTER(abi.GemvSeg), C.c_int, C.c_int, C.c_int, C.c_void_p]
        L.dsgx_fill_normal.argtypes = [C.c_uint64, C.c_uint64, C.c_size_t, C.c_double, C.c_void_p, C.c_int, C.c_void_p]
        L.dsgx_launch_floor.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        if hasattr(L, "dsgx_moe_prefill"):
            L.dsgx_prefill_ws_bytes.restype = C.c_size_t
            L.dsgx_prefill_ws_bytes.argtypes = [C.POINTER(abi.LayerW), C.c_int]
            L.dsgx_moe_prefill.argtypes = [C.POINTER(abi.LayerW), C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p,
                                           C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(abi.PrefillCfg)]
            L.dsgx_prefill_view_get.argtypes = [C.POINTER(abi.LayerW), C.c_void_p, C.c_int, C.POINTER(abi.PrefillView)]
        _lib = L
    return _lib


def _check(rc):
    if rc:
        raise DsgxError(rc, lib().dsgx_last_error().decode())


def _ptr(t):
    return None if t is None else t.data_ptr()


def _stream(stream=None):
    import torch
    s = stream if stream is not None else torch.cuda.current_stream()
    return s.cuda_stream


# ---- gx::route ------------------------------------------------------------------------------------------------------
def route(logits, bias, idx, w, route_scale=2.5, score_fn=0, stream=None):
    """logits f32 [M][E], bias f32 [E] or None -> idx i32 [M][topk], w f32 [M][topk] (filled)."""
    M, E = logits.shape
    topk = idx.shape[1]
    _check(lib().dsgx_route(_ptr(logits), _ptr(bias), M, E, topk, route_scale, score_fn, _ptr(idx), _ptr(w), _stream(stream)))


# ---- gx::moe_decode ---------------------------------------------------------------------------------------------------
def decode_ws_bytes(layer_w):
    return lib().dsgx_decode_ws_bytes(C.byref(layer_w))


def decode_ws_flag_offset(layer_w):
    return lib().dsgx_decode_ws_flag_offset(C.byref(layer_w))


def moe_decode(layer_w, x, idx, w, M, ws, yr, ys, stream=None, parts=3, ysum=False, logits=None, bias=None,
               route_scale=1.0, score_fn=0, up=-1, down=0, post=None):
    """ws None: the library's own workspace (dsgx_moe_decode_noalloc). up -1: the library's choice of variant."""
    cfg = abi.DecodeCfg(up, down, parts, int(ysum), _ptr(logits), _ptr(bias), route_scale, score_fn, post)
    if ws is None:
        _check(lib().dsgx_moe_decode_noalloc(C.byref(layer_w), _ptr(x), _ptr(idx), _ptr(w), M, _ptr(yr), _ptr(ys),
                                             _stream(stream), C.byref(cfg)))
        return
    _check(lib().dsgx_moe_decode(C.byref(layer_w), _ptr(x), _ptr(idx), _ptr(w), M, _ptr(ws), _ptr(yr), _ptr(ys),
                                 _stream(stream), C.byref(cfg)))


def dsk_moe(layer_w, xq, xs, idx, w, M, ws, y, ys, stream=None, limit=10.0, logits=None, bias=None, route_scale=1.0, parts=3):
    """DeepSeek's decode MoE (dsk::moe / moe_routed): MXFP4 experts + FP8 shared expert, rows given as act_quant(x)"""
    cfg = abi.DskCfg(limit, _ptr(logits), _ptr(bias), route_scale, parts)
    _check(lib().dsgx_dsk_moe(C.byref(layer_w), _ptr(xq), _ptr(xs), M, _ptr(idx), _ptr(w), _ptr(ws), _ptr(y), _ptr(ys), _stream(stream),
                              C.byref(cfg)))


def dsk_ws_bytes(H, I):
    return lib().dsgx_dsk_ws_bytes(H, I)


def dsk_moe_stacked(weights, xq, xs, idx, w, M, ws, y, stream=None, limit=10.0, logits=None, bias=None, route_scale=1.0, parts=3, idx_out=None,
                    wts_out=None):
    """dsk::moe / moe_routed on experts stacked by id (abi.DskWeights); the shared expert's rows stay in ws (dsk_ws_bytes)"""
    cfg = abi.DskCfg(limit, _ptr(logits), _ptr(bias), route_scale, parts)
    _check(lib().dsgx_dsk_moe_stacked(C.byref(weights), _ptr(xq), _ptr(xs), M, _ptr(idx), _ptr(w), _ptr(ws), _ptr(y), _stream(stream),
                                      C.byref(cfg), _ptr(idx_out), _ptr(wts_out)))


def dsk_prefill_ws_bytes(H, I, E, topk, T):
    return lib().dsgx_dsk_prefill_ws_bytes(H, I, E, topk, T)


def dsk_moe_prefill(weights, xq, xs, idx, w, T, ws, y, stream=None, limit=10.0, phases=31):
    """dsk::moe_prefill: a chunk of T quantised rows through the MXFP4 experts (abi.DskWeights) on the block-scaled MFMA"""
    cfg = abi.DskPrefillCfg(limit, phases)
    _check(lib().dsgx_dsk_moe_prefill(C.byref(weights), _ptr(xq), _ptr(xs), T, _ptr(idx), _ptr(w), _ptr(ws), _ptr(y), _stream(stream), C.byref(cfg)))


def dsk_prefill_view(weights, ws, T):
    v = abi.DskPrefillView()
    _check(lib().dsgx_dsk_prefill_view_get(C.byref(weights), _ptr(ws), T, C.byref(v)))
    return v


def probe_mfma_bf16(A, B, out, stream=None, acc=None):
    _check(lib().dsgx_probe_mfma_bf16(_ptr(A), _ptr(B), _ptr(acc), _ptr(out), _stream(stream)))


def probe_dot2_bf16(a, b, c, out, n, stream=None):
    """out[i] = c[i] + a[i].lo b[i].lo + a[i].hi b[i].hi by v_dot2_f32_bf16 (a, b packed bf16 pairs, c, out f32; device tensors)"""
    _check(lib().dsgx_probe_dot2_bf16(_ptr(a), _ptr(b), _ptr(c), _ptr(out), int(n), _stream(stream)))


def probe_mfma_scaled(A, SA, B, SB, a_fp4, out, stream=None, acc=None):
    _check(lib().dsgx_probe_mfma_scaled(_ptr(A), _ptr(SA), _ptr(B), _ptr(SB), int(a_fp4), _ptr(acc), _ptr(out), _stream(stream)))


def decode_status(layer_w, ws, stream=None):
    """waits for the stream; raises DsgxError(ETIMEOUT) if a fused decode step gave up at its grid barrier since the last
    check (ws None: the library's own workspace)"""
    _check(lib().dsgx_decode_status(C.byref(layer_w), _ptr(ws), _stream(stream)))


def finalize(R, S, n, out, stream=None):
    """out[i] = bf16(bf16(R[i]) + bf16(S[i])) for n = M * H values"""
    _check(lib().dsgx_finalize(_ptr(R), _ptr(S), n, _ptr(out), _stream(stream)))


def add_norm(part, part2, M, H, res, res_out, w, eps, xn, round2=False, stream=None):
    """h = bf16(f32(res) + sum) -> res_out; xn = bf16(w * bf16(h * rstd)): the local half of allreduce_add_norm"""
    _check(lib().dsgx_add_norm(_ptr(part), _ptr(part2), M, H, _ptr(res), _ptr(res_out), _ptr(w), eps, _ptr(xn), int(round2), _stream(stream)))


# ---- gx::moe_prefill --------------------------------------------------------------------------------------------------
def prefill_ws_bytes(layer_w, T):
    return lib().dsgx_prefill_ws_bytes(C.byref(layer_w), T)


def moe_prefill(layer_w, x, idx, w, T, ws, yr, ys, stream=None, shared=True, phases=31, act_fp8=True, fast_act=False, tile_order=-1):
    cfg = abi.PrefillCfg(int(shared), phases, int(act_fp8), int(fast_act), int(tile_order))
    _check(lib().dsgx_moe_prefill(C.byref(layer_w), _ptr(x), _ptr(idx), _ptr(w), T, _ptr(ws), _ptr(yr), _ptr(ys),
                                  _stream(stream), C.byref(cfg)))


def prefill_view(layer_w, ws, T):
    v = abi.PrefillView()
    _check(lib().dsgx_prefill_view_get(C.byref(layer_w), _ptr(ws), T, C.byref(v)))
    return v


# ---- glm::gemv ------------------------------------------------------------------------------------------------------------
def gemv(x, ldx, rows, K, segs, out, splitk=1, stream=None):
    """segs: list of dict(fmt, w, s, zp, n, y, ldy, rs=128, ks=128) with torch tensors."""
    arr = (abi.GemvSeg * len(segs))()
    for i, g in enumerate(segs):
        arr[i] = abi.GemvSeg(g["fmt"], _ptr(g["w"]), _ptr(g.get("s")), _ptr(g.get("zp")), g["n"], g.get("rs", 128),
                             g.get("ks", 128), _ptr(g["y"]), g["ldy"])
    _check(lib().dsgx_gemv(_ptr(x), ldx, rows, K, arr, len(segs), out, splitk, _stream(stream)))


def add_norm_gemv(part, part2, res, res_out, w, eps, xn, rows, K, segs, out, splitk=1, round2=False, stream=None):
    """dsgx_add_norm as the prologue of the GEMV that reads its rows: y = W RMSNorm(bf16(res + part)); res_out, xn optional"""
    arr = (abi.GemvSeg * len(segs))()
    for i, g in enumerate(segs):
        arr[i] = abi.GemvSeg(g["fmt"], _ptr(g["w"]), _ptr(g.get("s")), _ptr(g.get("zp")), g["n"], g.get("rs", 128),
                             g.get("ks", 128), _ptr(g["y"]), g["ldy"])
    n = abi.NormIn(_ptr(part), _ptr(part2), _ptr(res), _ptr(res_out), _ptr(w), eps, _ptr(xn), int(round2))
    _check(lib().dsgx_add_norm_gemv(C.byref(n), rows, K, arr, len(segs), out, splitk, _stream(stream)))


def fill_normal(seed, tid, n, sigma, out, bf16=False, stream=None):
    """out[i] = N(0, sigma) value i of tensor `tid` under `seed` (the oracle's generator), f32 or bf16 bits"""
    _check(lib().dsgx_fill_normal(C.c_uint64(seed), C.c_uint64(tid), C.c_size_t(n), C.c_double(sigma), _ptr(out), int(bf16), _stream(stream)))


def launch_floor(kind, buf=None, sink=None, stream=None):
    _check(lib().dsgx_launch_floor(kind, _ptr(buf), _ptr(sink), _stream(stream)))


def dequant_int4(packed, scale, zp, N, K, out, ld=None, stream=None, probe=False):
    f = lib().dsgx_probe_dequant_int4 if probe else lib().dsgx_dequant_int4
    _check(f(_ptr(packed), _ptr(scale), _ptr(zp), N, K, _ptr(out), ld or K, _stream(stream)))


def widen_fp8(codes, N, K, out, ld=None, stream=None):
    _check(lib().dsgx_widen_fp8(_ptr(codes), N, K, _ptr(out), ld or K, _stream(stream)))


def act_quant(x, T, K, q, s, stream=None):
    _check(lib().dsgx_act_quant(_ptr(x), T, K, _ptr(q), _ptr(s), _stream(stream)))


def stream_read(buf, nbytes, sink, stream=None):
    _check(lib().dsgx_stream_read(_ptr(buf), nbytes, _ptr(sink), _stream(stream)))


def stream_read_cfg(buf, nbytes, sink, wgs_per_cu, unroll, stream=None):
    _check(lib().dsgx_stream_read_cfg(_ptr(buf), nbytes, _ptr(sink), wgs_per_cu, unroll, _stream(stream)))


def stream_copy(src, dst, nbytes, stream=None):
    _check(lib().dsgx_stream_copy(_ptr(src), _ptr(dst), nbytes, _stream(stream)))


def probe_mfma_fp8(A, B, raw, form=0, stream=None):
    """raw f32 [64][16]: the accumulator registers of one e4m3 MFMA; form 0: 32x32x64 over A [32][64], B [32][64];
    form 1: 16x16x128 over A [16][128], B [16][128]"""
    _check(lib().dsgx_probe_mfma_fp8(_ptr(A), _ptr(B), _ptr(raw), form, _stream(stream)))
