"""ctypes mirror of include/dsgx.h: constants and structures only (loads nothing)."""
import ctypes as C

FMT_REF_NVFP4, FMT_REF_INT4, FMT_REF_BF16 = 0, 2, 3
FMT_FP8, FMT_INT4, FMT_BF16 = 16, 18, 19
FMT_MXFP4, FMT_FP8E = 20, 21  # DeepSeek's routed experts; their shared expert (ue8m0 scales per 32 x 32)
OUT_BF16, OUT_F32, OUT_SWIGLU = 0, 1, 2
MAX_ROWS, MAX_TOPK, MAX_UNION, SH_SLOT, MAX_EXPERTS, MAX_CHUNK = 16, 8, 128, 128, 512, 8192
UP_PREFILL_ORDER = 6  # dsgx_decode_cfg.up: the rows through the prefill kernels (gx::kUpPrefillOrder), bf16 activations
UP_PREFILL_ORDER_ACT_FP8 = 7  # ... with FP8 activations (the default prefill of FP8 layers)
OK, EINVAL, EFORMAT, EUNSUPPORTED, EHIP, ETIMEOUT = 0, 1, 2, 3, 4, 5
NOALLOC_MAX_H, NOALLOC_MAX_I = 6144, 2048


class MatDesc(C.Structure):
    _fields_ = [("off", C.c_uint64), ("s2", C.c_float), ("fmt", C.c_uint32), ("rsv", C.c_uint32 * 12)]


class SharedW(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("g", "u", "d", "gs", "us", "ds", "bgu", "bd")]


class LayerW(C.Structure):
    _fields_ = [("pool", C.c_void_p), ("desc", C.c_void_p), ("sh", SharedW), ("fmt", C.c_uint32),
                ("H", C.c_int32), ("I", C.c_int32), ("E", C.c_int32), ("topk", C.c_int32)]


class DskCfg(C.Structure):
    _fields_ = [("swiglu_limit", C.c_float), ("logits", C.c_void_p), ("bias", C.c_void_p), ("route_scale", C.c_float), ("parts", C.c_int32)]


class DskWeights(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("w1", "s1", "w3", "s3", "w2", "s2", "sh_w1", "sh_s1", "sh_w3", "sh_s3", "sh_w2", "sh_s2")] + \
               [(n, C.c_int32) for n in ("H", "I", "E", "topk")]


class DskPrefillCfg(C.Structure):
    _fields_ = [("swiglu_limit", C.c_float), ("phases", C.c_int32)]


class DskPrefillView(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("rpos", "re", "off", "perm", "h", "hsh", "d", "dsh", "hq", "hs")]


class DecodeCfg(C.Structure):
    _fields_ = [("up", C.c_int32), ("down", C.c_int32), ("parts", C.c_int32), ("ysum", C.c_int32),
                ("logits", C.c_void_p), ("bias", C.c_void_p), ("route_scale", C.c_float), ("score_fn", C.c_int32),
                ("post", C.c_void_p)]


class PrefillCfg(C.Structure):
    _fields_ = [("shared", C.c_int32), ("phases", C.c_int32), ("act_fp8", C.c_int32), ("fast_act", C.c_int32), ("tile_order", C.c_int32)]


class PrefillView(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("rpos", "re", "h", "hsh", "off", "perm")]


class NormIn(C.Structure):
    _fields_ = [("part", C.c_void_p), ("part2", C.c_void_p), ("res", C.c_void_p), ("res_out", C.c_void_p), ("w", C.c_void_p), ("eps", C.c_float),
                ("xn", C.c_void_p), ("round2", C.c_int32)]


class GemvSeg(C.Structure):
    _fields_ = [("fmt", C.c_int32), ("w", C.c_void_p), ("s", C.c_void_p), ("zp", C.c_void_p), ("n", C.c_int32),
                ("rs", C.c_int32), ("ks", C.c_int32), ("y", C.c_void_p), ("ldy", C.c_int32)]


assert C.sizeof(MatDesc) == 64

# every symbol include/dsgx.h declares
SYMBOLS = [
    "dsgx_mat_bytes", "dsgx_mat_scale_off", "dsgx_mat_zp_off", "dsgx_route", "dsgx_decode_cfg_default",
    "dsgx_decode_ws_bytes", "dsgx_decode_ws_flag_offset", "dsgx_decode_status", "dsgx_moe_decode", "dsgx_moe_decode_noalloc", "dsgx_finalize", "dsgx_add_norm", "dsgx_dsk_cfg_default", "dsgx_dsk_moe", "dsgx_dsk_ws_bytes", "dsgx_dsk_moe_stacked", "dsgx_prefill_cfg_default", "dsgx_prefill_ws_bytes",
    "dsgx_moe_prefill", "dsgx_prefill_view_get", "dsgx_gemv", "dsgx_dequant_int4", "dsgx_probe_dequant_int4", "dsgx_probe_mfma_fp8",
    "dsgx_widen_fp8", "dsgx_act_quant", "dsgx_last_error", "dsgx_version", "dsgx_stream_read", "dsgx_stream_read_cfg", "dsgx_stream_copy", "dsgx_add_norm_gemv", "dsgx_fill_normal", "dsgx_launch_floor",
    "dsgx_dsk_prefill_cfg_default", "dsgx_dsk_prefill_ws_bytes", "dsgx_dsk_moe_prefill", "dsgx_dsk_prefill_view_get", "dsgx_probe_mfma_scaled", "dsgx_probe_mfma_bf16", "dsgx_probe_dot2_bf16",
]
