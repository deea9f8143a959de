"""Host-side layer assembly: the checkpoint's canonical tensors placed into a weight pool with the 64-byte matrix
descriptors the kernels read (the role of the reference's TestLayer / make_desc: altar1-4xgx10-switchless/engine/experts/
tests/testdata.h:148-238, engine/experts/layout.h:165-183). numpy only; upload() needs torch and a GPU."""
import ctypes as C

import numpy as np

from . import abi

DESC_DTYPE = np.dtype([("off", "<u8"), ("s2", "<f4"), ("fmt", "<u4"), ("rsv", "<u4", (12,))])
assert DESC_DTYPE.itemsize == 64


def _al256(n):
    return (n + 255) // 256 * 256


def mat_bytes(fmt, N, K):
    """bytes of one [N][K] matrix in a pool format (dsgx_mat_bytes)."""
    if fmt == abi.FMT_FP8:
        return _al256(N * K) + _al256(((N + 127) // 128) * (K // 128) * 4)
    if fmt == abi.FMT_INT4:
        return _al256(N * K // 2) + _al256(N * (K // 32) * 2) + _al256((N // 8) * (K // 32) * 4)
    if fmt == abi.FMT_BF16:
        return _al256(N * K * 2)
    if fmt == abi.FMT_MXFP4:
        return _al256(N * K // 2) + _al256(N * (K // 32))
    raise ValueError("format %r is not FP8_B128 (16), INT4_G32 (18) or BF16 (19)" % (fmt,))


def mat_blob(fmt, parts):
    """One matrix's pool bytes from its canonical tensors: FP8 (codes u8 [N][K], scales f32), INT4 (packed u32 [N][K/8],
    scale bf16-bits u16 [N][K/32], zp u32 [N/8][K/32]), BF16 (bits u16 [N][K])."""
    if fmt == abi.FMT_FP8:
        codes, scales = parts
        N, K = codes.shape
        assert codes.dtype == np.uint8 and scales.dtype == np.float32 and scales.shape == ((N + 127) // 128, K // 128)
        chunks = [codes, scales]
    elif fmt == abi.FMT_INT4:
        packed, scale, zp = parts
        N, K = packed.shape[0], packed.shape[1] * 8
        assert packed.dtype == np.uint32 and scale.dtype == np.uint16 and zp.dtype == np.uint32
        assert scale.shape == (N, K // 32) and zp.shape == (N // 8, K // 32)
        chunks = [packed, scale, zp]
    elif fmt == abi.FMT_BF16:
        (w,) = parts
        N, K = w.shape
        assert w.dtype == np.uint16
        chunks = [w]
    elif fmt == abi.FMT_MXFP4:  # e2m1 pairs u8 [N][K/2] (low nibble the even k), ue8m0 u8 [N][K/32]
        packed, scale = parts
        N, K = packed.shape[0], packed.shape[1] * 2
        assert packed.dtype == np.uint8 and scale.dtype == np.uint8 and scale.shape == (N, K // 32)
        chunks = [packed, scale]
    else:
        raise ValueError("format %r" % (fmt,))
    out = np.zeros(mat_bytes(fmt, N, K), np.uint8)
    o = 0
    for c in chunks:
        b = np.ascontiguousarray(c).view(np.uint8).reshape(-1)
        out[o:o + b.size] = b
        o += _al256(b.size)
    return out, (N, K)


class HostLayer:
    """A layer of NS stored experts of one format; expert id e uses stored expert emap[e]."""

    def __init__(self, fmt, H, I, E, topk, experts, emap=None, shared_fp8=None, shared_bf16=None, s2=None):
        """experts: list of (gate_parts, up_parts, down_parts) canonical tensors. shared_fp8: ((gc, gs), (uc, us), (dc, ds)).
        shared_bf16: (bgu u16 [2I][H] interleaved, bd u16 [H][I])."""
        self.fmt, self.H, self.I, self.E, self.topk = fmt, H, I, E, topk
        self.emap = np.arange(E, dtype=np.int64) % len(experts) if emap is None else np.asarray(emap)
        offs, blobs, o = [], [], 0
        for ex in experts:
            for j, parts in enumerate(ex):
                b, (N, K) = mat_blob(fmt, parts)
                assert (N, K) == ((I, H) if j < 2 else (H, I)), (N, K, j)
                offs.append(o)
                blobs.append(b)
                o += b.size
        self.pool = np.zeros(max(o, 256), np.uint8)
        for off, b in zip(offs, blobs):
            self.pool[off:off + b.size] = b
        self.desc = np.zeros(E * 3, DESC_DTYPE)
        for e in range(E):
            for j in range(3):
                d = self.desc[e * 3 + j]
                d["off"] = offs[int(self.emap[e]) * 3 + j]
                d["s2"] = 1.0 if s2 is None else s2[j]
                d["fmt"] = fmt
        self.shared_fp8 = shared_fp8
        self.shared_bf16 = shared_bf16
        self.experts = experts
        self._keep = []

    @property
    def has_shared(self):
        return self.shared_fp8 is not None or self.shared_bf16 is not None

    def host_layer_w(self):
        """(LayerW with HOST pointers, desc array) for the CPU oracle."""
        L = abi.LayerW()
        L.pool = self.pool.ctypes.data
        L.desc = self.desc.ctypes.data
        L.fmt, L.H, L.I, L.E, L.topk = self.fmt, self.H, self.I, self.E, self.topk
        if self.shared_fp8 is not None:
            (gc, gs), (uc, us), (dc, ds) = self.shared_fp8
            L.sh.g, L.sh.u, L.sh.d = gc.ctypes.data, uc.ctypes.data, dc.ctypes.data
            L.sh.gs, L.sh.us, L.sh.ds = gs.ctypes.data, us.ctypes.data, ds.ctypes.data
        if self.shared_bf16 is not None:
            bgu, bd = self.shared_bf16
            L.sh.bgu, L.sh.bd = bgu.ctypes.data, bd.ctypes.data
        return L, self.desc

    def upload(self, device="cuda"):
        """Device copies; returns a DeviceLayer (holds the tensors, .w is the LayerW with device pointers)."""
        import torch
        t = lambda a: torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1)).to(device)
        return DeviceLayer(self, t)


class DeviceLayer:
    def __init__(self, hl, t):
        self.host = hl
        self.pool = t(hl.pool)
        self.desc = t(hl.desc)
        self.keep = []
        L = abi.LayerW()
        L.pool, L.desc = self.pool.data_ptr(), self.desc.data_ptr()
        L.fmt, L.H, L.I, L.E, L.topk = hl.fmt, hl.H, hl.I, hl.E, hl.topk
        if hl.shared_fp8 is not None:
            ts = [t(a) for pair in hl.shared_fp8 for a in pair]  # gc gs uc us dc ds
            self.keep += ts
            L.sh.g, L.sh.gs, L.sh.u, L.sh.us, L.sh.d, L.sh.ds = [x.data_ptr() for x in ts]
        if hl.shared_bf16 is not None:
            ts = [t(a) for a in hl.shared_bf16]
            self.keep += ts
            L.sh.bgu, L.sh.bd = [x.data_ptr() for x in ts]
        self.w = L
