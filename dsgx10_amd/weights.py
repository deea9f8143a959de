"""Binds a checkpoint's expert tensors into a layer of this library: safetensors shards -> HostLayer (weight pool +
64-byte descriptors) -> DeviceLayer. The role of the reference's expert loader and packer
(altar1-4xgx10-switchless/engine/weights/int4_pack.py:60-71 canon_int4, :320-366 Shards / load_expert, :175-205 the
descriptors; glw.py:419-431 the shared expert's interleaved gate/up), without its re-tiling: the pool formats of this
library ARE the checkpoint's canonical tensors (compressed-tensors INT4 group 32: weight_packed / weight_scale /
weight_zero_point; FP8: e4m3 weight + f32 weight_scale_inv per 128 x 128 block; BF16: weight), so binding is a copy and
the verifier reads every byte back.

    hl = load_layer("/ckpt", layer=5)     # format, sizes and expert count come from the tensors
    verify_layer(hl, shards, 5)           # every matrix of the pool equals its checkpoint tensors, byte for byte
    dl = hl.upload()                      # dl.w is the dsgx_layer_w for dsgx_moe_decode / dsgx_moe_prefill

numpy only (the shards are read with pread, no mmap and no tensor library: bf16 and e4m3 stay raw bits)."""
import json
import os
import struct

import numpy as np

from . import abi
from .layer import HostLayer, _al256, mat_bytes

PROJ = ("gate", "up", "down")
_DTYPES = {"I32": np.int32, "U32": np.uint32, "BF16": np.uint16, "F32": np.float32, "F8_E4M3": np.uint8, "U8": np.uint8,
           "I64": np.int64}


class Shards:
    """A checkpoint directory's tensors by name: model.safetensors.index.json (or every *.safetensors file's header when
    there is no index), each tensor read on demand."""

    def __init__(self, directory):
        self.dir = directory
        self._hdr = {}
        index = os.path.join(directory, "model.safetensors.index.json")
        if os.path.exists(index):
            with open(index) as f:
                self.where = dict(json.load(f)["weight_map"])
        else:
            self.where = {}
            for fn in sorted(os.listdir(directory)):
                if fn.endswith(".safetensors"):
                    for name in self._header(fn)[1]:
                        if name != "__metadata__":
                            self.where[name] = fn

    def _header(self, fn):
        if fn not in self._hdr:
            with open(os.path.join(self.dir, fn), "rb") as f:
                (n,) = struct.unpack("<Q", f.read(8))
                if n > (100 << 20):
                    raise ValueError("%s: header of %d bytes" % (fn, n))
                self._hdr[fn] = (8 + n, json.loads(f.read(n)))
        return self._hdr[fn]

    def __contains__(self, name):
        return name in self.where

    def get(self, name):
        """the tensor as a numpy array of raw bits (bf16 as uint16, e4m3 as uint8)"""
        fn = self.where[name]
        base, hdr = self._header(fn)
        ent = hdr[name]
        if ent["dtype"] not in _DTYPES:
            raise ValueError("%s: dtype %s" % (name, ent["dtype"]))
        lo, hi = ent["data_offsets"]
        fd = os.open(os.path.join(self.dir, fn), os.O_RDONLY)
        try:
            buf = os.pread(fd, hi - lo, base + lo)
        finally:
            os.close(fd)
        if len(buf) != hi - lo:
            raise IOError("%s: %d of %d bytes of %s" % (fn, len(buf), hi - lo, name))
        return np.frombuffer(buf, dtype=_DTYPES[ent["dtype"]]).reshape(ent["shape"])


def write_shard(path, tensors):
    """a safetensors file from {name: (dtype tag, numpy array)} (tests and small exports)"""
    hdr, blobs, o = {}, [], 0
    for name, (tag, a) in tensors.items():
        b = np.ascontiguousarray(a).view(np.uint8).reshape(-1).tobytes()
        hdr[name] = {"dtype": tag, "shape": list(a.shape), "data_offsets": [o, o + len(b)]}
        blobs.append(b)
        o += len(b)
    h = json.dumps(hdr, separators=(",", ":")).encode()
    h += b" " * (-len(h) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(h)))
        f.write(h)
        for b in blobs:
            f.write(b)


def _matrix(S, prefix):
    """(fmt, parts) of the matrix named prefix + 'weight...' in the canonical form layer.mat_blob takes"""
    if prefix + "weight_packed" in S:
        wp = S.get(prefix + "weight_packed")
        if wp.dtype != np.int32 or wp.ndim != 2:
            raise ValueError("%sweight_packed: int32 [N][K/8] expected" % prefix)
        N, K = wp.shape[0], wp.shape[1] * 8
        s, zp = S.get(prefix + "weight_scale"), S.get(prefix + "weight_zero_point")
        if s.dtype != np.uint16 or s.shape != (N, K // 32) or zp.dtype != np.int32 or zp.shape != (N // 8, K // 32):
            raise ValueError("%s: scales %s %s, zero points %s %s for [%d][%d]" % (prefix, s.dtype, s.shape, zp.dtype, zp.shape, N, K))
        if prefix + "weight_shape" in S:
            shp = tuple(int(v) for v in S.get(prefix + "weight_shape").reshape(-1))
            if shp != (N, K):
                raise ValueError("%sweight_shape %s, tensors [%d][%d]" % (prefix, shp, N, K))
        return abi.FMT_INT4, (wp.view(np.uint32), s, zp.view(np.uint32))
    w = S.get(prefix + "weight")
    if w.dtype == np.uint8:  # e4m3 codes with one f32 scale a 128 x 128 block
        N, K = w.shape
        s = S.get(prefix + "weight_scale_inv")
        if s.dtype != np.float32 or s.shape != ((N + 127) // 128, K // 128):
            raise ValueError("%sweight_scale_inv %s %s for [%d][%d]" % (prefix, s.dtype, s.shape, N, K))
        return abi.FMT_FP8, (w, s)
    if w.dtype != np.uint16 or w.ndim != 2:
        raise ValueError("%sweight: %s %s" % (prefix, w.dtype, w.shape))
    return abi.FMT_BF16, (w,)


def expert_count(S, layer):
    e = 0
    while "model.layers.%d.mlp.experts.%d.gate_proj.weight_packed" % (layer, e) in S or \
            "model.layers.%d.mlp.experts.%d.gate_proj.weight" % (layer, e) in S:
        e += 1
    return e


def load_layer(source, layer, topk=8, experts=None):
    """source: a checkpoint directory or a Shards. experts: the expert ids to bind (default: all of the layer); expert
    id e of the returned layer is experts[e]. The routed experts share one format; a shared expert
    (mlp.shared_experts.*) is fused when the kernels take the pair: FP8 beside FP8, BF16 beside INT4."""
    S = source if isinstance(source, Shards) else Shards(source)
    ids = list(range(expert_count(S, layer))) if experts is None else list(experts)
    if not ids:
        raise ValueError("layer %d holds no routed experts" % layer)
    mats, fmt, H, I = [], None, None, None
    for e in ids:
        ex = []
        for j, p in enumerate(PROJ):
            f, parts = _matrix(S, "model.layers.%d.mlp.experts.%d.%s_proj." % (layer, e, p))
            N = parts[0].shape[0]
            K = parts[0].shape[1] * (8 if f == abi.FMT_INT4 else 1)
            if fmt is None:
                fmt, I, H = f, N, K
            if f != fmt or (N, K) != ((I, H) if j < 2 else (H, I)):
                raise ValueError("expert %d %s_proj: format %d [%d][%d] in a layer of format %d, hidden %d, intermediate %d" % (e, p, f, N, K, fmt, H, I))
            ex.append(parts)
        mats.append(tuple(ex))
    sh8 = sh16 = None
    sp = "model.layers.%d.mlp.shared_experts." % layer
    if sp + "gate_proj.weight" in S:
        sh = [_matrix(S, sp + p + "_proj.") for p in PROJ]
        sf = sh[0][0]
        if any(f != sf for f, _ in sh):
            raise ValueError("layer %d: the shared expert's matrices differ in format" % layer)
        if sf == abi.FMT_FP8 and fmt == abi.FMT_FP8:
            sh8 = tuple(tuple(np.array(a) for a in parts) for _, parts in sh)  # (copies: the shard buffers are read-only)
        elif sf == abi.FMT_BF16 and fmt == abi.FMT_INT4:
            g, u, d = (parts[0] for _, parts in sh)
            bgu = np.empty((2 * g.shape[0], g.shape[1]), np.uint16)  # rows 2 c gate, 2 c + 1 up (glw.py:419-431)
            bgu[0::2], bgu[1::2] = g, u
            sh16 = (bgu, np.array(d))
        else:
            raise ValueError("layer %d: a format %d shared expert beside format %d experts is not built" % (layer, sf, fmt))
    return HostLayer(fmt, H, I, len(ids), min(topk, len(ids)), mats, emap=np.arange(len(ids)), shared_fp8=sh8, shared_bf16=sh16)


def read_back(hl, e, j):
    """the canonical tensors of matrix j (0 gate, 1 up, 2 down) of expert e, cut out of the pool through its descriptor
    (the independent reader: offsets from the descriptor and the format's layout rule, not from the packer's state)"""
    d = hl.desc[e * 3 + j]
    off, fmt = int(d["off"]), int(d["fmt"])
    N, K = (hl.I, hl.H) if j < 2 else (hl.H, hl.I)
    if off % 256 or off + mat_bytes(fmt, N, K) > hl.pool.size:
        raise ValueError("descriptor of expert %d matrix %d: offset %d" % (e, j, off))
    p = hl.pool
    if fmt == abi.FMT_INT4:
        nb, ns = N * K // 2, N * (K // 32) * 2
        o1, o2 = off + _al256(nb), off + _al256(nb) + _al256(ns)
        return (p[off:off + nb].view(np.uint32).reshape(N, K // 8), p[o1:o1 + ns].view(np.uint16).reshape(N, K // 32),
                p[o2:o2 + (N // 8) * (K // 32) * 4].view(np.uint32).reshape(N // 8, K // 32))
    if fmt == abi.FMT_FP8:
        o1 = off + _al256(N * K)
        nsb = (N + 127) // 128
        return (p[off:off + N * K].reshape(N, K), p[o1:o1 + nsb * (K // 128) * 4].view(np.float32).reshape(nsb, K // 128))
    if fmt == abi.FMT_BF16:
        return (p[off:off + N * K * 2].view(np.uint16).reshape(N, K),)
    raise ValueError("descriptor of expert %d matrix %d: format %d" % (e, j, fmt))


def verify_layer(hl, source, layer, experts=None):
    """every matrix of the pool, read back through its descriptor, against the checkpoint's tensors; returns the number
    of bytes compared, raises on the first difference"""
    S = source if isinstance(source, Shards) else Shards(source)
    ids = list(range(hl.E)) if experts is None else list(experts)
    total = 0
    for e, src in enumerate(ids):
        for j, p in enumerate(PROJ):
            f, parts = _matrix(S, "model.layers.%d.mlp.experts.%d.%s_proj." % (layer, src, p))
            back = read_back(hl, e, j)
            if f != int(hl.desc[e * 3 + j]["fmt"]) or len(back) != len(parts):
                raise ValueError("expert %d %s_proj: format %d in the checkpoint, %d in the pool" % (src, p, f, int(hl.desc[e * 3 + j]["fmt"])))
            for a, b in zip(parts, back):
                a = np.ascontiguousarray(a).view(np.uint8).reshape(-1)
                b = np.ascontiguousarray(b).view(np.uint8).reshape(-1)
                if a.size != b.size or not np.array_equal(a, b):
                    raise ValueError("expert %d %s_proj: the pool differs from the checkpoint" % (src, p))
                total += a.size
    return total
