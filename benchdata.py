"""Synthetic layers and timing loops for bench.py (GPU side only; torch is the allocator).

Values come from the generator the tests' oracle uses (splitmix64 keyed by seed, tensor id and index -> Box-Muller), made
on the GPU by the library's fill kernel (dsgx_fill_normal).

The layers have the benchmark's full shapes: weights ~ N(0, 0.02) quantised on the GPU with the reference's FP8
quantiser (per 128 x 128 block: scale = amax * f32(1/448), e4m3 round-to-nearest-even;
altar1-4xgx10-switchless/engine/attn/tools/pack.py:216-232) or this build's symmetric INT4-g32 quantiser (scale =
bf16(amax / 7), stored zero point 8), laid out in the pool formats of include/dsgx.h."""
import ctypes as C

import numpy as np
import torch

from dsgx10_amd import abi, lib
from dsgx10_amd.layer import DESC_DTYPE, HostLayer, mat_bytes

HBM_PEAK = 8.0e12


def _al256(n):
    return (n + 255) // 256 * 256


class Seeded:
    """N(0, sigma) tensors on the GPU from the oracle's generator: tensor number `tid` counts up with every draw"""

    def __init__(self, seed):
        self.seed, self.tid = seed, 0

    def normal(self, shape, sigma=1.0, dtype=torch.float32):
        n = int(np.prod(shape))
        out = torch.empty(shape, dtype=dtype, device="cuda")
        assert dtype in (torch.float32, torch.bfloat16)
        lib.fill_normal(self.seed, self.tid, n, sigma, out, bf16=dtype == torch.bfloat16)
        self.tid += 1
        return out


def time_graph(gr, reps=7):
    """seconds a replay: the median of `reps` replays, each between its own pair of events (and the fastest and slowest)"""
    torch.cuda.synchronize()
    ts = []
    for _ in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        gr.replay()
        e1.record()
        torch.cuda.synchronize()
        ts.append(e0.elapsed_time(e1) * 1e-3)
    return float(np.median(ts)), float(min(ts)), float(max(ts))


def fp8_quantize_gpu(w):
    """w f32 [N][K] on the GPU -> (codes u8 [N][K], scales f32 [N/128][K/128])"""
    N, K = w.shape
    blk = w.view(N // 128, 128, K // 128, 128)
    amax = blk.abs().amax(dim=(1, 3))
    scale = (amax * torch.tensor(1.0 / 448.0, dtype=torch.float32, device=w.device)).clamp_min(1e-12)
    q = (blk / scale[:, None, :, None]).to(torch.float8_e4m3fn)
    return q.view(torch.uint8).reshape(N, K), scale


def int4_quantize_gpu(w):
    """w f32 [N][K] -> (packed i32 [N][K/8], scale bf16 [N][K/32], zp i32 [N/8][K/32]) symmetric, stored zero point 8"""
    N, K = w.shape
    g = w.view(N, K // 32, 32)
    amax = g.abs().amax(-1)
    s = torch.where(amax > 0, amax / 7.0, torch.ones_like(amax)).to(torch.bfloat16)
    q = torch.clamp(torch.round(g / s.float()[..., None]), -8, 7).to(torch.int64) + 8
    sh = torch.arange(8, device=w.device, dtype=torch.int64) * 4
    words = (q.view(N, K // 8, 8) << sh).sum(-1)
    words = torch.where(words >= 2 ** 31, words - 2 ** 32, words).to(torch.int32)
    zp = torch.full((N // 8, K // 32), -0x77777778, dtype=torch.int32, device=w.device)  # 0x88888888
    return words, s, zp


def _put(pool, off, t):
    b = t.contiguous().view(torch.uint8).reshape(-1)
    pool[off:off + b.numel()] = b
    return _al256(b.numel())


class _LayerGen:
    """A full layer on the GPU: pool + descriptors + NSH rotating copies of the shared expert."""

    def layer_w(self, shared_copy):
        L = abi.LayerW()
        L.pool, L.desc = self.pool.data_ptr(), self.desc.data_ptr()
        L.fmt, L.H, L.I, L.E, L.topk = self.fmt, self.H, self.I, self.E, self.topk
        self._set_shared(L, shared_copy % self.NSH)
        return L

    def stream_read_gbs(self):
        sink = torch.zeros(4, dtype=torch.uint8, device="cuda")
        n = self.pool.numel() // 16 * 16
        lib.stream_read(self.pool, n, sink)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        lib.stream_read(self.pool, n, sink)
        e1.record()
        torch.cuda.synchronize()
        return n / (e0.elapsed_time(e1) * 1e-3) / 1e9


class Fp8LayerGen(_LayerGen):
    name = "fp8_moe_decode"
    fmt, H, I, E, topk, route_scale, NSH = abi.FMT_FP8, 4096, 2048, 256, 8, 1.0, 16

    def __init__(self, seed=0):
        g = Seeded(seed)
        H, I, E = self.H, self.I, self.E
        per = [mat_bytes(self.fmt, I, H), mat_bytes(self.fmt, I, H), mat_bytes(self.fmt, H, I)]
        self.expert_bytes = sum(per)
        self.pool = torch.zeros(E * self.expert_bytes, dtype=torch.uint8, device="cuda")
        desc = np.zeros(E * 3, DESC_DTYPE)
        o = 0
        for e in range(E):
            for j in range(3):
                N, K = (I, H) if j < 2 else (H, I)
                codes, scale = fp8_quantize_gpu(g.normal((N, K), 0.02))
                d = desc[e * 3 + j]
                d["off"], d["s2"], d["fmt"] = o, 1.0, self.fmt
                _put(self.pool, o, codes)
                _put(self.pool, o + _al256(N * K), scale)
                o += per[j]
        self.desc = torch.from_numpy(desc.view(np.uint8).reshape(-1)).cuda()
        self.shared = []
        for c in range(self.NSH):
            mats = []
            for j in range(3):
                N, K = (I, H) if j < 2 else (H, I)
                mats.append(fp8_quantize_gpu(g.normal((N, K), 0.02)))
            self.shared.append(mats)
        self.shared_bytes = self.expert_bytes

    def _set_shared(self, L, c):
        (gc, gs), (uc, us), (dc, ds) = self.shared[c]
        L.sh.g, L.sh.u, L.sh.d = gc.data_ptr(), uc.data_ptr(), dc.data_ptr()
        L.sh.gs, L.sh.us, L.sh.ds = gs.data_ptr(), us.data_ptr(), ds.data_ptr()

    def describe(self, M):
        return ("FP8 MoE decode layer: hidden 4096, 256 routed experts + 1 fused shared, intermediate 2048, e4m3 weights with "
                "128x128 f32 block scales, sigmoid top-8 renormalised (scale 1, no bias), M=%d bf16 rows" % M)

    def up_bytes(self, U):
        return (U + 1) * 2 * mat_bytes(self.fmt, self.I, self.H)

    def layer_bytes(self, U):
        return (U + 1) * self.expert_bytes

    def host_sublayer(self, experts, shared_copy):
        """the picked experts (ascending ids) and the shared copy as a HostLayer whose expert ids are 0..len-1"""
        H, I = self.H, self.I
        desc = np.frombuffer(self.desc.cpu().numpy().tobytes(), DESC_DTYPE)
        ex = []
        for e in experts:
            mats = []
            for j in range(3):
                N, K = (I, H) if j < 2 else (H, I)
                o = int(desc[e * 3 + j]["off"])
                codes = self.pool[o:o + N * K].cpu().numpy().reshape(N, K)
                so = o + _al256(N * K)
                sc = self.pool[so:so + (N // 128) * (K // 128) * 4].cpu().numpy().view(np.float32).reshape(N // 128, K // 128)
                mats.append((codes, sc))
            ex.append(tuple(mats))
        sh = tuple((c.cpu().numpy(), s.cpu().numpy()) for c, s in self.shared[shared_copy % self.NSH])
        return HostLayer(self.fmt, H, I, len(experts), self.topk, ex, emap=np.arange(len(experts)), shared_fp8=sh)


class Int4LayerGen(_LayerGen):
    name = "int4_moe_decode"
    fmt, H, I, E, topk, route_scale, NSH = abi.FMT_INT4, 6144, 2048, 168, 8, 2.5, 8

    def __init__(self, seed=0):
        g = Seeded(seed + 1)
        H, I, E = self.H, self.I, self.E
        per = [mat_bytes(self.fmt, I, H), mat_bytes(self.fmt, I, H), mat_bytes(self.fmt, H, I)]
        self.expert_bytes = sum(per)
        self.pool = torch.zeros(E * self.expert_bytes, dtype=torch.uint8, device="cuda")
        desc = np.zeros(E * 3, DESC_DTYPE)
        o = 0
        for e in range(E):
            for j in range(3):
                N, K = (I, H) if j < 2 else (H, I)
                words, s, zp = int4_quantize_gpu(g.normal((N, K), 0.02))
                d = desc[e * 3 + j]
                d["off"], d["s2"], d["fmt"] = o, 1.0, self.fmt
                _put(self.pool, o, words)
                _put(self.pool, o + _al256(N * K // 2), s)
                _put(self.pool, o + _al256(N * K // 2) + _al256(N * (K // 32) * 2), zp)
                o += per[j]
        self.desc = torch.from_numpy(desc.view(np.uint8).reshape(-1)).cuda()
        self.shared = []
        for c in range(self.NSH):
            bgu, bd = g.normal((2 * I, H), 0.02, torch.bfloat16), g.normal((H, I), 0.02, torch.bfloat16)
            self.shared.append((bgu, bd))
        self.shared_bytes = 3 * H * I * 2

    def _set_shared(self, L, c):
        bgu, bd = self.shared[c]
        L.sh.bgu, L.sh.bd = bgu.data_ptr(), bd.data_ptr()

    def describe(self, M):
        return ("INT4-g32 MoE decode layer (GLM-style): hidden 6144, 168 routed experts (compressed-tensors int4, bf16 group scales, "
                "stored zero points) + 1 fused bf16 shared expert, intermediate 2048, sigmoid top-8 x 2.5, M=%d bf16 rows" % M)

    def up_bytes(self, U):
        return U * 2 * mat_bytes(self.fmt, self.I, self.H) + 2 * self.I * self.H * 2

    def layer_bytes(self, U):
        return U * self.expert_bytes + self.shared_bytes

    def host_sublayer(self, experts, shared_copy):
        H, I = self.H, self.I
        desc = np.frombuffer(self.desc.cpu().numpy().tobytes(), DESC_DTYPE)
        ex = []
        for e in experts:
            mats = []
            for j in range(3):
                N, K = (I, H) if j < 2 else (H, I)
                o = int(desc[e * 3 + j]["off"])
                a, b = _al256(N * K // 2), _al256(N * (K // 32) * 2)
                p = self.pool[o:o + N * K // 2].cpu().numpy().view(np.uint32).reshape(N, K // 8)
                s = self.pool[o + a:o + a + N * (K // 32) * 2].cpu().numpy().view(np.uint16).reshape(N, K // 32)
                z = self.pool[o + a + b:o + a + b + (N // 8) * (K // 32) * 4].cpu().numpy().view(np.uint32).reshape(N // 8, K // 32)
                mats.append((p, s, z))
            ex.append(tuple(mats))
        bgu, bd = self.shared[shared_copy % self.NSH]
        sh = (bgu.view(torch.int16).cpu().numpy().view(np.uint16), bd.view(torch.int16).cpu().numpy().view(np.uint16))
        return HostLayer(self.fmt, H, I, len(experts), self.topk, ex, emap=np.arange(len(experts)), shared_bf16=sh)


class DecodeBench:
    """`steps` decode steps of M rows over a generated layer; step s routes logits[s] (seeded N(0,1))."""

    def __init__(self, gen, M, steps, seed=1234, up=0):
        """up: the decode variant (dsgx_decode_cfg::up): 0 the vector-unit kernels, 1 the MFMA kernels"""
        self.gen, self.M, self.steps, self.up = gen, M, steps, up
        g = Seeded(seed)
        self.x = g.normal((M, gen.H), 1.0, torch.bfloat16)
        self.logits = g.normal((steps, M, gen.E), 1.0)
        self.idx = torch.zeros(steps, M, gen.topk, dtype=torch.int32, device="cuda")
        self.w = torch.zeros(steps, M, gen.topk, dtype=torch.float32, device="cuda")
        self.layers = [gen.layer_w(c) for c in range(gen.NSH)]
        self.ws = torch.zeros(lib.decode_ws_bytes(self.layers[0]), dtype=torch.uint8, device="cuda")
        self.yr = torch.zeros(M, gen.H, dtype=torch.float32, device="cuda")
        self.ys = torch.zeros(M, gen.H, dtype=torch.float32, device="cuda")
        for s in range(steps):
            lib.route(self.logits[s], None, self.idx[s], self.w[s], gen.route_scale)
        torch.cuda.synchronize()
        idx = self.idx.cpu().numpy()
        self.union_sizes = np.array([len(np.unique(idx[s])) for s in range(steps)])

    def step(self, s, parts=3, route=True, fused_routing=True):
        """one layer: with fused_routing the router runs inside the expert kernel (the reference runner's default,
        DecodeCfg::logits), else as its own launch before it"""
        g = self.gen
        if fused_routing:
            lib.moe_decode(self.layers[s % g.NSH], self.x, None, None, self.M, self.ws, self.yr, self.ys, parts=parts,
                           logits=self.logits[s], route_scale=g.route_scale, up=self.up)
            return
        if route:
            lib.route(self.logits[s], None, self.idx[s], self.w[s], g.route_scale)
        lib.moe_decode(self.layers[s % g.NSH], self.x, self.idx[s], self.w[s], self.M, self.ws, self.yr, self.ys, parts=parts, up=self.up)

    def _graph(self, fn):
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr):
            fn()
        return gr


    def time_layer(self, warmup):
        for s in range(warmup):
            self.step(s % self.steps)
        torch.cuda.synchronize()
        gr = self._graph(lambda: [self.step(s) for s in range(self.steps)])
        gr.replay()  # untimed: uploads the graph
        sec, lo, hi = time_graph(gr)
        us = sec / self.steps * 1e6
        bytes_ = float(np.mean([self.gen.layer_bytes(u) for u in self.union_sizes]))
        return dict(us_per_layer=us, us_per_layer_min=lo / self.steps * 1e6, us_per_layer_max=hi / self.steps * 1e6, replays=7,
                    bytes_per_layer=bytes_, layer_hbm_frac=bytes_ / (us * 1e-6) / HBM_PEAK, mean_union=float(self.union_sizes.mean()))

    def time_up_kernel(self):
        """the dominant kernel alone: `steps` launches of the gate/up kernel back to back in one graph"""
        gr = self._graph(lambda: [self.step(s, parts=1, route=False) for s in range(self.steps)])
        gr.replay()
        sec = time_graph(gr)[0]
        us = sec / self.steps * 1e6
        b = float(np.mean([self.gen.up_bytes(u) for u in self.union_sizes]))
        gbs = b / (us * 1e-6) / 1e9
        return dict(up_us=us, up_bytes=b, up_gbs=gbs, up_frac=gbs * 1e9 / HBM_PEAK)

    def run_step_and_download(self, s):
        """runs step s eagerly; returns the host copies the CPU oracle needs and the GPU's outputs"""
        self.step(s)
        torch.cuda.synchronize()
        idx = self.idx[s].cpu().numpy()
        w = self.w[s].cpu().numpy()
        experts = sorted(set(int(e) for e in idx.reshape(-1)))
        remap = {e: i for i, e in enumerate(experts)}
        idx_local = np.vectorize(remap.get)(idx).astype(np.int32)
        hl = self.gen.host_sublayer(experts, s)
        x = self.x.view(torch.int16).cpu().numpy().view(np.uint16)
        return dict(layer=hl, x=x, idx=idx_local, w=w, yr=self.yr.cpu().numpy().copy(), ys=self.ys.cpu().numpy().copy(),
                    experts=experts)


class DskLayerGen(_LayerGen):
    """DeepSeek's MoE layer (ds41f-4xgx10-switchless/engine/kernels/dsk.h:199-241) at its unsharded shape: hidden 5120,
    intermediate 2304 (the reference's 576 a rank x 4), 256 MXFP4 experts, top-6 by the sqrt-softplus router, one FP8 shared
    expert with ue8m0 scales per 32 x 32; random e2m1 codes and scale bytes (the values' statistics do not change the bytes
    streamed)."""
    name = "dsk_mxfp4_moe_decode"
    fmt, H, I, E, topk, route_scale, NSH = abi.FMT_MXFP4, 5120, 2304, 256, 6, 1.5, 16

    def __init__(self, seed=0):
        g = torch.Generator(device="cuda")
        g.manual_seed(seed + 2)
        H, I, E = self.H, self.I, self.E
        per = [mat_bytes(self.fmt, I, H), mat_bytes(self.fmt, I, H), mat_bytes(self.fmt, H, I)]
        self.expert_bytes = sum(per)
        self.pool = torch.zeros(E * self.expert_bytes, dtype=torch.uint8, device="cuda")
        desc = np.zeros(E * 3, DESC_DTYPE)
        o = 0
        for e in range(E):
            for j in range(3):
                N, K = (I, H) if j < 2 else (H, I)
                d = desc[e * 3 + j]
                d["off"], d["s2"], d["fmt"] = o, 1.0, self.fmt
                _put(self.pool, o, torch.randint(0, 256, (N, K // 2), generator=g, device="cuda", dtype=torch.uint8))
                _put(self.pool, o + _al256(N * K // 2), torch.randint(114, 120, (N, K // 32), generator=g, device="cuda", dtype=torch.uint8))
                o += per[j]
        self.desc = torch.from_numpy(desc.view(np.uint8).reshape(-1)).cuda()
        self.shared = []
        for c in range(self.NSH):
            mats = []
            for j in range(3):
                N, K = (I, H) if j < 2 else (H, I)
                codes = (torch.randn(N, K, generator=g, device="cuda") * 40.0).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
                mats.append((codes, torch.randint(110, 116, (N // 32, K // 32), generator=g, device="cuda", dtype=torch.uint8)))
            self.shared.append(mats)
        self.shared_bytes = 3 * (H * I + (H // 32) * (I // 32))

    def _set_shared(self, L, c):
        (gc, gs), (uc, us), (dc, ds) = self.shared[c]
        L.sh.g, L.sh.u, L.sh.d = gc.data_ptr(), uc.data_ptr(), dc.data_ptr()
        L.sh.gs, L.sh.us, L.sh.ds = gs.data_ptr(), us.data_ptr(), ds.data_ptr()

    def layer_bytes(self, U):
        return U * self.expert_bytes + self.shared_bytes


class DskBench:
    """`steps` decode steps of M rows through dsgx_dsk_moe with the routing fused (dsk::moe_routed): step s routes logits[s]"""

    def __init__(self, gen, M, steps, seed=77):
        self.gen, self.M, self.steps = gen, M, steps
        g = Seeded(seed)
        x = g.normal((M, gen.H), 1.5)
        blk = x.view(M, gen.H // 32, 32)
        v = blk.abs().amax(-1).clamp_min(1e-4) * torch.tensor(1.0 / 448.0, device="cuda")
        bits = v.view(torch.int32)
        e = ((bits >> 23) & 0xFF) + ((bits & 0x7FFFFF) != 0).to(torch.int32)
        self.xs = e.to(torch.uint8).contiguous()
        self.xq = (blk * torch.ldexp(torch.ones_like(v), (127 - e).float())[..., None]).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).reshape(M, gen.H).contiguous()
        self.logits = g.normal((steps, M, gen.E), 1.0)
        idx = torch.zeros(steps, M, gen.topk, dtype=torch.int32, device="cuda")
        w = torch.zeros(steps, M, gen.topk, dtype=torch.float32, device="cuda")
        for s in range(steps):
            lib.route(self.logits[s], None, idx[s], w[s], gen.route_scale, score_fn=1)
        torch.cuda.synchronize()
        self.union_sizes = np.array([len(np.unique(idx[s].cpu().numpy())) for s in range(steps)])
        self.layers = [gen.layer_w(c) for c in range(gen.NSH)]
        self.ws = torch.zeros(lib.decode_ws_bytes(self.layers[0]), dtype=torch.uint8, device="cuda")
        self.y = torch.zeros(M, gen.H, dtype=torch.float32, device="cuda")
        self.ys = torch.zeros(M, gen.H, dtype=torch.float32, device="cuda")

    def step(self, s, parts=3):
        g = self.gen
        lib.dsk_moe(self.layers[s % g.NSH], self.xq, self.xs, None, None, self.M, self.ws, self.y, self.ys, logits=self.logits[s],
                    route_scale=g.route_scale, parts=parts)

    def time(self, parts=3):
        for s in range(4):
            self.step(s, parts)
        torch.cuda.synchronize()
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr):
            for s in range(self.steps):
                self.step(s, parts)
        gr.replay()
        us = time_graph(gr)[0] * 1e6 / self.steps
        lib.decode_status(self.layers[0], self.ws)
        b = float(np.mean([self.gen.layer_bytes(u) for u in self.union_sizes]))
        return dict(workload=self.gen.name, M=self.M, variant="mfma", us_per_layer=us, bytes=b, hbm_frac=b / (us * 1e-6) / HBM_PEAK,
                    outputs_finite=bool(torch.isfinite(self.y).all()))


class ChainBench:
    """A decode layer's dense projections and MoE step as the reference's runner chains them (model.cu:229-352; the sequence
    is dsgx10_amd/chain.py's), layer after layer in one graph: x-projection (BF16, K over 4), q_b and o_proj (the layer's
    format: INT4 or FP8 128 x 128), the add + norms, the router's logits (BF16, f32 out, K over 4) and the experts with the
    routing, the shared expert and yr += ys fused. Shapes: the whole layer on one GPU (GLM / altar-1: hidden 6144, x-projection
    2752 rows, q_lora 2048, 64 heads x 256; the FP8 layer: hidden 4096, 2112, 1536, 64 x 256). Every layer rotates over
    weight sets that together exceed the caches and routes by its own data. fused: each add + norm inside the GEMV that
    reads it (the router's: 6 launches a layer, 7 with the MFMA variant's ordered sum) or as launches of their own (7 / 8)."""

    def __init__(self, gen, M, layers, seed=99, up=-1, moe_only=False):
        from dsgx10_amd.chain import LayerChain
        self.gen, self.M, self.layers, self.up, self.moe_only = gen, M, layers, up, moe_only
        g = Seeded(seed)
        H, E = gen.H, gen.E
        fp8 = gen.fmt == abi.FMT_FP8
        self.XR, self.QL, self.NQ = (2112, 1536, 16384) if fp8 else (2752, 2048, 16384)
        XR, QL, NQ = self.XR, self.QL, self.NQ
        quant = fp8_quantize_gpu if fp8 else int4_quantize_gpu

        def mat(N, K):
            t = quant(g.normal((N, K), 0.02))
            return dict(fmt=gen.fmt, w=t[0], s=t[1], zp=t[2] if len(t) > 2 else None)
        self.nsets = 4
        lw = [gen.layer_w(c) for c in range(gen.NSH)]
        self.ws = torch.zeros(lib.decode_ws_bytes(lw[0]), dtype=torch.uint8, device="cuda")
        self.sets = []
        for c in range(self.nsets):
            self.sets.append(dict(attn_norm=(1.0 + g.normal((H,), 0.1)).to(torch.bfloat16), ffn_norm=(1.0 + g.normal((H,), 0.1)).to(torch.bfloat16),
                                  xproj=g.normal((XR, H), 0.02, torch.bfloat16), router=g.normal((E, H), 0.05, torch.bfloat16),
                                  qb=mat(NQ, QL), oproj=mat(H, NQ)))
        self.lw = lw
        self.dense_bytes = XR * H * 2 + E * H * 2 + mat_bytes(gen.fmt, NQ, QL) + mat_bytes(gen.fmt, H, NQ)
        self.ch = LayerChain(M, H, XR, QL, NQ, E, gen.route_scale, lambda n: torch.zeros(n, dtype=torch.uint8, device="cuda"))
        self.x0 = g.normal((M, H), 1.0, torch.bfloat16)

    def layer(self, l, fused):
        W = dict(self.sets[l % self.nsets], moe=self.lw[l % self.gen.NSH], ws=self.ws)
        if self.moe_only:  # the MoE half alone: router GEMV (+ add + norm) and the experts
            ch, g = self.ch, self.gen
            a, b = ch.res[ch.cur], ch.res[ch.cur ^ 1]
            rt = [dict(fmt=abi.FMT_BF16, w=W["router"], n=g.E, y=ch.logits, ldy=g.E)]
            if fused:
                lib.add_norm_gemv(ch.yr, None, a, b, W["ffn_norm"], 1e-5, ch.xn, self.M, g.H, rt, abi.OUT_F32, splitk=4)
            else:
                lib.add_norm(ch.yr, None, self.M, g.H, a, b, W["ffn_norm"], 1e-5, ch.xn)
                lib.gemv(ch.xn, g.H, self.M, g.H, rt, abi.OUT_F32, splitk=4)
            ch.cur ^= 1
            lib.moe_decode(W["moe"], ch.xn, None, None, self.M, W["ws"], ch.yr, ch.ys, logits=ch.logits, route_scale=g.route_scale, ysum=True, up=self.up)
            return
        self.ch.layer(W, fused=fused, up=self.up)

    def _reset(self):
        self.ch.cur = 0
        self.ch.res[0].copy_(self.x0.view(torch.uint8).reshape(-1))
        self.ch.yr.zero_()

    def time(self, fused=True):
        self._reset()
        for l in range(4):
            self.layer(l, fused)
        torch.cuda.synchronize()
        self._reset()
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr):
            for l in range(self.layers):
                self.layer(l, fused)
        gr.replay()
        torch.cuda.synchronize()
        sec, lo, hi = time_graph(gr)
        lib.decode_status(self.lw[0], self.ws)
        finite = bool(torch.isfinite(self.ch.yr.view(torch.float32)).all())
        us = sec * 1e6 / self.layers
        moe_bytes = self.gen.layer_bytes(self.gen.topk * self.M if self.M == 1 else self.gen.topk)  # (M = 1: eight experts + shared)
        total = moe_bytes + (self.gen.E * self.gen.H * 2 if self.moe_only else self.dense_bytes)
        names = (["k_gemv_sk (router logits, add + norm in its prologue)" if fused else "k_add_norm, k_gemv_sk (router logits)", "k_decode / k_decode_mfma (+ its ordered sum)"]
                 if self.moe_only else
                 ["k_add_norm", "k_gemv_sk (x-projection)", "k_gemv (q_b)", "k_gemv (o_proj)",
                  "k_gemv_sk (router logits%s)" % (", add + norm in its prologue" if fused else "; k_add_norm before it"), "k_decode / k_decode_mfma (+ its ordered sum)"])
        return dict(workload=self.gen.name.replace("decode", "moe_half_chain" if self.moe_only else "layer_chain"), M=self.M, layers=self.layers, fused_add_norm=fused,
                    launches_per_layer=names, us_per_layer=us, us_per_layer_min=lo * 1e6 / self.layers, us_per_layer_max=hi * 1e6 / self.layers,
                    bytes_per_layer=total, hbm_frac=total / (us * 1e-6) / HBM_PEAK, outputs_finite=finite)


def launch_floors(reps=64):
    """what a graph node costs with nothing in it: an empty kernel, and one wavefront doing two dependent loads and a store"""
    buf = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    sink = torch.zeros(16, dtype=torch.uint8, device="cuda")
    out = {}
    for name, kind in (("empty_kernel_us", 0), ("two_dependent_loads_us", 1)):
        lib.launch_floor(kind, buf, sink)
        torch.cuda.synchronize()
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr):
            for _ in range(reps):
                lib.launch_floor(kind, buf, sink)
        gr.replay()
        out[name] = time_graph(gr)[0] * 1e6 / reps
    return out


def gemv_bench(reps=64):
    """the two dense GEMV configurations: FP8 [2048 x 4096] at 1 row, INT4 [1536 x 6144] at 1, 2, 4, 6 rows, and the router's
    logits (BF16 [E x H], f32 out, 1 row), each with K unsplit and split over 2 and 4 waves; weights rotate over copies that
    exceed the caches; beside them what an empty graph node and a node of two dependent memory round trips cost"""
    out = []
    g = Seeded(7)
    floors = launch_floors(reps)
    for name, fmt, N, K, rows, kind in (("dense_fp8_gemv_2048x4096", abi.FMT_FP8, 2048, 4096, (1,), abi.OUT_BF16),
                                        ("dense_int4_gemv_1536x6144", abi.FMT_INT4, 1536, 6144, (1, 2, 4, 6), abi.OUT_BF16),
                                        ("router_bf16_gemv_256x4096", abi.FMT_BF16, 256, 4096, (1,), abi.OUT_F32),
                                        ("router_bf16_gemv_168x6144", abi.FMT_BF16, 168, 6144, (1,), abi.OUT_F32)):
        per = mat_bytes(fmt, N, K)
        copies = max(8, int(600e6 // per))
        mats = []
        for c in range(copies):
            w = g.normal((N, K), 0.02)
            mats.append(fp8_quantize_gpu(w) if fmt == abi.FMT_FP8 else int4_quantize_gpu(w) if fmt == abi.FMT_INT4 else (w.to(torch.bfloat16), None))
        for M in rows:
            x = g.normal((M, K), 1.0, torch.bfloat16)
            y = torch.zeros(M, N, dtype=torch.float32 if kind == abi.OUT_F32 else torch.bfloat16, device="cuda")
            for sk in (1, 2, 4):
                def one(c):
                    m = mats[c % copies]
                    seg = dict(fmt=fmt, w=m[0], s=m[1], zp=m[2] if len(m) > 2 else None, n=N, y=y, ldy=N)
                    lib.gemv(x, K, M, K, [seg], kind, splitk=sk)
                for c in range(4):
                    one(c)
                torch.cuda.synchronize()
                gr = torch.cuda.CUDAGraph()
                with torch.cuda.graph(gr):
                    for c in range(reps):
                        one(c)
                gr.replay()
                us = time_graph(gr)[0] * 1e6 / reps
                b = per + M * K * 2 + M * N * y.element_size()
                out.append(dict(workload=name, M=M, splitk=sk, us_per_call=us, bytes=b, hbm_frac=b / (us * 1e-6) / HBM_PEAK, floors=floors))
    return out


class DskPrefillBench:
    """One prefill chunk of T rows through dsgx_dsk_moe_prefill (dsk::moe_prefill, ds41f-4xgx10-switchless/engine/kernels/
    dsk.h:268-295) at DeepSeek's unsharded layer shape: hidden 5120, intermediate 2304 (the reference's 576 a rank x 4), 256 MXFP4
    experts stacked by id, top-6 drawn from a Zipf(s) popularity with uniform weights, one FP8 shared expert; random e2m1
    codes and scale bytes, rows N(0, 1.5) quantised per 32 (ue8m0) as the reference's act_quant does."""
    name = "dsk_mxfp4_moe_prefill"
    H, I, E, topk = 5120, 2304, 256, 6

    def __init__(self, T, zipf_s=1.1, seed=4321):
        H, I, E, topk = self.H, self.I, self.E, self.topk
        self.T = T
        g = torch.Generator(device="cuda")
        g.manual_seed(seed)
        rnd = lambda shape, lo, hi: torch.randint(lo, hi, shape, generator=g, device="cuda", dtype=torch.uint8)
        self.t = {}
        for n, (N, K) in (("1", (I, H)), ("3", (I, H)), ("2", (H, I))):
            self.t["w" + n], self.t["s" + n] = rnd((E, N, K // 2), 0, 256), rnd((E, N, K // 32), 114, 120)
            self.t["sh_w" + n] = (torch.randn(N, K, generator=g, device="cuda") * 40.0).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
            self.t["sh_s" + n] = rnd((N // 32, K // 32), 110, 116)
        self.weights = abi.DskWeights(*[self.t[k].data_ptr() for k in ("w1", "s1", "w3", "s3", "w2", "s2", "sh_w1", "sh_s1", "sh_w3", "sh_s3", "sh_w2", "sh_s2")],
                                      H, I, E, topk)
        x = Seeded(seed).normal((T, H), 1.5)
        blk = x.view(T, H // 32, 32)
        v = blk.abs().amax(-1).clamp_min(1e-4) * torch.tensor(1.0 / 448.0, device="cuda")
        bits = v.view(torch.int32)
        e = ((bits >> 23) & 0xFF) + ((bits & 0x7FFFFF) != 0).to(torch.int32)
        self.xs = e.to(torch.uint8).contiguous()
        self.xq = (blk * torch.ldexp(torch.ones_like(v), (127 - e).float())[..., None]).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).reshape(T, H).contiguous()
        rank = torch.randperm(E, generator=g, device="cuda").to(torch.float32) + 1.0
        self.idx = torch.multinomial(rank.pow(-zipf_s).expand(T, E), topk, replacement=False, generator=g).to(torch.int32).contiguous()
        self.w = torch.full((T, topk), 1.0 / topk, dtype=torch.float32, device="cuda")
        self.ws = torch.empty(lib.dsk_prefill_ws_bytes(H, I, E, topk, T), dtype=torch.uint8, device="cuda")
        self.y = torch.zeros(T, H, dtype=torch.float32, device="cuda")
        self.flops_routed = 2.0 * T * topk * 3 * I * H
        self.flops_shared = 2.0 * T * 3 * I * H
        self.expert_bytes = 3 * (I * H // 2 + I * H // 32)

    def run(self, phases=31):
        lib.dsk_moe_prefill(self.weights, self.xq, self.xs, self.idx, self.w, self.T, self.ws, self.y, phases=phases)

    def time(self, phases=31, reps=8, samples=7):
        self.run(phases)
        torch.cuda.synchronize()
        ts = []
        for _ in range(samples):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                self.run(phases)
            e1.record()
            torch.cuda.synchronize()
            ts.append(e0.elapsed_time(e1) * 1e-3 / reps)
        return float(np.median(ts))


class PrefillBench:
    """One prefill chunk of T rows over a generated FP8 layer: each row picks top-k distinct experts drawn from a
    Zipf(s) popularity over a seeded permutation of the experts, uniform weights 1/top-k (the reference's
    bench_prefill input shape, engine/experts/tests/bench_prefill.inc)."""

    def __init__(self, gen, T, zipf_s=1.1, seed=4321):
        self.gen, self.T = gen, T
        g = torch.Generator(device="cuda")   # (the Zipf draw: torch's multinomial)
        g.manual_seed(seed)
        self.x = Seeded(seed).normal((T, gen.H), 1.0, torch.bfloat16)
        rank = torch.randperm(gen.E, generator=g, device="cuda").to(torch.float32) + 1.0
        p = rank.pow(-zipf_s)
        self.idx = torch.multinomial(p.expand(T, gen.E), gen.topk, replacement=False, generator=g).to(torch.int32).contiguous()
        self.w = torch.full((T, gen.topk), 1.0 / gen.topk, dtype=torch.float32, device="cuda")
        self.layer = gen.layer_w(0)
        self.ws = torch.zeros(lib.prefill_ws_bytes(self.layer, T), dtype=torch.uint8, device="cuda")
        self.yr = torch.zeros(T, gen.H, dtype=torch.float32, device="cuda")
        self.ys = torch.zeros(T, gen.H, dtype=torch.float32, device="cuda")
        # useful multiply-adds only: routed picks (and, apart, the shared expert on every row)
        self.flops_routed = 2.0 * T * gen.topk * 3 * gen.I * gen.H
        self.flops_shared = 2.0 * T * 3 * gen.I * gen.H

    def run(self, phases=31, shared=True):
        lib.moe_prefill(self.layer, self.x, self.idx, self.w, self.T, self.ws, self.yr, self.ys, shared=shared, phases=phases)

    def time(self, phases=31, shared=True, reps=8, samples=7):
        """Seconds per call: `reps` calls back to back between two events (a model's layers follow each other the same
        way; a lone launch after an idle gap runs at a lower clock), the median of `samples` such runs."""
        self.run(phases, shared)
        torch.cuda.synchronize()
        ts = []
        for _ in range(samples):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                self.run(phases, shared)
            e1.record()
            torch.cuda.synchronize()
            ts.append(e0.elapsed_time(e1) * 1e-3 / reps)
        return float(np.median(ts))
