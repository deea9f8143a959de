"""One decode layer's dense projections and MoE step chained as the reference's runner chains them
(altar1-4xgx10-switchless/engine/model/model.cu:229-352), on the C ABI. The attention kernels between the projections
(norms, RoPE, the indexer, sparse attention, the absorbed per-head W_UK / W_UV products) are not part of this build, so the
chain hands q_b's output to o_proj directly; every launch, shape and dependency of the GEMVs and of the MoE half is the
runner's:

    x-projection   BF16 [XR][H], K split 4                 model.cu:236-247   <- RMSNorm(res + the layer before's yr)
    q_b            INT4 or FP8 [NQ][QL] on the first QL columns of the x-projection's output        model.cu:262-267
    o_proj         INT4 or FP8 [H][NQ], f32 partials                                                 model.cu:291-294
    add + norm     h = bf16(res + part), xn = RMSNorm(h) with the layer's ffn norm                   model.cu:299
    router         BF16 [E][H], f32 logits, K split 4                                                model.cu:311-313
    experts        routing, shared expert and yr += ys fused                                         model.cu:334-343
    add + norm     the next layer's attention norm                                                   model.cu:346-352

fused = True runs the add + norm in front of the router as the prologue of the router's GEMV (dsgx_add_norm_gemv): six
launches a layer (seven with the MFMA variant's ordered sum) instead of seven (eight); the bits are the same. fuse_xproj does
the same for the x-projection: right for the bits, but that GEMV has ten times the router's workgroups, each of which would
redo the rows' norm, and the layer gets slower (measured: +4 us at hidden 4096, +10 us at 6144), so it is off by default."""
from . import abi, lib


class LayerChain:
    def __init__(self, M, H, XR, QL, NQ, E, route_scale, alloc):
        """alloc(nbytes) -> a zeroed device buffer (the caller's allocator: torch in the tests and the bench)"""
        self.M, self.H, self.XR, self.QL, self.NQ, self.E, self.route_scale = M, H, XR, QL, NQ, E, route_scale
        self.res = [alloc(M * H * 2), alloc(M * H * 2)]   # the residual stream, ping-pong (a fused add + norm reads one, writes the other)
        self.xn = alloc(M * H * 2)
        self.xg = alloc(M * XR * 2)
        self.q = alloc(M * NQ * 2)
        self.part = alloc(M * H * 4)
        self.logits = alloc(M * E * 4)
        self.yr = alloc(M * H * 4)
        self.ys = alloc(M * H * 4)
        self.cur = 0

    def layer(self, W, fused=True, up=-1, stream=None, tap=None, fuse_xproj=False):
        """W: dict(attn_norm, ffn_norm bf16 [H]; xproj bf16 [XR][H]; qb, oproj: dict(fmt, w, s, zp) [NQ][QL], [H][NQ]; router bf16
        [E][H]; moe: a dsgx_layer_w; ws: its decode workspace). Reads res[cur] and yr, leaves the new residual in res[cur].
        tap(name): called after each stage (tests read the stage's buffers then)."""
        M, H, XR, QL, NQ, E = self.M, self.H, self.XR, self.QL, self.NQ, self.E
        a, b = self.res[self.cur], self.res[self.cur ^ 1]
        tap = tap or (lambda name: None)
        xp = [dict(fmt=abi.FMT_BF16, w=W["xproj"], n=XR, y=self.xg, ldy=XR)]
        if fused and fuse_xproj:
            lib.add_norm_gemv(self.yr, None, a, b, W["attn_norm"], 1e-5, None, M, H, xp, abi.OUT_BF16, splitk=2, stream=stream)
        else:
            lib.add_norm(self.yr, None, M, H, a, b, W["attn_norm"], 1e-5, self.xn, stream=stream)
            tap("norm1")
            # (K over 2 waves: 7.2 / 9.1 us for the two layers' shapes against 8.7 / 11.2 over 4 and 8.0 / 10.1 unsplit, measured)
            lib.gemv(self.xn, H, M, H, xp, abi.OUT_BF16, splitk=2, stream=stream)
        tap("xproj")
        lib.gemv(self.xg, XR, M, QL, [dict(W["qb"], n=NQ, y=self.q, ldy=NQ)], abi.OUT_BF16, stream=stream)
        tap("qb")
        lib.gemv(self.q, NQ, M, NQ, [dict(W["oproj"], n=H, y=self.part, ldy=H)], abi.OUT_F32, stream=stream)
        tap("oproj")
        rt = [dict(fmt=abi.FMT_BF16, w=W["router"], n=E, y=self.logits, ldy=E)]
        if fused:
            lib.add_norm_gemv(self.part, None, b, a, W["ffn_norm"], 1e-5, self.xn, M, H, rt, abi.OUT_F32, splitk=4, stream=stream)
        else:
            lib.add_norm(self.part, None, M, H, b, a, W["ffn_norm"], 1e-5, self.xn, stream=stream)
            tap("norm2")
            lib.gemv(self.xn, H, M, H, rt, abi.OUT_F32, splitk=4, stream=stream)
        tap("router")
        lib.moe_decode(W["moe"], self.xn, None, None, M, W["ws"], self.yr, self.ys, logits=self.logits, route_scale=self.route_scale,
                       ysum=True, up=up, stream=stream)
        tap("experts")
        # (the new residual is in res[cur] again: two add + norms a layer)

    def finish(self, norm_w, stream=None):
        """the add + norm after the last layer: the final residual into res[cur ^ 1], its norm into xn"""
        lib.add_norm(self.yr, None, self.M, self.H, self.res[self.cur], self.res[self.cur ^ 1], norm_w, 1e-5, self.xn, stream=stream)
        self.cur ^= 1
