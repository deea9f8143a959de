"""The reference runner's MoE step, call by call (altar1-4xgx10-switchless/engine/model/model.cu:309-343): the router's
logits by the BF16 GEMV with f32 output and K split four ways, then either (a) the expert kernel with fused routing, the fused BF16 shared
expert and yr += ys, or (b) the shared expert through two GEMVs (interleaved gate/up with the SwiGLU epilogue, down to
f32) and the expert kernel over the routed experts with the caller's ys; then the caller's bf16(f32(residual) + sum) and the next
layer's RMSNorm (glmcoll.h:44-52 at one rank).
Each call is checked against the oracle's call of the same name fed with the GPU's own inputs of that stage, and the
whole chain against the oracle's chain."""
import numpy as np
import pytest

from dsgx10_amd import abi, lib
from dsgx10_amd.layer import HostLayer
from tests import gpu, orc
from tests.helpers import check_outputs, check_sums, make_layer

pytestmark = pytest.mark.gpu


def _gemv(x, fmt, parts, N, K, out_kind, splitk=1):
    ncol = N // 2 if out_kind == abi.OUT_SWIGLU else N
    y = gpu.empty(x.shape[0] * ncol * (4 if out_kind == abi.OUT_F32 else 2), 0xFF)
    keep = [gpu.dev(p) for p in parts]
    lib.gemv(gpu.dev(x), x.shape[1], x.shape[0], K, [dict(fmt=fmt, w=keep[0], s=None, zp=None, n=N, y=y, ldy=ncol)], out_kind, splitk=splitk)
    return gpu.host(y, np.float32 if out_kind == abi.OUT_F32 else np.uint16, (x.shape[0], ncol))


@pytest.mark.parametrize("up", [0, 1], ids=["vector", "mfma"])
def test_moe_step_as_the_runner_calls_it(up):
    H, I, E, topk, M, scale = 2048, 2048, 24, 8, 3, 2.5
    hl = make_layer(abi.FMT_INT4, H, I, E, topk, NS=4, seed=8, shared="bf16")
    dl = hl.upload()
    x = orc.normal_bf16(8, 1, (M, H), 1.0)
    res = orc.normal_f32(8, 2, (M, H), 1.0)  # the residual stream (f32 here; finalize rounds it to bf16 first)
    wr = orc.normal_bf16(8, 3, (E, H), 0.05)
    bias = orc.normal_f32(8, 4, (E,), 0.1)
    # 1. the router's logits: fp32 products of bf16 values, f32 sums, K split four ways (model.cu:309-312)
    logits = _gemv(x, abi.FMT_BF16, (wr,), E, H, abi.OUT_F32, splitk=4)
    o = orc.gemv(x, abi.FMT_BF16, wr, None, None, E, H, abi.OUT_F32)
    worst, bad = check_sums(logits, o["yd"], o["ymag"], 1e-4)
    assert bad == 0, worst
    idx, w = orc.route(logits, bias, topk, scale)  # the oracle's picks from the GPU's logits
    uni = orc.union(idx, E)
    # 2a. fused: routing, shared expert and the sum inside the expert kernel (kTuneRoute, kTuneShFused, decision 8)
    yr_a, ys_a, ws = gpu.decode_layer(dl, x, None, None, M, logits=gpu.dev(logits), bias=gpu.dev(bias), route_scale=scale, ysum=True, up=up)
    hg = gpu.h_of(ws, dl, M, len(uni))
    dn = orc.moe_down(hl, hg, idx, w, uni, ysum=True)
    worst, bad = check_sums(yr_a, dn["yr64"], dn["yrmag"] + dn["ysmag"], 1e-4)
    assert bad == 0, worst
    # 2b. the shared expert through the GEMV (model.cu:326-332), the routed experts with the caller's ys
    bgu, bd = hl.shared_bf16
    hm = _gemv(x, abi.FMT_BF16, (bgu,), 2 * I, H, abi.OUT_SWIGLU)
    ys_b = _gemv(hm, abi.FMT_BF16, (bd,), H, I, abi.OUT_F32)
    routed = HostLayer(hl.fmt, H, I, E, topk, hl.experts, hl.emap)
    dr = routed.upload()
    yr_b, ys_out, _ = gpu.decode_layer(dr, x, idx, w, M, ysum=True, ys_in=ys_b, up=up)
    assert np.array_equal(ys_out, ys_b)
    # the GEMV's shared expert against the fused one: the same h rule, another order of adds
    assert (hm == hg[-1]).mean() >= 0.995
    check_outputs(ys_b, ys_a)
    check_outputs(yr_b, yr_a)
    # 3. the caller's residual add, and the whole chain against the oracle's chain from x
    out = gpu.empty(M * H * 2)
    lib.finalize(gpu.dev(res), gpu.dev(yr_a), M * H, out)
    out = gpu.host(out, np.uint16, (M, H))
    assert np.array_equal(out, orc.finalize(res, yr_a))
    up_o = orc.moe_up(hl, x, uni, want_range=False)
    full = orc.moe_down(hl, up_o["h32"], idx, w, uni, ysum=True)
    check_outputs(yr_a, full["yr32"])
    ref_out = orc.bf16_to_f32(orc.finalize(res, full["yr32"]))
    assert np.abs(orc.bf16_to_f32(out) - ref_out).max() <= 2e-2 + 2.0 ** -7 * np.abs(ref_out).max()
    # 3'. the runner's own step 3 (model.cu:343, glmcoll.h:44-52): h = bf16(bf16 residual + yr), the next layer's RMSNorm of h
    res16, nw = orc.normal_bf16(8, 5, (M, H), 1.0), orc.normal_bf16(8, 6, (H,), 1.0)
    ro, xn = gpu.empty(M * H * 2, 0xFF), gpu.empty(M * H * 2, 0xFF)
    lib.add_norm(gpu.dev(yr_a), None, M, H, gpu.dev(res16), ro, gpu.dev(nw), 1e-5, xn)
    o_ro, o_xn, _ = orc.add_norm(yr_a, None, res16, nw, 1e-5)
    assert np.array_equal(gpu.host(ro, np.uint16, (M, H)), o_ro)
    xn = gpu.host(xn, np.uint16, (M, H))
    assert (xn == o_xn).mean() >= 0.999 and np.abs(xn.astype(np.int32) - o_xn.astype(np.int32)).max() <= 1


def _chain_weights(seed, l, fmt, H, XR, QL, NQ, E):
    qb = orc.normal_f32(seed, 100 * l + 1, (NQ, QL), 0.03)
    op = orc.normal_f32(seed, 100 * l + 2, (H, NQ), 0.03)
    if fmt == abi.FMT_FP8:
        qb, op = orc.fp8_quantize(qb), orc.fp8_quantize(op)
    else:
        qb, op = orc.int4_quantize_sym(qb), orc.int4_quantize_sym(op)
    return dict(attn_norm=orc.f32_to_bf16(1.0 + orc.normal_f32(seed, 100 * l + 3, (H,), 0.1)), ffn_norm=orc.f32_to_bf16(1.0 + orc.normal_f32(seed, 100 * l + 4, (H,), 0.1)),
                xproj=orc.normal_bf16(seed, 100 * l + 5, (XR, H), 0.03), router=orc.normal_bf16(seed, 100 * l + 6, (E, H), 0.05), qb=qb, oproj=op)


def _oracle_chain(layers, hls, fmt, x0, H, XR, QL, NQ, E, topk, scale, final_norm):
    """the same chain on the CPU: orc_add_norm, orc_gemv, orc_route, orc_moe_up / orc_moe_down; returns (residual bf16, xn bf16)"""
    M = x0.shape[0]
    res, yr = x0.copy(), np.zeros((M, H), np.float32)
    g = lambda x, parts, N, K, kind, f: orc.gemv(x, f, parts[0], parts[1] if len(parts) > 1 else None, parts[2] if len(parts) > 2 else None, N, K, kind, want64=False)
    for W, hl in zip(layers, hls):
        res, xn, _ = orc.add_norm(yr, None, res, W["attn_norm"], 1e-5)
        xg = g(xn, (W["xproj"],), XR, H, abi.OUT_BF16, abi.FMT_BF16)["y16"]
        q = g(np.ascontiguousarray(xg[:, :QL]), W["qb"], NQ, QL, abi.OUT_BF16, fmt)["y16"]
        part = g(q, W["oproj"], H, NQ, abi.OUT_F32, fmt)["yf"]
        res, xn, _ = orc.add_norm(part, None, res, W["ffn_norm"], 1e-5)
        logits = g(xn, (W["router"],), E, H, abi.OUT_F32, abi.FMT_BF16)["yf"]
        idx, w = orc.route(logits, None, topk, scale)
        uni = orc.union(idx, E)
        up = orc.moe_up(hl, xn, uni, want_range=False)
        yr = orc.moe_down(hl, up["h32"], idx, w, uni, ysum=True)["yr32"]
    return orc.add_norm(yr, None, res, final_norm, 1e-5)[:2]


def _bf16_close(got, ref, what, share=0.99):
    """bf16 outputs of one stage from the same inputs: nearly all equal, none more than one step apart"""
    d = np.abs(got.astype(np.int32) - ref.astype(np.int32))
    assert (d == 0).mean() >= share and d.max() <= 1, (what, float((d == 0).mean()), int(d.max()))


@pytest.mark.parametrize("fmt,shared,scale", [(abi.FMT_FP8, "fp8", 1.0), (abi.FMT_INT4, "bf16", 2.5)], ids=["fp8", "int4"])
def test_chained_layers_against_the_oracle_chain(fmt, shared, scale):
    """Three decode layers as the runner chains them (dsgx10_amd/chain.py: x-projection, q_b, o_proj, add + norm, router, experts,
    add + norm), every layer with weights of its own and routing by its own data.
    (1) each add + norm fused into the GEMV that reads it gives the bits of the separate launches;
    (2) every stage of every layer against the oracle's call of the same name fed with the GPU's own inputs of that stage: the
        residual adds bit for bit, bf16 outputs equal in >= 99% and never more than a step apart, f32 sums within 1e-4 of their
        sums of |terms|, the experts' yr at the benchmark's bar (2e-2 / 1e-3);
    (3) the free-running chain against the oracle's free-running chain. A chain of bf16 roundings is chaotic in the small: one
        value that rounds the other way (a step is 0.4-0.8% of it) moves every sum downstream by ~1e-4 relative, which flips a
        few % of the next roundings, and so on: after three layers a third of the residual's values differ by a step, which is
        3e-3 in relative L2 although every stage holds the bar. Checked: relative L2 <= 1e-2, no value off by more than 2% of the
        largest."""
    from dsgx10_amd.chain import LayerChain
    H, XR, QL, NQ, I, E, topk, M, NL = 2048, 512, 256, 1024, 1024, 16, 4, 2, 3
    hls = [make_layer(fmt, H, I, E, topk, NS=4, seed=40 + l, shared=shared) for l in range(NL)]
    dls = [h.upload() for h in hls]
    Ws = [_chain_weights(7, l, fmt, H, XR, QL, NQ, E) for l in range(NL)]
    x0 = orc.normal_bf16(7, 999, (M, H), 1.0)
    fin = orc.f32_to_bf16(1.0 + orc.normal_f32(7, 998, (H,), 0.1))
    keep = []

    def mat(parts):
        t = [gpu.dev(p) for p in parts]
        keep.append(t)
        return dict(fmt=fmt, w=t[0], s=t[1], zp=t[2] if len(t) > 2 else None)
    devW = []
    for W, dl in zip(Ws, dls):
        d = dict(attn_norm=gpu.dev(W["attn_norm"]), ffn_norm=gpu.dev(W["ffn_norm"]), xproj=gpu.dev(W["xproj"]), router=gpu.dev(W["router"]),
                 qb=mat(W["qb"]), oproj=mat(W["oproj"]), moe=dl.w, ws=gpu.empty(lib.decode_ws_bytes(dl.w), 0))
        devW.append(d)
    g = lambda x, parts, N, K, kind, f: orc.gemv(x, f, parts[0], parts[1] if len(parts) > 1 else None, parts[2] if len(parts) > 2 else None, N, K, kind)
    outs = {}
    for fused in (False, True):
        ch = LayerChain(M, H, XR, QL, NQ, E, scale, lambda n: gpu.empty(n, 0))
        ch.res[0].copy_(gpu.dev(x0))
        for l, (d, W, hl) in enumerate(zip(devW, Ws, hls)):
            got = {}

            def tap(name):
                a, b = ch.res[ch.cur], ch.res[ch.cur ^ 1]
                for k, t, dt, shp in (("res_a", a, np.uint16, (M, H)), ("res_b", b, np.uint16, (M, H)), ("xn", ch.xn, np.uint16, (M, H)),
                                      ("xg", ch.xg, np.uint16, (M, XR)), ("q", ch.q, np.uint16, (M, NQ)), ("part", ch.part, np.float32, (M, H)),
                                      ("logits", ch.logits, np.float32, (M, E)), ("yr", ch.yr, np.float32, (M, H))):
                    got[name + "." + k] = gpu.host(t, dt, shp)
            yr_prev, res_prev = gpu.host(ch.yr, np.float32, (M, H)), gpu.host(ch.res[ch.cur], np.uint16, (M, H))
            ch.layer(d, fused=fused, up=0 if fmt == abi.FMT_FP8 else 1, tap=None if fused else tap, fuse_xproj=fused)
            if fused:
                continue
            # (2) stage by stage, the oracle fed with the GPU's own inputs
            o_res, o_xn, _ = orc.add_norm(yr_prev, None, res_prev, W["attn_norm"], 1e-5)
            assert np.array_equal(got["norm1.res_b"], o_res), (l, "residual after the attention-side add")
            _bf16_close(got["norm1.xn"], o_xn, (l, "norm1"), 0.999)
            o = g(got["norm1.xn"], (W["xproj"],), XR, H, abi.OUT_BF16, abi.FMT_BF16)
            _bf16_close(got["xproj.xg"], o["y16"], (l, "xproj"))
            o = g(np.ascontiguousarray(got["xproj.xg"][:, :QL]), W["qb"], NQ, QL, abi.OUT_BF16, fmt)
            _bf16_close(got["qb.q"], o["y16"], (l, "q_b"))
            o = g(got["qb.q"], W["oproj"], H, NQ, abi.OUT_F32, fmt)
            worst, bad = check_sums(got["oproj.part"], o["yd"], o["ymag"], 1e-4)
            assert bad == 0, (l, "o_proj", worst)
            o_res, o_xn, _ = orc.add_norm(got["oproj.part"], None, got["norm1.res_b"], W["ffn_norm"], 1e-5)
            assert np.array_equal(got["norm2.res_a"], o_res), (l, "residual after the MoE-side add")
            _bf16_close(got["norm2.xn"], o_xn, (l, "norm2"), 0.999)
            o = g(got["norm2.xn"], (W["router"],), E, H, abi.OUT_F32, abi.FMT_BF16)
            worst, bad = check_sums(got["router.logits"], o["yd"], o["ymag"], 1e-4)
            assert bad == 0, (l, "router", worst)
            idx, w = orc.route(got["router.logits"], None, topk, scale)
            uni = orc.union(idx, E)
            up_o = orc.moe_up(hl, got["norm2.xn"], uni, want_range=False)
            full = orc.moe_down(hl, up_o["h32"], idx, w, uni, ysum=True)
            check_outputs(got["experts.yr"], full["yr32"])
        ch.finish(gpu.dev(fin))
        for d, dl in zip(devW, dls):
            lib.decode_status(dl.w, d["ws"])
        outs[fused] = (gpu.host(ch.res[ch.cur], np.uint16, (M, H)), gpu.host(ch.xn, np.uint16, (M, H)))
    assert np.array_equal(outs[True][0], outs[False][0]) and np.array_equal(outs[True][1], outs[False][1]), "fused add + norm changes bits"
    r_ref, xn_ref = _oracle_chain(Ws, hls, fmt, x0, H, XR, QL, NQ, E, topk, scale, fin)
    for got, ref, what in ((outs[True][0], r_ref, "residual"), (outs[True][1], xn_ref, "normed row")):
        gf, rf = orc.bf16_to_f32(got).astype(np.float64), orc.bf16_to_f32(ref).astype(np.float64)
        rel = np.sqrt(((gf - rf) ** 2).sum() / (rf ** 2).sum())
        print("free-running chain, %s after %d layers: equal %.2f%%, rel-L2 %.2e, max-abs %.2e (|ref| max %.1f)"
              % (what, NL, 100 * (got == ref).mean(), rel, np.abs(gf - rf).max(), np.abs(rf).max()))
        assert rel <= 1e-2 and np.abs(gf - rf).max() <= 0.02 * np.abs(rf).max(), what
