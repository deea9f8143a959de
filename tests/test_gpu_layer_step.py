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
