"""The C++ mirror headers on the GPU (marked gpu): tests/mirror_run (tests/mirror_run.cpp, compiled by
dsgx10_amd.build against include/gx/experts.h and include/glm/attn.h) runs route -> moe_decode -> finalize, the fused
form, a dense GEMV and the residual add + RMSNorm through the gx:: / glm:: / comm::glm:: forwarders; every output must equal, bit for bit, what the same calls
give through the ctypes binding of the C ABI."""
import os
import subprocess
import tempfile

import numpy as np
import pytest
import torch

from dsgx10_amd import abi, lib
from tests import gpu, orc
from tests.helpers import make_layer, rows_and_routing

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "mirror_run")


@pytest.mark.parametrize("fmt,shared,scale,up", [(abi.FMT_FP8, "fp8", 1.0, -1), (abi.FMT_FP8, "fp8", 1.0, 0), (abi.FMT_INT4, "bf16", 2.5, 1), (abi.FMT_FP8, "fp8", 1.0, abi.UP_PREFILL_ORDER)])
def test_cpp_mirrors_give_the_c_abi_bits(fmt, shared, scale, up):
    assert os.path.exists(EXE), "tests/mirror_run is not built (python -m dsgx10_amd.build)"
    H, I, E, topk, M = 2048, 2048, 32, 8, 3
    hl = make_layer(fmt, H, I, E, topk, 4, seed=12, shared=shared)
    dl = hl.upload()
    x, logits, _, _ = rows_and_routing(51, M, H, E, topk, scale)
    bias = orc.normal_f32(51, 3, (E,), 0.3)
    resid = orc.normal_f32(51, 4, (M, H), 1.0)
    res16, normw = orc.normal_bf16(51, 5, (M, H), 1.0), orc.normal_bf16(51, 6, (H,), 1.0)
    with tempfile.TemporaryDirectory() as d:
        def put(name, a):
            np.ascontiguousarray(a).tofile(os.path.join(d, name + ".bin"))
        put("pool", hl.pool), put("desc", hl.desc), put("x", x), put("logits", logits), put("bias", bias), put("resid", resid)
        put("res16", res16), put("normw", normw)
        if hl.shared_fp8 is not None:
            for n, (c, s) in zip("gud", hl.shared_fp8):
                put("sh_" + n, c), put("sh_" + n + "s", s)
        if hl.shared_bf16 is not None:
            put("sh_bgu", hl.shared_bf16[0]), put("sh_bd", hl.shared_bf16[1])
        r = subprocess.run([EXE, d, str(fmt), str(H), str(I), str(E), str(topk), str(M), repr(scale), str(up)], capture_output=True, text=True, timeout=120)
        assert r.returncode == 0 and "CHECK mirror_run ok" in r.stdout, r.stdout + r.stderr
        got = {n: np.fromfile(os.path.join(d, "o_%s.bin" % n), dt) for n, dt in
               (("idx", np.int32), ("w", np.uint32), ("yr", np.uint32), ("ys", np.uint32), ("out", np.uint16), ("yr2", np.uint32), ("ys2", np.uint32), ("gemv", np.uint32), ("h", np.uint16), ("xn", np.uint16))}
    # the same calls through ctypes
    dlog, dbias = gpu.dev(logits), gpu.dev(bias)
    gi, gw = gpu.empty(M * topk * 4), gpu.empty(M * topk * 4)
    lib.route(dlog.view(torch.float32).view(M, E), dbias, gi.view(torch.int32).view(M, topk), gw.view(torch.float32).view(M, topk), scale)
    idx, w = gpu.host(gi, np.int32, (M, topk)), gpu.host(gw, np.float32, (M, topk))
    assert np.array_equal(got["idx"], idx.reshape(-1)) and np.array_equal(got["w"], w.view(np.uint32).reshape(-1))
    ridx, rw = orc.route(logits, bias, topk, scale)
    assert np.array_equal(idx, ridx) and np.array_equal(w.view(np.uint32), rw.view(np.uint32))
    yr, ys, _ = gpu.decode_layer(dl, x, idx, w, M, up=up)
    assert np.array_equal(got["yr"], yr.view(np.uint32).reshape(-1)) and np.array_equal(got["ys"], ys.view(np.uint32).reshape(-1))
    out = gpu.empty(M * H * 2, 0)
    lib.finalize(gpu.dev(resid), gpu.dev(yr), M * H, out)
    assert np.array_equal(got["out"], gpu.host(out, np.uint16, (-1,)))
    yr2, ys2, _ = gpu.decode_layer(dl, x, None, None, M, logits=dlog, bias=dbias, route_scale=scale, ysum=True, up=up)
    assert np.array_equal(got["yr2"], yr2.view(np.uint32).reshape(-1)) and np.array_equal(got["ys2"], ys2.view(np.uint32).reshape(-1))
    assert np.array_equal(yr2, yr + ys)
    # the dense GEMV
    gn = I if shared == "fp8" else 2 * I
    y = gpu.empty(M * gn * 4, 0)
    if shared == "fp8":
        seg = dict(fmt=abi.FMT_FP8, w=gpu.dev(hl.shared_fp8[0][0]), s=gpu.dev(hl.shared_fp8[0][1]), n=gn, y=y, ldy=gn)
    else:
        seg = dict(fmt=abi.FMT_BF16, w=gpu.dev(hl.shared_bf16[0]), n=gn, y=y, ldy=gn)
    lib.gemv(gpu.dev(x), H, M, H, [seg], abi.OUT_F32, splitk=4)
    assert np.array_equal(got["gemv"], gpu.host(y, np.uint32, (-1,)))
    # comm::glm::allreduce_add_norm at a world of one
    r16, xn = gpu.dev(res16), gpu.empty(M * H * 2, 0)
    lib.add_norm(gpu.dev(yr2), None, M, H, r16, r16, gpu.dev(normw), 1e-5, xn)
    assert np.array_equal(got["h"], gpu.host(r16, np.uint16, (-1,))) and np.array_equal(got["xn"], gpu.host(xn, np.uint16, (-1,)))
    assert np.array_equal(got["h"], orc.add_norm(yr2, None, res16, normw, 1e-5)[0].reshape(-1))


@pytest.mark.parametrize("H,I,E,M,shared", [(1024, 512, 16, 3, True), (2048, 768, 32, 12, True), (1024, 256, 8, 16, False)])
def test_dsk_mirror_gives_the_c_abi_bits(H, I, E, M, shared):
    """include/dsk/dsk.h with the reference's own argument lists (tests/mirror_run_dsk.cpp): experts stacked by id after
    tile_fp4 / tile_fp8, router_topk -> moe, moe_routed with idx_out / wts_out, moe_prefill_rows; against dsgx_route and
    dsgx_dsk_moe on a pooled layer of the same weights (whose parity with the oracle tests/test_gpu_dsk.py holds), bit for bit;
    moe_prefill against dsgx_dsk_moe_prefill on the same stacked tensors (parity: tests/test_gpu_dsk_prefill.py), bit for bit.
    12 and 16 rows take two passes of the decode kernels."""
    from tests.test_gpu_dsk import _layer
    exe = os.path.join(ROOT, "tests", "mirror_run_dsk")
    assert os.path.exists(exe), "tests/mirror_run_dsk is not built (python -m dsgx10_amd.build)"
    topk, scale = 6, 1.5
    hl = _layer(33, H, I, E, topk, 5, shared)
    dl = hl.upload()
    x = orc.normal_bf16(33, 1, (M, H), 1.5)
    xq, xs = orc.act_quant_ue8m0(x)
    logits, bias = orc.normal_f32(33, 2, (M, E), 1.0), orc.normal_f32(33, 3, (E,), 0.2)
    with tempfile.TemporaryDirectory() as d:
        def put(name, a):
            np.ascontiguousarray(a).tofile(os.path.join(d, name + ".bin"))
        for j, n in enumerate(("1", "3", "2")):
            put("w" + n, np.stack([hl.experts[int(hl.emap[e])][j][0] for e in range(E)]))
            put("s" + n, np.stack([hl.experts[int(hl.emap[e])][j][1] for e in range(E)]))
            if shared:
                put("sh_w" + n, hl.shared_fp8[j][0]), put("sh_s" + n, hl.shared_fp8[j][1])
        put("xq", xq), put("xs", xs), put("logits", logits), put("bias", bias)
        stacks = {}
        for j, n in enumerate(("1", "3", "2")):
            stacks["w" + n] = gpu.dev(np.stack([hl.experts[int(hl.emap[e])][j][0] for e in range(E)]))
            stacks["s" + n] = gpu.dev(np.stack([hl.experts[int(hl.emap[e])][j][1] for e in range(E)]))
            if shared:
                stacks["sh_w" + n], stacks["sh_s" + n] = gpu.dev(hl.shared_fp8[j][0]), gpu.dev(hl.shared_fp8[j][1])
        r = subprocess.run([exe, d, str(H), str(I), str(E), str(M), repr(scale), str(int(shared))], capture_output=True, text=True, timeout=120)
        assert r.returncode == 0 and "CHECK mirror_run_dsk ok" in r.stdout, r.stdout + r.stderr
        got = {n: np.fromfile(os.path.join(d, "o_%s.bin" % n), dt) for n, dt in
               (("idx", np.int32), ("w", np.uint32), ("idx2", np.int32), ("w2", np.uint32), ("y", np.uint32), ("y2", np.uint32), ("y3", np.uint32), ("y4", np.uint32))}
    idx, w = orc.route(logits, bias, topk, scale, score_fn=1)
    for k in ("idx", "idx2"):
        assert np.array_equal(got[k], idx.reshape(-1)), k
    for k in ("w", "w2"):
        assert np.array_equal(got[k], w.view(np.uint32).reshape(-1)), k
    ws = gpu.empty(lib.decode_ws_bytes(dl.w), 0)
    y, ys = gpu.empty(M * H * 4, 0xFF), gpu.empty(M * H * 4, 0xFF)
    lib.dsk_moe(dl.w, gpu.dev(xq), gpu.dev(xs), gpu.dev(idx), gpu.dev(w), M, ws, y, ys)
    want = gpu.host(y, np.uint32, (-1,))
    assert np.isfinite(want.view(np.float32)).all()
    for k in ("y", "y2", "y4"):
        assert np.array_equal(got[k], want), (k, int((got[k] != want).sum()))
    ptr = lambda k: stacks[k].data_ptr() if k in stacks else None
    dw = abi.DskWeights(*[ptr(k) for k in ("w1", "s1", "w3", "s3", "w2", "s2", "sh_w1", "sh_s1", "sh_w3", "sh_s3", "sh_w2", "sh_s2")], H, I, E, topk)
    pws, yp = gpu.empty(lib.dsk_prefill_ws_bytes(H, I, E, topk, M), 0xEE), gpu.empty(M * H * 4, 0xFF)
    lib.dsk_moe_prefill(dw, gpu.dev(xq), gpu.dev(xs), gpu.dev(idx), gpu.dev(w), M, pws, yp)
    wantp = gpu.host(yp, np.uint32, (-1,))
    assert np.array_equal(got["y3"], wantp), int((got["y3"] != wantp).sum())
    rel = np.linalg.norm(wantp.view(np.float32) - want.view(np.float32)) / np.linalg.norm(want.view(np.float32))
    assert rel <= 5e-3, rel  # the two operators agree to their tolerance
