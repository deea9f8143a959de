"""GPU parity of DeepSeek's decode MoE (dsgx_dsk_moe = dsk::moe / dsk::moe_routed of the reference,
ds41f-4xgx10-switchless/engine/kernels/dsk.h:199-241): MXFP4 routed experts + FP8 shared expert with ue8m0 scales, rows
given as act_quant(x), against the CPU oracle, stage by stage as the reference tests its kernels
(engine/kernels/tests/test_kernels.cu:218-377: moe_up's quantised output against an fp64 host reference, then y):
  h (bf16, before its quantisation; read from the workspace) within the range the oracle allows at the reference's sum
  tolerance and equal to the oracle's in >= 99% of bits; each expert's w2 from the GPU's own h: the f32 sums behind y within
  1e-4 * sum|terms| + one bf16 step of the f64 sums; y against the oracle's chain at max-abs 2e-2 / rel-L2 1e-3."""
import numpy as np
import pytest

from dsgx10_amd import abi, lib
from dsgx10_amd.layer import HostLayer
from tests import gpu, orc

pytestmark = pytest.mark.gpu


def _fp4_mat(rng, N, K, lo=116, hi=121):
    codes = rng.integers(0, 16, (N, K), dtype=np.uint8)
    return (codes[:, 0::2] | (codes[:, 1::2] << 4)).astype(np.uint8), rng.integers(lo, hi, (N, K // 32), dtype=np.uint8)


def _fp8e_mat(rng, N, K, lo=112, hi=117):
    w = orc.f32_to_e4m3(np.clip(rng.standard_normal((N, K)).astype(np.float32) * 40.0, -448, 448))
    return w, rng.integers(lo, hi, (N // 32, K // 32), dtype=np.uint8)


def _layer(seed, H, I, E, topk, NS, shared):
    rng = np.random.default_rng(seed)
    experts = [(_fp4_mat(rng, I, H), _fp4_mat(rng, I, H), _fp4_mat(rng, H, I, 118, 123)) for _ in range(NS)]
    sh = (_fp8e_mat(rng, I, H), _fp8e_mat(rng, I, H), _fp8e_mat(rng, H, I, 114, 119)) if shared else None
    return HostLayer(abi.FMT_MXFP4, H, I, E, topk, experts, emap=np.array([(7 * e + 3) % NS for e in range(E)]), shared_fp8=sh)


@pytest.mark.parametrize("H,I,E,M,shared,fused", [(1024, 512, 16, 1, True, False), (2048, 768, 32, 3, True, True), (1024, 256, 8, 8, False, False),
                                                  (5120, 2304, 48, 2, True, True)])
def test_dsk_moe_against_oracle(H, I, E, M, shared, fused):
    topk = 6
    hl = _layer(21, H, I, E, topk, 5, shared)
    dl = hl.upload()
    x = orc.normal_bf16(21, 1, (M, H), 1.5)
    xq, xs = orc.act_quant_ue8m0(x)
    xd = orc.dequant_act_ue8m0(xq, xs)
    logits = orc.normal_f32(21, 2, (M, E), 1.0)
    bias = orc.normal_f32(21, 3, (E,), 0.2)
    idx, w = orc.route(logits, bias, topk, 1.5, score_fn=1)
    ws = gpu.empty(lib.decode_ws_bytes(dl.w), 0)
    y, ys = gpu.empty(M * H * 4, 0xFF), gpu.empty(M * H * 4, 0xFF)
    if fused:
        lib.dsk_moe(dl.w, gpu.dev(xq), gpu.dev(xs), None, None, M, ws, y, ys, logits=gpu.dev(logits), bias=gpu.dev(bias), route_scale=1.5)
    else:
        lib.dsk_moe(dl.w, gpu.dev(xq), gpu.dev(xs), gpu.dev(idx), gpu.dev(w), M, ws, y, ys)
    lib.decode_status(dl.w, ws)
    y, ys = gpu.host(y, np.float32, (M, H)), gpu.host(ys, np.float32, (M, H))
    uni = orc.union(idx, E)
    hg = gpu.h_of(ws, dl, M, len(uni))  # [slots (+ shared last)][M][I], bf16 before the quantisation
    deq = lambda parts: orc.mxfp4_dequant(*parts)
    ref = np.zeros((M, H), np.float64)      # the oracle's chain from x
    ref_own = np.zeros((M, H), np.float32)  # the fold of the oracle's w2 outputs from the GPU's own h
    nh = nbad = 0
    worst = 0.0
    slots = [(u, int(e)) for u, e in enumerate(uni)] + ([(len(uni), -1)] if shared else [])
    for u, e in slots:
        if e >= 0:
            ex = hl.experts[int(hl.emap[e])]
            w1, w3, w2 = deq(ex[0]), deq(ex[1]), deq(ex[2])
            rw = np.array([w[m][list(idx[m]).index(e)] if e in idx[m] else 0.0 for m in range(M)], np.float32)
            rows = [m for m in range(M) if e in idx[m]]
        else:
            w1, w3, w2 = (orc.fp8e_dequant(*p) for p in hl.shared_fp8)
            rw, rows = None, list(range(M))
        up = orc.dsk_up(w1, w3, xd, rw)
        for m in rows:
            hf = orc.bf16_to_f32(hg[u][m])
            assert np.all(hf >= up["lo"][m] - 1e-30) and np.all(hf <= up["hi"][m] + 1e-30), (u, m)
            nbad += int((hg[u][m] != up["h64"][m]).sum())
            nh += I
        dn_own = orc.dsk_down(w2, hg[u])
        dn_ref = orc.dsk_down(w2, up["h32"])
        for m in rows:
            ref[m] += orc.bf16_to_f32(dn_ref["outb"][m])
            ref_own[m] = ref_own[m] + orc.bf16_to_f32(dn_own["outb"][m])
        if e < 0:  # the shared expert's own output: bf16 values, within a step of the oracle's from the same h
            err = np.abs(ys.astype(np.float64) - dn_own["out64"])
            tol = 1e-4 * dn_own["mag"] + np.abs(dn_own["out64"]) * 2.0 ** -8
            assert np.all(err <= tol), (err / tol).max()
            assert np.array_equal(orc.bf16_to_f32(orc.f32_to_bf16(ys)), ys)
            worst = max(worst, float((err / np.maximum(tol, 1e-300)).max()))
    assert nbad <= 0.01 * nh, (nbad, nh)
    # y from the GPU's own h: every term is a bf16 value that may round the other way; a term's step is 2^-8 of it
    assert np.abs(y - ref_own).max() <= 2e-2 and np.linalg.norm(y - ref_own) <= 1e-3 * np.linalg.norm(ref_own) + 1e-12
    # and the whole chain
    assert np.abs(y - ref).max() <= 2e-2 + 2.0 ** -7 * np.abs(ref).max()
    rl2 = np.linalg.norm(y - ref) / max(np.linalg.norm(ref), 1e-30)
    print("dsk moe H=%d I=%d M=%d: h equal %.2f%%, end-to-end rel-L2 %.2e max-abs %.2e (|y| max %.2f)"
          % (H, I, M, 100 - 100.0 * nbad / nh, rl2, np.abs(y - ref).max(), np.abs(ref).max()))
    assert rl2 <= 3e-3


@pytest.mark.parametrize("H,I,E,M,shared", [(1024, 512, 16, 1, True), (2048, 768, 32, 3, True), (1024, 256, 8, 8, False), (5120, 2304, 48, 2, True)])
def test_dsk_moe_every_bit_against_the_matrix_unit_oracle(H, I, E, M, shared):
    """with the bf16 MFMA's order of adds and the decode kernels' slicing of K restated in the oracle (orc.set_dsk_dot_rule;
    the instruction's rule is pinned on the CPU by tests/golden/mfma_bf16_k32.npz) DeepSeek's decode layer is checked bit
    for bit: h of every slot and row, the shared expert's output, and the fold y"""
    topk = 6
    hl = _layer(23, H, I, E, topk, 5, shared)
    dl = hl.upload()
    x = orc.normal_bf16(23, 1, (M, H), 1.5)
    xq, xs = orc.act_quant_ue8m0(x)
    xd = orc.dequant_act_ue8m0(xq, xs)
    idx, w = orc.route(orc.normal_f32(23, 2, (M, E), 1.0), orc.normal_f32(23, 3, (E,), 0.2), topk, 1.5, score_fn=1)
    ws = gpu.empty(lib.decode_ws_bytes(dl.w), 0)
    y, ys = gpu.empty(M * H * 4, 0xFF), gpu.empty(M * H * 4, 0xFF)
    lib.dsk_moe(dl.w, gpu.dev(xq), gpu.dev(xs), gpu.dev(idx), gpu.dev(w), M, ws, y, ys)
    lib.decode_status(dl.w, ws)
    y, ys = gpu.host(y, np.float32, (M, H)), gpu.host(ys, np.float32, (M, H))
    uni = orc.union(idx, E)
    hg = gpu.h_of(ws, dl, M, len(uni))
    want = np.zeros((M, H), np.float32)
    try:
        for u, e in enumerate(uni):
            ex = hl.experts[int(hl.emap[int(e)])]
            w1, w3, w2 = (orc.mxfp4_dequant(*p) for p in ex)
            rw = np.array([w[m][list(idx[m]).index(e)] if e in idx[m] else 0.0 for m in range(M)], np.float32)
            orc.set_dsk_dot_rule(1)
            up = orc.dsk_up(w1, w3, xd, rw)
            assert np.array_equal(hg[u], up["h32"]), (u, int((hg[u] != up["h32"]).sum()))
            dn = orc.dsk_down(w2, up["h32"])
            for m in range(M):
                if e in idx[m]:
                    want[m] = want[m] + orc.bf16_to_f32(dn["outb"][m])
        if shared:
            orc.set_dsk_dot_rule(3)
            w1, w3, w2 = (orc.fp8e_dequant(*p) for p in hl.shared_fp8)
            up = orc.dsk_up(w1, w3, xd, None)
            assert np.array_equal(hg[len(uni)], up["h32"]), int((hg[len(uni)] != up["h32"]).sum())
            dn = orc.dsk_down(w2, up["h32"])
            sh = orc.bf16_to_f32(dn["outb"])
            assert np.array_equal(ys.view(np.uint32), sh.view(np.uint32)), int((ys != sh).sum())
            want = want + sh
    finally:
        orc.set_dsk_dot_rule(0)
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32)), int((y != want).sum())


@pytest.mark.parametrize("M", [12, 16])
def test_dsk_moe_nine_to_sixteen_rows(M):
    """9-16 rows run as two passes of the kernels built for eight (dsk.h:211-223's up16 / down16 range): every row's bits are
    what the row gives in a call of its own, whose parity with the oracle the test above holds; routing fused and apart"""
    H, I, E, topk = 2048, 768, 32, 6
    hl = _layer(22, H, I, E, topk, 5, True)
    dl = hl.upload()
    x = orc.normal_bf16(22, 1, (M, H), 1.5)
    xq, xs = orc.act_quant_ue8m0(x)
    logits, bias = orc.normal_f32(22, 2, (M, E), 1.0), orc.normal_f32(22, 3, (E,), 0.2)
    idx, w = orc.route(logits, bias, topk, 1.5, score_fn=1)
    ws = gpu.empty(lib.decode_ws_bytes(dl.w), 0)

    def run(rows, fused):
        n = len(rows)
        y, ys = gpu.empty(n * H * 4, 0xFF), gpu.empty(n * H * 4, 0xFF)
        if fused:
            lib.dsk_moe(dl.w, gpu.dev(xq[rows]), gpu.dev(xs[rows]), None, None, n, ws, y, ys, logits=gpu.dev(logits[rows]), bias=gpu.dev(bias), route_scale=1.5)
        else:
            lib.dsk_moe(dl.w, gpu.dev(xq[rows]), gpu.dev(xs[rows]), gpu.dev(idx[rows]), gpu.dev(w[rows]), n, ws, y, ys)
        lib.decode_status(dl.w, ws)
        return gpu.host(y, np.uint32, (n, H)), gpu.host(ys, np.uint32, (n, H))
    all_rows = list(range(M))
    y, ys = run(all_rows, False)
    yf, ysf = run(all_rows, True)
    assert np.array_equal(y, yf) and np.array_equal(ys, ysf)
    for m in (0, 7, 8, M - 1):
        y1, ys1 = run([m], False)
        assert np.array_equal(y[m], y1[0]) and np.array_equal(ys[m], ys1[0]), m
    assert np.isfinite(y.view(np.float32)).all()
