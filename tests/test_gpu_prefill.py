"""GPU tests of the prefill pieces (marked gpu): MFMA layouts, bucketing, the grouped GEMMs, the whole step."""
import numpy as np
import pytest

from dsgx10_amd import lib
from tests import gpu, orc

pytestmark = pytest.mark.gpu


def test_mfma_fp8_layout():
    """one 32x32x64 e4m3 MFMA, operands loaded as the prefill kernels load them, against an exact integer product"""
    rng = np.random.default_rng(5)
    vals = np.array([0.0, 1.0, -1.0, 2.0, -2.0, 3.0, 0.5, -4.0], dtype=np.float32)
    A = vals[rng.integers(0, len(vals), (32, 64))]
    B = vals[rng.integers(0, len(vals), (32, 64))]
    qa, qb = orc.f32_to_e4m3(A), orc.f32_to_e4m3(B)
    assert np.array_equal(orc.e4m3_table()[qa], A)
    raw = gpu.empty(64 * 16 * 4, 0xFF)
    lib.probe_mfma_fp8(gpu.dev(qa), gpu.dev(qb), raw)
    raw = gpu.host(raw, np.float32, (64, 16))
    D = A.astype(np.float64) @ B.astype(np.float64).T
    got = np.empty((32, 32), dtype=np.float64)
    for l in range(64):
        for r in range(16):
            got[8 * (r // 4) + 4 * (l // 32) + r % 4, l % 32] = raw[l, r]
    assert np.array_equal(got, D)


def test_mfma_fp8_k128_layout():
    """one 16x16x128 e4m3 MFMA with the prefill kernels' k order, against an exact integer product"""
    rng = np.random.default_rng(6)
    vals = np.array([0.0, 1.0, -1.0, 2.0, -2.0, 3.0, 0.5, -4.0], dtype=np.float32)
    A = vals[rng.integers(0, len(vals), (16, 128))]
    B = vals[rng.integers(0, len(vals), (16, 128))]
    raw = gpu.empty(64 * 16 * 4, 0xFF)
    lib.probe_mfma_fp8(gpu.dev(orc.f32_to_e4m3(A)), gpu.dev(orc.f32_to_e4m3(B)), raw, form=1)
    raw = gpu.host(raw, np.float32, (64, 16))
    got = np.empty((16, 16), dtype=np.float64)
    for l in range(64):
        for r in range(4):
            got[4 * (l // 16) + r, l % 16] = raw[l, r]
    assert np.array_equal(got, A.astype(np.float64) @ B.astype(np.float64).T)


def test_mfma_fp8_accuracy():
    """What the e4m3 MFMA's own sums are worth: against exact sums of 64 products, the error stays under 1e-4 of
    sum|terms| on data shaped like quantised activations and weights (the GEMV tolerance of the reference,
    test_experts.cu:352-361), but it is far from f32 rounding (a sequential f32 sum: ~1e-8)."""
    rng = np.random.default_rng(7)
    tab = orc.e4m3_table().astype(np.float64)
    worst = 0.0
    for it in range(4):
        qa = orc.f32_to_e4m3((rng.standard_normal((32, 64)) * 100).astype(np.float32))
        qb = orc.f32_to_e4m3((rng.standard_normal((32, 64)) * 100).astype(np.float32))
        raw = gpu.empty(64 * 16 * 4, 0xFF)
        lib.probe_mfma_fp8(gpu.dev(qa), gpu.dev(qb), raw)
        raw = gpu.host(raw, np.float32, (64, 16))
        A, B = tab[qa], tab[qb]
        got = np.empty((32, 32))
        for l in range(64):
            for r in range(16):
                got[8 * (r // 4) + 4 * (l // 32) + r % 4, l % 32] = raw[l, r]
        worst = max(worst, float((np.abs(got - A @ B.T) / (np.abs(A) @ np.abs(B).T)).max()))
    assert worst <= 1e-4, worst


# ---- the whole step against the oracle (FP8 weights, FP8 activations) ------------------------------------------------
from dsgx10_amd import abi  # noqa: E402
from tests import helpers  # noqa: E402


def _prefill(hl, x, idx, w, T, **kw):
    dl = hl.upload()
    ws = gpu.empty(lib.prefill_ws_bytes(dl.w, T), 0)
    yr, ys = gpu.empty(T * hl.H * 4, 0xFF), gpu.empty(T * hl.H * 4, 0xFF)
    lib.moe_prefill(dl.w, gpu.dev(x), gpu.dev(idx), gpu.dev(w), T, ws, yr, ys, **kw)
    return gpu.host(yr, np.float32, (T, hl.H)), gpu.host(ys, np.float32, (T, hl.H)), ws, dl


@pytest.mark.parametrize("H,I,E,topk,T,shared", [(512, 256, 16, 4, 70, "fp8"), (256, 384, 4, 2, 300, None), (1024, 128, 8, 8, 129, "fp8")])
def test_prefill_fp8_against_oracle(H, I, E, topk, T, shared):
    hl = helpers.make_layer(abi.FMT_FP8, H, I, E, topk, min(E, 6), seed=3, shared=shared)
    x, _, idx, w = helpers.rows_and_routing(11, T, H, E, topk, 2.5)
    yr, ys, ws, dl = _prefill(hl, x, idx, w, T)
    v = lib.prefill_view(dl.w, ws, T)
    # the buckets: offsets are the expert counts' prefix sums, perm lists each expert's rows in row order
    P = T * topk
    off = gpu.host(gpu.view(ws, v.off, (E + 1) * 4), np.int32, (E + 1,))
    perm = gpu.host(gpu.view(ws, v.perm, P * 4), np.int32, (P,))
    cnt = np.bincount(idx.reshape(-1), minlength=E)
    assert np.array_equal(off, np.concatenate([[0], np.cumsum(cnt)]))
    for e in range(E):
        assert np.array_equal(perm[off[e]:off[e + 1]], np.nonzero((idx == e).any(axis=1))[0])
    re = gpu.host(gpu.view(ws, v.re, P * 4), np.int32, (T, topk))
    rpos = gpu.host(gpu.view(ws, v.rpos, P * 4), np.int32, (T, topk))
    assert np.array_equal(re, np.sort(idx, axis=1))
    assert all(perm[rpos[t, r]] == t and off[re[t, r]] <= rpos[t, r] < off[re[t, r] + 1] for t in range(T) for r in range(topk))
    hg = gpu.host(gpu.view(ws, v.h, P * I * 2), np.uint16, (P, I))
    hsh = gpu.host(gpu.view(ws, v.hsh, T * I * 2), np.uint16, (T, I)) if shared else None
    nh = nbad = 0
    worst_sum = 0.0
    ref_r, ref_s = np.empty((T, H), np.float32), np.empty((T, H), np.float32)
    for t in range(T):
        # (1) gate/up + SwiGLU. The e4m3 MFMA does not add its products in full f32 precision (test_mfma_fp8_accuracy:
        # ~2e-6 of sum|terms| on data like this), so g and u straddle a bf16 rounding far more often than the f32
        # sums of the decode path do (test_experts.cu:366-407 asks 99.5% there): most h equal, all within a few steps (a step each of g, silu g and u)
        o = orc.moe_prefill_fp8_row(hl, x[t], idx[t], w[t])
        ref_r[t], ref_s[t] = o["yr"], o["ys"]
        mine = [hg[rpos[t, r]] for r in range(topk)] + [hsh[t] if shared else np.zeros(I, np.uint16)]
        for r in range(topk + (1 if shared else 0)):
            nbad += int((mine[r] != o["h"][r]).sum())
            nh += I
            a, b = orc.bf16_to_f32(mine[r]).astype(np.float64), orc.bf16_to_f32(o["h"][r]).astype(np.float64)
            step = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(b), 2.0 ** -100))) - 7)
            assert np.all(np.abs(a - b) <= 4 * step + 5e-5), np.abs(a - b).max()  # (5e-5: values that are a difference of large terms)
        # (2) down + combine from the very h the GPU made: the GEMV tolerance of the reference (:352-361) and the bar
        o = orc.moe_prefill_fp8_row(hl, x[t], idx[t], w[t], h_in=np.stack(mine))
        worst, bad = helpers.check_sums(yr[t], o["yr64"], o["yrmag"])
        assert bad == 0, (t, worst)
        worst_sum = max(worst_sum, worst)
        helpers.check_outputs(yr[t], o["yr"], bf16_rel=False)  # (the MFMA's ~1e-5 relative error flips bf16 roundings too)
        if shared:
            worst, bad = helpers.check_sums(ys[t], o["ys64"], o["ysmag"])
            assert bad == 0, (t, worst)
            worst_sum = max(worst_sum, worst)
            helpers.check_outputs(ys[t], o["ys"], bf16_rel=False)
    assert nbad <= 0.05 * nh, (nbad, nh)
    print("fp8 prefill H=%d I=%d T=%d: h equal %.2f%%, staged |err|/sum|terms| %.2e, end-to-end rel-L2 routed %.2e%s, max-abs %.2e"
          % (H, I, T, 100 - 100.0 * nbad / nh, worst_sum, helpers.rel_l2(yr, ref_r),
             " shared %.2e" % helpers.rel_l2(ys, ref_s) if shared else "", np.abs(yr - ref_r).max()))
    # (3) end to end against the oracle's own h. A bf16 step of one h is, one time in ten or so, an e4m3 step of its
    # quantised value (6-12% of it), or of its whole block of 128 when it is the block's maximum: two correct
    # evaluations of this contract differ by about 1e-3 in relative L2 (measured here: 0.6e-3 to 1.4e-3). The bar of
    # 1e-3 / 2e-2 is held by (2), where both sides start from the same h; here the chunk stays within 3e-3 / 2e-2.
    assert helpers.rel_l2(yr, ref_r) <= 3e-3 and np.abs(yr - ref_r).max() <= 2e-2
    if shared:
        assert helpers.rel_l2(ys, ref_s) <= 3e-3 and np.abs(ys - ref_s).max() <= 2e-2


def test_prefill_rows_do_not_depend_on_the_chunk():
    """a row's result is the same bits whatever else is in the chunk (bucket positions differ)"""
    H, I, E, topk = 256, 256, 8, 2
    hl = helpers.make_layer(abi.FMT_FP8, H, I, E, topk, 5, seed=4, shared="fp8")
    x, _, idx, w = helpers.rows_and_routing(12, 200, H, E, topk, 1.0)
    yr, ys, _, _ = _prefill(hl, x, idx, w, 200)
    yr2, ys2, _, _ = _prefill(hl, x[50:60], idx[50:60], w[50:60], 10)
    assert np.array_equal(yr[50:60], yr2) and np.array_equal(ys[50:60], ys2)


def test_prefill_argument_errors():
    hl = helpers.make_layer(abi.FMT_BF16, 512, 256, 8, 2, 4, seed=1)
    dl = hl.upload()
    assert lib.prefill_ws_bytes(dl.w, 16) == 0
    with pytest.raises(lib.DsgxError):
        lib.moe_prefill(dl.w, gpu.empty(16), gpu.empty(16), gpu.empty(16), 16, gpu.empty(16), gpu.empty(16), gpu.empty(16))


# ---- bf16 activations (INT4 layers; FP8 layers with act_fp8 = 0): the decode contract row by row -----------------------
def _rows_are_decode_rows(fmt, H, I, E, topk, T, shared, seed, per_row=True, **kw):
    """a chunk row is a decode row (engine/experts/tests/test_prefill.inc:307-373): h and the outputs against the decode oracle.
    per_row: the benchmark's output bar (relative L2 1e-3, max-abs 2e-2) is applied to every row by itself; else to the
    chunk's output tensor as a whole (the FP8 test layers are random codes with a wide range of magnitudes: ONE h value
    that falls on the other side of a bf16 rounding, inside the range of valid f32 sums, moves a small row by 2e-3)."""
    hl = helpers.make_layer(fmt, H, I, E, topk, min(E, 5), seed=seed, shared=shared)
    x, _, idx, w = helpers.rows_and_routing(13, T, H, E, topk, 2.5)
    yr, ys, ws, dl = _prefill(hl, x, idx, w, T, **kw)
    v = lib.prefill_view(dl.w, ws, T)
    P = T * topk
    rpos = gpu.host(gpu.view(ws, v.rpos, P * 4), np.int32, (T, topk))
    re = gpu.host(gpu.view(ws, v.re, P * 4), np.int32, (T, topk))
    hg = gpu.host(gpu.view(ws, v.h, P * I * 2), np.uint16, (P, I))
    hsh = gpu.host(gpu.view(ws, v.hsh, T * I * 2), np.uint16, (T, I)) if shared else None
    assert np.array_equal(re, np.sort(idx, axis=1))
    exact = total = 0
    ref_yr, ref_ys = [], []
    for t in range(T):
        uni = orc.union(idx[t:t + 1], E)
        up = orc.moe_up(hl, x[t:t + 1], uni)
        mine = np.stack([hg[rpos[t, r]] for r in range(topk)] + ([hsh[t]] if shared else []))[:, None, :]
        hv = orc.bf16_to_f32(mine)
        assert np.all((hv >= up["lo"]) & (hv <= up["hi"])), "h outside the range of f32 sums"
        exact += int(((mine == up["h64"]) | ((hv == 0) & (orc.bf16_to_f32(up["h64"]) == 0))).sum())
        total += mine.size
        dn = orc.moe_down(hl, mine, idx[t:t + 1], w[t:t + 1], uni)
        worst, bad = helpers.check_sums(yr[t:t + 1], dn["yr64"], dn["yrmag"], 1e-4)
        assert bad == 0, worst
        full = orc.moe_down(hl, up["h32"], idx[t:t + 1], w[t:t + 1], uni)
        ref_yr.append(full["yr32"][0])
        if per_row:
            helpers.check_outputs(yr[t:t + 1], full["yr32"])
        if shared:
            worst, bad = helpers.check_sums(ys[t:t + 1], dn["ys64"], dn["ysmag"], 1e-4)
            assert bad == 0, worst
            ref_ys.append(full["ys32"][0])
            if per_row:
                helpers.check_outputs(ys[t:t + 1], full["ys32"])
    assert exact >= 0.995 * total, (exact, total)
    helpers.check_outputs(yr, np.stack(ref_yr))
    if shared:
        helpers.check_outputs(ys, np.stack(ref_ys))


@pytest.mark.parametrize("H,I,E,topk,T,shared", [(512, 256, 8, 2, 150, "bf16"), (256, 128, 16, 4, 37, None)])
def test_prefill_int4_against_oracle(H, I, E, topk, T, shared):
    _rows_are_decode_rows(abi.FMT_INT4, H, I, E, topk, T, shared, seed=6)


@pytest.mark.parametrize("H,I,E,topk,T,shared", [(512, 256, 8, 2, 150, "fp8"), (1024, 128, 16, 4, 37, None)])
def test_prefill_fp8_bf16_activations_against_oracle(H, I, E, topk, T, shared):
    """FP8 weights under the engine's own prefill contract (prefill.cu:337-352: bf16 activations, per 128-k block the sum
    from zero, then fma(S, sum, acc)): act_fp8 = 0"""
    _rows_are_decode_rows(abi.FMT_FP8, H, I, E, topk, T, shared, seed=8, per_row=False, act_fp8=False)
