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


def test_mfma_fp8_block_rule_live():
    """the oracle's statement of the e4m3 MFMA's block sum (pinned on the CPU by tests/golden/mfma_fp8_k128.npz) against the
    instruction itself on fresh operands: every bit"""
    rng = np.random.default_rng(2718)
    for sa, sb, dens in ((104, 160, 1.0), (30, 300, 1.0), (104, 160, 0.1), (None, None, 1.0), (None, None, 0.05)):
        if sa is None:
            qa, qb = rng.integers(0, 256, (16, 128)).astype(np.uint8), rng.integers(0, 256, (16, 128)).astype(np.uint8)
            qa[(qa & 0x7F) == 0x7F] = 0x21
            qb[(qb & 0x7F) == 0x7F] = 0xA2
        else:
            qa = orc.f32_to_e4m3(np.clip(rng.standard_normal((16, 128)) * sa, -448, 448).astype(np.float32))
            qb = orc.f32_to_e4m3(np.clip(rng.standard_normal((16, 128)) * sb, -448, 448).astype(np.float32))
        qa[rng.random((16, 128)) > dens] = 0
        raw = gpu.empty(64 * 16 * 4, 0xFF)
        lib.probe_mfma_fp8(gpu.dev(qa), gpu.dev(qb), raw, 1)
        raw = gpu.host(raw, np.float32, (64, 16))
        got = np.empty((16, 16), np.float32)
        for l in range(64):
            for r in range(4):
                got[4 * (l // 16) + r, l % 16] = raw[l, r]
        want = orc.mfma_fp8_k128(qa, qb)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), int((got != want).sum())


@pytest.fixture
def unit_rule():
    """the oracle adds a 128-k block's products by the matrix unit's rule (orc_mfma_fp8_k128) instead of sequentially"""
    orc.set_fp8_block_rule(1)
    yield
    orc.set_fp8_block_rule(0)


@pytest.mark.parametrize("H,I,E,topk,T,shared", [(512, 256, 16, 4, 70, "fp8"), (256, 384, 4, 2, 300, None), (1024, 128, 8, 8, 129, "fp8")])
def test_prefill_fp8_against_oracle(H, I, E, topk, T, shared, unit_rule):
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
    seq_r, seq_s = np.empty((T, H), np.float32), np.empty((T, H), np.float32)
    for t in range(T):
        # (1) gate/up + SwiGLU against the oracle that adds each 128-k block by the matrix unit's rule: the same sums, so h
        # differs only where the device's expf() and the host's round silu to different bf16 values (rare), by one step
        o = orc.moe_prefill_fp8_row(hl, x[t], idx[t], w[t])
        ref_r[t], ref_s[t] = o["yr"], o["ys"]
        mine = [hg[rpos[t, r]] for r in range(topk)] + [hsh[t] if shared else np.zeros(I, np.uint16)]
        for r in range(topk + (1 if shared else 0)):
            nbad += int((mine[r] != o["h"][r]).sum())
            nh += I
            a, b = orc.bf16_to_f32(mine[r]).astype(np.float64), orc.bf16_to_f32(o["h"][r]).astype(np.float64)
            step = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(b), 2.0 ** -100))) - 7)
            assert np.all(np.abs(a - b) <= step), np.abs(a - b).max()
        # (2) down + combine from the very h the GPU made: the GEMV tolerance of the reference (test_experts.cu:352-361)
        # against exact sums, and the f32 outputs bit for bit against the oracle's (same block sums, same order of adds)
        o = orc.moe_prefill_fp8_row(hl, x[t], idx[t], w[t], h_in=np.stack(mine))
        worst, bad = helpers.check_sums(yr[t], o["yr64"], o["yrmag"])
        assert bad == 0, (t, worst)
        worst_sum = max(worst_sum, worst)
        assert np.array_equal(yr[t].view(np.uint32), o["yr"].view(np.uint32)), (t, int((yr[t] != o["yr"]).sum()))
        if shared:
            worst, bad = helpers.check_sums(ys[t], o["ys64"], o["ysmag"])
            assert bad == 0, (t, worst)
            worst_sum = max(worst_sum, worst)
            assert np.array_equal(ys[t].view(np.uint32), o["ys"].view(np.uint32)), (t, int((ys[t] != o["ys"]).sum()))
        if t < 24:  # the contract with sequential f32 block sums (the reference's CPU stand-in), for the record below
            orc.set_fp8_block_rule(0)
            o0 = orc.moe_prefill_fp8_row(hl, x[t], idx[t], w[t])
            orc.set_fp8_block_rule(1)
            seq_r[t], seq_s[t] = o0["yr"], o0["ys"]
    assert nbad <= 0.002 * nh, (nbad, nh)
    print("fp8 prefill H=%d I=%d T=%d: h equal %.3f%%, staged |err|/sum|terms| %.2e, end-to-end rel-L2 routed %.2e%s, max-abs %.2e; "
          "against sequential f32 block sums (24 rows): rel-L2 routed %.2e"
          % (H, I, T, 100 - 100.0 * nbad / nh, worst_sum, helpers.rel_l2(yr, ref_r),
             " shared %.2e" % helpers.rel_l2(ys, ref_s) if shared else "", np.abs(yr - ref_r).max(), helpers.rel_l2(yr[:24], seq_r[:24])))
    # (3) end to end against the oracle's own h, the benchmark's bar: relative L2 1e-3, max-abs 2e-2, on the f32 outputs and
    # on their bf16 roundings
    helpers.check_outputs(yr, ref_r)
    if shared:
        helpers.check_outputs(ys, ref_s)
    # (4) the same chunk against the oracle with sequential f32 block sums: inside what evaluations whose sums differ by
    # 2e-6 of their sums of |terms| differ by (tests/test_oracle_moe.py records that spread at the benchmark's shape)
    assert helpers.rel_l2(yr[:24], seq_r[:24]) <= 6e-3
    if shared:
        assert helpers.rel_l2(ys[:24], seq_s[:24]) <= 6e-3


def test_prefill_rows_do_not_depend_on_the_chunk():
    """a row's result is the same bits whatever else is in the chunk (bucket positions differ)"""
    H, I, E, topk = 256, 256, 8, 2
    hl = helpers.make_layer(abi.FMT_FP8, H, I, E, topk, 5, seed=4, shared="fp8")
    x, _, idx, w = helpers.rows_and_routing(12, 200, H, E, topk, 1.0)
    yr, ys, _, _ = _prefill(hl, x, idx, w, 200)
    yr2, ys2, _, _ = _prefill(hl, x[50:60], idx[50:60], w[50:60], 10)
    assert np.array_equal(yr[50:60], yr2) and np.array_equal(ys[50:60], ys2)


def test_prefill_tile_order_does_not_change_a_bit():
    """dsgx_prefill_cfg::tile_order (the reference's prefill_tuning tord, ds41f engine/kernels/dsk.h:252) only changes which
    workgroup takes which tile: experts of 0, a few, 128, 129, 256 and several hundred rows (remainders, 256-position
    tiles and both), every order, the same yr, ys and workspace views as the order by expert id"""
    H, I, E, topk, T = 256, 256, 12, 2, 900
    hl = helpers.make_layer(abi.FMT_FP8, H, I, E, topk, 5, seed=9, shared="fp8")
    x, _, _, w = helpers.rows_and_routing(21, T, H, E, topk, 1.0)
    # rows an expert: 0, 1, 17, 128, 129, 256, 257, 300, 421, ... (pairs (a, b), a < b, dealt so that the counts come out)
    want = [0, 1, 17, 128, 129, 256, 257, 300, 421, 291, 0, 0]
    want[10] = (2 * T - sum(want)) // 2
    want[11] = 2 * T - sum(want)
    left = list(want)
    idx = np.zeros((T, topk), np.int32)
    for t in range(T):
        a = int(np.argmax(left))
        left[a] -= 1
        b = int(np.argmax([v if j != a else -1 for j, v in enumerate(left)]))
        left[b] -= 1
        idx[t] = (a, b)
    assert min(left) == 0 and max(left) == 0 and (idx[:, 0] != idx[:, 1]).all()
    ref = None
    for order in (0, 1, 2, -1):
        yr, ys, ws, dl = _prefill(hl, x, idx, w, T, tile_order=order)
        got = (yr.view(np.uint32), ys.view(np.uint32))
        if ref is None:
            ref = got
            assert np.isfinite(yr).all() and np.isfinite(ys).all() and np.abs(yr).max() > 0
        assert np.array_equal(ref[0], got[0]) and np.array_equal(ref[1], got[1]), order
    with pytest.raises(lib.DsgxError):
        _prefill(hl, x, idx, w, T, tile_order=3)


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


def test_prefill_int4_lds_staged_kernels_give_the_register_ring_kernels_bits():
    """the INT4 experts' grouped GEMMs (pf_gemm_i4.cuh: both operands staged in LDS by DMA, weights decoded a turn ahead) add
    in the k order of the kernel they replaced (k_pf_gemm16: register ring, kept behind DSGX_PF_I4_OLD=1): yr, ys and h equal
    bit for bit, on a chunk with full and ragged tiles"""
    import os
    H, I, E, topk, T = 512, 256, 4, 2, 300
    hl = helpers.make_layer(abi.FMT_INT4, H, I, E, topk, 4, seed=9, shared="bf16")
    x, _, idx, w = helpers.rows_and_routing(17, T, H, E, topk, 2.5)
    outs = []
    for old in ("0", "1"):
        os.environ["DSGX_PF_I4_OLD"] = old
        try:
            yr, ys, ws, dl = _prefill(hl, x, idx, w, T)
            v = lib.prefill_view(dl.w, ws, T)
            outs.append((yr.view(np.uint32), ys.view(np.uint32), gpu.host(gpu.view(ws, v.h, T * topk * I * 2), np.uint16, (-1,))))
        finally:
            os.environ.pop("DSGX_PF_I4_OLD", None)
    for a, b in zip(*outs):
        assert np.array_equal(a, b)


@pytest.mark.parametrize("H,I,E,topk,T,shared", [(512, 256, 8, 2, 150, "fp8"), (1024, 128, 16, 4, 37, None)])
def test_prefill_fp8_bf16_activations_against_oracle(H, I, E, topk, T, shared):
    """FP8 weights under the engine's own prefill contract (prefill.cu:337-352: bf16 activations, per 128-k block the sum
    from zero, then fma(S, sum, acc)): act_fp8 = 0"""
    _rows_are_decode_rows(abi.FMT_FP8, H, I, E, topk, T, shared, seed=8, per_row=False, act_fp8=False)


@pytest.mark.parametrize("fmt,H,I,E,topk,T,shared,kw", [
    (abi.FMT_INT4, 512, 256, 8, 2, 150, "bf16", {}),
    (abi.FMT_INT4, 256, 384, 4, 4, 300, None, {}),
    (abi.FMT_FP8, 512, 256, 8, 2, 150, "fp8", dict(act_fp8=False)),
    (abi.FMT_FP8, 1024, 128, 16, 4, 37, None, dict(act_fp8=False)),
])
def test_prefill_bf16_activations_every_bit_against_the_matrix_unit_oracle(fmt, H, I, E, topk, T, shared, kw):
    """with the bf16 MFMA's order of adds restated in the oracle (pinned on the CPU by tests/golden/mfma_bf16_k32.npz) the
    bf16-activation prefill is checked bit for bit: h of every pick and of the shared expert, yr, ys, on chunks with full
    and ragged tiles (INT4 experts: pf_gemm_i4.cuh; the BF16 and FP8 matrices: k_pf_gemm16)"""
    hl = helpers.make_layer(fmt, H, I, E, topk, min(E, 5), seed=21, shared=shared)
    x, _, idx, w = helpers.rows_and_routing(29, T, H, E, topk, 2.5)
    yr, ys, ws, dl = _prefill(hl, x, idx, w, T, **kw)
    v = lib.prefill_view(dl.w, ws, T)
    P = T * topk
    rpos = gpu.host(gpu.view(ws, v.rpos, P * 4), np.int32, (T, topk))
    hg = gpu.host(gpu.view(ws, v.h, P * I * 2), np.uint16, (P, I))
    hsh = gpu.host(gpu.view(ws, v.hsh, T * I * 2), np.uint16, (T, I)) if shared else None
    rows = list(range(T)) if T <= 40 else sorted(set(np.random.default_rng(1).integers(0, T, 24).tolist()) | {0, T - 1})
    for t in rows:
        o = orc.moe_prefill_b16_row_mfma(hl, x[t], idx[t], w[t])
        mine = np.stack([hg[rpos[t, r]] for r in range(topk)] + ([hsh[t]] if shared else []))
        assert np.array_equal(mine, o["h"]), (t, int((mine != o["h"]).sum()))
        assert np.array_equal(yr[t].view(np.uint32), o["yr"].view(np.uint32)), (t, int((yr[t] != o["yr"]).sum()))
        if shared:
            assert np.array_equal(ys[t].view(np.uint32), o["ys"].view(np.uint32)), (t, int((ys[t] != o["ys"]).sum()))
