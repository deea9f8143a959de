"""GPU parity of the dense GEMV (dsgx_gemv = glm::gemv of the reference) against the CPU oracle: the two dense
configurations of the benchmark (FP8 [2048 x 4096], INT4 [1536 x 6144], rows 1, 2, 4, 6), one-hot rows (exact weights),
every row count, every output kind, partial last segments and several segments a launch.

Tolerances: bf16 outputs max-abs-err <= 2e-2 and relative L2 <= 1e-3 against the f32-accumulated oracle, and the
reference's own rule |err| <= 1e-4 * sum|terms| against f64 (altar1-4xgx10-switchless/engine/experts/tests/
test_experts.cu:352-361, micro/gemv.cu:1170)."""
import numpy as np
import pytest

from dsgx10_amd import abi, lib
from tests import gpu, orc
from tests.helpers import check_sums, quant_fp8, quant_int4, rel_l2

pytestmark = pytest.mark.gpu


def _run(x16, fmt, parts, N, K, out_kind, rows=None, ldx=None, splitk=1):
    M = x16.shape[0] if rows is None else rows
    ldx = ldx or x16.shape[1]
    ncol = N // 2 if out_kind == abi.OUT_SWIGLU else N
    esz = 4 if out_kind == abi.OUT_F32 else 2
    y = gpu.empty(M * ncol * esz, 0xFF)
    keep = [gpu.dev(p) for p in parts]
    seg = dict(fmt=fmt, w=keep[0], s=keep[1] if len(keep) > 1 else None, zp=keep[2] if len(keep) > 2 else None, n=N, y=y, ldy=ncol)
    lib.gemv(gpu.dev(x16), ldx, M, K, [seg], out_kind, splitk=splitk)
    return gpu.host(y, np.float32 if out_kind == abi.OUT_F32 else np.uint16, (M, ncol))


def _oracle(x16, fmt, parts, N, K, out_kind):
    p = list(parts) + [None] * (3 - len(parts))
    return orc.gemv(x16, fmt, p[0], p[1], p[2], N, K, out_kind)


def _check_bf16(got16, o):
    got = orc.bf16_to_f32(got16)
    ref = orc.bf16_to_f32(o["y16"])
    # 2e-2, or one bf16 step where the value is large enough for a step to exceed it
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(ref), 2.0 ** -126))) - 7)
    assert np.all(np.abs(got - ref) <= np.maximum(2e-2, ulp))
    assert rel_l2(got, ref) <= 1e-3
    # within one bf16 step of the f64 result wherever the f32 sum is not at a rounding boundary
    worst, bad = check_sums(got, o["yd"], o["ymag"] + np.abs(o["yd"]) * 2.0 ** -8 / 1e-4, 1e-4)
    assert bad == 0, worst


def test_config1_dense_fp8_gemv():
    """x [1 x 4096] bf16 ~ N(0,1); W [2048 x 4096] ~ N(0, 0.02) -> e4m3 + f32 scale per 128 x 128; seed 0"""
    N, K = 2048, 4096
    x = orc.normal_bf16(0, 1, (1, K), 1.0)
    parts = quant_fp8(0, 2, N, K)
    o = _oracle(x, abi.FMT_FP8, parts, N, K, abi.OUT_BF16)
    _check_bf16(_run(x, abi.FMT_FP8, parts, N, K, abi.OUT_BF16), o)
    yf = _run(x, abi.FMT_FP8, parts, N, K, abi.OUT_F32)
    worst, bad = check_sums(yf, o["yd"], o["ymag"], 1e-4)
    assert bad == 0, worst
    assert worst < 2e-6  # f32 accumulation: far inside the reference's bar


@pytest.mark.parametrize("M", [1, 2, 4, 6])
def test_config2_dense_int4_gemv(M):
    """W [1536 x 6144] ~ N(0, 0.02), symmetric int4 g32 (u_z = 8), bf16 scales; x [M x 6144]"""
    N, K = 1536, 6144
    x = orc.normal_bf16(0, 1, (M, K), 1.0)
    parts = quant_int4(0, 3, N, K)
    o = _oracle(x, abi.FMT_INT4, parts, N, K, abi.OUT_BF16)
    _check_bf16(_run(x, abi.FMT_INT4, parts, N, K, abi.OUT_BF16), o)
    yf = _run(x, abi.FMT_INT4, parts, N, K, abi.OUT_F32)
    worst, bad = check_sums(yf, o["yd"], o["ymag"], 1e-4)
    assert bad == 0 and worst < 2e-6, worst
    # the same outputs as the BF16 GEMV over the dequantised matrix (same decode, same order): bit for bit
    wb = orc.int4_dequant(*parts)
    yb = _run(x, abi.FMT_BF16, (wb,), N, K, abi.OUT_F32)
    assert rel_l2(yf, yb) < 1e-6


@pytest.mark.parametrize("fmt", [abi.FMT_FP8, abi.FMT_INT4, abi.FMT_BF16])
def test_one_hot_rows_give_exact_weights(fmt):
    N, K = 64, 4096
    ks = [0, 15, 16, 31, 1023, 1024, 2047, 2048, 4095]
    x = np.zeros((8, K), np.uint16)
    for r, k in enumerate(ks[:8]):
        x[r, k] = 0x3F80
    parts = {abi.FMT_FP8: lambda: orc.fp8_random(7, N, K, 1.0 / 256), abi.FMT_INT4: lambda: orc.int4_random(8, N, K),
             abi.FMT_BF16: lambda: (orc.normal_bf16(0, 4, (N, K), 0.02),)}[fmt]()
    yf = _run(x, fmt, parts, N, K, abi.OUT_F32)
    o = _oracle(x, fmt, parts, N, K, abi.OUT_F32)
    assert np.array_equal(yf.view(np.uint32), o["yf"].view(np.uint32))  # a single non-zero term: no order, exact


@pytest.mark.parametrize("fmt", [abi.FMT_FP8, abi.FMT_INT4, abi.FMT_BF16])
@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 6, 7, 8, 9, 16])
def test_every_row_count(fmt, M):
    N, K = 256, 2048
    x = orc.normal_bf16(M, 1, (M, K), 1.0)
    parts = {abi.FMT_FP8: lambda: quant_fp8(1, 2, N, K), abi.FMT_INT4: lambda: orc.int4_random(9, N, K),
             abi.FMT_BF16: lambda: (orc.normal_bf16(0, 4, (N, K), 0.02),)}[fmt]()
    o = _oracle(x, fmt, parts, N, K, abi.OUT_F32)
    yf = _run(x, fmt, parts, N, K, abi.OUT_F32)
    worst, bad = check_sums(yf, o["yd"], o["ymag"], 1e-4)
    assert bad == 0 and worst < 2e-6, worst
    # batch invariance: row 0 alone gives the same bits as row 0 in the batch
    y0 = _run(x[:1], fmt, parts, N, K, abi.OUT_F32)
    assert np.array_equal(y0[0].view(np.uint32), yf[0].view(np.uint32))


def test_swiglu_output_and_bf16_rounding():
    N, K, M = 512, 1024, 3     # rows interleaved gate/up
    x = orc.normal_bf16(2, 1, (M, K), 1.0)
    for fmt, parts in [(abi.FMT_BF16, (orc.normal_bf16(0, 4, (N, K), 0.02),)), (abi.FMT_INT4, orc.int4_random(10, N, K))]:
        o = _oracle(x, fmt, parts, N, K, abi.OUT_SWIGLU)
        got = _run(x, fmt, parts, N, K, abi.OUT_SWIGLU)
        g, r = orc.bf16_to_f32(got), orc.bf16_to_f32(o["y16"])
        assert (got != o["y16"]).mean() < 0.02 and np.abs(g - r).max() <= 2e-2 and rel_l2(g, r) <= 2e-3


def test_partial_segments_strides_and_two_segments():
    # K that is not a whole number of 1024 / 2048 / 512-k segments, ldx > K, two segments of different rows
    M = 2
    for fmt, K in [(abi.FMT_FP8, 1536), (abi.FMT_FP8, 128), (abi.FMT_INT4, 2560), (abi.FMT_INT4, 32), (abi.FMT_BF16, 320)]:
        N1, N2, ldx = 40, 24, K + 64
        xfull = orc.normal_bf16(5, 1, (M, ldx), 1.0)
        mk = {abi.FMT_FP8: lambda n, t: quant_fp8(2, t, n, K), abi.FMT_INT4: lambda n, t: orc.int4_random(t, n, K),
              abi.FMT_BF16: lambda n, t: (orc.normal_bf16(0, t, (n, K), 0.02),)}[fmt]
        p1, p2 = mk(N1, 31), mk(N2, 32)
        y1, y2 = gpu.empty(M * N1 * 4, 0xFF), gpu.empty(M * 100 * 4, 0xFF)
        keep = [[gpu.dev(a) for a in p] for p in (p1, p2)]
        segs = []
        for k, n, y, ldy in ((keep[0], N1, y1, N1), (keep[1], N2, y2, 100)):
            segs.append(dict(fmt=fmt, w=k[0], s=k[1] if len(k) > 1 else None, zp=k[2] if len(k) > 2 else None, n=n, y=y, ldy=ldy))
        lib.gemv(gpu.dev(xfull), ldx, M, K, segs, abi.OUT_F32)
        xk = np.ascontiguousarray(xfull[:, :K])
        for p, n, y, ldy in ((p1, N1, y1, N1), (p2, N2, y2, 100)):
            o = _oracle(xk, fmt, p, n, K, abi.OUT_F32)
            got = gpu.host(y, np.float32, (M, ldy))[:, :n]
            worst, bad = check_sums(got, o["yd"], o["ymag"], 1e-4)
            assert bad == 0 and worst < 2e-6, (fmt, K, worst)


@pytest.mark.parametrize("sk", [2, 4])
@pytest.mark.parametrize("case", ["router168", "router256", "fp8_cfg1", "int4_cfg2", "int4_tail", "swiglu"])
def test_split_k(case, sk):
    """K over 2 or 4 waves of a workgroup, the slices added in slice order (the reference's router GEMV: split 4, f32 out,
    altar1-4xgx10-switchless/engine/model/model.cu:309-312). Same bars as the unsplit kernel; the order of adds differs,
    so bits may."""
    fmt, N, K, M, kind = {
        "router168": (abi.FMT_BF16, 168, 6144, 4, abi.OUT_F32),
        "router256": (abi.FMT_BF16, 256, 4096, 1, abi.OUT_F32),
        "fp8_cfg1": (abi.FMT_FP8, 2048, 4096, 1, abi.OUT_BF16),
        "int4_cfg2": (abi.FMT_INT4, 1536, 6144, 6, abi.OUT_BF16),
        "int4_tail": (abi.FMT_INT4, 72, 1280, 3, abi.OUT_F32),  # a partial last segment, fewer segments than slices
        "swiglu": (abi.FMT_BF16, 512, 2048, 2, abi.OUT_SWIGLU),
    }[case]
    x = orc.normal_bf16(11, 1, (M, K), 1.0)
    if fmt == abi.FMT_FP8:
        parts = quant_fp8(11, 2, N, K)
    elif fmt == abi.FMT_INT4:
        parts = quant_int4(11, 2, N, K)
    else:
        parts = (orc.normal_bf16(11, 2, (N, K), 0.05),)
    o = _oracle(x, fmt, parts, N, K, kind)
    got = _run(x, fmt, parts, N, K, kind, splitk=sk)
    if kind == abi.OUT_F32:
        worst, bad = check_sums(got, o["yd"], o["ymag"], 1e-4)
        assert bad == 0 and worst < 2e-6, worst
    elif kind == abi.OUT_BF16:
        _check_bf16(got, o)
    else:
        one = _run(x, fmt, parts, N, K, kind)
        assert (got == one).mean() >= 0.99
        assert np.abs(orc.bf16_to_f32(got) - orc.bf16_to_f32(o["y16"])).max() <= 2e-2


@pytest.mark.parametrize("sk", [1, 2, 4])
@pytest.mark.parametrize("case", ["router168", "fp8_cfg1", "int4_cfg2", "int4_tail", "swiglu"])
def test_gemv_every_bit_against_the_oracle(case, sk):
    """with v_dot2_f32_bf16's rule (pinned on the CPU by tests/golden/dot2_bf16.npz), the lanes' split of K, the wave's tree
    and the split-K order restated in the oracle (orc.set_dot_rule(4, splitk)) the dense GEMV is checked bit for bit:
    f32 sums, bf16 outputs, SwiGLU outputs, a partial last segment"""
    fmt, N, K, M, kind = {
        "router168": (abi.FMT_BF16, 168, 6144, 4, abi.OUT_F32),
        "fp8_cfg1": (abi.FMT_FP8, 2048, 4096, 1, abi.OUT_BF16),
        "int4_cfg2": (abi.FMT_INT4, 1536, 6144, 6, abi.OUT_BF16),
        "int4_tail": (abi.FMT_INT4, 72, 1280, 3, abi.OUT_F32),
        "swiglu": (abi.FMT_BF16, 512, 2048, 2, abi.OUT_SWIGLU),
    }[case]
    x = orc.normal_bf16(13, 1, (M, K), 1.0)
    if fmt == abi.FMT_FP8:
        parts = quant_fp8(13, 2, N, K)
    elif fmt == abi.FMT_INT4:
        parts = quant_int4(13, 2, N, K)
    else:
        parts = (orc.normal_bf16(13, 2, (N, K), 0.05),)
    got = _run(x, fmt, parts, N, K, kind, splitk=sk)
    orc.set_dot_rule(4, sk)
    try:
        o = _oracle(x, fmt, parts, N, K, kind)
    finally:
        orc.set_dot_rule(0)
    want = o["yf"] if kind == abi.OUT_F32 else o["y16"]
    assert np.array_equal(got.view(np.uint32 if kind == abi.OUT_F32 else np.uint16), want.view(np.uint32 if kind == abi.OUT_F32 else np.uint16)), int((got != want).sum())


@pytest.mark.parametrize("H", [2048, 4096, 6144])
@pytest.mark.parametrize("mode", ["contract", "round2", "two_partials"])
def test_add_norm(H, mode):
    """The residual add and RMSNorm after the expert step (glmcoll.h:34-62 at one rank, prep.cu:12-66): h bit for bit,
    xn within one bf16 step of the oracle's (f64 statistics) on at most 0.1% of the values, equal elsewhere."""
    M = 5
    part = orc.normal_f32(12, 1, (M, H), 0.7)
    part2 = orc.normal_f32(12, 2, (M, H), 0.3) if mode == "two_partials" else None
    res, w = orc.normal_bf16(12, 3, (M, H), 1.5), orc.normal_bf16(12, 4, (H,), 1.0)
    ro, xn = gpu.empty(M * H * 2, 0xFF), gpu.empty(M * H * 2, 0xFF)
    lib.add_norm(gpu.dev(part), None if part2 is None else gpu.dev(part2), M, H, gpu.dev(res), ro, gpu.dev(w), 1e-5, xn,
                 round2=mode == "round2")
    o_ro, o_xn, o_xn32 = orc.add_norm(part, part2, res, w, 1e-5, round2=mode == "round2")
    assert np.array_equal(gpu.host(ro, np.uint16, (M, H)), o_ro)
    xn = gpu.host(xn, np.uint16, (M, H))
    for ref in (o_xn, o_xn32):
        assert (xn == ref).mean() >= 0.999 and np.abs(xn.astype(np.int32) - ref.astype(np.int32)).max() <= 1
    # in place, and the residual alone
    r2 = gpu.dev(res)
    lib.add_norm(gpu.dev(part), None if part2 is None else gpu.dev(part2), M, H, r2, r2, None, 1e-5, None, round2=mode == "round2")
    assert np.array_equal(gpu.host(r2, np.uint16, (M, H)), o_ro)
