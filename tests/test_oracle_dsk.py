"""Pins of the oracle's DeepSeek MXFP4 x FP8 expert (oracle/oracle.cpp: orc_e2m1_value, orc_ue8m0_value, orc_act_scale_byte,
orc_act_quant_ue8m0, orc_mxfp4_dequant, orc_fp8e_dequant, orc_dsk_up, orc_dsk_down): the codecs against closed forms, the
scale byte against exact rational arithmetic, the expert against vectors computed by the reference's own torch kernels
(tests/golden/dsk_mxfp4_expert.npz, written by tests/golden/make_dsk_mxfp4_vectors.py), with negative controls."""
import os
from fractions import Fraction

import numpy as np

from tests import orc

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "dsk_mxfp4_expert.npz")


def test_e2m1_and_ue8m0_codecs():
    # OCP MX e2m1: sign, 2 exponent bits (bias 1), 1 mantissa bit; exponent 0 is subnormal (0, 0.5)
    want = []
    for c in range(16):
        s, e, m = c >> 3, (c >> 1) & 3, c & 1
        mag = m * 0.5 if e == 0 else (1 + m * 0.5) * 2.0 ** (e - 1)
        want.append(-mag if s else mag)
    got = orc.e2m1_table()
    assert np.array_equal(got, np.array(want, np.float32)) and np.signbit(got[8])
    for b in (1, 2, 100, 127, 128, 200, 254):
        assert orc.ue8m0_value(b) == np.ldexp(np.float32(1), b - 127)


def test_act_scale_byte_is_the_smallest_power_of_two_that_covers():
    """e = the smallest integer with 2^(e-127) >= v, v = f32(max(amax, 1e-4) * f32(1/448)): exact rational comparison"""
    rng = np.random.default_rng(5)
    r448 = np.float32(1.0) / np.float32(448.0)
    amaxes = list(np.exp(rng.uniform(np.log(1e-6), np.log(1e6), 4000)).astype(np.float32))
    for k in range(-20, 20):  # around the points where v crosses a power of two
        a = np.float32(448.0 * 2.0 ** k)
        amaxes += [a, np.nextafter(a, np.float32(0)), np.nextafter(a, np.float32(1e30))]
    for a in amaxes:
        v = np.float32(max(a, np.float32(1e-4))) * r448
        e = orc.act_scale_byte(float(a))
        fv = Fraction(float(v))
        assert Fraction(2) ** (e - 127) >= fv and Fraction(2) ** (e - 128) < fv, (a, e)


def test_act_quant_ue8m0_and_dequant_against_the_reference_vectors():
    g = np.load(GOLD)
    q, s = orc.act_quant_ue8m0(g["x"])
    assert np.array_equal(orc.dequant_act_ue8m0(q, s), g["x_deq"])
    assert np.array_equal(np.array([[orc.ue8m0_value(b) for b in row] for row in s], np.float32), g["x_scale"])
    # every dequantised activation is a bf16 value (what the GPU path relies on)
    d = orc.dequant_act_ue8m0(q, s)
    assert np.array_equal(orc.bf16_to_f32(orc.f32_to_bf16(d)), d)


def _steps(a, b):
    """difference of two bf16 bit arrays in units of the larger value's bf16 step"""
    fa, fb = orc.bf16_to_f32(a).astype(np.float64), orc.bf16_to_f32(b).astype(np.float64)
    step = 2.0 ** (np.floor(np.log2(np.maximum(np.maximum(np.abs(fa), np.abs(fb)), 2.0 ** -120))) - 7)
    return np.abs(fa - fb) / step


def test_expert_against_the_reference_vectors():
    """h (before its quantisation) and the expert's bf16 output against the reference's: equal in nearly all bits, never
    more than a few bf16 steps apart (torch sums the products in another order; a gate or up that rounds the other way
    moves h by a step or two). Controls: the nibbles swapped, the routing weight applied after w2, no clamp."""
    g = np.load(GOLD)
    xd = g["x_deq"]
    for kind in ("routed", "shared"):
        if kind == "routed":
            w1, w3, w2 = (orc.mxfp4_dequant(g["r%d_w" % i], g["r%d_s" % i]) for i in (1, 3, 2))
            rw = g["rw"]
        else:
            w1, w3, w2 = (orc.fp8e_dequant(g["s%d_w" % i], g["s%d_s" % i]) for i in (1, 3, 2))
            rw = None
        # the dequantised weights are bf16 values too
        assert all(np.array_equal(orc.bf16_to_f32(orc.f32_to_bf16(w)), w) for w in (w1, w3, w2))
        up = orc.dsk_up(w1, w3, xd, rw)
        href = g["h_" + kind]
        st = _steps(up["h32"], href)
        assert (up["h32"] == href).mean() >= 0.97 and st.max() <= 4, ((up["h32"] == href).mean(), st.max())
        hf = orc.bf16_to_f32(href)
        assert np.all(hf >= up["lo"] - 1e-30) and np.all(hf <= up["hi"] + 1e-30)
        # w2 from the reference's own h: the bf16 outputs
        dn = orc.dsk_down(w2, href)
        yref = g["y_" + kind]
        sty = _steps(dn["outb"], yref)
        assert (dn["outb"] == yref).mean() >= 0.98 and sty.max() <= 1.01, ((dn["outb"] == yref).mean(), sty.max())
        err = np.abs(orc.bf16_to_f32(yref).astype(np.float64) - dn["out64"])
        assert np.all(err <= 1e-4 * dn["mag"] + np.abs(dn["out64"]) * 2.0 ** -8)
        if kind == "routed":
            # controls
            swapped = ((g["r1_w"] >> 4) | (g["r1_w"] << 4)).astype(np.uint8)
            bad = orc.dsk_up(orc.mxfp4_dequant(swapped, g["r1_s"]), w3, xd, rw, want_range=False)
            assert (bad["h32"] == href).mean() < 0.2
            late = orc.dsk_up(w1, w3, xd, None, want_range=False)  # no weight before w2 ...
            dl = orc.dsk_down(w2, late["h32"])
            y_late = orc.f32_to_bf16(dl["out32"] * rw[:, None])     # ... but after it
            assert (y_late == yref).mean() < 0.9
            noclamp = orc.dsk_up(w1, w3, xd, rw, limit=1e30, want_range=False)
            assert np.any(noclamp["h32"] != up["h32"])


def test_matrix_unit_variant_stays_inside_the_contract():
    """orc_dsk_up_mx / orc_dsk_down_mx (every dot product added as gfx950's block-scaled MFMA adds it; the rule itself is pinned
    by tests/golden/mfma_scaled_k128.npz) against orc_dsk_up / orc_dsk_down (pinned above by the reference's vectors): h inside
    the range of the reference's sum tolerance and mostly equal, outputs within one bf16 step; the shared expert's form too"""
    rng = np.random.default_rng(9)
    H, I, M = 512, 256, 3
    x = orc.normal_bf16(9, 1, (M, H), 1.5)
    xq, xs = orc.act_quant_ue8m0(x)
    xd = orc.dequant_act_ue8m0(xq, xs)
    rw = np.array([0.3, 1.1, 0.7], np.float32)

    def fp4(N, K, lo, hi):
        codes = rng.integers(0, 16, (N, K), dtype=np.uint8)
        return (codes[:, 0::2] | (codes[:, 1::2] << 4)).astype(np.uint8), rng.integers(lo, hi, (N, K // 32), dtype=np.uint8)

    def fp8(N, K, lo, hi):
        return orc.f32_to_e4m3(np.clip(rng.standard_normal((N, K)).astype(np.float32) * 40.0, -448, 448)), rng.integers(lo, hi, (N // 32, K // 32), dtype=np.uint8)
    for f4, mk, deq, r in ((1, fp4, orc.mxfp4_dequant, rw), (0, fp8, orc.fp8e_dequant, None)):
        (w1, s1), (w3, s3), (w2, s2) = mk(I, H, 116, 121), mk(I, H, 116, 121), mk(H, I, 118, 123)
        up = orc.dsk_up(deq(w1, s1), deq(w3, s3), xd, r, sum_tol=1e-4)
        hm = orc.dsk_up_mx(w1, s1, w3, s3, f4, xq, xs, r)
        hf = orc.bf16_to_f32(hm)
        assert np.all(hf >= up["lo"]) and np.all(hf <= up["hi"])
        assert (hm == up["h32"]).mean() >= 0.97, (hm == up["h32"]).mean()
        dn = orc.dsk_down(deq(w2, s2), hm)
        dm = orc.dsk_down_mx(w2, s2, f4, hm)
        assert np.array_equal(dm["hq"], dn["hq"]) and np.array_equal(dm["hs"], dn["hs"])
        err = np.abs(orc.bf16_to_f32(dm["outb"]).astype(np.float64) - dn["out64"])
        assert np.all(err <= 1e-4 * dn["mag"] + np.abs(dn["out64"]) * 2.0 ** -8)
        assert (dm["outb"] == dn["outb"]).mean() >= 0.97
