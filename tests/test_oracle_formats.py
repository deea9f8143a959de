"""Pins the oracle's INT4-g32 and FP8-128x128 readers, dequantisers and quantisers.

INT4: the contract W = bf16_rne((u - u_z) s) is checked on the whole domain (every finite bf16 scale x every (u, u_z))
against compressed-tensors' own expression evaluated with torch's bf16 arithmetic, (q.to(bf16) - z.to(bf16)) * s
(reference: altar1-4xgx10-switchless/docs/model.md:166-195), and against the reference's known answers
(engine/weights/int4_pack.py:301-305). The nibble and zero-point bit order is checked on hand-made words
(docs/model.md:111-114,136-139). FP8: the quantiser is checked against the reference's formula evaluated with torch
primitives (engine/attn/tools/pack.py:216-232), the cast being torch's own."""
import numpy as np
import torch

from tests import orc


def test_int4_known_answers():
    L = orc.lib()
    assert L.orc_int4_value_bits(15, 0, 0x3F81) == 0x4172   # int4_pack.py:301-305
    assert L.orc_int4_value_bits(0, 0, 0x3F81) == 0x0000
    assert L.orc_int4_value_bits(8, 8, 0x3F81) == 0x0000
    assert L.orc_int4_value_bits(7, 8, 0x3F80) == 0xBF80    # -1


def test_int4_contract_whole_domain():
    """16,711,680 cases: equal to torch's bf16 arithmetic (the library's expression) and to one RNE of the exact product."""
    sb = np.arange(0x10000, dtype=np.uint32)
    sb = sb[((sb & 0x7F80) != 0x7F80)].astype(np.uint16)            # every finite bf16, both signs: 65,280
    assert sb.size == 65280
    s_t = torch.from_numpy(sb.view(np.int16).copy()).view(torch.bfloat16)
    inexact = 0
    for uz in range(16):
        # a matrix [65280 rows? no: rows = scales] x 32 columns: u = column % 16 (two copies), one group a row
        N = sb.size
        Np = (N + 7) // 8 * 8
        u = np.tile(np.arange(16, dtype=np.uint32), 2)
        words = np.zeros(4, np.uint32)
        for i in range(32):
            words[i // 8] |= u[i] << np.uint32(4 * (i % 8))
        packed = np.tile(words, (Np, 1))
        scale = np.zeros((Np, 1), np.uint16)
        scale[:N, 0] = sb
        zp = np.full((Np // 8, 1), uz * 0x11111111, np.uint32)
        got = orc.int4_dequant(packed, scale, zp)[:N]
        q = torch.tensor(u.astype(np.int64) - 8, dtype=torch.int8)
        z = torch.tensor(uz - 8, dtype=torch.int8)
        want_t = (q.to(torch.bfloat16) - z.to(torch.bfloat16))[None, :] * s_t[:, None]
        want = want_t.view(torch.int16).numpy().view(np.uint16)
        nan = torch.isnan(want_t).numpy()
        assert np.array_equal(got[~nan], want[~nan]), uz
        # one rounding of the exact product (f64 holds it exactly)
        exact = (u.astype(np.float64) - uz)[None, :] * orc.bf16_to_f32(sb).astype(np.float64)[:, None]
        with np.errstate(over="ignore"):
            rne = torch.from_numpy(exact.astype(np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
        with np.errstate(over="ignore"):
            fin = np.isfinite(exact.astype(np.float32)) & ~nan
        assert np.array_equal(got[fin], rne[fin])
        inexact += int((orc.bf16_to_f32(got[fin]).astype(np.float64) != exact[fin]).sum())
    assert inexact > 0.3 * 65280 * 256 * 2 * 0.9  # the rounding is real (about 43 % of the products are inexact)


def test_int4_bit_order():
    # value k of a row is nibble k % 8 (lowest first) of word k / 8; row n's zero point is nibble n % 8 of word n / 8
    N, K = 8, 32
    packed = np.zeros((N, K // 8), np.uint32)
    packed[:, 0] = 0x76543210
    packed[:, 1] = 0xFEDCBA98
    packed[:, 2] = 0x00000008
    packed[:, 3] = 0x80000000
    scale = np.full((N, 1), 0x3F80, np.uint16)  # 1.0
    zp = np.array([[0x76543210]], np.uint32)    # row n has u_z = n
    w = orc.bf16_to_f32(orc.int4_dequant(packed, scale, zp))
    u = np.array(list(range(16)) + [8] + [0] * 7 + [0] * 7 + [8], np.float32)
    for n in range(N):
        assert np.array_equal(w[n], u - n), n


def test_int4_quantize_sym_properties():
    w = orc.normal_f32(0, 11, (16, 256), 0.02)
    packed, scale, zp = orc.int4_quantize_sym(w)
    assert np.all(zp == 0x88888888)
    dq = orc.bf16_to_f32(orc.int4_dequant(packed, scale, zp))
    s = orc.bf16_to_f32(scale)
    amax = np.abs(w.reshape(16, 8, 32)).max(-1)
    assert np.array_equal(scale, orc.f32_to_bf16(amax / np.float32(7)))
    # error at most half a step (plus the bf16 rounding of the product), except where q clamps at +7 (amax / s may exceed 7.5 never)
    err = np.abs(dq - w).reshape(16, 8, 32)
    assert np.all(err <= 0.56 * s[..., None] + 1e-9)  # half a step + the scale's and the product's bf16 roundings
    z = w.copy()
    z[3, 64:96] = 0
    p2, s2, _ = orc.int4_quantize_sym(z)
    assert s2[3, 2] == 0x3F80 and np.all(orc.int4_dequant(p2, s2, zp)[3, 64:96] == 0)


def _fp8_from_master_torch(w):
    """the reference's fp8_from_master (pack.py:216-232) with torch primitives"""
    w = torch.from_numpy(w).float()
    N, K = w.shape
    nb, kb = (N + 127) // 128, K // 128
    pad = torch.zeros(nb * 128, K)
    pad[:N] = w
    blk = pad.view(nb, 128, kb, 128)
    amax = blk.abs().amax(dim=(1, 3))
    scale = (amax * torch.tensor(1.0 / 448.0, dtype=torch.float32)).clamp_min(1e-12)
    q = (blk / scale[:, None, :, None]).to(torch.float8_e4m3fn)
    return q.view(torch.uint8).reshape(nb * 128, K)[:N].contiguous().numpy(), scale.numpy()


def test_fp8_quantiser_matches_reference_formula():
    for (N, K, sig) in [(256, 512, 0.02), (200, 256, 1.0), (128, 128, 1e-6)]:
        w = orc.normal_f32(0, 100 + N, (N, K), sig)
        w[5, 7] = 0.0
        if N == 200:
            w[128:200, 128:256] = 0  # an all-zero block: scale 1e-12
        c, s = orc.fp8_quantize(w)
        ct, st = _fp8_from_master_torch(w)
        assert np.array_equal(s, st) and np.array_equal(c, ct)
        # amax / 448 differs from amax * (1/448) in some blocks: the multiply form is the contract
        dq = orc.fp8_dequant(c, s)
        v = torch.from_numpy(c).view(torch.float8_e4m3fn).float().numpy()
        sfull = np.repeat(np.repeat(s, 128, 0)[:N], 128, 1)
        assert np.array_equal(dq, (v * sfull).astype(np.float32))       # pack.py:235-241
        assert np.abs(dq - w).max() <= np.abs(w).max() * 2.0 ** -4 + 1e-20
        assert not np.any((c & 0x7F) == 0x7F)


def test_act_quant_matches_reference_formula():
    x16 = orc.normal_bf16(0, 5, (37, 512), 1.0)
    x16[3, :128] = 0                      # amax clamps at 1e-4
    q, s = orc.act_quant(x16)
    x = torch.from_numpy(orc.bf16_to_f32(x16))
    xf = x.unflatten(-1, (4, 128))
    amax = xf.abs().amax(-1, keepdim=True).clamp_min(1e-4)
    st = amax * torch.tensor(1.0 / 448.0, dtype=torch.float32)
    qt = (xf / st).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8).flatten(-2).numpy()
    assert np.array_equal(s, st.squeeze(-1).numpy()) and np.array_equal(q, qt)
    assert s[3, 0] == np.float32(1e-4) * np.float32(1.0 / 448.0)


def test_random_tensors_follow_the_reference_generators():
    packed, scale, zp = orc.int4_random(6, 24, 1024)
    # scales: positive bf16 in [2^-9, 2^-5) (testdata.h:45-48); every nibble and zero-point value occurs
    s = orc.bf16_to_f32(scale)
    assert s.min() >= 2.0 ** -9 and s.max() < 2.0 ** -5
    nib = (packed[:, :, None] >> (np.arange(8, dtype=np.uint32) * 4)) & 15
    assert set(np.unique(nib)) == set(range(16))
    c, fs = orc.fp8_random(7, 128, 256, 1.0 / 1024)
    assert not np.any((c & 0x7F) == 0x7F) and np.all((c & 0x78) <= 0x48)
    assert fs.min() >= 0.5 / 1024 and fs.max() < 1.5 / 1024
