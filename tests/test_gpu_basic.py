"""GPU parity, through the C ABI, of the bit-exact classes: the INT4 and FP8 decode (both the operator and the
streaming kernels' own in-register routine), the router's ids and weight bits, finalize and act_quant.
Mirrors the reference's test_deq / test_route (altar1-4xgx10-switchless/engine/experts/tests/test_experts.cu:217-319)."""
import numpy as np
import pytest

from dsgx10_amd import abi, lib
from tests import gpu, orc

pytestmark = pytest.mark.gpu


def _i4_test_scales():
    # test_experts.cu:62-68: extremes, subnormals, random normal ones, any positive finite bf16
    v = [0x0001, 0x0002, 0x0017, 0x0040, 0x007F, 0x0080, 0x0081, 0x00FF, 0x0100, 0x3F80, 0x3F81, 0x3FFF, 0x7F00, 0x7F7F,
         0x3B80, 0x3C00, 0x3D00]
    m = orc.lib().orc_mix64
    for i in range(64):
        h = m(i + 5)
        v.append(((118 + h % 4) << 7) | ((h >> 8) & 0x7F))
    for i in range(64):
        v.append(m(i + 99) % 0x7F7F + 1)
    return np.array(v, np.uint16)


def _dequant(packed, scale, zp, probe):
    N, K = packed.shape[0], packed.shape[1] * 8
    out = gpu.empty(N * K * 2, 0xEE)
    lib.dequant_int4(gpu.dev(packed), gpu.dev(scale), gpu.dev(zp), N, K, out, probe=probe)
    return gpu.host(out, np.uint16, (N, K))


@pytest.mark.parametrize("probe", [False, True])
def test_int4_dequant_random_matrices(probe):
    for (N, K, seed) in [(2048, 6144, 40), (6144, 2048, 42), (24, 1024, 6)]:
        packed, scale, zp = orc.int4_random(seed, N, K)
        assert np.array_equal(_dequant(packed, scale, zp, probe), orc.int4_dequant(packed, scale, zp)), (N, K)


def test_int4_dequant_whole_domain_operator():
    """every finite positive and negative bf16 scale x every (u, u_z): the operator equals the contract bit for bit"""
    sb = np.arange(0x10000, dtype=np.uint32)
    sb = sb[(sb & 0x7F80) != 0x7F80].astype(np.uint16)
    N = (sb.size + 7) // 8 * 8
    words = np.zeros(4, np.uint32)
    for i in range(32):
        words[i // 8] |= np.uint32(i % 16) << np.uint32(4 * (i % 8))
    packed = np.tile(words, (N, 16))           # K = 512: 16 groups a row, group g has u_z = g
    scale = np.zeros((N, 16), np.uint16)
    scale[: sb.size] = sb[:, None]
    zp = np.tile((np.arange(16, dtype=np.uint32) * 0x11111111)[None, :], (N // 8, 1)).astype(np.uint32)
    got = _dequant(packed, scale, zp, False)
    want = orc.int4_dequant(packed, scale, zp)
    nan = np.isnan(orc.bf16_to_f32(want))      # inf * 0 at the two largest scales' overflow: NaN payloads are not compared
    assert np.array_equal(got[~nan], want[~nan])
    assert nan.mean() < 1e-3


def test_int4_hot_decode_scales():
    """the streaming kernels' own decode on the reference's 145 test scales (subnormal, extreme) and on every finite scale
    below 2^124, all (u, u_z)"""
    sc = _i4_test_scales()
    sb = np.arange(0x10000, dtype=np.uint32)
    sb = sb[((sb & 0x7F80) != 0x7F80) & ((sb & 0x7FFF) < 0x7D80) & ((sb & 0x7FFF) != 0)].astype(np.uint16)   # 0 < |s| < 2^124
    sc = np.concatenate([sc[(sc & 0x7FFF) < 0x7D80], sb])
    N = (sc.size + 7) // 8 * 8
    words = np.zeros(4, np.uint32)
    for i in range(32):
        words[i // 8] |= np.uint32(i % 16) << np.uint32(4 * (i % 8))
    packed = np.tile(words, (N, 16))
    scale = np.full((N, 16), 0x3F80, np.uint16)
    scale[: sc.size] = sc[:, None]
    zp = np.tile((np.arange(16, dtype=np.uint32) * 0x11111111)[None, :], (N // 8, 1)).astype(np.uint32)
    got, want = _dequant(packed, scale, zp, True), orc.int4_dequant(packed, scale, zp)
    pos = (scale[:, 0] & 0x8000) == 0
    assert np.array_equal(got[pos], want[pos])          # the format's scales are positive: bit for bit
    # negative scales (refused by the loader's scale check) differ only in the sign of a zero: u = u_z gives +0, not -0
    z = (want & 0x7FFF) == 0
    assert np.array_equal(got[~pos][~z[~pos]], want[~pos][~z[~pos]]) and np.all((got[z] & 0x7FFF) == 0)


def test_fp8_widen_every_code():
    codes = np.tile(np.arange(256, dtype=np.uint8), (8, 4))      # [8][1024]
    out = gpu.empty(codes.size * 2, 0xEE)
    lib.widen_fp8(gpu.dev(codes), 8, 1024, out)
    got = gpu.host(out, np.uint16, codes.shape)
    want = orc.f32_to_bf16(orc.e4m3_table()[codes])
    ok = (codes & 0x7F) != 0x7F
    assert np.array_equal(got[ok], want[ok])                     # the 254 non-NaN values widen exactly
    assert np.all(np.isnan(orc.bf16_to_f32(got[~ok])))


def _route_gpu(l, bias, topk, scale, score_fn=0):
    M, E = l.shape
    di, dw = gpu.empty(M * topk * 4, 0xFF), gpu.empty(M * topk * 4, 0xFF)
    dl, db = gpu.dev(l), (None if bias is None else gpu.dev(bias))
    rc = lib.lib().dsgx_route(dl.data_ptr(), None if db is None else db.data_ptr(), M, E, topk, scale, score_fn, di.data_ptr(),
                              dw.data_ptr(), None)
    assert rc == 0, lib.lib().dsgx_last_error()
    return gpu.host(di, np.int32, (M, topk)), gpu.host(dw, np.float32, (M, topk))


def _rnd_logits(M, E, seed, ties):
    m = orc.lib().orc_mix64
    l = np.empty((M, E), np.float32)
    for i in range(M * E):
        h = m(seed * 13 + i)
        v = (np.float32(h >> 40) * np.float32(2.0 ** -24) - np.float32(0.5)) * np.float32(6.0)
        l.flat[i] = np.float32(1.25) if ties and (h & 7) == 0 else v
    return l


@pytest.mark.parametrize("E,topk,scale", [(168, 8, 2.5), (256, 8, 1.0), (64, 6, 1.5), (512, 8, 2.5), (8, 8, 1.0)])
def test_route_ids_and_weight_bits(E, topk, scale):
    m = orc.lib().orc_mix64
    for ties in range(3):
        M = 16 + 3 * (ties > 0)
        l = _rnd_logits(M, E, 11 + ties, ties == 1)
        bias = np.array([28.25 if ties else 28.2 + 0.37 * ((m(e) % 1000) / 1000.0) for e in range(E)], np.float32)
        if ties == 2 and E >= 168:   # three experts share the 8th key, the rest distinct (test_experts.cu:295-301)
            for r in range(M):
                for e in range(E):
                    l[r, e] = -4.0 + 0.01 * ((e * 37 + r * 11) % E)
                a, b, c, top = (r * 13) % E, (r * 13 + 50) % E, (r * 13 + 101) % E, (r * 13 + 7) % E
                for k in range(7):
                    l[r, (top + 3 * k) % E] = 5.0 + k
                l[r, a] = l[r, b] = l[r, c] = 4.5
        ri, rw = orc.route(l, bias, topk, scale)
        gi, gw = _route_gpu(l, bias, topk, scale)
        assert np.array_equal(gi, ri), (E, ties)
        assert np.array_equal(gw.view(np.uint32), rw.view(np.uint32)), (E, ties)
    # no bias, N(0,1) logits: the DeepSeek-shaped configuration
    l = orc.normal_f32(0, 2, (33, E), 1.0)
    ri, rw = orc.route(l, None, topk, scale)
    gi, gw = _route_gpu(l, None, topk, scale)
    assert np.array_equal(gi, ri) and np.array_equal(gw.view(np.uint32), rw.view(np.uint32))


def test_route_sqrt_softplus_bits():
    """DeepSeek's score sqrt(softplus(l)) is built from IEEE operations only on both sides (as the sigmoid is): ids and
    weight bits equal the oracle's, on random rows, on rows with a bias, on logits across the whole range incl. both sides of
    the switch at 20, and on engineered ties"""
    l = orc.normal_f32(3, 2, (16, 384), 1.0)
    wide = np.linspace(-95, 30, 16 * 384, dtype=np.float32).reshape(16, 384)[:, ::-1].copy()
    ties = l.copy()
    ties[:, 7] = ties[:, 300] = ties[:, 301] = 3.25   # a three-way tie at the top: lower ids first
    bias = orc.normal_f32(3, 9, (384,), 0.1)
    for logits, b in ((l, None), (l * 4, bias), (wide, None), (ties, None), (ties, bias)):
        ri, rw = orc.route(logits, b, 6, 1.5, score_fn=1)
        gi, gw = _route_gpu(logits, b, 6, 1.5, score_fn=1)
        assert np.array_equal(gi, ri) and np.array_equal(gw.view(np.uint32), rw.view(np.uint32))


def test_finalize_bits():
    R, S = orc.normal_f32(0, 1, (6144 * 3,), 1.0), orc.normal_f32(0, 2, (6144 * 3,), 0.3)
    out = gpu.empty(R.size * 2, 0)
    lib.finalize(gpu.dev(R), gpu.dev(S), R.size, out)
    assert np.array_equal(gpu.host(out, np.uint16, R.shape), orc.finalize(R, S))


def test_act_quant_bits():
    x = orc.normal_bf16(0, 5, (37, 4096), 1.0)
    x[3, :128] = 0
    x[4, 128:256] = orc.f32_to_bf16(np.full(128, 3e-5, np.float32))
    q, s = gpu.empty(x.size, 0xEE), gpu.empty(37 * 32 * 4, 0xEE)
    lib.act_quant(gpu.dev(x), 37, 4096, q, s)
    oq, os_ = orc.act_quant(x)
    assert np.array_equal(gpu.host(s, np.float32, os_.shape), os_)
    assert np.array_equal(gpu.host(q, np.uint8, oq.shape), oq)


def test_stream_read_and_copy_run():
    a = gpu.dev(np.arange(1 << 20, dtype=np.uint32))
    b = gpu.empty(a.numel(), 0)
    sink = gpu.empty(4, 0)
    lib.stream_read(a, a.numel(), sink)
    lib.stream_copy(a, b, a.numel())
    assert np.array_equal(gpu.host(b, np.uint32, (-1,)), np.arange(1 << 20, dtype=np.uint32))


def test_bf16_mfma_probe_is_the_f32_product_sum():
    """one v_mfma_f32_16x16x32_bf16 (the instruction of decode variant 1 and of the bf16-activation prefill GEMMs), operands as the
    kernels hand them over (a lane of part p holds k = 8 p .. 8 p + 7 of its row), with an accumulator going in: within 1e-6 of
    the sum of |terms| of the f64 result, and equal bit for bit to the oracle's statement of how the unit adds (orc_mfma_bf16_k32,
    pinned on the CPU by tests/golden/mfma_bf16_k32.npz) on these fresh operands"""
    rng = np.random.default_rng(4)
    for trial in range(4):
        a = orc.f32_to_bf16((rng.standard_normal((16, 32)) * 2.0 ** rng.integers(-3, 4, (16, 32))).astype(np.float32))
        b = orc.f32_to_bf16(rng.standard_normal((16, 32)).astype(np.float32))
        c = (rng.standard_normal((16, 16)) * 3).astype(np.float32) if trial % 2 else None
        out = gpu.empty(16 * 16 * 4, 0xFF)
        lib.probe_mfma_bf16(gpu.dev(a), gpu.dev(b), out, acc=None if c is None else gpu.dev(c))
        got = gpu.host(out, np.float32, (16, 16)).astype(np.float64)
        av, bv = orc.bf16_to_f32(a).astype(np.float64), orc.bf16_to_f32(b).astype(np.float64)
        want = av @ bv.T + (0 if c is None else c.astype(np.float64))
        mag = np.abs(av) @ np.abs(bv).T + (0 if c is None else np.abs(c).astype(np.float64))
        assert np.all(np.abs(got - want) <= 1e-6 * mag), float((np.abs(got - want) / mag).max())
        mine = gpu.host(out, np.float32, (16, 16))
        assert np.array_equal(mine.view(np.uint32), orc.mfma_bf16_k32(a, b, c).view(np.uint32))
