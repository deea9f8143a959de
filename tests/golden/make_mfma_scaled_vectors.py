"""Writes tests/golden/mfma_scaled_k128.npz: operands and results of gfx950's v_mfma_scale_f32_16x16x128_f8f6f4, the
instruction DeepSeek's prefill GEMMs run on (e2m1 or e4m3 weights, e4m3 rows, a ue8m0 scale byte per 32 k for each, the
accumulator carried from block to block). RUN ON THE GPU: it calls the library's own probe (dsgx_probe_mfma_scaled), nothing of
the reference. The CPU tests check the oracle's statement of the unit's summation rule (orc_mfma_scaled_k128) against these
vectors bit for bit.

    python tests/golden/make_mfma_scaled_vectors.py [out.npz]

Per case c: fp4[c] (1: a holds e2m1 pairs [16][64], the low nibble the even k; 0: e4m3 codes [16][128], stored in the first
or all 128 columns of a[c]), b[c] e4m3 [16][128], sa[c], sb[c] ue8m0 [16][4], acc[c] f32 [16][16] (the accumulator going in;
zeros in every third case), d[c] f32 [16][16]: d[i][j] = acc[i][j] + sum over k of a[i][k] 2^(sa[i][k/32] - 127) b[j][k]
2^(sb[j][k/32] - 127) as the instruction adds it, k as stored.
Cases: operands shaped like quantised rows and weights with unit scales; uniformly random codes; scale bytes spread over
+-3, +-6 and +-10 around 127; sparse rows; accumulators of 1e-3 to 1e3 times a standard normal; two crafted cases that
sit on the edge of the accumulator adder's width, six with accumulators just above a power of two, and two whose sums carry out of the accumulator's binade (the last two)."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)


def main(out):
    from dsgx10_amd import lib
    from tests import gpu

    def e4m3_of(v):  # round-to-nearest-even e4m3 codes of f32 values (torch's cast: the maker runs where torch has a GPU)
        import torch
        return torch.from_numpy(np.clip(v, -448, 448).astype(np.float32)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()

    rng = np.random.default_rng(11)
    fp4s, A, B, SA, SB, ACC, D = [], [], [], [], [], [], []
    for trial in range(30):
        fp4, style = trial % 2, (trial // 2) % 5
        a = np.zeros((16, 128), np.uint8)
        if fp4:
            codes = rng.integers(0, 16, (16, 128), dtype=np.uint8)
            if style == 3:
                codes = np.where(rng.random((16, 128)) < 0.1, codes, 0).astype(np.uint8)
            a[:, :64] = codes[:, 0::2] | (codes[:, 1::2] << 4)
        else:
            a = e4m3_of(rng.standard_normal((16, 128)) * 40.0) if style != 1 else rng.integers(0, 256, (16, 128), dtype=np.uint8)
            a = np.where((a & 0x7F) == 0x7F, a & 0x80, a).astype(np.uint8)  # (no NaN codes)
            if style == 3:
                a = np.where(rng.random((16, 128)) < 0.1, a, 0).astype(np.uint8)
        b = e4m3_of(rng.standard_normal((16, 128)) * 30.0) if style != 1 else rng.integers(0, 256, (16, 128), dtype=np.uint8)
        b = np.where((b & 0x7F) == 0x7F, b & 0x80, b).astype(np.uint8)
        if style == 4:
            b = np.where(rng.random((16, 128)) < 0.15, b, 0).astype(np.uint8)
        spread = (0, 0, 3, 6, 10)[style]
        sa = (127 + rng.integers(-spread, spread + 1, (16, 4))).astype(np.uint8)
        sb = (127 + rng.integers(-spread, spread + 1, (16, 4))).astype(np.uint8)
        acc = np.zeros((16, 16), np.float32) if trial % 3 == 0 else (rng.standard_normal((16, 16)) * (10.0 ** rng.integers(-3, 4))).astype(np.float32)
        o = gpu.empty(16 * 16 * 4, 0xFF)
        lib.probe_mfma_scaled(gpu.dev(np.ascontiguousarray(a[:, :64]) if fp4 else a), gpu.dev(sa), gpu.dev(b), gpu.dev(sb), fp4, o,
                              acc=None if trial % 3 == 0 else gpu.dev(acc))
        fp4s.append(fp4), A.append(a), B.append(b), SA.append(sa), SB.append(sb), ACC.append(acc), D.append(gpu.host(o, np.float32, (16, 16)))
    # crafted: the accumulator adder's width and rounding. Row i of a case pairs with row i of b (its result is d[i][i]): the
    # accumulator is 2^30 (or -(2^30 + 2^29)... its ulp is 128), the unit adds (or subtracts) 2^6 - half an ulp - from one group
    # and 2^p from the other, p = 5 .. -6: the result moves by a whole ulp exactly while 2^p still reaches the adder
    import torch
    code = lambda v: int(torch.tensor([v], dtype=torch.float32).to(torch.float8_e4m3fn).view(torch.uint8)[0])
    for sign, accv in ((1.0, 2.0 ** 30), (-1.0, 2.0 ** 30 + 2.0 ** 29)):
        a, b = np.zeros((16, 128), np.uint8), np.zeros((16, 128), np.uint8)
        sa, sb = np.full((16, 4), 127, np.uint8), np.full((16, 4), 127, np.uint8)
        acc = np.zeros((16, 16), np.float32)
        for i in range(12):
            e = (5 - i) - 6
            e1 = max(e, -6)
            sa[i, 0] = 127 + 6
            a[i, 0], b[i, 0] = code(sign), code(1.0)
            a[i, 8], b[i, 8] = code(sign * 2.0 ** e1), code(2.0 ** (e - e1))
            acc[i, i] = accv
        o = gpu.empty(16 * 16 * 4, 0xFF)
        lib.probe_mfma_scaled(gpu.dev(a), gpu.dev(sa), gpu.dev(b), gpu.dev(sb), 0, o, acc=gpu.dev(acc))
        fp4s.append(0), A.append(a), B.append(b), SA.append(sa), SB.append(sb), ACC.append(acc), D.append(gpu.host(o, np.float32, (16, 16)))
    # cancellation: accumulators just above a power of two against small sums of either sign (results that fall below it)
    for trial in range(6):
        a = e4m3_of(rng.standard_normal((16, 128)) * (2.0, 6.0, 1.0)[trial % 3])
        b = e4m3_of(rng.standard_normal((16, 128)) * 4.0)
        if trial % 2:
            a[:, 16 * (1 + trial):] = 0
        sa, sb = np.full((16, 4), 127 - 6, np.uint8), np.full((16, 4), 127 - 4, np.uint8)
        acc = (np.where(rng.random((16, 16)) < 0.5, 1.0, -1.0) * 2.0 ** rng.integers(-2, 4, (16, 16)) * (1.0 + rng.random((16, 16)) * (0.002, 0.02)[trial % 2])).astype(np.float32)
        o = gpu.empty(16 * 16 * 4, 0xFF)
        lib.probe_mfma_scaled(gpu.dev(a), gpu.dev(sa), gpu.dev(b), gpu.dev(sb), 0, o, acc=gpu.dev(acc))
        fp4s.append(0), A.append(a), B.append(b), SA.append(sa), SB.append(sb), ACC.append(acc), D.append(gpu.host(o, np.float32, (16, 16)))
    # crafted: a sum that carries out of the accumulator's binade: the accumulator is +-(2 - 2^-8); with both scale bytes of the
    # block at 2^-13 / 2^0 one group holds 2^5 (-> 2^-8), the unit's other group 2^-10 (-> 2^-23, half an ulp of the result) and
    # 2^-16 .. 2^-18 (-> 2^-29 .. 2^-31): the last is inside the accumulator's window and outside the sum's
    for sign in (1.0, -1.0):
        a, b = np.zeros((16, 128), np.uint8), np.zeros((16, 128), np.uint8)
        sa, sb = np.full((16, 4), 127, np.uint8), np.full((16, 4), 127, np.uint8)
        acc = np.zeros((16, 16), np.float32)
        for i in range(3):
            sa[i, 0] = 127 - 13
            a[i, 0], b[i, 0] = code(sign * 32.0), code(1.0)
            a[i, 8], b[i, 8] = code(sign * 2.0 ** -5), code(2.0 ** -5)
            t = -16 - i
            a[i, 9], b[i, 9] = code(sign * 2.0 ** -9), code(2.0 ** (t + 9))
            acc[i, i] = sign * (2.0 - 2.0 ** -8)
        o = gpu.empty(16 * 16 * 4, 0xFF)
        lib.probe_mfma_scaled(gpu.dev(a), gpu.dev(sa), gpu.dev(b), gpu.dev(sb), 0, o, acc=gpu.dev(acc))
        fp4s.append(0), A.append(a), B.append(b), SA.append(sa), SB.append(sb), ACC.append(acc), D.append(gpu.host(o, np.float32, (16, 16)))
    np.savez_compressed(out, fp4=np.array(fp4s, np.int32), a=np.stack(A), b=np.stack(B), sa=np.stack(SA), sb=np.stack(SB), acc=np.stack(ACC), d=np.stack(D))
    print("wrote", out, len(fp4s), "cases")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else os.path.join(os.path.dirname(os.path.abspath(__file__)), "mfma_scaled_k128.npz"))
