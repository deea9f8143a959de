"""Writes tests/golden/dot2_bf16.npz: operands and results of gfx950's v_dot2_f32_bf16, the multiply-add of the vector-unit
decode kernels and the dense GEMV. RUN ON THE GPU: it calls the library's own probe (dsgx_probe_dot2_bf16), nothing of the
reference. The CPU tests check the oracle's statement of the instruction (orc_dot2_bf16) against these vectors bit for bit.

    python tests/golden/make_dot2_bf16_vectors.py [out.npz]

a, b: packed bf16 pairs (uint32, the low half first), c f32, d f32 = c + a.lo b.lo + a.hi b.hi as the instruction adds it.
Cases: standard normals times 2^r, r uniform in +-0, 2, 6, 12, 20, with c of comparable or far smaller / larger size and
zero in a tenth of the cases; operands with bf16 subnormals; zero operands; c just above a power of two with products that
take the result below it; and crafted cases on the edge of the adder's width
(c = 2^30 whose ulp is 128, one product 2^6 - half an ulp - and the other 2^p, p = 5 .. -6) and on a sum that carries out of
c's binade (c = 2 - 2^e + 2^-23, the products 2^e and 2^p, p = -26 .. -33)."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)


def main(out):
    from dsgx10_amd import lib
    from tests import gpu, orc

    rng = np.random.default_rng(41)
    n = 2048
    A, B, Cc = [], [], []
    pack = lambda v: v[:, 0].astype(np.uint32) | (v[:, 1].astype(np.uint32) << 16)
    for spread in (0, 2, 6, 12, 20):
        mk = lambda: orc.f32_to_bf16((rng.standard_normal((n, 2)) * 2.0 ** rng.integers(-spread, spread + 1, (n, 2))).astype(np.float32))
        c = (rng.standard_normal(n) * 2.0 ** rng.integers(-spread - 2, spread + 3, n)).astype(np.float32)
        c[rng.random(n) < 0.1] = 0
        a = mk()
        a[rng.random((n, 2)) < 0.05] = 0
        A.append(pack(a)), B.append(pack(mk())), Cc.append(c)
    # bf16 subnormals against large values
    a = rng.integers(1, 128, (n, 2)).astype(np.uint16) | (rng.integers(0, 2, (n, 2)).astype(np.uint16) << 15)
    b = orc.f32_to_bf16((rng.standard_normal((n, 2)) * 2.0 ** 120).astype(np.float32))
    A.append(pack(a)), B.append(pack(b)), Cc.append((rng.standard_normal(n) * 1e-3).astype(np.float32))
    # cancellation: c just above a power of two, products of either sign
    a = orc.f32_to_bf16((rng.standard_normal((n, 2)) * 0.05).astype(np.float32))
    b = orc.f32_to_bf16(rng.standard_normal((n, 2)).astype(np.float32))
    c = (np.where(rng.random(n) < 0.5, 1.0, -1.0) * 2.0 ** rng.integers(-2, 4, n) * (1.0 + rng.random(n) * 0.01)).astype(np.float32)
    A.append(pack(a)), B.append(pack(b)), Cc.append(c)
    # the adder's width
    one = lambda v: int(orc.f32_to_bf16(np.array([v], np.float32))[0])
    a, b, c = np.zeros((n, 2), np.uint16), np.zeros((n, 2), np.uint16), np.zeros(n, np.float32)
    i = 0
    for sign, accv in ((1.0, 2.0 ** 30), (-1.0, 2.0 ** 30 + 2.0 ** 29), (1.0, -(2.0 ** 30)), (-1.0, -(2.0 ** 30 + 2.0 ** 29))):
        for p in range(5, -7, -1):
            a[i] = (one(sign * 64.0), one(sign * 2.0 ** p))
            b[i] = (one(1.0), one(1.0))
            c[i] = accv
            i += 1
    # a sum that carries out of the accumulator's binade: c = +-(2 - 2^e - 2^-23 ...): c = +-(2 - 2^e), products 2^e + 2^-23 (one
    # bf16 value times 1 cannot hold both: 2^e from one product, 2^p from the other, c carrying the half ulp itself)
    for sign in (1.0, -1.0):
        for e in (-8, -6):
            for p in range(-26, -34, -1):
                a[i] = (one(sign * 2.0 ** e), one(sign * 2.0 ** p))
                b[i] = (one(1.0), one(1.0))
                c[i] = sign * (2.0 - 2.0 ** e + 2.0 ** -23)
                i += 1
    A.append(pack(a)), B.append(pack(b)), Cc.append(c)
    a, b, c = np.concatenate(A), np.concatenate(B), np.concatenate(Cc)
    o = gpu.empty(a.size * 4, 0xFF)
    lib.probe_dot2_bf16(gpu.dev(a), gpu.dev(b), gpu.dev(c), o, a.size)
    np.savez_compressed(out, a=a, b=b, c=c, d=gpu.host(o, np.float32, (a.size,)))
    print("wrote", out, a.size, "cases")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else os.path.join(os.path.dirname(os.path.abspath(__file__)), "dot2_bf16.npz"))
