#!/usr/bin/env python3
"""Writes tests/golden/dsk_mxfp4_expert.npz: input/output vectors of the reference's MXFP4 routed expert and FP8 shared
expert (ds41f-4xgx10-switchless/ref/inference/model.py:841-851 Expert.forward over linear() :181-205) computed by the
reference's own pure-torch kernels (ds41f-4xgx10-switchless/ref/torchref/kernel.py: act_quant :56-77 with block 32 and
ue8m0 scales, fp4_gemm :135-138 / dequant_fp4_weight :111-117, fp8_gemm :120-125 / dequant_fp8_weight :105-108 with
32 x 32 blocks), swiglu_limit 10, a routing weight on the routed expert.

Run in the build container only (the reference is not on the GPU box):  python tests/golden/make_dsk_mxfp4_vectors.py
The vectors pin oracle/oracle.cpp: orc_act_quant_ue8m0, orc_mxfp4_dequant, orc_fp8e_dequant, orc_dsk_up and orc_dsk_down as
a chain (tests/test_oracle_dsk.py).
"""
import importlib.util
import os

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
REF = "/root/reference/ds41f-4xgx10-switchless/ref/torchref/kernel.py"


def main():
    spec = importlib.util.spec_from_file_location("ds41f_torchref_kernel", REF)
    ref = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(ref)
    torch.set_default_dtype(torch.bfloat16)  # the reference runs with bf16 as the default dtype (the gemms cast to it)
    g = torch.Generator().manual_seed(20261126)
    M, H, I, LIMIT = 5, 256, 192, 10.0
    E8 = torch.float8_e8m0fnu

    def fp4_weight(N, K):
        """packed e2m1 u8 [N][K/2] (low nibble the even k) and ue8m0 scales [N][K/32]; scales differ from group to group"""
        codes = torch.randint(0, 16, (N, K), generator=g, dtype=torch.uint8)
        packed = (codes[:, 0::2] | (codes[:, 1::2] << 4)).contiguous()
        sb = torch.randint(118, 125, (N, K // 32), generator=g, dtype=torch.uint8)  # 2^-9 .. 2^-3: gate and up reach beyond the clamp
        return packed, sb

    def fp8_weight(N, K):
        """e4m3 codes [N][K] and ue8m0 scales [N/32][K/32]"""
        w = (torch.randn(N, K, generator=g, dtype=torch.float32) * 40.0).clamp(-448, 448).to(torch.float8_e4m3fn)
        sb = torch.randint(114, 120, (N // 32, K // 32), generator=g, dtype=torch.uint8)
        return w, sb

    def lin4(x, packed, sb):
        a, a_s = ref.act_quant(x, 32, "ue8m0", E8)
        return ref.fp4_gemm(a, a_s, packed, sb.view(E8))

    def lin8(x, q, sb):
        a, a_s = ref.act_quant(x, 32, "ue8m0", E8)
        return ref.fp8_gemm(a, a_s, q, sb.view(E8), E8, block_size=32)

    def expert(x, lin, w1, w3, w2, weights):
        gate, up = lin(x, *w1).float(), lin(x, *w3).float()
        up = torch.clamp(up, min=-LIMIT, max=LIMIT)
        gate = torch.clamp(gate, max=LIMIT)
        h = F.silu(gate) * up
        if weights is not None:
            h = weights * h
        h = h.to(torch.bfloat16)
        return h, lin(h, *w2)

    x = (torch.randn(M, H, generator=g, dtype=torch.float32) * 1.5).to(torch.bfloat16)
    rw = (torch.rand(M, 1, generator=g, dtype=torch.float32) * 0.5 + 0.1)
    r1, r3, r2 = fp4_weight(I, H), fp4_weight(I, H), fp4_weight(H, I)
    s1, s3, s2 = fp8_weight(I, H), fp8_weight(I, H), fp8_weight(H, I)
    hr, yr = expert(x, lin4, r1, r3, r2, rw)
    hs, ys = expert(x, lin8, s1, s3, s2, None)
    xa, xs = ref.act_quant(x, 32, "ue8m0", E8)
    bits = lambda t: t.contiguous().view(torch.int16).numpy().view(np.uint16)
    u8 = lambda t: t.contiguous().view(torch.uint8).numpy()
    np.savez_compressed(os.path.join(HERE, "dsk_mxfp4_expert.npz"), x=bits(x), rw=rw.numpy().reshape(-1), x_deq=xa.deq.float().numpy(),
                        x_scale=xs.float().numpy(),
                        r1_w=u8(r1[0]), r1_s=u8(r1[1]), r3_w=u8(r3[0]), r3_s=u8(r3[1]), r2_w=u8(r2[0]), r2_s=u8(r2[1]),
                        s1_w=u8(s1[0]), s1_s=u8(s1[1]), s3_w=u8(s3[0]), s3_s=u8(s3[1]), s2_w=u8(s2[0]), s2_s=u8(s2[1]),
                        h_routed=bits(hr), y_routed=bits(yr), h_shared=bits(hs), y_shared=bits(ys))
    print("wrote dsk_mxfp4_expert.npz", os.path.getsize(os.path.join(HERE, "dsk_mxfp4_expert.npz")), "bytes")


if __name__ == "__main__":
    main()
