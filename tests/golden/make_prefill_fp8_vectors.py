#!/usr/bin/env python3
"""Writes tests/golden/prefill_fp8_expert.npz: input/output vectors of the reference's FP8-activation expert
(ds41f-4xgx10-switchless/ref/inference/model.py:841-851 over linear() :181-205) computed by the reference's own
pure-torch kernels (ds41f-4xgx10-switchless/ref/torchref/kernel.py: act_quant :56-77, fp8_gemm :118-125), in the
128 x 128 / 1 x 128 f32-scale form of the benchmark's FP8 prefill configuration (act_quant(x, 128, None),
fp8_gemm(..., block_size=128)).

Run in the build container only (the reference is not on the GPU box):  python tests/golden/make_prefill_fp8_vectors.py
The vectors pin oracle/oracle.cpp: orc_moe_prefill_fp8_row as a whole (tests/test_oracle_prefill_golden.py); no other
function of the oracle needs an import of the reference.
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
    torch.set_default_dtype(torch.bfloat16)  # the reference runs with bf16 as the default dtype (fp8_gemm casts to it)
    g = torch.Generator().manual_seed(20261125)
    T, H, I = 6, 256, 256  # two k blocks and two row blocks each way, every block with a scale of its own

    def weight(N, K):
        """e4m3 codes [N][K] and f32 scales [N/128][K/128]: N(0, 0.02) weights times a per-block factor, scale = amax / 448"""
        w = torch.randn(N, K, generator=g, dtype=torch.float32) * 0.02
        w = w * (1.0 + torch.arange((N // 128) * (K // 128), dtype=torch.float32).view(N // 128, K // 128)
                 ).repeat_interleave(128, 0).repeat_interleave(128, 1)
        blocks = w.view(N // 128, 128, K // 128, 128)
        s = blocks.abs().amax((1, 3)).clamp_min(1e-12) * torch.tensor(1.0 / 448.0, dtype=torch.float32)
        q = (blocks / s[:, None, :, None]).reshape(N, K).to(torch.float8_e4m3fn)
        return q, s

    def lin(x, q, s):
        a, a_s = ref.act_quant(x, 128, None)
        return ref.fp8_gemm(a, a_s, q, s, block_size=128)

    x = torch.randn(T, H, generator=g, dtype=torch.float32).to(torch.bfloat16)
    (gq, gs), (uq, us), (dq, ds) = weight(I, H), weight(I, H), weight(H, I)
    gate, up = lin(x, gq, gs), lin(x, uq, us)
    h = (F.silu(gate.float()) * up.float()).to(torch.bfloat16)
    d = lin(h, dq, ds)
    bits = lambda t: t.view(torch.int16).numpy().view(np.uint16)
    codes = lambda t: t.view(torch.uint8).numpy()
    np.savez_compressed(os.path.join(HERE, "prefill_fp8_expert.npz"), x=bits(x), gate_codes=codes(gq), gate_scales=gs.numpy(),
                        up_codes=codes(uq), up_scales=us.numpy(), down_codes=codes(dq), down_scales=ds.numpy(),
                        gate=bits(gate), up=bits(up), h=bits(h), d=bits(d))
    print("wrote prefill_fp8_expert.npz", os.path.getsize(os.path.join(HERE, "prefill_fp8_expert.npz")), "bytes")


if __name__ == "__main__":
    main()
