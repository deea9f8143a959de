"""The oracle's FP8-activation expert (oracle.cpp: orc_moe_prefill_fp8_row) against vectors computed by the reference's own
pure-torch kernels (tests/golden/make_prefill_fp8_vectors.py; ds41f-4xgx10-switchless/ref/torchref/kernel.py:56-125,
ref/inference/model.py:841-851): x -> act_quant 1x128 -> gate / up (e4m3 128x128 block scales) -> SiLU(gate) up -> bf16
-> act_quant -> down.

The two are not the same arithmetic bit for bit, on purpose: the reference dequantises both operands to f32 and sums
their products in one matmul, then rounds to bf16; the oracle sums the e4m3 products of a 128-k block from zero and
applies the two scales once a block (the engine's order), rounds SiLU(g) to bf16 before the product (the engine's h:
decode.cu:110-113) and keeps the down result in f32. What the vectors pin is everything a restatement can get wrong
without failing its own parts: the scale of (row block, k block), the block order of both operands, the quantiser's
clamp and reciprocal, the two re-quantisations, which matrix is which. Stage by stage the agreement is at the bit level:
h from the reference's gate / up under the engine's rounding rule, and bf16(down) from the reference's h."""
import os

import numpy as np

from dsgx10_amd import abi
from dsgx10_amd.layer import HostLayer
from tests import orc
from tests.helpers import rel_l2

FIX = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "prefill_fp8_expert.npz")


def _layer(v, down_scales=None):
    H, I = v["x"].shape[1], v["gate_codes"].shape[0]
    ex = ((v["gate_codes"], v["gate_scales"]), (v["up_codes"], v["up_scales"]),
          (v["down_codes"], v["down_scales"] if down_scales is None else down_scales))
    return HostLayer(abi.FMT_FP8, H, I, 1, 1, [ex])


def _run(hl, v, h_in=None):
    T = v["x"].shape[0]
    rows = [orc.moe_prefill_fp8_row(hl, v["x"][t], np.zeros(1, np.int32), np.ones(1, np.float32),
                                    h_in=None if h_in is None else np.stack([h_in[t], h_in[t]])) for t in range(T)]
    return np.stack([r["h"][0] for r in rows]), np.stack([r["yr"] for r in rows])


def _ulps(a, b):
    return np.abs(a.astype(np.int32) - b.astype(np.int32))


def test_gate_up_and_swiglu_against_the_reference_vectors():
    v = np.load(FIX)
    h, _ = _run(_layer(v), v)
    # the engine's h from the REFERENCE's gate and up (bf16): bf16(bf16(silu(g)) u). Equal bits unless the oracle's g or u
    # straddles a bf16 rounding under its other order of f32 adds (1 of 1536 here).
    g, u = orc.bf16_to_f32(v["gate"]), orc.bf16_to_f32(v["up"])
    silu = (g / (np.float32(1) + np.exp(-g))).astype(np.float32)
    h_engine = orc.f32_to_bf16((orc.bf16_to_f32(orc.f32_to_bf16(silu)) * u).astype(np.float32))
    assert (h == h_engine).mean() >= 0.995, (h == h_engine).mean()
    assert _ulps(h, h_engine).max() <= 1
    # and against the reference's own h, which rounds silu(g) u once: never more than one bf16 step apart
    assert _ulps(h, v["h"]).max() <= 1
    assert (h == v["h"]).mean() >= 0.6


def test_requantise_and_down_against_the_reference_vectors():
    v = np.load(FIX)
    _, d = _run(_layer(v), v, h_in=v["h"])  # the down projection from the reference's h
    db = orc.f32_to_bf16(d)
    assert (db == v["d"]).mean() >= 0.995, (db == v["d"]).mean()  # (all 1536 here)
    assert _ulps(db, v["d"]).max() <= 1
    # end to end (the oracle's own h): two evaluations of a contract with an e4m3 re-quantisation in the middle
    _, d2 = _run(_layer(v), v)
    assert rel_l2(d2, orc.bf16_to_f32(v["d"])) <= 3e-2


def test_the_vectors_tell_a_wrong_scale_index_apart():
    """the checks above have teeth: the down scales transposed (block (n, k) taking the scale of (k, n)) fail them by far"""
    v = np.load(FIX)
    _, d = _run(_layer(v, down_scales=np.ascontiguousarray(v["down_scales"].T)), v, h_in=v["h"])
    assert (orc.f32_to_bf16(d) == v["d"]).mean() < 0.6
    assert rel_l2(d, orc.bf16_to_f32(v["d"])) > 5e-2
