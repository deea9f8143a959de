"""Shared builders for the tests: seeded synthetic layers in the pool formats and tolerance checks."""
import numpy as np

from dsgx10_amd import abi
from dsgx10_amd.layer import HostLayer
from tests import orc


def quant_fp8(seed, tid, N, K, sigma=0.02):
    """W ~ N(0, sigma) quantised to e4m3 with 128x128 block scales (the reference's quantiser)."""
    return orc.fp8_quantize(orc.normal_f32(seed, tid, (N, K), sigma))


def quant_int4(seed, tid, N, K, sigma=0.02):
    return orc.int4_quantize_sym(orc.normal_f32(seed, tid, (N, K), sigma))


def make_layer(fmt, H, I, E, topk, NS, seed=0, shared=None, random_codes=False):
    """NS stored experts; expert id e uses stored expert mix64(seed + 99 + e) % NS (testdata.h:197).
    shared: None | 'fp8' | 'bf16'. random_codes: the reference's random-byte tensors (asymmetric INT4 with every zero
    point; random FP8 codes) instead of quantised normal weights."""
    experts = []
    for e in range(NS):
        mats = []
        for j in range(3):
            N, K = (I, H) if j < 2 else (H, I)
            tid = 1000 + e * 3 + j
            if fmt == abi.FMT_FP8:
                mats.append(orc.fp8_random(seed * 131 + tid, N, K, 1.0 / 1024 if j < 2 else 1.0 / 256) if random_codes
                            else quant_fp8(seed, tid, N, K))
            elif fmt == abi.FMT_INT4:
                mats.append(orc.int4_random(seed * 131 + tid, N, K) if random_codes else quant_int4(seed, tid, N, K))
            else:
                mats.append((orc.normal_bf16(seed, tid, (N, K), 0.02),))
        experts.append(tuple(mats))
    emap = np.array([orc.lib().orc_mix64(seed + 99 + e) % NS for e in range(E)], np.int64)
    sh8 = sh16 = None
    if shared == "fp8":
        sh8 = (quant_fp8(seed, 17, I, H), quant_fp8(seed, 18, I, H), quant_fp8(seed, 19, H, I))
    elif shared == "bf16":
        sh16 = (orc.normal_bf16(seed, 27, (2 * I, H), 0.02), orc.normal_bf16(seed, 28, (H, I), 0.02))
    return HostLayer(fmt, H, I, E, topk, experts, emap, shared_fp8=sh8, shared_bf16=sh16)


def rows_and_routing(seed, M, H, E, topk, scale, bias=None):
    x = orc.normal_bf16(seed, 1, (M, H), 1.0)
    logits = orc.normal_f32(seed, 2, (M, E), 1.0)
    idx, w = orc.route(logits, bias, topk, scale)
    return x, logits, idx, w


def rel_l2(got, ref):
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    return float(np.sqrt(((got - ref) ** 2).sum() / max((ref ** 2).sum(), 1e-300)))


def check_sums(got, ref64, mag, tol=1e-4):
    """the reference's rule for GEMV / down outputs: |got - ref| <= tol * sum|terms| (test_experts.cu:352-361,525)"""
    got, ref64, mag = np.asarray(got, np.float64), np.asarray(ref64), np.asarray(mag)
    e = np.abs(got - ref64) / np.where(mag > 0, mag, 1.0)
    return float(e.max()), int((~(e <= tol)).sum())


def check_outputs(got, ref, bf16_rel=True, stress=False):
    """The benchmark's bar on outputs against the f32-accumulated oracle: relative L2 <= 1e-3 and max-abs-err <= 2e-2,
    on the f32 outputs and on their bf16 roundings. The absolute bar is stated for outputs of order one (weights
    ~ N(0, 0.02), activations ~ N(0, 1)); a value large enough for one bf16 step to exceed 2e-2 is allowed that step.
    stress: the layers made of random codes (outputs of order 1e3), where the absolute bar scales with max|ref| / 8."""
    got, ref = np.asarray(got, np.float32), np.asarray(ref, np.float32)
    scale = max(1.0, float(np.abs(ref).max()) / 8.0) if stress else 1.0
    assert rel_l2(got, ref) <= 1e-3, rel_l2(got, ref)
    assert np.abs(got - ref).max() <= 2e-2 * scale, np.abs(got - ref).max()
    g16, r16 = orc.bf16_to_f32(orc.f32_to_bf16(got)), orc.bf16_to_f32(orc.f32_to_bf16(ref))
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(r16), 2.0 ** -126))) - 7)
    assert np.all(np.abs(g16 - r16) <= np.maximum(2e-2 * scale, ulp)), np.abs(g16 - r16).max()
    # (bf16_rel off: where activations are re-quantised to e4m3 on the way, as in the FP8 prefill, got and ref differ by
    # ~5e-4 relative in single terms, which flips ~10% of the bf16 roundings: a step of 4e-3 each, above 1e-3 in L2
    # although the f32 values agree within the bar)
    if bf16_rel:
        assert rel_l2(g16, r16) <= 1e-3


def zipf_picks(T, E, topk, s=1.1, seed=4321):
    """top-k distinct experts a row drawn (without replacement) from a Zipf(s) popularity over a seeded permutation of the
    experts: the k largest of log p + Gumbel noise; uniform weights 1 / top-k (the bench's prefill input)"""
    rng = np.random.default_rng(seed)
    logp = -s * np.log(rng.permutation(E) + 1.0)
    idx = np.argsort(-(logp[None, :] + rng.gumbel(size=(T, E))), axis=1, kind="stable")[:, :topk]
    return np.ascontiguousarray(idx, np.int32), np.full((T, topk), 1.0 / topk, np.float32)


def prefill_fp8_spread(hl, x, idx, w, rows, eps_list=(0.0, 2e-6, 2e-5, 1e-4)):
    """How far two correct evaluations of the FP8-activation prefill contract lie apart END TO END on the rows given:
    the oracle's f32-contract evaluation against evaluations whose gate and up sums are the f64 sums moved by
    eps * r * sum|terms| (r uniform in [-1, 1); eps = 0: the f64 sums themselves), each then re-quantised to e4m3 and put
    through the same down projection. Returns {eps: dict(h_equal, rel_r, rel_s, max_abs)} against the f32 contract's
    outputs: the reference tolerates 2e-5 on such sums for h and 1e-4 for outputs (test_experts.cu:352-407)."""
    base = [orc.moe_prefill_fp8_row(hl, x[t], idx[t], w[t]) for t in rows]
    ref_r, ref_s = np.stack([o["yr"] for o in base]), np.stack([o["ys"] for o in base])
    out = {}
    for eps in eps_list:
        got_r, got_s, same, total = [], [], 0, 0
        for o, t in zip(base, rows):
            hp = orc.moe_prefill_fp8_row_h_perturbed(hl, x[t], idx[t], eps, seed=1000 + t)
            same += int((hp == o["h"]).sum())
            total += hp.size
            o2 = orc.moe_prefill_fp8_row(hl, x[t], idx[t], w[t], h_in=hp)
            got_r.append(o2["yr"]), got_s.append(o2["ys"])
        got_r, got_s = np.stack(got_r), np.stack(got_s)
        out[eps] = dict(h_equal=same / total, rel_r=rel_l2(got_r, ref_r), rel_s=rel_l2(got_s, ref_s),
                        max_abs=float(max(np.abs(got_r - ref_r).max(), np.abs(got_s - ref_s).max())))
    return out
