#!/usr/bin/env python3
"""Benchmark of the quantised-MoE hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extra] [--no-cpu]

A step is one MoE layer: the router kernel plus the decode expert step (gate/up + SwiGLU, down + weighted sum) for M
rows, inputs resident in HBM. The headline workload is the FP8 MoE decode layer at M = 1 (hidden 4096, 256 routed
experts + 1 shared, intermediate 2048, e4m3 weights with 128 x 128 block scales, sigmoid top-8 renormalised). Every
step routes a different seeded logits row, so its experts come from a 6.4 GB pool and not from the caches; the shared
expert rotates over copies that together exceed the 256 MB Infinity Cache.

Prints ONE JSON line: metric us_per_moe_layer (lower is better), the roofline of the kernel the timed step launches
(the layer's algorithmic bytes over its time in the timed graph, HIP events on the launch stream; the gate/up kernel
launched alone is an extra field), the CPU baseline (the C++ oracle on the host cores over the same step, which also
checks the GPU's outputs) and, unless --no-extra, the other benchmark configurations, each decode configuration with
both kernel variants (dsgx_decode_cfg::up: 0 = dot products on the vector unit; 1 = on the bf16 MFMA) and each prefill
chunk with a few of its rows checked against the oracle.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published


def log(*a):
    print(*a, file=sys.stderr, flush=True)


# HBM bytes a launch of the FP8 M=1 decode kernel (k_decode), from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs of this
# script, each scaled by what the counter reads for a kernel of known size in the same run (profiles/): the algorithmic
# bytes are 226,547,712
LAYER_TRAFFIC_FP8_M1 = 229540000


def prefill_extra(gen, T, name, peak, check=True):
    """a prefill chunk of the benchmark: T rows, top-8 experts drawn from a Zipf(1.1) popularity, uniform weights; FP8
    weights and activations on the e4m3 MFMA (peak 5 PFLOP/s), or INT4 weights decoded to bf16 on the bf16 MFMA
    (2.5 PFLOP/s); TFLOP/s over the useful multiply-adds of the routed experts (T * 8 * 3 * I * H * 2)"""
    from benchdata import PrefillBench
    pb = PrefillBench(gen, T)
    t_routed, t_all = pb.time(15, False), pb.time(31, True)
    d = dict(workload=name, T=T, zipf_s=1.1, ms_routed=t_routed * 1e3, ms_with_shared=t_all * 1e3,
             tflops_routed=pb.flops_routed / t_routed / 1e12, tflops_with_shared=(pb.flops_routed + pb.flops_shared) / t_all / 1e12,
             mfma_peak_tflops=peak / 1e12, mfma_frac=pb.flops_routed / t_routed / peak,
             phases_ms={n: pb.time(ph, sh) * 1e3 for n, ph, sh in (("bucket", 1, False), ("up", 2, False), ("down", 4, False),
                                                                      ("combine", 8, False), ("shared", 16, True))})
    # the other roofline: every picked expert's weights once, x in, yr out (a chunk of few rows an expert is bound by these)
    import torch
    picked = int((torch.bincount(pb.idx.reshape(-1).long(), minlength=gen.E) > 0).sum())
    d["algorithmic_bytes_routed"] = picked * gen.expert_bytes + T * gen.H * (2 + 4)
    d["hbm_bound_ms"] = d["algorithmic_bytes_routed"] / (HBM_PEAK_GBS * 1e9) * 1e3
    d["mfma_bound_ms"] = pb.flops_routed / peak * 1e3
    d["hbm_frac"] = d["hbm_bound_ms"] / d["ms_routed"]
    d["bound"] = "hbm" if d["hbm_bound_ms"] > d["mfma_bound_ms"] else "mfma"
    log("  %s T=%d: routed %.3f ms (%.0f TFLOP/s, %.1f%% of %.1f PFLOP/s; %.2f GB of weights and rows at least: %.1f%% of 8 TB/s), with shared %.3f ms" %
        (name, T, d["ms_routed"], d["tflops_routed"], 100 * d["mfma_frac"], peak / 1e15, d["algorithmic_bytes_routed"] / 1e9,
         100 * d["hbm_frac"], d["ms_with_shared"]))
    if check:
        d["gpu_vs_oracle"] = prefill_check_rows(pb)
        log("  %s: rows %s against the oracle: max-abs %.2e, rel-L2 %.2e%s" %
            (name, d["gpu_vs_oracle"]["rows"], d["gpu_vs_oracle"]["max_abs_err"], d["gpu_vs_oracle"]["rel_l2"],
             "; against the oracle with sequential f32 block sums (the spread of correct evaluations): rel-L2 %.2e" % d["gpu_vs_oracle"]["vs_sequential_block_sums_rel_l2"]
             if "vs_sequential_block_sums_rel_l2" in d["gpu_vs_oracle"] else ""))
    del pb
    return d


def dsk_prefill_extra(T=8192, check=True):
    """DeepSeek's prefill MoE chunk (dsgx_dsk_moe_prefill): T rows, top-6 of 256 MXFP4 experts (Zipf(1.1)) + the FP8 shared expert,
    on the block-scaled e4m3 / e2m1 MFMA (peak 5 PFLOP/s: the wider operand sets the rate); phases: 1 bucketing, 2 shared
    expert, 4 gate/up, 8 down, 16 combine"""
    from benchdata import DskPrefillBench
    import torch
    pb = DskPrefillBench(T)
    peak = 5.0e15
    t_routed, t_all = pb.time(1 | 4 | 8 | 16), pb.time(31)
    picked = int((torch.bincount(pb.idx.reshape(-1).long(), minlength=pb.E) > 0).sum())
    d = dict(workload=pb.name, T=T, zipf_s=1.1, ms_routed=t_routed * 1e3, ms_with_shared=t_all * 1e3, tflops_routed=pb.flops_routed / t_routed / 1e12,
             tflops_with_shared=(pb.flops_routed + pb.flops_shared) / t_all / 1e12, mfma_peak_tflops=peak / 1e12, mfma_frac=pb.flops_routed / t_routed / peak,
             phases_ms={n: pb.time(ph) * 1e3 for n, ph in (("bucket", 1), ("shared", 2), ("up", 4), ("down", 8), ("combine", 16))},
             algorithmic_bytes_routed=picked * pb.expert_bytes + T * pb.H * (1 + 4) + T * pb.H // 32)
    d["hbm_bound_ms"] = d["algorithmic_bytes_routed"] / (HBM_PEAK_GBS * 1e9) * 1e3
    d["mfma_bound_ms"] = pb.flops_routed / peak * 1e3
    d["hbm_frac"] = d["hbm_bound_ms"] / d["ms_routed"]
    d["bound"] = "hbm" if d["hbm_bound_ms"] > d["mfma_bound_ms"] else "mfma"
    log("  %s T=%d: routed %.3f ms (%.0f TFLOP/s, %.1f%% of %.1f PFLOP/s; %.2f GB of weights and rows at least: %.1f%% of 8 TB/s), with shared %.3f ms; phases %s" %
        (pb.name, T, d["ms_routed"], d["tflops_routed"], 100 * d["mfma_frac"], peak / 1e15, d["algorithmic_bytes_routed"] / 1e9, 100 * d["hbm_frac"],
         d["ms_with_shared"], {k: round(v, 3) for k, v in d["phases_ms"].items()}))
    if check:
        d["gpu_vs_oracle"] = dsk_prefill_check_rows(pb)
        log("  %s: rows %s against the oracle's chain (the matrix unit's sums): max-abs %.2e, rel-L2 %.2e; against the oracle with sequential f32 sums: rel-L2 %.2e" %
            (pb.name, d["gpu_vs_oracle"]["rows"], d["gpu_vs_oracle"]["max_abs_err"], d["gpu_vs_oracle"]["rel_l2"], d["gpu_vs_oracle"]["vs_sequential_f32_sums_rel_l2"]))
    del pb
    return d


def dsk_prefill_check_rows(pb, rows=(0, 4097, 8191)):
    """Part of the CPU leg: a few rows of the chunk just timed against the C++ oracle's chain (each picked expert and the shared
    one: gate/up, clamped SwiGLU times the routing weight, h quantised per 32, w2, rounded to bf16; summed in expert-id order),
    with every dot product added as the block-scaled MFMA adds it (the rule pinned by tests/golden/mfma_scaled_k128.npz), and,
    beside it, with sequential f32 sums (two correct evaluations of the contract: their distance is what h's 3-bit-mantissa
    quantisation makes of sums that differ in the last bits)"""
    import torch
    from tests import orc   # the oracle: test infrastructure, used here as the checker only
    pb.run(31)
    torch.cuda.synchronize()
    rows = [t for t in rows if t < pb.T] or [0]
    host = lambda t: t.cpu().numpy()
    sh = tuple(orc.fp8e_dequant(host(pb.t["sh_w" + n]), host(pb.t["sh_s" + n])) for n in ("1", "3", "2"))
    worst = dict(rows=rows, max_abs_err=0.0, rel_l2=0.0, vs_sequential_f32_sums_rel_l2=0.0, vs_sequential_f32_sums_max_abs=0.0,
                 oracle="C++ oracle, DeepSeek's expert arithmetic with every dot product added as the block-scaled MFMA adds it")
    for t in rows:
        xq, xs = host(pb.xq[t:t + 1]), host(pb.xs[t:t + 1])
        xd = orc.dequant_act_ue8m0(xq, xs)
        ref, seq = np.zeros(pb.H, np.float32), np.zeros(pb.H, np.float32)
        idx, w = host(pb.idx[t]), host(pb.w[t])
        for e in sorted(int(v) for v in idx):
            raw = [(host(pb.t["w" + n][e]), host(pb.t["s" + n][e])) for n in ("1", "3", "2")]
            rw = np.array([w[list(idx).index(e)]], np.float32)
            hm = orc.dsk_up_mx(raw[0][0], raw[0][1], raw[1][0], raw[1][1], 1, xq, xs, rw)
            ref = ref + orc.bf16_to_f32(orc.dsk_down_mx(raw[2][0], raw[2][1], 1, hm)["outb"][0])
            w1, w3, w2 = (orc.mxfp4_dequant(*r) for r in raw)
            up = orc.dsk_up(w1, w3, xd, rw, want_range=False)
            seq = seq + orc.bf16_to_f32(orc.dsk_down(w2, up["h32"])["outb"][0])
        rawsh = [(host(pb.t["sh_w" + n]), host(pb.t["sh_s" + n])) for n in ("1", "3", "2")]
        hm = orc.dsk_up_mx(rawsh[0][0], rawsh[0][1], rawsh[1][0], rawsh[1][1], 0, xq, xs, None)
        ref = ref + orc.bf16_to_f32(orc.dsk_down_mx(rawsh[2][0], rawsh[2][1], 0, hm)["outb"][0])
        up = orc.dsk_up(sh[0], sh[1], xd, None, want_range=False)
        seq = seq + orc.bf16_to_f32(orc.dsk_down(sh[2], up["h32"])["outb"][0])
        got = host(pb.y[t])
        worst["max_abs_err"] = max(worst["max_abs_err"], float(np.abs(got - ref).max()))
        worst["rel_l2"] = max(worst["rel_l2"], float(np.linalg.norm(got - ref) / max(np.linalg.norm(ref), 1e-30)))
        worst["vs_sequential_f32_sums_max_abs"] = max(worst["vs_sequential_f32_sums_max_abs"], float(np.abs(got - seq).max()))
        worst["vs_sequential_f32_sums_rel_l2"] = max(worst["vs_sequential_f32_sums_rel_l2"], float(np.linalg.norm(got - seq) / max(np.linalg.norm(seq), 1e-30)))
    return worst


def chain_entries(gen, layers=96):
    """the layer chains of one format at one row: the MoE half alone (router GEMV + experts + add + norm) and the whole chain
    with the dense projections, each with the add + norms as launches of their own and fused into the GEMVs that read them"""
    from benchdata import ChainBench
    out = []
    for moe_only in (True, False):
        cb = ChainBench(gen, 1, layers, moe_only=moe_only)
        for fused in (False, True):
            d = cb.time(fused)
            log("  %s M=1 (add + norm %s): %.2f us a layer [%.2f .. %.2f] (%d layers in one graph, %.1f%% of 8 TB/s over %.0f MB)" %
                (d["workload"], "fused" if fused else "apart", d["us_per_layer"], d["us_per_layer_min"], d["us_per_layer_max"], d["layers"],
                 100 * d["hbm_frac"], d["bytes_per_layer"] / 1e6))
            out.append(d)
        del cb
    return out


def prefill_check_rows(pb, nrows=4):
    """Part of the CPU leg: a few rows of the chunk just timed against the C++ oracle (FP8 layers: the FP8-activation
    contract row by row; INT4 layers: a chunk row is a decode row). Returns the worst errors over the rows."""
    import torch
    from dsgx10_amd import abi
    from tests import orc   # the oracle: test infrastructure, used here as the checker only
    pb.run(31, True)
    torch.cuda.synchronize()
    T, gen = pb.T, pb.gen
    cnt = torch.bincount(pb.idx.reshape(-1).long(), minlength=gen.E).cpu().numpy()
    idx_h = pb.idx.cpu().numpy()
    hot, cold = int(np.argmax(cnt)), int(np.argmin(np.where(cnt > 0, cnt, 1 << 30)))
    rows = []
    for t in (int(np.nonzero((idx_h == hot).any(1))[0][-1]), int(np.nonzero((idx_h == cold).any(1))[0][0]), 0, T - 1, T // 2, T // 3):
        if t not in rows and len(rows) < nrows:
            rows.append(t)
    worst = dict(rows=rows, max_abs_err=0.0, rel_l2=0.0, oracle="C++ oracle; FP8 activations: each 128-k block added by the e4m3 MFMA's rule" if gen.fmt == abi.FMT_FP8 else "C++ oracle; a chunk row is a decode row, each sum added by the bf16 MFMA's rule in the kernels' k order")
    for t in rows:
        experts = sorted(int(e) for e in idx_h[t])
        hl = gen.host_sublayer(experts, 0)
        li = np.array([experts.index(int(e)) for e in idx_h[t]], np.int32)
        x = pb.x[t:t + 1].view(torch.int16).cpu().numpy().view(np.uint16)
        w = pb.w[t:t + 1].cpu().numpy()
        if gen.fmt == abi.FMT_FP8:
            # the contract's oracle with each 128-k block added by the matrix unit's rule (pinned by tests/golden/mfma_fp8_k128.npz:
            # what the e4m3 MFMA computes) ...
            orc.set_fp8_block_rule(1)
            o = orc.moe_prefill_fp8_row(hl, x[0], li, w[0])
            orc.set_fp8_block_rule(0)
            ref = [o["yr"], o["ys"]]
            # ... and with sequential f32 block sums (the reference's CPU stand-in): two correct evaluations whose sums differ by
            # ~1.5e-6 of their sums of |terms|, apart by what h's re-quantisation to e4m3 makes of that
            o0 = orc.moe_prefill_fp8_row(hl, x[0], li, w[0])
            for got, r in zip((pb.yr[t].cpu().numpy(), pb.ys[t].cpu().numpy()), (o0["yr"], o0["ys"])):
                worst["vs_sequential_block_sums_rel_l2"] = max(worst.get("vs_sequential_block_sums_rel_l2", 0.0),
                                                               float(np.sqrt(((got - r).astype(np.float64) ** 2).sum() / max((r.astype(np.float64) ** 2).sum(), 1e-300))))
                worst["vs_sequential_block_sums_max_abs"] = max(worst.get("vs_sequential_block_sums_max_abs", 0.0), float(np.abs(got - r).max()))
        else:
            # every sum added as the bf16 MFMA adds it in the kernels' k order (pinned by tests/golden/mfma_bf16_k32.npz) ...
            o = orc.moe_prefill_b16_row_mfma(hl, x[0], li, w[0])
            ref = [o["yr"], o["ys"]]
            # ... and the decode contract's sequential f32 sums
            uni = np.arange(len(experts), dtype=np.int32)
            up = orc.moe_up(hl, x, uni, want_range=False)
            dn = orc.moe_down(hl, up["h32"], li[None, :], w, uni)
            for got, r in zip((pb.yr[t].cpu().numpy(), pb.ys[t].cpu().numpy()), (dn["yr32"][0], dn["ys32"][0])):
                worst["vs_sequential_block_sums_rel_l2"] = max(worst.get("vs_sequential_block_sums_rel_l2", 0.0),
                                                               float(np.sqrt(((got - r).astype(np.float64) ** 2).sum() / max((r.astype(np.float64) ** 2).sum(), 1e-300))))
                worst["vs_sequential_block_sums_max_abs"] = max(worst.get("vs_sequential_block_sums_max_abs", 0.0), float(np.abs(got - r).max()))
        for got, r in zip((pb.yr[t].cpu().numpy(), pb.ys[t].cpu().numpy()), ref):
            worst["max_abs_err"] = max(worst["max_abs_err"], float(np.abs(got - r).max()))
            worst["rel_l2"] = max(worst["rel_l2"], float(np.sqrt(((got - r).astype(np.float64) ** 2).sum() / max((r.astype(np.float64) ** 2).sum(), 1e-300))))
    return worst


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=512)
    ap.add_argument("--warmup", type=int, default=64)
    ap.add_argument("--no-extra", action="store_true", help="only the headline workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--workload", default="fp8_m1", help="headline workload: fp8_m1 | int4_m1; fp8_prefill | int4_prefill time only that prefill chunk; gemv only the dense GEMVs; chain only the layer chains; dsk only the MXFP4 layer's decode steps; dsk_prefill only its prefill chunk")
    ap.add_argument("--variant", default="vector", choices=("vector", "mfma"),
                    help="the headline's decode kernels (dsgx_decode_cfg::up = 0 | 1); --no-extra then runs nothing else")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on one GPU (the whole layer is resident; no collectives are built); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    from dsgx10_amd import abi, lib
    from benchdata import DecodeBench, Fp8LayerGen, Int4LayerGen

    if not torch.cuda.is_available():
        print("bench.py: no GPU", file=sys.stderr)
        sys.exit(2)
    lib.lib()  # fails loudly when the HIP extension is not built
    torch.cuda.set_device(0)
    K, W = args.steps, args.warmup
    t_start = time.time()

    VARIANTS = ("vector", "mfma")  # dsgx_decode_cfg::up = 0, 1

    def run_decode(gen, M, steps, warmup, up=0):
        b = DecodeBench(gen, M, steps, up=up)
        r = b.time_layer(warmup)
        r.update(b.time_up_kernel())
        log("  %s M=%d (%s kernels): %.2f us/layer (%.1f%% of 8 TB/s), gate/up kernel %.2f us (%.1f%%)" %
            (gen.name, M, VARIANTS[up], r["us_per_layer"], 100 * r["layer_hbm_frac"], r["up_us"], 100 * r["up_frac"]))
        return b, r

    def decode_entry(gen, M, e, up):
        return dict(workload=gen.name, M=M, variant=VARIANTS[up], us_per_layer=e["us_per_layer"], bytes=e["bytes_per_layer"],
                    hbm_frac=e["layer_hbm_frac"], up_kernel_us=e["up_us"], up_hbm_frac=e["up_frac"])

    def cpu_baseline(b, budget_s):
        """The C++ oracle on the host cores over step 0 of the same workload (f32 contract sums only), repeated for about
        budget_s seconds; its result is also the checker of the GPU's outputs for that step."""
        from tests import orc   # the oracle: test infrastructure, used here as baseline and checker only
        d = b.run_step_and_download(0)
        hl, uni = d["layer"], np.arange(len(d["experts"]), dtype=np.int32)
        orc.set_f32_only(True)
        ts = []
        while (sum(ts) < budget_s and len(ts) < 200) or len(ts) < 3:
            t0 = time.perf_counter()
            up = orc.moe_up(hl, d["x"], uni, want_range=False)
            dn = orc.moe_down(hl, up["h32"], d["idx"], d["w"], uni)
            ts.append(time.perf_counter() - t0)
        orc.set_f32_only(False)
        def err(got, ref):
            return dict(max_abs_err=float(np.abs(got - ref).max()),
                        rel_l2=float(np.sqrt(((got - ref).astype(np.float64) ** 2).sum() / max((ref.astype(np.float64) ** 2).sum(), 1e-300))))
        par = {"yr": err(d["yr"], dn["yr32"])}
        if hl.has_shared:
            par["ys"] = err(d["ys"], dn["ys32"])
        # the same step with every dot product added in the kernels' own order (the oracle's restatement of v_dot2_f32_bf16 /
        # the bf16 MFMA, the lanes' split of K and the reduction tree): the outputs then agree bit for bit
        orc.set_dot_rule(2 if getattr(b, "up", 0) == 1 else 3)
        try:
            up2 = orc.moe_up(hl, d["x"], uni, want_range=False)
            dn2 = orc.moe_down(hl, up2["h32"], d["idx"], d["w"], uni)
        finally:
            orc.set_dot_rule(0)
        par["bits_equal_in_kernel_order"] = bool(np.array_equal(d["yr"].view(np.uint32), dn2["yr32"].view(np.uint32)) and
                                                 (not hl.has_shared or np.array_equal(d["ys"].view(np.uint32), dn2["ys32"].view(np.uint32))))
        return dict(value=float(np.mean(ts[1:]) * 1e6), unit="us", cores=orc.threads(), kind="port",
                    sample="step 0 of the same workload (M=%d, %d routed experts + shared), %d repetitions after one warm-up, "
                           "C++ oracle, OpenMP, f32 sums" % (b.M, len(d["experts"]), len(ts) - 1),
                    gpu_vs_oracle=par)

    if args.workload in ("fp8_prefill", "int4_prefill"):
        # only the prefill chunk (for profiler runs of the grouped-GEMM kernels): its own JSON line, TFLOP/s over useful MACs
        fp8 = args.workload == "fp8_prefill"
        gen = Fp8LayerGen(seed=0) if fp8 else Int4LayerGen(seed=0)
        d = prefill_extra(gen, 8192 if fp8 else 2048, args.workload.replace("_", "_moe_"), 5.0e15 if fp8 else 2.5e15, not args.no_cpu)
        print(json.dumps({"metric": "prefill_grouped_gemm_tflops", "value": d["tflops_routed"], "unit": "TFLOP/s", "n_gpus": 1, "steps": 8,
                          "warmup": 1, "ms_per_step": d["ms_routed"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
                          "dtype": "fp8 (e4m3 x e4m3, f32 sums)" if fp8 else "bf16 (INT4 weights decoded to bf16, f32 sums)", "data": "synthetic",
                          "config": {"workload": d["workload"], "T": d["T"]},
                          "roofline": ({"bound": "hbm", "achieved": d["algorithmic_bytes_routed"] / d["ms_routed"] * 1e-6, "peak": HBM_PEAK_GBS,
                                        "unit": "GB/s", "frac": d["hbm_frac"], "traffic": None, "mfma_frac": d["mfma_frac"]} if d["bound"] == "hbm" else
                                       {"bound": "mfma", "achieved": d["tflops_routed"], "peak": d["mfma_peak_tflops"], "unit": "TFLOP/s",
                                        "frac": d["mfma_frac"], "traffic": None, "hbm_frac": d["hbm_frac"]}),
                          "cpu_baseline": None, "extra": [d], "wall_s": round(time.time() - t_start, 1)}))
        return
    if args.workload == "dsk":
        # only DeepSeek's MXFP4 layer (dsgx_dsk_moe, routing fused), M = 1, 2, 4, 8
        from benchdata import DskBench, DskLayerGen
        dg = DskLayerGen(seed=0)
        ds = []
        for M in (1, 2, 4, 8):
            ds.append(DskBench(dg, M, 128).time())
            log("  %s M=%d: %.2f us/layer (%.1f%% of 8 TB/s)" % (ds[-1]["workload"], M, ds[-1]["us_per_layer"], 100 * ds[-1]["hbm_frac"]))
        print(json.dumps({"metric": "us_per_moe_layer", "value": ds[0]["us_per_layer"], "unit": "us", "n_gpus": 1, "steps": 128, "warmup": 4,
                          "ms_per_step": ds[0]["us_per_layer"] * 1e-3, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
                          "dtype": "f32 sums of exact bf16 x bf16 products (MXFP4 / e4m3 values times power-of-two scales)", "data": "synthetic",
                          "config": {"workload": ds[0]["workload"], "rows_M": 1},
                          "roofline": {"bound": "hbm", "achieved": ds[0]["bytes"] / ds[0]["us_per_layer"] * 1e-3, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                       "frac": ds[0]["hbm_frac"], "traffic": None},
                          "cpu_baseline": None, "extra": ds, "wall_s": round(time.time() - t_start, 1)}))
        return
    if args.workload == "dsk_prefill":
        d = dsk_prefill_extra(8192, check=not args.no_cpu)
        print(json.dumps({"metric": "ms_per_prefill_chunk", "value": d["ms_routed"], "unit": "ms", "n_gpus": 1, "steps": 8, "warmup": 1, "ms_per_step": d["ms_routed"],
                          "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "e2m1 / e4m3 x e4m3 with ue8m0 scales, f32 sums (block-scaled MFMA)",
                          "data": "synthetic", "config": {"workload": d["workload"], "T": d["T"]},
                          "roofline": {"bound": "mfma", "achieved": d["tflops_routed"], "peak": d["mfma_peak_tflops"], "unit": "TFLOP/s", "frac": d["mfma_frac"],
                                       "traffic": None, "hbm_frac": d["hbm_frac"]},
                          "cpu_baseline": None, "extra": [d], "wall_s": round(time.time() - t_start, 1)}))
        return
    if args.workload == "chain":
        # only the layer chains (router GEMV -> experts -> add + norm, 128 layers a graph), FP8 then INT4
        from benchdata import ChainBench
        ds = []
        for cls in (Fp8LayerGen, Int4LayerGen):
            g2 = cls(seed=0)
            ds += chain_entries(g2)
            del g2
        print(json.dumps({"metric": "us_per_moe_layer_step", "value": ds[0]["us_per_layer"], "unit": "us", "n_gpus": 1, "steps": 128, "warmup": 4,
                          "ms_per_step": ds[0]["us_per_layer"] * 1e-3, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
                          "dtype": "f32 sums of bf16 x bf16 products", "data": "synthetic", "config": {"workload": ds[0]["workload"], "rows_M": 1},
                          "roofline": None, "cpu_baseline": None, "extra": ds, "wall_s": round(time.time() - t_start, 1)}))
        return
    if args.workload == "gemv":
        # only the dense GEMVs (for profiler runs): one line, the FP8 [2048 x 4096] row-1 call as the value
        from benchdata import gemv_bench
        g = gemv_bench()
        head = min((d for d in g if d["workload"].startswith("dense_fp8")), key=lambda d: d["us_per_call"])
        print(json.dumps({"metric": "dense_gemv_us", "value": head["us_per_call"], "unit": "us", "n_gpus": 1, "steps": 64, "warmup": 4,
                          "ms_per_step": head["us_per_call"] * 1e-3, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
                          "dtype": "f32 sums of bf16 x bf16 products", "data": "synthetic", "config": {"workload": head["workload"], "rows_M": 1},
                          "roofline": {"bound": "hbm", "achieved": head["bytes"] / head["us_per_call"] * 1e-3, "peak": 8000.0, "unit": "GB/s",
                                       "frac": head["hbm_frac"], "traffic": None},
                          "cpu_baseline": None, "extra": g, "wall_s": round(time.time() - t_start, 1)}))
        return
    head_fp8 = args.workload == "fp8_m1"
    log("generating the %s layer ..." % ("FP8 256-expert" if head_fp8 else "INT4 168-expert"))
    gen = Fp8LayerGen(seed=0) if head_fp8 else Int4LayerGen(seed=0)
    log("  %.1f s, pool %.2f GB" % (time.time() - t_start, gen.pool.numel() / 1e9))
    stream_gbs = gen.stream_read_gbs()
    head_up = 1 if args.variant == "mfma" else 0
    b, r = run_decode(gen, 1, K, W, head_up)
    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(b, 10.0)
        log("  cpu baseline: %.0f us on %d cores; gpu vs oracle %s" % (cpu["value"], cpu["cores"], cpu["gpu_vs_oracle"]))
    extra = []
    if not args.no_extra:
        ks = min(K, 128)
        del b
        _, e = run_decode(gen, 1, K, W, up=1 - head_up)
        extra.append(decode_entry(gen, 1, e, 1 - head_up))
        for M in (4, 8):
            for up in (0, 1):
                _, e = run_decode(gen, M, ks, min(W, 16), up)
                extra.append(decode_entry(gen, M, e, up))
        extra.append(prefill_extra(gen, 8192, "fp8_moe_prefill", 5.0e15, not args.no_cpu) if head_fp8 else prefill_extra(gen, 2048, "int4_moe_prefill", 2.5e15, not args.no_cpu))
        other = Int4LayerGen(seed=0) if head_fp8 else Fp8LayerGen(seed=0)
        for M in (1, 8):
            for up in (0, 1):
                ob, e = run_decode(other, M, ks if M > 1 else K, min(W, 16), up)
                d = decode_entry(other, M, e, up)
                if M == 1 and not args.no_cpu:
                    d["cpu_baseline"] = cpu_baseline(ob, 3.0)
                extra.append(d)
                del ob
        extra.append(prefill_extra(other, 2048, "int4_moe_prefill", 2.5e15, not args.no_cpu) if head_fp8 else prefill_extra(other, 8192, "fp8_moe_prefill", 5.0e15, not args.no_cpu))
        from benchdata import ChainBench, DskBench, DskLayerGen, gemv_bench
        for g2 in (gen, other):
            extra += chain_entries(g2)
        del other
        dg = DskLayerGen(seed=0)
        for M in (1, 8):
            d = DskBench(dg, M, 128).time()
            log("  %s M=%d: %.2f us/layer (%.1f%% of 8 TB/s)" % (d["workload"], M, d["us_per_layer"], 100 * d["hbm_frac"]))
            extra.append(d)
        del dg
        import torch
        torch.cuda.empty_cache()
        extra.append(dsk_prefill_extra(8192, check=not args.no_cpu))
        extra += gemv_bench()

    out = {
        "metric": "us_per_moe_layer",
        "value": r["us_per_layer"],
        "unit": "us",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": r["us_per_layer"] / 1000.0,
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic (seeded splitmix64 / Box-Muller values: N(0,0.02) weights quantised on the GPU, N(0,1) bf16 rows and f32 logits)",
        "config": {"workload": gen.describe(1), "arithmetic": "f32 sums of bf16 x bf16 products (weights decoded to bf16 in registers)", "rows_M": 1, "steps_route_different_experts": True,
                   "bytes_per_layer": r["bytes_per_layer"], "layer_hbm_frac_of_8TBs": r["layer_hbm_frac"],
                   "variant": args.variant,
                   "kernels_per_step": ["k_decode (routing + gate/up + SwiGLU + down + weighted sum, one persistent launch)"] if head_up == 0 else
                                       ["k_decode_mfma (routing + gate/up + SwiGLU + down, one persistent launch)", "k_down_combine (weighted sum in expert order)"],
                   "timed_as": "one HIP graph of all steps; the median of 7 replays", "us_min_max_of_replays": [r["us_per_layer_min"], r["us_per_layer_max"]]},
        # the kernel(s) of the timed step: the algorithmic bytes of a layer (every weight byte of the picked experts and the
        # shared expert once, scales included) over the step's time in the timed graph (HIP events on the launch stream)
        "roofline": {"bound": "hbm",
                     "kernel": "k_decode<FP8_B128, FP8_B128, 1, 2>" if head_fp8 and head_up == 0 else
                               ("k_decode" if head_up == 0 else "k_decode_mfma + k_down_combine"),
                     "achieved": r["bytes_per_layer"] / (r["us_per_layer"] * 1e-6) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": r["layer_hbm_frac"], "traffic": LAYER_TRAFFIC_FP8_M1 if head_fp8 and head_up == 0 else None,
                     "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of an earlier run of this command (profiles/k_decode_fp8_m1_one_launch.md), not measured in this run",
                     "bytes_per_launch": r["bytes_per_layer"], "avg_launch_us": r["us_per_layer"],
                     "gate_up_kernel_alone": {"kernel": "k_up" if head_up == 0 else "k_up_mfma", "avg_launch_us": r["up_us"],
                                              "bytes_per_launch": r["up_bytes"], "achieved": r["up_gbs"], "frac": r["up_frac"]},
                     "measured_stream_read_gbs": stream_gbs},
        "cpu_baseline": cpu,
        "extra": extra,
        "wall_s": round(time.time() - t_start, 1),
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
