"""GPU parity of DeepSeek's prefill MoE (dsgx_dsk_moe_prefill = dsk::moe_prefill of the reference,
ds41f-4xgx10-switchless/engine/kernels/dsk.h:268-295, prefill.cu:1605-1675) against the CPU oracle, stage by stage as the
reference tests its prefill kernels (engine/kernels/tests/test_kernels.cu: each GEMM against an fp64 host reference from the
kernel's own inputs, then y):
  the block-scaled matrix instruction itself against the dequantised products (one instruction, both weight formats);
  h (bf16, before its quantisation) inside the range the oracle allows at the reference's sum tolerance (1e-4 sum|terms|) and
  equal to the oracle's in >= 98.5% of bits (the reference's bar for a prefill chunk, experts/tests/test_prefill.inc:183-186);
  h's quantisation (codes and scale bytes) equal to the oracle's act_quant of the GPU's own h, bit for bit;
  each pick's w2 output (bf16) from the GPU's own h within 1e-4 sum|terms| + one bf16 step of the f64 sums;
  y equal, bit for bit, to the f32 fold of the GPU's own outputs in expert-id order with the shared expert last;
  y against the oracle's chain at max-abs 2e-2 / rel-L2 3e-3, and against the decode operator on the same rows;
  and, bit for bit, against the oracle variant that adds every dot product as the matrix instruction does (orc_dsk_up_mx /
  orc_dsk_down_mx over the rule of tests/golden/mfma_scaled_k128.npz): each pick's w2 output from the GPU's own h equal in
  every bit, h equal but for the rare value where expf() on the two sides rounds apart."""
import ctypes as C

import numpy as np
import pytest

from dsgx10_amd import abi, lib
from tests import gpu, orc
from tests.test_gpu_dsk import _fp4_mat, _fp8e_mat

pytestmark = pytest.mark.gpu


def test_scaled_mfma_is_the_dequantised_product():
    """one v_mfma_scale_f32_16x16x128_f8f6f4 with e2m1 or e4m3 weights: the lane's scale byte belongs to its 32 k, the low
    nibble is the even k, out[i][j] pairs A's row i with B's row j"""
    rng = np.random.default_rng(5)
    e2m1, e4m3 = orc.e2m1_table(), orc.e4m3_table()
    for a_fp4 in (1, 0):
        for trial in range(4):
            sa, sb = rng.integers(120, 131, (16, 4), dtype=np.uint8), rng.integers(121, 130, (16, 4), dtype=np.uint8)
            b = orc.f32_to_e4m3(np.clip(rng.standard_normal((16, 128)).astype(np.float32) * 30.0, -448, 448))
            if a_fp4:
                codes = rng.integers(0, 16, (16, 128), dtype=np.uint8)
                a = (codes[:, 0::2] | (codes[:, 1::2] << 4)).astype(np.uint8)
                av = e2m1[codes].astype(np.float64)
            else:
                a = orc.f32_to_e4m3(np.clip(rng.standard_normal((16, 128)).astype(np.float32) * 30.0, -448, 448))
                av = e4m3[a].astype(np.float64)
            if trial == 3:  # a sparse case whose sums are exact in f32: the result must be exact
                keep = np.zeros((16, 128), bool)
                keep[:, rng.integers(0, 128, 5)] = True
                b = np.where(keep, b, 0).astype(np.uint8)
            av = av * np.repeat(2.0 ** (sa.astype(np.float64) - 127), 32, axis=1)
            bv = e4m3[b].astype(np.float64) * np.repeat(2.0 ** (sb.astype(np.float64) - 127), 32, axis=1)
            want, mag = av @ bv.T, np.abs(av) @ np.abs(bv).T
            out = gpu.empty(16 * 16 * 4, 0xFF)
            lib.probe_mfma_scaled(gpu.dev(a), gpu.dev(sa), gpu.dev(b), gpu.dev(sb), a_fp4, out)
            got = gpu.host(out, np.float32, (16, 16)).astype(np.float64)
            err = np.abs(got - want)
            assert np.all(err <= 1e-4 * mag + 1e-30), (a_fp4, trial, float((err / np.maximum(mag, 1e-30)).max()))
            if trial == 3:
                assert np.array_equal(got.astype(np.float32), want.astype(np.float32)), (a_fp4, "sparse")
            # and, on these fresh operands, bit for bit what the oracle's statement of the instruction's summation gives
            rule = orc.mfma_scaled_k128(a, sa, a_fp4, b, sb)
            assert np.array_equal(rule.view(np.uint32), got.astype(np.float32).view(np.uint32)), (a_fp4, trial, int((rule != got.astype(np.float32)).sum()))


class Stacked:
    """experts stacked by id as dsk::MoeWeights wants them, from `ns` distinct experts mapped onto E ids"""

    def __init__(self, seed, H, I, E, topk, ns, shared):
        rng = np.random.default_rng(seed)
        self.H, self.I, self.E, self.topk = H, I, E, topk
        self.experts = [(_fp4_mat(rng, I, H), _fp4_mat(rng, I, H), _fp4_mat(rng, H, I, 118, 123)) for _ in range(ns)]
        self.shared = (_fp8e_mat(rng, I, H), _fp8e_mat(rng, I, H), _fp8e_mat(rng, H, I, 114, 119)) if shared else None
        self.emap = np.array([(7 * e + 3) % ns for e in range(E)])
        import torch
        self.dev = {}
        for j, n in enumerate(("1", "3", "2")):
            wsrc = torch.stack([torch.from_numpy(ex[j][0]) for ex in self.experts]).cuda()
            ssrc = torch.stack([torch.from_numpy(ex[j][1]) for ex in self.experts]).cuda()
            sel = torch.from_numpy(self.emap).cuda()
            self.dev["w" + n], self.dev["s" + n] = wsrc[sel].contiguous(), ssrc[sel].contiguous()
            if shared:
                self.dev["sh_w" + n], self.dev["sh_s" + n] = gpu.dev(self.shared[j][0]), gpu.dev(self.shared[j][1])
        p = lambda k: self.dev[k].data_ptr() if k in self.dev else None
        self.w = abi.DskWeights(p("w1"), p("s1"), p("w3"), p("s3"), p("w2"), p("s2"), p("sh_w1"), p("sh_s1"), p("sh_w3"), p("sh_s3"), p("sh_w2"), p("sh_s2"),
                                H, I, E, topk)
        self._deq = {}

    def raw(self, e):
        """the stored tensors ((w1, s1), (w3, s3), (w2, s2)) of expert id e (-1: the shared expert) and whether they are e2m1"""
        return (self.shared, 0) if e < 0 else (self.experts[int(self.emap[e])], 1)

    def deq(self, e):
        """dequantised (w1, w3, w2) of expert id e (-1: the shared expert)"""
        k = -1 if e < 0 else int(self.emap[e])
        if k not in self._deq:
            src = self.shared if k < 0 else self.experts[k]
            f = orc.fp8e_dequant if k < 0 else orc.mxfp4_dequant
            self._deq[k] = tuple(f(*src[j]) for j in range(3))
        return self._deq[k]


def run_prefill(L, xq, xs, idx, w, phases=31):
    T, H, I, topk = xq.shape[0], L.H, L.I, L.topk
    ws = gpu.empty(lib.dsk_prefill_ws_bytes(H, I, L.E, topk, T), 0xEE)
    y = gpu.empty(T * H * 4, 0xFF)
    lib.dsk_moe_prefill(L.w, gpu.dev(xq), gpu.dev(xs), gpu.dev(idx), gpu.dev(w), T, ws, y, phases=phases)
    v = lib.dsk_prefill_view(L.w, ws, T)
    P = T * topk
    take = lambda ptr, n, dt, shape: gpu.host(gpu.view(ws, ptr, n), dt, shape)
    out = dict(y=gpu.host(y, np.float32, (T, H)), rpos=take(v.rpos, P * 4, np.int32, (T, topk)), re=take(v.re, P * 4, np.int32, (T, topk)),
               perm=take(v.perm, P * 4, np.int32, (P,)), off=take(v.off, (L.E + 1) * 4, np.int32, (L.E + 1,)),
               h=take(v.h, P * I * 2, np.uint16, (P, I)), hq=take(v.hq, P * I, np.uint8, (P, I)), hs=take(v.hs, P * (I // 32), np.uint8, (P, I // 32)),
               d=take(v.d, P * H * 2, np.uint16, (P, H)))
    if L.shared is not None:
        out["hsh"] = take(v.hsh, T * I * 2, np.uint16, (T, I))
        out["dsh"] = take(v.dsh, T * H * 2, np.uint16, (T, H))
    return out


def check_chunk(L, x, idx, w, rows, got, note="", e2e=3e-3):
    """parity of the sampled rows of a chunk (every stage; see the module's docstring); returns the figures it prints"""
    H, I, topk = L.H, L.I, L.topk
    xq, xs = orc.act_quant_ue8m0(x)
    xd = orc.dequant_act_ue8m0(xq, xs)
    T = x.shape[0]
    # the bucketing: ids ascending per row, positions inside their expert's bucket, in token order
    for t in rows:
        assert np.array_equal(got["re"][t], np.sort(idx[t])), t
        for r in range(topk):
            e, pos = got["re"][t][r], got["rpos"][t][r]
            assert got["off"][e] <= pos < got["off"][e + 1] and got["perm"][pos] == t
    assert np.all(np.diff(got["perm"][got["off"][3]:got["off"][4]]) > 0)
    nh = nbad = nbad_mx = ny = nybad = 0
    ref = np.zeros((len(rows), H), np.float64)
    worst_d = 0.0
    for i, t in enumerate(rows):
        fold = np.zeros(H, np.float32)
        slots = [(int(got["re"][t][r]), int(got["rpos"][t][r])) for r in range(topk)] + ([(-1, t)] if L.shared is not None else [])
        for e, pos in slots:
            w1, w3, w2 = L.deq(e)
            rw = None if e < 0 else np.array([w[t][list(idx[t]).index(e)]], np.float32)
            up = orc.dsk_up(w1, w3, xd[t:t + 1], rw, sum_tol=1e-4)
            hg = (got["hsh"] if e < 0 else got["h"])[pos]
            hf = orc.bf16_to_f32(hg)
            assert np.all(hf >= up["lo"][0] - 1e-30) and np.all(hf <= up["hi"][0] + 1e-30), (t, e, note)
            nbad += int((hg != up["h64"][0]).sum())
            nh += I
            # the oracle that adds every dot product as the matrix instruction does (its rule: tests/golden/mfma_scaled_k128.npz):
            # h equal but for the rare value where the two exponential routines round apart, everything after it bit for bit
            (r1, r3, r2), f4 = L.raw(e)
            hm = orc.dsk_up_mx(r1[0], r1[1], r3[0], r3[1], f4, xq[t:t + 1], xs[t:t + 1], rw)[0]
            nbad_mx += int((hg != hm).sum())
            dm = orc.dsk_down_mx(r2[0], r2[1], f4, hg[None, :])
            chain = orc.dsk_down_mx(r2[0], r2[1], f4, hm[None, :])["outb"][0]
            own = orc.dsk_down(w2, hg[None, :])
            if e >= 0:  # the quantisation of h as the down GEMM read it
                assert np.array_equal(got["hq"][pos], own["hq"][0]) and np.array_equal(got["hs"][pos], own["hs"][0]), (t, e)
            dg = (got["dsh"] if e < 0 else got["d"])[pos]
            assert np.array_equal(dg, dm["outb"][0]), (t, e, "w2 from the GPU's own h: the matrix unit's sums", int((dg != dm["outb"][0]).sum()))
            ny += H
            nybad += int((dg != chain).sum())
            err = np.abs(orc.bf16_to_f32(dg).astype(np.float64) - own["out64"][0])
            tol = 1e-4 * own["mag"][0] + np.abs(own["out64"][0]) * 2.0 ** -8
            assert np.all(err <= tol), (t, e, float((err / tol).max()))
            worst_d = max(worst_d, float((err / np.maximum(tol, 1e-300)).max()))
            fold = fold + orc.bf16_to_f32(dg)
            ref[i] += orc.bf16_to_f32(orc.dsk_down(w2, up["h32"])["outb"][0])
        assert np.array_equal(got["y"][t].view(np.uint32), fold.view(np.uint32)), (t, "the ordered fold")
    y = got["y"][rows]
    rl2 = np.linalg.norm(y - ref) / max(np.linalg.norm(ref), 1e-30)
    print("dsk prefill %s H=%d I=%d T=%d: %d rows checked, h equal %.2f%%, w2 worst %.2f of its tolerance, end-to-end rel-L2 %.2e max-abs %.2e (|y| max %.2f)"
          % (note, H, I, T, len(rows), 100 - 100.0 * nbad / nh, worst_d, rl2, np.abs(y - ref).max(), np.abs(ref).max()))
    print("  against the oracle with the matrix unit's sums: h differs in %d of %d values, the picks' outputs from the oracle's own h in %d of %d"
          % (nbad_mx, nh, nybad, ny))
    assert nbad_mx <= 2e-4 * nh + 1, (nbad_mx, nh)
    assert nybad <= 2e-3 * ny + 8, (nybad, ny)
    assert nbad <= 0.015 * nh, (nbad, nh)
    assert np.abs(y - ref).max() <= 2e-2 + 2.0 ** -7 * np.abs(ref).max()
    assert rl2 <= e2e
    return rl2


@pytest.mark.parametrize("H,I,E,T,shared", [(1024, 512, 16, 300, True), (2048, 768, 8, 700, True), (1024, 256, 32, 37, False), (1024, 512, 16, 1, True)])
def test_dsk_prefill_against_oracle(H, I, E, T, shared):
    """T = 700 over 8 experts: buckets of ~500 rows, i.e. 256-position tiles and ragged remainders; T = 37 over 32: experts
    with no rows at all; T = 1"""
    topk = 6
    L = Stacked(41, H, I, E, topk, 5, shared)
    x = orc.normal_bf16(41, 1, (T, H), 1.5)
    logits, bias = orc.normal_f32(41, 2, (T, E), 1.0), orc.normal_f32(41, 3, (E,), 0.2)
    idx, w = orc.route(logits, bias, topk, 1.5, score_fn=1)
    xq, xs = orc.act_quant_ue8m0(x)
    got = run_prefill(L, xq, xs, idx, w)
    rows = sorted(set([0, T - 1] + list(np.random.default_rng(1).integers(0, T, 10))))
    check_chunk(L, x, idx, w, rows, got)
    # against the decode operator on the same rows (different sums inside a dot product: close, not equal)
    M = min(T, 8)
    ws = gpu.empty(lib.dsk_ws_bytes(H, I), 0)
    yd = gpu.empty(M * H * 4, 0xFF)
    lib.dsk_moe_stacked(L.w, gpu.dev(xq[:M]), gpu.dev(xs[:M]), gpu.dev(idx[:M]), gpu.dev(w[:M]), M, ws, yd)
    yd = gpu.host(yd, np.float32, (M, H))
    rel = np.linalg.norm(got["y"][:M] - yd) / np.linalg.norm(yd)
    print("  against dsk::moe on the first %d rows: rel-L2 %.2e" % (M, rel))
    assert rel <= 5e-3
    # phases apart give the same bits as the whole step
    if T == 300:
        ws2 = gpu.empty(lib.dsk_prefill_ws_bytes(H, I, E, topk, T), 0x11)
        y2 = gpu.empty(T * H * 4, 0)
        for ph in (1, 2, 4, 8, 16):
            lib.dsk_moe_prefill(L.w, gpu.dev(xq), gpu.dev(xs), gpu.dev(idx), gpu.dev(w), T, ws2, y2, phases=ph)
        assert np.array_equal(gpu.host(y2, np.uint32, (T, H)), got["y"].view(np.uint32))


def test_dsk_prefill_refuses_what_it_cannot_run():
    L = Stacked(42, 1024, 512, 16, 6, 2, False)
    xq = gpu.empty(4 * 1024, 0)
    with pytest.raises(lib.DsgxError):
        lib.dsk_moe_prefill(L.w, xq, None, xq, xq, 4, xq, xq)  # null scales
    bad = abi.DskWeights.from_buffer_copy(L.w)
    bad.H = 1000
    assert lib.dsk_prefill_ws_bytes(1000, 512, 16, 6, 4) == 0
    with pytest.raises(lib.DsgxError):
        lib.dsk_moe_prefill(bad, xq, xq, xq, xq, 4, xq, xq)
    assert C.sizeof(abi.DskPrefillCfg) == 8


def test_dsk_prefill_at_the_layer_shape():
    """DeepSeek's unsharded layer (hidden 5120, intermediate 2304, 256 experts, top-6 + shared) on a whole chunk of 8192 rows
    with Zipf(1.1) picks: six stored experts aliased under all ids (the reference's testdata.h:197 does the same), every
    index, offset and launch shape the benchmark's. Sampled rows stage by stage; chunk independence (a row's y in a chunk of
    its own equals its y in the big chunk: the grouped GEMMs' sums do not depend on the tile a row falls in). The K = 5120
    sums of the block-scaled MFMA move ~1% of h by a bf16 step, which h's e4m3 quantisation (3 mantissa bits) carries into y:
    measured 8e-4 of relative L2 end to end here; the stage-wise bounds are the tight ones."""
    from tests.helpers import zipf_picks
    H, I, E, topk, T = 5120, 2304, 256, 6, 8192
    L = Stacked(43, H, I, E, topk, 6, True)
    x = orc.normal_bf16(43, 1, (T, H), 1.5)
    idx, _ = zipf_picks(T, E, topk, 1.1, seed=43)
    w = np.abs(orc.normal_f32(43, 4, (T, topk), 0.3)).astype(np.float32) + 0.05
    xq, xs = orc.act_quant_ue8m0(x)
    got = run_prefill(L, xq, xs, idx, w)
    cnt = np.bincount(idx.reshape(-1), minlength=E)
    assert np.array_equal(got["off"], np.concatenate([[0], np.cumsum(cnt)]))
    assert np.array_equal(np.sort(got["perm"].reshape(-1)), np.sort(np.repeat(np.arange(T), topk)))
    hot, cold = int(np.argmax(cnt)), int(np.argmin(np.where(cnt > 0, cnt, 1 << 30)))
    rows = sorted(set([0, T - 1, T // 2, int(np.nonzero((idx == hot).any(1))[0][-1]), int(np.nonzero((idx == cold).any(1))[0][0])]))
    check_chunk(L, x, idx, w, rows, got, note="layer shape")
    assert np.isfinite(got["y"]).all()
    sub = rows[:3]
    got1 = run_prefill(L, xq[sub], xs[sub], idx[sub], w[sub])
    assert np.array_equal(got1["y"].view(np.uint32), got["y"][sub].view(np.uint32))
