"""The checkpoint binder (dsgx10_amd/weights.py): synthetic safetensors shards with the reference's tensor names
(altar1-4xgx10-switchless/engine/weights/int4_pack.py:354-366 load_expert, glw.py:419-431 the shared expert) -> layer ->
every byte read back. The pattern of the reference's packer tests: a packer, an independent reader, a round trip
(int4_pack.py:207-227 untile, :269-318 selftest)."""
import json
import os

import numpy as np
import pytest

from dsgx10_amd import abi, weights
from dsgx10_amd.layer import HostLayer
from tests import orc

H, I, E, LAYER = 256, 128, 5, 7


def _int4_ckpt(tmp, with_shape=True):
    mats = [[orc.int4_random(100 + 3 * e + j, *((I, H) if j < 2 else (H, I))) for j in range(3)] for e in range(E)]
    sh = [orc.normal_bf16(3, 40 + j, (I, H) if j < 2 else (H, I), 0.02) for j in range(3)]
    shards = [{}, {}]
    for e in range(E):
        for j, p in enumerate(weights.PROJ):
            n = "model.layers.%d.mlp.experts.%d.%s_proj." % (LAYER, e, p)
            packed, scale, zp = mats[e][j]
            t = shards[e % 2]
            t[n + "weight_packed"] = ("I32", packed.view(np.int32))
            t[n + "weight_scale"] = ("BF16", scale)
            t[n + "weight_zero_point"] = ("I32", zp.view(np.int32))
            if with_shape:
                t[n + "weight_shape"] = ("I64", np.array(((I, H) if j < 2 else (H, I)), np.int64))
    for j, p in enumerate(weights.PROJ):
        shards[1]["model.layers.%d.mlp.shared_experts.%s_proj.weight" % (LAYER, p)] = ("BF16", sh[j])
    wm = {}
    for i, t in enumerate(shards):
        fn = "model-%05d-of-00002.safetensors" % (i + 1)
        weights.write_shard(os.path.join(tmp, fn), t)
        wm.update({k: fn for k in t})
    with open(os.path.join(tmp, "model.safetensors.index.json"), "w") as f:
        json.dump({"weight_map": wm}, f)
    return mats, sh


def test_int4_layer_with_bf16_shared_expert_binds_and_reads_back(tmp_path):
    mats, sh = _int4_ckpt(str(tmp_path))
    hl = weights.load_layer(str(tmp_path), LAYER)
    assert (hl.fmt, hl.H, hl.I, hl.E, hl.topk) == (abi.FMT_INT4, H, I, E, E)
    # the same pool and descriptors as the layer assembled from the arrays directly
    bgu = np.empty((2 * I, H), np.uint16)
    bgu[0::2], bgu[1::2] = sh[0], sh[1]
    direct = HostLayer(abi.FMT_INT4, H, I, E, E, [tuple(m) for m in mats], emap=np.arange(E), shared_bf16=(bgu, sh[2]))
    assert np.array_equal(hl.pool, direct.pool) and hl.desc.tobytes() == direct.desc.tobytes()
    assert np.array_equal(hl.shared_bf16[0], bgu) and np.array_equal(hl.shared_bf16[1], sh[2])
    nbytes = weights.verify_layer(hl, str(tmp_path), LAYER)
    assert nbytes == E * 3 * (I * H // 2 + I * (H // 32) * 2 + (I // 8) * (H // 32) * 4)
    # the values the kernels will see: the dequantised matrix of (expert 3, down) from the bound pool
    packed, scale, zp = weights.read_back(hl, 3, 2)
    assert np.array_equal(orc.int4_dequant(packed, scale, zp), orc.int4_dequant(*mats[3][2]))
    # a subset of experts, renumbered
    sub = weights.load_layer(str(tmp_path), LAYER, experts=[4, 1])
    assert sub.E == 2 and weights.verify_layer(sub, str(tmp_path), LAYER, experts=[4, 1]) > 0
    assert np.array_equal(weights.read_back(sub, 0, 0)[0], mats[4][0][0])


def test_verifier_sees_one_flipped_byte(tmp_path):
    _int4_ckpt(str(tmp_path), with_shape=False)
    hl = weights.load_layer(str(tmp_path), LAYER)
    hl.pool[int(hl.desc[2 * 3 + 1]["off"]) + 17] ^= 0x10
    with pytest.raises(ValueError, match="expert 2 up_proj"):
        weights.verify_layer(hl, str(tmp_path), LAYER)


def test_fp8_layer_without_an_index_file(tmp_path):
    t = {}
    mats = []
    for e in range(3):
        ex = []
        for j, p in enumerate(weights.PROJ):
            codes, scales = orc.fp8_random(7 + 3 * e + j, *((I, H) if j < 2 else (H, I)), 1.0 / 512)
            n = "model.layers.0.mlp.experts.%d.%s_proj." % (e, p)
            t[n + "weight"] = ("F8_E4M3", codes)
            t[n + "weight_scale_inv"] = ("F32", scales)
            ex.append((codes, scales))
        mats.append(tuple(ex))
    shared = []
    for j, p in enumerate(weights.PROJ):
        codes, scales = orc.fp8_random(90 + j, *((I, H) if j < 2 else (H, I)), 1.0 / 512)
        t["model.layers.0.mlp.shared_experts.%s_proj.weight" % p] = ("F8_E4M3", codes)
        t["model.layers.0.mlp.shared_experts.%s_proj.weight_scale_inv" % p] = ("F32", scales)
        shared.append((codes, scales))
    weights.write_shard(os.path.join(str(tmp_path), "model.safetensors"), t)
    hl = weights.load_layer(str(tmp_path), 0, topk=2)
    assert (hl.fmt, hl.E, hl.topk) == (abi.FMT_FP8, 3, 2) and hl.shared_fp8 is not None
    assert weights.verify_layer(hl, str(tmp_path), 0) == 3 * 3 * (I * H + 2 * 4)  # codes + two block scales a matrix
    for e in range(3):
        for j in range(3):
            back = weights.read_back(hl, e, j)
            assert np.array_equal(back[0], mats[e][j][0]) and np.array_equal(back[1], mats[e][j][1])
    # the oracle runs over the bound layer: one row through expert 1 equals the same row over the arrays bound directly
    direct = HostLayer(abi.FMT_FP8, H, I, 3, 2, mats, emap=np.arange(3), shared_fp8=tuple(shared))
    x = orc.normal_bf16(1, 2, (1, H))
    uni = np.array([1], np.int32)
    assert np.array_equal(orc.moe_up(hl, x, uni, want_range=False)["h32"], orc.moe_up(direct, x, uni, want_range=False)["h32"])


def test_mixed_formats_and_missing_tensors_are_refused(tmp_path):
    packed, scale, zp = orc.int4_random(1, I, H)
    t = {}
    for j, p in enumerate(weights.PROJ):
        n = "model.layers.2.mlp.experts.0.%s_proj." % p
        if j == 1:
            t[n + "weight"] = ("BF16", orc.normal_bf16(1, 3, (I, H)))
        else:
            pk = orc.int4_random(1 + j, *((I, H) if j < 2 else (H, I)))
            t[n + "weight_packed"], t[n + "weight_scale"], t[n + "weight_zero_point"] = ("I32", pk[0].view(np.int32)), ("BF16", pk[1]), ("I32", pk[2].view(np.int32))
    weights.write_shard(os.path.join(str(tmp_path), "a.safetensors"), t)
    with pytest.raises(ValueError, match="format"):
        weights.load_layer(str(tmp_path), 2)
    with pytest.raises(ValueError, match="no routed experts"):
        weights.load_layer(str(tmp_path), 3)
