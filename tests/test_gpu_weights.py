"""A layer bound from safetensors shards (dsgx10_amd/weights.py) runs through dsgx_moe_decode like one assembled from
arrays: the checks of test_gpu_decode on a small INT4 layer with its BF16 shared expert, both kernel variants."""
import os

import numpy as np
import pytest

from dsgx10_amd import abi, weights
from tests import orc
from tests.helpers import rows_and_routing
from tests.test_gpu_decode import _check_step

pytestmark = pytest.mark.gpu


def test_decode_over_a_layer_bound_from_shards(tmp_path):
    H, I, E, topk = 2048, 2048, 3, 2
    t = {}
    for e in range(E):
        for j, p in enumerate(weights.PROJ):
            N, K = (I, H) if j < 2 else (H, I)
            w = orc.normal_f32(11, 50 + 3 * e + j, (N, K), 0.02)
            packed, scale, zp = orc.int4_quantize_sym(w)
            n = "model.layers.4.mlp.experts.%d.%s_proj." % (e, p)
            t[n + "weight_packed"], t[n + "weight_scale"] = ("I32", packed.view(np.int32)), ("BF16", scale)
            t[n + "weight_zero_point"] = ("I32", zp.view(np.int32))
    for j, p in enumerate(weights.PROJ):
        t["model.layers.4.mlp.shared_experts.%s_proj.weight" % p] = ("BF16", orc.normal_bf16(11, 90 + j, (I, H) if j < 2 else (H, I), 0.02))
    weights.write_shard(os.path.join(str(tmp_path), "model.safetensors"), t)
    hl = weights.load_layer(str(tmp_path), 4, topk=topk)
    assert weights.verify_layer(hl, str(tmp_path), 4) > 0
    dl = hl.upload()
    x, logits, idx, w = rows_and_routing(3, 4, H, E, topk, 2.5)
    for up in (0, 1):
        _check_step(hl, dl, x, idx, w, 4, up=up)
