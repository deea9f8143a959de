"""GPU test of dsgx_moe_decode_noalloc (the decode step on the library's built-in workspace, for callers that cannot
allocate): the same bits as dsgx_moe_decode with a caller's workspace, on two calls in a row, the second with a smaller
input, for both kernel variants and both weight formats; sizes beyond the built-in workspace are refused."""
import numpy as np
import pytest
import torch

from dsgx10_amd import abi, lib
from tests import gpu
from tests.helpers import make_layer, rows_and_routing

pytestmark = pytest.mark.gpu


def _both(dl, x, idx, w, M, **kw):
    """(yr, ys) through the caller's workspace and through the built-in one"""
    H = dl.host.H
    dx, di, dw = gpu.dev(x[:M]), gpu.dev(idx[:M]), gpu.dev(w[:M])
    out = []
    for own_ws in (True, False):
        ws = gpu.empty(lib.decode_ws_bytes(dl.w), 0) if own_ws else None
        yr, ys = gpu.empty(M * H * 4, 0xFF), gpu.empty(M * H * 4, 0xFF)
        lib.moe_decode(dl.w, dx, di, dw, M, ws, yr, ys, **kw)
        lib.decode_status(dl.w, ws)
        out.append((gpu.host(yr, np.uint32, (M, H)), gpu.host(ys, np.uint32, (M, H))))
    return out


@pytest.mark.parametrize("fmt,shared,scale", [(abi.FMT_FP8, "fp8", 1.0), (abi.FMT_INT4, "bf16", 2.5)])
def test_noalloc_equals_caller_workspace_twice(fmt, shared, scale):
    big = make_layer(fmt, 2048, 2048, 32, 8, 4, seed=2, shared=shared).upload()
    small = make_layer(fmt, 2048 if fmt == abi.FMT_INT4 else 1024, 2048 if fmt == abi.FMT_INT4 else 1024, 16, 4, 3, seed=4, shared=None).upload()
    xb, _, ib, wb = rows_and_routing(41, 8, big.host.H, 32, 8, scale)
    xs, _, is_, ws_ = rows_and_routing(42, 8, small.host.H, 16, 4, scale)
    for up in (0, 1):
        # first call: 8 rows of the larger layer (a large union: the slot-partitioned down phase and its f32 buffer);
        # second call: fewer rows, then a smaller layer (the workspace still holds the first call's contents)
        for dl, x, idx, w, M in ((big, xb, ib, wb, 8), (big, xb, ib, wb, 3), (small, xs, is_, ws_, 1), (big, xb, ib, wb, 8)):
            (yr_a, ys_a), (yr_b, ys_b) = _both(dl, x, idx, w, M, up=up)
            assert np.array_equal(yr_a, yr_b), (fmt, up, M)
            if dl.host.has_shared:
                assert np.array_equal(ys_a, ys_b), (fmt, up, M)
            assert not np.all(yr_b == 0xFFFFFFFF)


def test_noalloc_fused_routing_and_default_variant():
    dl = make_layer(abi.FMT_FP8, 2048, 1024, 32, 8, 4, seed=2, shared="fp8").upload()
    x, logits, idx, w = rows_and_routing(43, 4, 2048, 32, 8, 1.0)
    for M in (4, 1):
        a, b = _both(dl, x, idx, w, M, logits=gpu.dev(logits[:M]), route_scale=1.0)
        assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])


def test_noalloc_refuses_layers_beyond_its_workspace():
    L = abi.LayerW()
    L.pool, L.desc, L.fmt, L.H, L.I, L.E, L.topk = 256, 256, abi.FMT_FP8, 8192, 2048, 8, 2
    t = gpu.empty(256, 0)
    with pytest.raises(lib.DsgxError) as e:
        lib.moe_decode(L, t, t, t, 1, None, t, t)
    assert e.value.code == abi.EINVAL and "built-in workspace" in str(e.value)
    L.H, L.I = 4096, 4096
    with pytest.raises(lib.DsgxError):
        lib.moe_decode(L, t, t, t, 1, None, t, t)
    torch.cuda.synchronize()
