"""Pins the oracle's router (route_sigmoid, sum order, top-k order and ties) with the reference's own CPU checks
(altar1-4xgx10-switchless/engine/experts/tests/test_experts.cu:187-212) and brute force."""
import numpy as np

from tests import orc


def _logits(M, E, seed, ties):
    # rnd_logits of the reference (testdata.h:329-336)
    l = np.empty((M, E), np.float32)
    for i in range(M * E):
        h = orc.lib().orc_mix64(seed * 13 + i)
        v = (np.float32(h >> 40) * np.float32(2.0 ** -24) - np.float32(0.5)) * np.float32(6.0)
        if ties and (h & 7) == 0:
            v = np.float32(1.25)
        l.flat[i] = v
    return l


def test_sigmoid_accuracy_and_limits():
    L = orc.lib()
    xs = np.linspace(-30, 30, 4001).astype(np.float32)
    got = np.array([L.orc_route_sigmoid(float(v)) for v in xs], np.float64)
    want = 1 / (1 + np.exp(-xs.astype(np.float64)))
    assert np.max(np.abs(got - want) / want) < 3e-7
    assert L.orc_route_sigmoid(100.0) == 1.0 and L.orc_route_sigmoid(-100.0) == 0.0 and L.orc_route_sigmoid(0.0) == 0.5
    assert np.all(np.diff(got) >= 0)


def test_route_order_ties_sum():
    # the reference's check at 168 experts: many tied logits, equal bias, three experts tied inside the top 8
    E, M, topk = 168, 64, 8
    l = _logits(M, E, 3, True)
    bias = np.full(E, 28.25, np.float32)
    for m in range(M):
        for j in range(3):
            l[m, (m * 29 + 53 * j) % E] = 3.5
    idx, w = orc.route(l, bias, topk, 2.5)
    ties = 0
    for m in range(M):
        key = np.array([np.float32(orc.lib().orc_route_sigmoid(float(v))) for v in l[m]], np.float32) + bias
        assert abs(float(w[m].astype(np.float64).sum()) - 2.5) < 1e-5
        assert idx[m].min() >= 0 and idx[m].max() < E and len(set(idx[m])) == topk
        for k in range(1, topk):
            a, b = idx[m, k - 1], idx[m, k]
            assert key[a] > key[b] or (key[a] == key[b] and a < b)
            ties += key[a] == key[b]
        # brute force: stable sort by (-key, id)
        order = sorted(range(E), key=lambda e: (-float(key[e]), e))[:topk]
        assert list(idx[m]) == order
    assert ties > 0


def test_route_weights_sum_order():
    # w_k = s_k / (((p0+p4)+(p2+p6)) + ((p1+p5)+(p3+p7)) + 1e-20) * scale, one divide then one multiply, in f32
    E, M = 256, 32
    l = orc.normal_f32(0, 2, (M, E), 1.0)
    idx, w = orc.route(l, None, 8, 1.0)
    other_order = 0
    for m in range(M):
        p = np.array([orc.lib().orc_route_sigmoid(float(l[m, e])) for e in idx[m]], np.float32)
        s = ((p[0] + p[4]) + (p[2] + p[6])) + ((p[1] + p[5]) + (p[3] + p[7]))
        s = np.float32(s + np.float32(1e-20))
        want = (p / s) * np.float32(1.0)
        assert np.array_equal(w[m], want.astype(np.float32))
        seq = np.float32(0)
        for v in p:
            seq = np.float32(seq + v)
        other_order += not np.array_equal((p / np.float32(seq + np.float32(1e-20))).astype(np.float32), w[m])
    assert other_order > 0  # a sequential sum would give other bits on some rows: the order is pinned


def test_route_top6_sum_order_and_bias_is_selection_only():
    E, M = 64, 16
    l = orc.normal_f32(1, 2, (M, E), 1.0)
    bias = orc.normal_f32(1, 3, (E,), 0.5)
    idx, w = orc.route(l, bias, 6, 1.5)
    for m in range(M):
        s = np.array([orc.lib().orc_route_sigmoid(float(v)) for v in l[m]], np.float32)
        key = s + bias
        order = sorted(range(E), key=lambda e: (-float(key[e]), e))[:6]
        assert list(idx[m]) == order
        p = s[idx[m]]
        tot = np.float32(((p[0] + p[4]) + p[2]) + ((p[1] + p[5]) + p[3]))  # ds41f common.cuh:310
        want = (p / np.float32(tot + np.float32(1e-20))) * np.float32(1.5)
        assert np.array_equal(w[m], want.astype(np.float32))


def test_union_sorted_unique():
    idx = np.array([[5, 3, 9], [3, 200, 0]], np.int32)
    assert list(orc.union(idx, 256)) == [0, 3, 5, 9, 200]


# ---- DeepSeek's score function: sqrt(softplus(l)) (ds41f-4xgx10-switchless/engine/kernels/common.cuh:266-315) ----------
def _ulp32(v):
    v = np.abs(np.asarray(v, np.float64))
    return 2.0 ** (np.floor(np.log2(np.maximum(v, 2.0 ** -126))) - 23)


def test_sqrt_softplus_score_against_f64():
    """score(l) = sqrt(l > 20 ? l : log1p(exp(l))) within 2 f32 ulp of the f64 value on a grid that covers both branches,
    the switch at 20 itself, large negative logits (softplus -> exp(l)) and the overflow side of expf"""
    L = orc.lib()
    xs = np.concatenate([np.linspace(-30, 30, 6001), np.linspace(19.9, 20.1, 401), [20.0, np.nextafter(np.float32(20), np.float32(21)), 25.0, 60.0, 88.0, 100.0, -80.0, 0.0]]).astype(np.float32)
    got = np.array([L.orc_route_score(float(v), 1) for v in xs], np.float64)
    x64 = xs.astype(np.float64)
    want = np.sqrt(np.where(xs > np.float32(20), x64, np.log1p(np.exp(np.minimum(x64, 50.0)))))
    assert np.all(np.abs(got - want) <= 2 * _ulp32(want)), float((np.abs(got - want) / _ulp32(want)).max())
    assert np.all(np.diff(got[:6001]) >= 0)  # monotone over the grid
    # the branch: exactly l above 20 (the square root of the logit itself, correctly rounded)
    for v in (20.5, 33.0, 100.0):
        assert L.orc_route_score(v, 1) == float(np.sqrt(np.float32(v)))
    # a different function (the sigmoid, or softplus without the root) is far outside the tolerance
    assert abs(L.orc_route_score(1.0, 1) - L.orc_route_score(1.0, 0)) > 0.1
    assert abs(L.orc_route_score(1.0, 1) - np.log1p(np.exp(1.0))) > 0.1


def test_sqrt_softplus_route_top6_order_and_sum_order():
    """the whole DeepSeek selection (router_row, common.cuh:266-315): keys = score + bias, top-6 by (key descending, id
    ascending) found by brute force, weights = score / (((p0+p4)+p2)+((p1+p5)+p3) + 1e-20) * scale with the bias left
    out of the weights; a sequential sum of the six gives other bits on some rows"""
    E, M, topk, scale = 384, 64, 6, 1.5
    l = orc.normal_f32(7, 2, (M, E), 1.0)
    l[0, :4] = [25.0, 21.0, 30.0, 20.5]      # rows that take the l > 20 branch
    l[1, 5] = l[1, 300] = l[1, 17] = 3.25      # a three-way tie inside the top six
    bias = orc.normal_f32(7, 3, (E,), 0.05)
    bias[5] = bias[300] = bias[17] = 0.0
    idx, w = orc.route(l, bias, topk, scale, score_fn=1)
    other_order = 0
    for m in range(M):
        s = np.array([orc.lib().orc_route_score(float(v), 1) for v in l[m]], np.float32)
        key = (s + bias).astype(np.float32)
        order = sorted(range(E), key=lambda e: (-float(key[e]), e))[:topk]
        assert list(idx[m]) == order
        p = s[idx[m]]
        tot = np.float32(np.float32(np.float32(p[0] + p[4]) + p[2]) + np.float32(np.float32(p[1] + p[5]) + p[3]))
        want = (p / np.float32(tot + np.float32(1e-20))) * np.float32(scale)
        assert np.array_equal(w[m].view(np.uint32), want.astype(np.float32).view(np.uint32))
        seq = np.float32(0)
        for v in p:
            seq = np.float32(seq + v)
        other_order += not np.array_equal((p / np.float32(seq + np.float32(1e-20)) * np.float32(scale)).astype(np.float32), w[m])
        assert abs(float(w[m].astype(np.float64).sum()) - scale) < 1e-5
    assert list(idx[1][:3]) == [5, 17, 300] or {5, 17, 300} <= set(idx[1])  # ties go to the lower id, in id order
    pos = [list(idx[1]).index(e) for e in (5, 17, 300)]
    assert pos == sorted(pos)
    assert other_order > 0
    # no bias (null) is bias 0
    i2, w2 = orc.route(l, None, topk, scale, score_fn=1)
    i3, w3 = orc.route(l, np.zeros(E, np.float32), topk, scale, score_fn=1)
    assert np.array_equal(i2, i3) and np.array_equal(w2.view(np.uint32), w3.view(np.uint32))
