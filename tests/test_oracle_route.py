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
