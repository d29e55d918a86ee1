"""CPU: the NumPy statement of the Gibipel decoder (oracle/gibipel_oracle.py) against closed forms and second spellings of its
mechanisms, so that the GPU tests compare the library with something that has itself been pinned."""
import math

import numpy as np

from oracle import gibipel_oracle as O
from tests import gibipel_util as U


def test_one_number_norm():
    x = np.array([[3.0, -4.0, 0.0, 0.0]])
    out = O.scalar_norm(x, np.array(2.0), 0.0)
    assert np.allclose(out, x / 2.5 * 2.0)
    assert np.allclose(O.scalar_norm(np.zeros((1, 4)), np.array(2.0), 1e-4), 0.0)


def test_rotation_of_halves_depends_on_the_distance_only_and_leaves_the_tail():
    rs = np.random.RandomState(0)
    f = O.rotation_frequencies(dict(base=100.0, dims=6))
    assert np.allclose(f, [1.0, 100.0 ** (-1 / 3), 100.0 ** (-2 / 3)])
    x = rs.randn(9, 2, 10)
    r = O.rotate_halves(x, f, 6)
    assert np.array_equal(r[..., 6:], x[..., 6:]) and np.allclose(r[0], x[0])
    q, k = np.tile(rs.randn(1, 1, 10), (9, 1, 1)), np.tile(rs.randn(1, 1, 10), (9, 1, 1))
    rq, rk = O.rotate_halves(q, f, 6), O.rotate_halves(k, f, 6)
    assert abs(rq[7, 0] @ rk[3, 0] - rq[5, 0] @ rk[1, 0]) < 1e-12
    # element i turns together with element i + dims / 2
    one = np.zeros((2, 1, 10)); one[:, 0, 1] = 1.0
    t = O.rotate_halves(one, f, 6)[1, 0]
    assert np.allclose(t[[1, 4]], [math.cos(f[1]), math.sin(f[1])]) and np.count_nonzero(np.abs(t) > 1e-15) == 2


def test_frequency_bands():
    rot = dict(base=10000.0, dims=32, scaling=dict(factor=8.0, low=1.0, high=4.0, original=256))
    plain = O.rotation_frequencies(dict(base=10000.0, dims=32))
    f = O.rotation_frequencies(rot)
    wl = 2 * math.pi / plain
    short, long_ = wl < 256 / 4.0, wl > 256 / 1.0
    assert short.any() and long_.any() and (~short & ~long_).any()
    assert np.array_equal(f[short], plain[short]) and np.allclose(f[long_], plain[long_] / 8.0)
    mid = ~short & ~long_
    assert ((f[mid] > plain[mid] / 8.0) & (f[mid] < plain[mid])).all()
    t = (256 / wl[mid] - 1.0) / 3.0
    assert np.allclose(f[mid], (1 - t) * plain[mid] / 8.0 + t * plain[mid])


def test_what_a_position_sees():
    assert O.visible_tokens(7, 5) == [3, 4, 5, 6, 7] and O.visible_tokens(2, 5) == [0, 1, 2]
    # blocks of three in front of a window of five: block b is seen from position 3 b + 2 + 5 on
    assert O.visible_blocks(6, 5, 3) == [] and O.visible_blocks(7, 5, 3) == [0] and O.visible_blocks(9, 5, 3) == [0]
    assert O.visible_blocks(10, 5, 3) == [0, 1]
    for i in range(40):
        seen = set(O.visible_tokens(i, 5))
        for b in O.visible_blocks(i, 5, 3):
            assert not seen & set(range(3 * b, 3 * b + 3))
        gap = set(range(i + 1)) - seen - {j for b in O.visible_blocks(i, 5, 3) for j in range(3 * b, 3 * b + 3)}
        assert len(gap) <= 2                       # positions that left the window and whose block is not whole yet


def test_pooled_window_attention_as_explicit_sums():
    rs = np.random.RandomState(1)
    T, H, G, d, e, w, P = 23, 4, 2, 6, 5, 7, 3
    q, k, v, sink = rs.randn(T, H, d), rs.randn(T, G, d), rs.randn(T, G, e), rs.randn(H)
    out = O.pooled_window_attention(q, k, v, sink, 0.4, w, P)
    for hd in range(H):
        g = hd // 2
        for i in (0, 6, 7, 9, 10, 22):
            num, den = np.zeros(e), math.exp(sink[hd])
            for j in range(i + 1):
                if i - j < w:
                    p = math.exp(0.4 * q[i, hd] @ k[j, g]); num += p * v[j, g]; den += p
            for b in range(T // P):
                if b * P + P - 1 <= i - w:
                    p = math.exp(0.4 * q[i, hd] @ k[b * P:(b + 1) * P, g].mean(0)); num += p * v[b * P:(b + 1) * P, g].mean(0); den += p
            assert np.allclose(out[i, hd], num / den)
    # a large sink takes the weight away
    assert np.abs(O.pooled_window_attention(q, k, v, sink + 30.0, 0.4, w, P)).max() < 1e-6


def test_matrix_memory_against_the_unstabilised_sums_and_across_a_cut():
    rs = np.random.RandomState(2)
    T, H, d, e = 17, 2, 4, 3
    q, k, v = rs.randn(T, H, d), rs.randn(T, H, d), rs.randn(T, H, e)
    li, lf = rs.randn(T, H) * 2.0, O.log_sigmoid(rs.randn(T, H) * 2.0)
    out, (S, n, m) = O.matrix_memory(q, k, v, li, lf)
    for hd in range(H):
        F = np.cumsum(lf[:, hd])
        for t in range(T):
            wts = np.exp(F[t] - F[:t + 1] + li[:t + 1, hd])
            St = (wts[:, None, None] * k[:t + 1, hd, :, None] * v[:t + 1, hd, None, :]).sum(0)
            nt = (wts[:, None] * k[:t + 1, hd]).sum(0)
            mt = F[t] + max(0.0, (li[:t + 1, hd] - F[:t + 1]).max())
            want = St.T @ q[t, hd] * math.exp(-mt) / (max(abs(nt @ q[t, hd]) * math.exp(-mt), math.exp(-mt)) + 1e-6)
            assert np.allclose(out[t, hd], want, rtol=1e-9, atol=1e-12)
        assert np.isclose(m[hd], F[-1] + max(0.0, (li[:, hd] - F).max()))
    a, st = O.matrix_memory(q[:6], k[:6], v[:6], li[:6], lf[:6])
    b, st2 = O.matrix_memory(q[6:], k[6:], v[6:], li[6:], lf[6:], st)
    assert np.allclose(np.concatenate([a, b]), out) and np.allclose(st2[0], S) and np.allclose(st2[1], n)


def test_gate_cap_and_logarithm_of_the_forget_gate():
    assert np.allclose(O.capped(np.array([0.1, 100.0, -100.0]), 5.0), [5 * math.tanh(0.02), 5.0, -5.0])
    assert np.allclose(O.log_sigmoid(np.array([0.0, 40.0, -40.0])), [-math.log(2.0), 0.0, -40.0], atol=1e-12)


def test_router_groups_correction_identity_and_weights():
    W = 4
    P = {"r.router": np.eye(6, W) * 0 + np.array([[2.0, 0, 0, 0], [1.0, 0, 0, 0], [0.5, 0, 0, 0], [1.9, 0, 0, 0], [0.0, 0, 0, 0], [-1.0, 0, 0, 0]]),
         "r.correction": np.array([0.0, 0.0, 0.0, 0.0, 0.0, 0.0])}
    h = np.array([[1.0, 0, 0, 0]])
    rt = dict(experts=4, identity=2, top=2, groups=dict(count=2, keep=1))
    z = np.array([2.0, 1.0, 0.5, 1.9, 0.0, -1.0]); s = np.exp(z) / np.exp(z).sum()
    sel, w = O.route(h, P, "r.", rt)
    assert list(sel[0]) == [0, 1] and np.allclose(w[0], s[[0, 1]] / s[[0, 1]].sum())      # the second group is out although 1.9 > 1
    # the correction moves the choice, not the weights; choice scores below zero still beat a group that is out
    P["r.correction"] = np.array([-5.0, -5.0, -5.0, 0.0, 0.0, 0.0])
    sel, w = O.route(h, P, "r.", rt)
    assert list(sel[0]) == [3, 4] and np.allclose(w[0], s[[3, 4]] / s[[3, 4]].sum())
    P["r.correction"] = np.array([-5.0, -5.0, -5.0, -6.0, -7.0, -8.0])
    sel, w = O.route(h, P, "r.", rt)
    assert sorted(sel[0]) == [0, 1] and abs(w[0].sum() - 1.0) < 1e-12
    rt1 = dict(experts=4, identity=2, top=3)
    P["r.correction"] = np.zeros(6)
    sel, _ = O.route(h, P, "r.", rt1)
    assert list(sel[0]) == [0, 3, 1]


def test_identity_and_shared_experts_in_the_mixture():
    cfg = U.config([U.layer(U.left(), U.right(), U.moe(experts=2, top=3, identity=1, groups=1, keep=1, shared=8))], width=16)
    P = U.random_weights(cfg, 3)
    rs = np.random.RandomState(3)
    h = rs.randn(5, 16)
    ml = cfg["layers"][0]["mlp"]
    out = O.mixture_ff(h, P, "l0.mlp.", ml)
    sel, w = O.route(h, P, "l0.mlp.", ml["router"])
    assert (np.sort(sel, 1) == [0, 1, 2]).all()              # top = all outputs: every token uses both experts and the identity
    for t in range(5):
        want = O.gated_ff(h[t:t + 1], P, "l0.mlp.shared.")[0]
        for j, wt in zip(sel[t], w[t]):
            want = want + wt * (h[t] if j == 2 else O.gated_ff(h[t:t + 1], P, f"l0.mlp.e{j}.")[0])
        assert np.allclose(out[t], want)


def test_planted_key_shows_exactly_where_the_mask_lets_it():
    size, pool = 20, 6
    cfg, P, QT, KT = U.planted(size, pool)
    for kp, qp in [(0, 19), (0, 20), (0, 24), (0, 25), (5, 25), (6, 25), (6, 30), (6, 31), (40, 60), (41, 66), (3, 89), (69, 89), (70, 89)]:
        toks = U.tokens(90, 65, kp * 1000 + qp)
        toks[kp], toks[qp] = KT, QT
        plain = list(toks); plain[kp] = (toks[kp - 1] + 1) % 65 if kp else 1
        a, b = O.forward(cfg, P, toks)[qp], O.forward(cfg, P, plain)[qp]
        moved = float(np.abs(a - b).max() / np.abs(a).max())
        seen = kp in O.visible_tokens(qp, size) or kp // pool in O.visible_blocks(qp, size, pool)
        assert (moved > 0.1) == seen and (seen or moved < 0.01), (kp, qp, moved)


def test_layers_and_greedy_tokens():
    cfg = U.small_config()
    P = U.random_weights(cfg, 4)
    toks = U.tokens(30, cfg["vocab"], 4)
    logits, layers = O.forward(cfg, P, toks, True)
    assert logits.shape == (30, cfg["vocab"]) and layers.shape == (3, 30, cfg["width"])
    assert np.allclose(O.forward(cfg, P, toks[:11]), logits[:11])          # causal
    new = O.greedy(cfg, P, toks[:5], 3)
    assert len(new) == 3 and new[0] == int(np.argmax(O.forward(cfg, P, toks[:5])[-1]))
