"""CPU: the NumPy statement of the Nevotar decoder (oracle/nevotar_oracle.py) against closed forms and second spellings of its
mechanisms, so that the GPU tests compare the library with something that has itself been pinned."""
import math

import numpy as np

from oracle import nevotar_oracle as O
from tests import nevotar_util as U


def test_norm_in_parts():
    x = np.array([[3.0, -4.0, 0.0, 5.0, 12.0, 0.0]])
    w = np.arange(1.0, 7.0)
    assert np.allclose(O.group_norm(x, w, 1, 0.0), x / math.sqrt((9 + 16 + 25 + 144) / 6) * w)
    two = O.group_norm(x, w, 2, 0.0)
    assert np.allclose(two[0, :3], x[0, :3] / math.sqrt(25 / 3) * w[:3]) and np.allclose(two[0, 3:], x[0, 3:] / math.sqrt(169 / 3) * w[3:])
    assert np.allclose(O.group_norm(x, np.ones(6), 6, 1e-12), np.sign(x))
    assert np.allclose(O.group_norm(np.zeros((1, 6)), w, 3, 1e-4), 0.0)      # eps sits inside the root


def test_query_temperature_steps_with_the_position():
    t = O.query_temperature(20, 0.5, 4)
    assert np.allclose(t[:3], 1.0)                                           # floor((p + 1) / 4) = 0 up to p = 2
    assert np.allclose(t[3:7], 1.0 + 0.5 * math.log(2.0)) and np.allclose(t[7], 1.0 + 0.5 * math.log(3.0))
    assert np.allclose(O.query_temperature(5, 0.3, 1), 1.0 + 0.3 * np.log(np.arange(5) + 2.0))


def test_window_softmax_sees_itself_and_the_tokens_before_it():
    rs = np.random.RandomState(0)
    p = O.causal_softmax(rs.randn(9, 9), 3)
    assert np.allclose(p.sum(-1), 1.0)
    for i in range(9):
        seen = np.nonzero(p[i] > 0)[0]
        assert list(seen) == list(range(max(0, i - 2), i + 1))
    assert np.allclose(O.causal_softmax(rs.randn(4, 4), 1), np.eye(4))
    full = O.causal_softmax(np.zeros((5, 5)))
    assert np.allclose(full[4], 0.2) and np.allclose(full[0], [1, 0, 0, 0, 0])


def test_differential_attention_as_explicit_sums():
    rs = np.random.RandomState(1)
    mx = U.attn(heads=2, kv_heads=1, dim=3, vdim=4, diff=0.4, coef=0.5, every=2, scale=0.7)
    W, T = 5, 6
    cfg = U.config([U.layer("attention", mx, None)], width=W)
    P = U.random_weights(cfg, 1)
    h = rs.randn(T, W)
    got = O.differential_attention(h, P, "l0.mix.", mx, 1e-6)
    lam = math.exp(P["l0.mix.lq1"].astype(float) @ P["l0.mix.lk1"].astype(float)) - math.exp(P["l0.mix.lq2"].astype(float) @ P["l0.mix.lk2"].astype(float)) + 0.4
    assert abs(lam - O.differential_lambda(P, "l0.mix.", 0.4)) < 1e-12
    q = h @ P["l0.mix.q"].astype(float).T + P["l0.mix.q.b"]
    k = h @ P["l0.mix.k"].astype(float).T + P["l0.mix.k.b"]
    v = h @ P["l0.mix.v"].astype(float).T + P["l0.mix.v.b"]
    out = np.zeros((T, 2, 4))
    for t in range(T):
        temp = 1.0 + 0.5 * math.log((t + 1) // 2 + 1)
        for hd in range(2):
            maps = []
            for mp in range(2):
                qq = q[t, hd * 6 + mp * 3: hd * 6 + mp * 3 + 3] * temp              # a head's row: [map 1 | map 2]
                s = np.array([qq @ k[j, mp * 3: mp * 3 + 3] * 0.7 for j in range(t + 1)])
                p = np.exp(s - s.max()); p /= p.sum()
                maps.append(p @ v[:t + 1])
            o = maps[0] - lam * maps[1]
            out[t, hd] = o / math.sqrt((o * o).mean() + 1e-6) * 0.6
    assert np.allclose(got, out.reshape(T, 8) @ P["l0.mix.o"].astype(float).T)


def test_equal_maps_leave_a_unit_vector_whatever_lambda_is():
    mx = U.attn(heads=2, kv_heads=2, dim=4, vdim=6, diff=0.25, coef=0.0, every=1)
    cfg = U.config([U.layer("attention", mx, None)], width=8)
    P = U.random_weights(cfg, 2)
    for n in ("q", "k"):                                                  # second map = first map
        m = P["l0.mix." + n].reshape(2, 2, 4, 8); m[:, 1] = m[:, 0]
        b = P["l0.mix." + n + ".b"].reshape(2, 2, 4); b[:, 1] = b[:, 0]
    h = np.random.RandomState(2).randn(5, 8)
    P["l0.mix.o"] = np.eye(12, dtype=np.float32)[:8].copy()
    cfg["width"] = 8
    out = O.differential_attention(h, {**P, "l0.mix.o": np.eye(12)}, "l0.mix.", mx, 0.0).reshape(5, 2, 6)
    lam = O.differential_lambda(P, "l0.mix.", 0.25)
    assert lam < 1.0
    assert np.allclose(np.sqrt((out * out).mean(-1)), 0.75)               # (1 - lambda) a, normed, times (1 - diff)


def test_rotation_of_halves_depends_on_the_distance_only_and_leaves_the_tail():
    rs = np.random.RandomState(3)
    x = rs.randn(9, 2, 10)
    r = O.rotate_halves(x, 6, 100.0)
    assert np.array_equal(r[..., 6:], x[..., 6:]) and np.allclose(r[0], x[0])
    q, k = np.tile(rs.randn(1, 1, 10), (9, 1, 1)), np.tile(rs.randn(1, 1, 10), (9, 1, 1))
    rq, rk = O.rotate_halves(q, 6, 100.0), O.rotate_halves(k, 6, 100.0)
    assert abs(rq[7, 0] @ rk[3, 0] - rq[5, 0] @ rk[1, 0]) < 1e-12
    one = np.zeros((2, 1, 10)); one[:, 0, 1] = 1.0
    t = O.rotate_halves(one, 6, 100.0)[1, 0]
    f1 = 100.0 ** (-2.0 / 6)
    assert np.allclose(t[[1, 4]], [math.cos(f1), math.sin(f1)]) and np.count_nonzero(np.abs(t) > 1e-15) == 2


def test_mixing_matrix_identity_is_plain_attention_and_a_permutation_swaps_heads():
    mx = U.left(heads=2, kv_heads=1, dim=4, vdim=4, size=3, dims=2)
    cfg = U.config([U.layer("parallel", U.side(mx, U.right()), None)], width=8)
    P = U.random_weights(cfg, 4)
    h = np.random.RandomState(4).randn(7, 8)
    pre = "l0.mix.left."
    P[pre + "o"] = np.eye(8, dtype=np.float32)
    P[pre + "talk"] = np.eye(2, dtype=np.float32)
    plain = O.window_talking_attention(h, P, pre, mx, 1e-6).reshape(7, 2, 4)
    # head 0 by hand
    q = O.unit_rms((h @ P[pre + "q"].astype(float).T + P[pre + "q.b"]).reshape(7, 2, 4), 1e-6) * P[pre + "q.norm"]
    k = O.unit_rms((h @ P[pre + "k"].astype(float).T + P[pre + "k.b"]).reshape(7, 1, 4), 1e-6) * P[pre + "k.norm"]
    v = (h @ P[pre + "v"].astype(float).T + P[pre + "v.b"]).reshape(7, 1, 4)
    q, k = O.rotate_halves(q, 2, mx["rot"]["base"]), O.rotate_halves(k, 2, mx["rot"]["base"])
    t = 5
    s = np.array([q[t, 0] @ k[j, 0] * mx["scale"] for j in (3, 4, 5)])
    p = np.exp(s - s.max()); p /= p.sum()
    assert np.allclose(plain[t, 0], p @ v[3:6, 0])
    P[pre + "talk"] = np.array([[0, 1], [1, 0]], np.float32)
    swapped = O.window_talking_attention(h, P, pre, mx, 1e-6).reshape(7, 2, 4)
    assert np.allclose(swapped[:, 0], plain[:, 1]) and np.allclose(swapped[:, 1], plain[:, 0])      # one value head: the weights swap


def test_gated_recurrence_as_an_explicit_sum():
    mx = U.hgrn(heads=2, dim=3, vdim=4)
    cfg = U.config([U.layer("hgrn2", mx, None)], width=6)
    P = U.random_weights(cfg, 5)
    P["l0.mix.o"] = np.eye(8, dtype=np.float32)[:6].copy()
    h = np.random.RandomState(5).randn(6, 6)
    got = O.hgrn2(h, {**P, "l0.mix.o": np.eye(8)}, "l0.mix.", mx, 0.0).reshape(6, 2, 4)
    q = O.silu(h @ P["l0.mix.q"].astype(float).T).reshape(6, 2, 3)
    v = (h @ P["l0.mix.v"].astype(float).T).reshape(6, 2, 4)
    lo = P["l0.mix.lower"].astype(float)
    f = (lo + (1 - lo) * O.sigmoid(h @ P["l0.mix.f"].astype(float).T + P["l0.mix.f.b"])).reshape(6, 2, 3)
    assert (f > lo.reshape(2, 3)).all() and (f < 1).all()
    t = 5
    for hd in range(2):
        o = np.zeros(4)
        for s in range(t + 1):
            keep = np.prod(f[s + 1:t + 1, hd], axis=0)                    # the gates after s, per channel
            o += ((q[t, hd] * keep * (1 - f[s, hd])).sum()) * v[s, hd]
        o = o / math.sqrt((o * o).mean()) * P["l0.mix.norm"]
        assert np.allclose(got[t, hd], o)


def test_causal_convolution():
    x = np.arange(12.0).reshape(6, 2)
    w = np.array([[0.0, 0.0, 1.0], [1.0, 0.0, 0.0]])                      # channel 0: the current token; channel 1: two tokens back
    y = O.causal_conv(x, w, np.array([0.5, -1.0]))
    assert np.allclose(y[:, 0], x[:, 0] + 0.5)
    assert np.allclose(y[:, 1], np.concatenate([[0, 0], x[:4, 1]]) - 1.0)
    assert np.allclose(O.causal_conv(x, np.array([[2.0], [3.0]]), np.zeros(2)), x * [2.0, 3.0])


def test_state_space_mixer_as_an_explicit_double_sum():
    mx = U.right(heads=4, vdim=3, state=5, groups=2, conv=3, norm_groups=2)
    cfg = U.config([U.layer("parallel", U.side(U.left(), mx), None)], width=10)
    P = U.random_weights(cfg, 6)
    pre = "l0.mix.right."
    h = np.random.RandomState(6).randn(7, 10)
    got = O.mamba2(h, {**P, pre + "o": np.eye(12)}, pre, mx, 1e-6)
    zz = h @ P[pre + "in"].astype(float).T
    z, xbc, dt = zz[:, :12], zz[:, 12:12 + 12 + 20], zz[:, 44:]
    xbc = O.silu(O.causal_conv(xbc, P[pre + "conv"], P[pre + "conv.b"]))
    x, B, C = xbc[:, :12].reshape(7, 4, 3), xbc[:, 12:22].reshape(7, 2, 5), xbc[:, 22:].reshape(7, 2, 5)
    dt = np.log1p(np.exp(dt + P[pre + "dt_bias"]))
    A = -np.exp(P[pre + "A_log"].astype(float))
    y = np.zeros((7, 4, 3))
    for t in range(7):
        for hd in range(4):
            g = hd // 2
            for s in range(t + 1):
                y[t, hd] += math.exp(A[hd] * dt[s + 1:t + 1, hd].sum()) * dt[s, hd] * (C[t, g] @ B[s, g]) * x[s, hd]
            y[t, hd] += P[pre + "D"][hd] * x[t, hd]
    y = y.reshape(7, 12) * O.silu(z)
    y = O.group_norm(y, P[pre + "norm"], 2, 1e-6)
    assert np.allclose(got, y)


def test_expert_weight_multiplies_the_input_and_the_activation_is_capped():
    ml = U.moe(experts=3, top=2, ff=4, limit=0.5, shared=3, shared_limit=2.0)
    cfg = U.config([U.layer("hgrn2", U.hgrn(), ml)], width=6)
    P = U.random_weights(cfg, 7)
    h = np.random.RandomState(7).randn(5, 6) * 3
    got = O.mixture_ff(h, P, "l0.mlp.", ml)
    s = O.sigmoid(h @ P["l0.mlp.router"].astype(float).T)

    def expert(x, pre, lim):
        g = np.minimum(P[pre + "gate"].astype(float) @ x, lim)
        u = np.clip(P[pre + "up"].astype(float) @ x, -lim, lim)
        return P[pre + "down"].astype(float) @ (g / (1 + np.exp(-1.702 * g)) * (u + 1))

    for t in range(5):
        order = sorted(range(3), key=lambda j: (-s[t, j], j))[:2]
        want = sum(expert(s[t, j] * h[t], f"l0.mlp.e{j}.", 0.5) for j in order) + expert(h[t], "l0.mlp.shared.", 2.0)
        assert np.allclose(got[t], want)
    big = O.capped_expert(np.full((1, 6), 50.0), {**P, "l0.mlp.e0.gate": np.ones((4, 6)), "l0.mlp.e0.up": np.ones((4, 6))}, "l0.mlp.e0.", 0.5)
    assert np.allclose(big, P["l0.mlp.e0.down"].astype(float) @ np.full(4, 0.5 / (1 + math.exp(-0.851)) * 1.5))


def test_a_layer_on_another_layers_tensors_equals_a_copy_of_them():
    cfg = U.small_config()
    P = U.random_weights(cfg, 8)
    toks = U.tokens(30, cfg["vocab"], 8)
    want = O.forward(cfg, P, toks)
    plain = {k: v for k, v in cfg.items()}
    plain["layers"] = [{k: v for k, v in ly.items() if k != "weights_of"} for ly in cfg["layers"]]
    Q = dict(P)
    for li, ly in enumerate(cfg["layers"]):
        if ly.get("weights_of") is not None:
            src = f"l{ly['weights_of']}."
            for k, v in P.items():
                if k.startswith(src):
                    Q[f"l{li}." + k[len(src):]] = v
    assert np.allclose(O.forward(plain, Q, toks), want)
    assert not any(k.startswith("l3.") or k.startswith("l4.") for k in P)


def test_logits_come_from_the_embedding_table_and_prefix_logits_do_not_change():
    cfg = U.small_config()
    P = U.random_weights(cfg, 9)
    toks = U.tokens(40, cfg["vocab"], 9)
    full, layers = O.forward(cfg, P, toks, True)
    assert layers.shape == (6, 40, cfg["width"]) and full.shape == (40, cfg["vocab"])
    assert np.allclose(full[-1], O.group_norm(layers[-1][-1], P["final.norm"], 4, cfg["norm"]["eps"]) @ P["embed"].astype(float).T)
    assert np.allclose(O.forward(cfg, P, toks[:17]), full[:17])            # causal throughout
    assert O.greedy(cfg, P, toks[:5], 3) == O.greedy(cfg, P, toks[:5], 4)[:3]


def test_planted_keys_dominate_their_scores():
    cfg, P, QT, KT = U.planted_window(size=6)
    toks = U.tokens(20, 65, 1)
    toks[10], toks[14] = KT, QT
    a = O.forward(cfg, P, toks)
    b = list(toks); b[10] = 1
    assert np.abs(O.forward(cfg, P, b)[14] - a[14]).max() > 0.1 * np.abs(a[14]).max()
    toks2 = list(toks); toks2[10], toks2[8] = toks[8], KT                  # six back: just outside
    c = list(toks2); c[8] = 1
    assert np.abs(O.forward(cfg, P, c)[14] - O.forward(cfg, P, toks2)[14]).max() < 0.01 * np.abs(a[14]).max()
    cfg, P, QT, KT = U.planted_causal()
    toks = U.tokens(300, 65, 2)
    toks[3], toks[290] = KT, QT
    a = O.forward(cfg, P, toks)
    b = list(toks); b[3] = 1
    assert np.abs(O.forward(cfg, P, b)[290] - a[290]).max() > 0.1 * np.abs(a[290]).max()
