"""Plain NumPy statement of the Gibipel decoder, one function per mechanism (float64, whole sequences, no cache).

Test infrastructure only: nothing here is imported by the product.  A model is a config dict in the checkpoint's own
spelling (``architecture``, ``width``, ``vocab``, ``norm.eps``, ``embedding.scale``, ``logit_scale``, ``layers[...]``) and a
dict of arrays under the checkpoint's tensor names (``embed``, ``l<i>.norm1``, ``l<i>.mix.left.q``, ``l<i>.mix.right.q``,
``l<i>.mlp.e<j>.gate``, ..., ``final.norm``, ``head``).

Notation: T tokens, W model width.  Left mixer (softmax attention): H query heads, G key/value heads, d key size, e value
size, window w, pooled blocks of P positions.  Right mixer (matrix memory): H heads, d key size, e value size.
"""
from __future__ import annotations

import math

import numpy as np


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    x = np.asarray(x, np.float64)
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-np.asarray(z, np.float64)))


def silu(z):
    return z * sigmoid(z)


def log_sigmoid(z):
    z = np.asarray(z, np.float64)
    return np.minimum(z, 0.0) - np.log1p(np.exp(-np.abs(z)))


def scalar_norm(x, g, eps):
    """Unit root mean square times ONE learned number."""
    return unit_rms(x, eps) * float(np.asarray(g).reshape(-1)[0])


# ---- rotation -------------------------------------------------------------------------------------------------------
def rotation_frequencies(rot):
    """Angle per position of pair i: base^(-2i / dims); with "scaling", long wavelengths are stretched by `factor`, short
    ones are kept, and the band between original / low and original / high blends the two linearly in original / wavelength."""
    dims, base = rot["dims"], rot["base"]
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)], np.float64)
    sc = rot.get("scaling")
    if sc:
        out = f.copy()
        for i, fi in enumerate(f):
            wavelength = 2.0 * math.pi / fi
            if wavelength < sc["original"] / sc["high"]:
                continue
            if wavelength > sc["original"] / sc["low"]:
                out[i] = fi / sc["factor"]
            else:
                t = (sc["original"] / wavelength - sc["low"]) / (sc["high"] - sc["low"])
                out[i] = (1.0 - t) * fi / sc["factor"] + t * fi
        f = out
    return f


def rotate_halves(x, freq, dims):
    """x: [T, heads, n]; element i < dims / 2 of row t pairs with element i + dims / 2 and the pair turns by t * freq[i];
    elements from dims on stay."""
    x = np.asarray(x, np.float64)
    out = x.copy()
    half = dims // 2
    ang = np.arange(x.shape[0], dtype=np.float64)[:, None] * freq[None, :]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    out[..., :half] = a * c - b * s
    out[..., half:dims] = b * c + a * s
    return out


# ---- left mixer: window attention with pooled blocks ----------------------------------------------------------------
def visible_tokens(i, window):
    """Positions j that position i sees as themselves."""
    return list(range(max(0, i - window + 1), i + 1))


def visible_blocks(i, window, pool):
    """Blocks [bP, bP + P) that lie wholly in front of position i's window (no pooling: none)."""
    if not pool:
        return []
    return [b for b in range((i + 1) // pool + 1) if b * pool + pool - 1 <= i - window]


def left_keys_values(h, P, pre, mx, eps):
    """Cached rows of the left mixer: keys after the norm over all heads at once and the rotation, values as projected."""
    T = h.shape[0]
    G, d, e = mx["kv_heads"], mx["dim"], mx["vdim"]
    k = h @ P[pre + "k"].T + P[pre + "k.b"]
    k = (unit_rms(k, eps) * P[pre + "k.norm"]).reshape(T, G, d)
    rot = mx.get("rot")
    if rot and rot.get("dims", 0) > 0:
        k = rotate_halves(k, rotation_frequencies(rot), rot["dims"])
    v = (h @ P[pre + "v"].T + P[pre + "v.b"]).reshape(T, G, e)
    return k, v


def left_queries(h, P, pre, mx, eps):
    T = h.shape[0]
    q = h @ P[pre + "q"].T + P[pre + "q.b"]
    q = (unit_rms(q, eps) * P[pre + "q.norm"]).reshape(T, mx["heads"], mx["dim"])
    rot = mx.get("rot")
    if rot and rot.get("dims", 0) > 0:
        q = rotate_halves(q, rotation_frequencies(rot), rot["dims"])
    return q


def pooled_window_attention(q, k, v, sink, scale, window, pool):
    """q [T, H, d], k [T, G, d], v [T, G, e].  Position i attends its window's tokens and, through the mean key and mean value
    of each, the blocks in front of the window; exp(sink) of the head joins the denominator once."""
    T, H, _ = q.shape
    G, e = k.shape[1], v.shape[2]
    out = np.zeros((T, H, e))
    nb = T // pool if pool else 0
    kb = k[:nb * pool].reshape(nb, pool, G, -1).mean(1) if nb else np.zeros((0,) + k.shape[1:])
    vb = v[:nb * pool].reshape(nb, pool, G, -1).mean(1) if nb else np.zeros((0,) + v.shape[1:])
    for hd in range(H):
        g = hd // (H // G)
        for i in range(T):
            js, bs = visible_tokens(i, window), visible_blocks(i, window, pool)
            keys = np.concatenate([kb[bs, g], k[js, g]], 0)
            vals = np.concatenate([vb[bs, g], v[js, g]], 0)
            s = keys @ q[i, hd] * scale
            top = max(s.max(), sink[hd])
            p = np.exp(s - top)
            out[i, hd] = (p[:, None] * vals).sum(0) / (p.sum() + math.exp(sink[hd] - top))
    return out


def left_mixer(h, P, pre, mx, eps):
    T = h.shape[0]
    q = left_queries(h, P, pre, mx, eps)
    k, v = left_keys_values(h, P, pre, mx, eps)
    o = pooled_window_attention(q, k, v, P[pre + "sink"], mx["scale"], mx["mask"]["size"], mx["mask"].get("pool", 0))
    return o.reshape(T, -1) @ P[pre + "o"].T


# ---- right mixer: matrix memory with exponential gates --------------------------------------------------------------
def capped(z, cap):
    return cap * np.tanh(np.asarray(z, np.float64) / cap)


def matrix_memory(q, k, v, li, lf, state=None):
    """q, k [T, H, d], v [T, H, e], li / lf [T, H] logarithms of the input and forget gates.  Per head a matrix S [d, e], a
    vector n [d] and a running maximum m (all zero at the start):
        m' = max(lf + m, li);  S' = exp(lf + m - m') S + exp(li - m') k v^T;  n' likewise with k alone
        o = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)
    Returns o [T, H, e] and the final (S, n, m)."""
    T, H, d = q.shape
    e = v.shape[2]
    if state is None:
        state = (np.zeros((H, d, e)), np.zeros((H, d)), np.zeros(H))
    S, n, m = (np.array(a, np.float64) for a in state)
    out = np.zeros((T, H, e))
    for t in range(T):
        for hd in range(H):
            mn = max(lf[t, hd] + m[hd], li[t, hd])
            keep, take = math.exp(lf[t, hd] + m[hd] - mn), math.exp(li[t, hd] - mn)
            S[hd] = keep * S[hd] + take * np.outer(k[t, hd], v[t, hd])
            n[hd] = keep * n[hd] + take * k[t, hd]
            m[hd] = mn
            out[t, hd] = S[hd].T @ q[t, hd] / (max(abs(n[hd] @ q[t, hd]), math.exp(-mn)) + 1e-6)
    return out, (S, n, m)


def right_mixer(h, P, pre, mx, eps):
    T = h.shape[0]
    H, d, e, cap = mx["heads"], mx["dim"], mx["vdim"], mx["gate_cap"]
    q = (h @ P[pre + "q"].T).reshape(T, H, d) * d ** -0.5
    k = (h @ P[pre + "k"].T).reshape(T, H, d)
    v = (h @ P[pre + "v"].T).reshape(T, H, e)
    li = capped(h @ P[pre + "i"].T + P[pre + "i.b"], cap)
    lf = log_sigmoid(capped(h @ P[pre + "f"].T + P[pre + "f.b"], cap))
    o, _ = matrix_memory(q, k, v, li, lf)
    o = unit_rms(o, eps).reshape(T, H * e) * P[pre + "norm"] * sigmoid(h @ P[pre + "g"].T)
    return o @ P[pre + "o"].T


def parallel_mixer(h, P, pre, mx, eps):
    return mx["left_scale"] * left_mixer(h, P, pre + "left.", mx["left"], eps) + \
        mx["right_scale"] * right_mixer(h, P, pre + "right.", mx["right"], eps)


# ---- feed-forward ---------------------------------------------------------------------------------------------------
def gated_ff(h, P, pre):
    return (silu(h @ P[pre + "gate"].T) * (h @ P[pre + "up"].T)) @ P[pre + "down"].T


def route(h, P, pre, rt):
    """Per token: the chosen outputs of the router (indices into experts + identity experts) and their weights.
    Softmax over all outputs; the choice goes by score + correction, inside the `keep` groups of neighbours whose best
    choice score is largest; the weights are the plain scores of the chosen, normalised to sum one."""
    z = np.asarray(h, np.float64) @ P[pre + "router"].T
    z = z - z.max(-1, keepdims=True)
    s = np.exp(z) / np.exp(z).sum(-1, keepdims=True)
    choice = s + P[pre + "correction"]
    n_out = s.shape[1]
    gr = rt.get("groups") or {"count": 1, "keep": 1}
    per = n_out // gr["count"]
    sel, wts = [], []
    for t in range(s.shape[0]):
        c = choice[t].copy()
        best = c.reshape(gr["count"], per).max(1)
        kept = np.argsort(-best, kind="stable")[:gr["keep"]]
        allowed = np.zeros(n_out, bool)
        for g in kept:
            allowed[g * per:(g + 1) * per] = True
        c[~allowed] = -np.inf
        pick = np.argsort(-c, kind="stable")[:rt["top"]]
        w = s[t, pick]
        sel.append(pick)
        wts.append(w / (w.sum() + 1e-20))
    return np.array(sel), np.array(wts)


def mixture_ff(h, P, pre, ml):
    rt = ml["router"]
    n_real = rt["experts"]
    sel, wts = route(h, P, pre, rt)
    out = np.zeros_like(h, dtype=np.float64)
    for t in range(h.shape[0]):
        for j, w in zip(sel[t], wts[t]):
            out[t] += w * (h[t] if j >= n_real else gated_ff(h[t:t + 1], P, f"{pre}e{j}.")[0])
    if ml.get("shared"):
        out += gated_ff(h, P, pre + "shared.")
    return out


# ---- the model ------------------------------------------------------------------------------------------------------
def forward(cfg, P, ids, return_layers=False):
    """Logits [T, vocab] of one sequence (and the residual stream after every layer)."""
    eps = cfg["norm"]["eps"]
    x = np.asarray(P["embed"], np.float64)[np.asarray(ids)] * cfg["embedding"]["scale"]
    layers = []
    for li, ly in enumerate(cfg["layers"]):
        p = f"l{li}."
        if ly["type"] != "parallel":
            raise ValueError(ly["type"])
        x = x + scalar_norm(parallel_mixer(x, P, p + "mix.", ly["mixer"], eps), P[p + "norm1"], eps)
        if ly.get("mlp") is not None:
            x = x + scalar_norm(mixture_ff(x, P, p + "mlp.", ly["mlp"]), P[p + "norm2"], eps)
        layers.append(x.copy())
    logits = scalar_norm(x, P["final.norm"], eps) @ np.asarray(P["head"], np.float64).T * cfg["logit_scale"]
    return (logits, np.stack(layers)) if return_layers else logits


def greedy(cfg, P, prompt, n_new):
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(np.argmax(forward(cfg, P, ids)[-1])))
    return ids[len(prompt):]
