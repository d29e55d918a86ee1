"""Plain NumPy statement of the Nevotar decoder, one function per mechanism (float64, whole sequences, no cache).

Test infrastructure only: nothing here is imported by the product.  A model is a config dict in the checkpoint's own
spelling (``architecture``, ``width``, ``vocab``, ``norm.eps``, ``norm.groups``, ``layers[...]``) and a dict of arrays under
the checkpoint's tensor names (``embed``, ``l<i>.norm1``, ``l<i>.mix.q``, ``l<i>.mix.left.q``, ``l<i>.mix.right.in``,
``l<i>.mlp.e<j>.gate``, ..., ``final.norm``).  The logits come from the embedding table itself.

Notation: T tokens, W model width.  Softmax attention: H query heads, G key / value heads, d key size, e value size.
Recurrent mixers: H heads, state [d or N][e].
"""
from __future__ import annotations

import math

import numpy as np


def f64(a):
    return np.asarray(a, np.float64)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-f64(z)))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    z = f64(z)
    return np.maximum(z, 0.0) + np.log1p(np.exp(-np.abs(z)))


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    x = f64(x)
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def group_norm(x, w, groups, eps):
    """The last axis in `groups` equal consecutive parts, each over its own root mean square; the whole times w."""
    x = f64(x)
    parts = x.reshape(x.shape[:-1] + (groups, x.shape[-1] // groups))
    return unit_rms(parts, eps).reshape(x.shape) * f64(w)


def linear(h, P, name, bias=False):
    y = f64(h) @ f64(P[name]).T
    return y + f64(P[name + ".b"]) if bias else y


# ---- softmax attention ----------------------------------------------------------------------------------------------
def causal_softmax(score, window=None):
    """score [T, T] -> weights; row i sees j <= i (and i - j < window)."""
    T = score.shape[0]
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    seen = j <= i
    if window is not None:
        seen &= (i - j) < window
    z = np.where(seen, score, -np.inf)
    z = z - z.max(-1, keepdims=True)
    p = np.exp(z)
    return p / p.sum(-1, keepdims=True)


def query_temperature(T, coef, every):
    """Factor on the query at positions 0..T-1: 1 + coef ln(floor((p + 1) / every) + 1)."""
    p = np.arange(T)
    return 1.0 + coef * np.log(np.floor_divide(p + 1, every) + 1.0)


def differential_lambda(P, pre, diff):
    return math.exp(float(f64(P[pre + "lq1"]) @ f64(P[pre + "lk1"]))) - math.exp(float(f64(P[pre + "lq2"]) @ f64(P[pre + "lk2"]))) + diff


def differential_attention(h, P, pre, mx, eps):
    """Two causal softmax maps per head over the same values: (a1 - lambda a2), unit RMS per head, times (1 - diff)."""
    T = h.shape[0]
    H, G, d, e = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = linear(h, P, pre + "q", True).reshape(T, H, 2, d)
    k = linear(h, P, pre + "k", True).reshape(T, G, 2, d)
    v = linear(h, P, pre + "v", True).reshape(T, G, e)
    if mx.get("q_temp"):
        q = q * query_temperature(T, mx["q_temp"]["coef"], mx["q_temp"]["every"])[:, None, None, None]
    lam = differential_lambda(P, pre, mx["diff"])
    out = np.zeros((T, H, e))
    for hd in range(H):
        g = hd // (H // G)
        a = [causal_softmax(q[:, hd, m] @ k[:, g, m].T * mx["scale"]) @ v[:, g] for m in range(2)]
        out[:, hd] = unit_rms(a[0] - lam * a[1], eps) * (1.0 - mx["diff"])
    return out.reshape(T, H * e) @ f64(P[pre + "o"]).T


def rotate_halves(x, dims, base):
    """x [T, heads, n]: element i < dims / 2 turns with element i + dims / 2 by t * base^(-2i / dims); the rest stays."""
    x = f64(x)
    out = x.copy()
    half = dims // 2
    freq = np.array([base ** (-2.0 * i / dims) for i in range(half)])
    ang = np.arange(x.shape[0], dtype=np.float64)[:, None] * freq[None, :]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    out[..., :half] = a * c - b * s
    out[..., half:dims] = b * c + a * s
    return out


def window_talking_attention(h, P, pre, mx, eps):
    """Sliding-window attention: per-head query / key norm, partial rotation, the heads' scores mixed before the softmax."""
    T = h.shape[0]
    H, G, d, e = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = linear(h, P, pre + "q", True).reshape(T, H, d)
    k = linear(h, P, pre + "k", True).reshape(T, G, d)
    v = linear(h, P, pre + "v", True).reshape(T, G, e)
    q = unit_rms(q, eps) * f64(P[pre + "q.norm"])
    k = unit_rms(k, eps) * f64(P[pre + "k.norm"])
    if mx.get("rot"):
        q = rotate_halves(q, mx["rot"]["dims"], mx["rot"]["base"])
        k = rotate_halves(k, mx["rot"]["dims"], mx["rot"]["base"])
    score = np.stack([q[:, hd] @ k[:, hd // (H // G)].T * mx["scale"] for hd in range(H)])      # [H, T, T]
    mixed = np.einsum("hg,gij->hij", f64(P[pre + "talk"]), score)
    window = mx["mask"]["size"] if mx.get("mask") else None
    out = np.zeros((T, H, e))
    for hd in range(H):
        out[:, hd] = causal_softmax(mixed[hd], window) @ v[:, hd // (H // G)]
    return out.reshape(T, H * e) @ f64(P[pre + "o"]).T


# ---- recurrent mixers -----------------------------------------------------------------------------------------------
def hgrn2(h, P, pre, mx, eps):
    """Gated linear recurrence whose forget gate also sets what is written: S <- diag(f) S + (1 - f) v^T, o = S^T q."""
    T = h.shape[0]
    H, d, e = mx["heads"], mx["dim"], mx["vdim"]
    q = silu(linear(h, P, pre + "q")).reshape(T, H, d)
    v = linear(h, P, pre + "v").reshape(T, H, e)
    low = f64(P[pre + "lower"])
    f = (low + (1.0 - low) * sigmoid(linear(h, P, pre + "f", True))).reshape(T, H, d)
    S = np.zeros((H, d, e))
    o = np.zeros((T, H, e))
    for t in range(T):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        o[t] = np.einsum("hde,hd->he", S, q[t])
    o = unit_rms(o, eps) * f64(P[pre + "norm"])
    return o.reshape(T, H * e) @ f64(P[pre + "o"]).T


def causal_conv(x, w, b):
    """x [T, C], w [C, taps] (last column: the current token), zeros before the start."""
    T, taps = x.shape[0], w.shape[1]
    xp = np.concatenate([np.zeros((taps - 1, x.shape[1])), f64(x)])
    return sum(xp[j:j + T] * f64(w)[:, j] for j in range(taps)) + f64(b)


def mamba2(h, P, pre, mx, eps):
    """State-space mixer: S <- exp(-exp(A_log) dt) S + dt B x^T, y = S^T C + D x; gate silu(z), grouped norm, output."""
    T = h.shape[0]
    H, e, N, G = mx["heads"], mx["vdim"], mx["state"], mx["groups"]
    inner = H * e
    zxbcdt = linear(h, P, pre + "in")
    z, xbc, dt = zxbcdt[:, :inner], zxbcdt[:, inner:2 * inner + 2 * G * N], zxbcdt[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, f64(P[pre + "conv"]), P[pre + "conv.b"]))
    x = xbc[:, :inner].reshape(T, H, e)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + f64(P[pre + "dt_bias"]))
    A = -np.exp(f64(P[pre + "A_log"]))
    D = f64(P[pre + "D"])
    S = np.zeros((H, N, e))
    y = np.zeros((T, H, e))
    for t in range(T):
        for hd in range(H):
            g = hd // (H // G)
            S[hd] = math.exp(A[hd] * dt[t, hd]) * S[hd] + dt[t, hd] * np.outer(B[t, g], x[t, hd])
            y[t, hd] = S[hd].T @ C[t, g] + D[hd] * x[t, hd]
    y = y.reshape(T, inner) * silu(z)
    y = group_norm(y, P[pre + "norm"], mx["norm_groups"], eps)
    return y @ f64(P[pre + "o"]).T


def parallel_mixer(h, P, pre, mx, eps):
    return mx["left_scale"] * window_talking_attention(h, P, pre + "left.", mx["left"], eps) + \
        mx["right_scale"] * mamba2(h, P, pre + "right.", mx["right"], eps)


# ---- feed-forward ---------------------------------------------------------------------------------------------------
def capped_expert(h, P, pre, limit):
    """g = min(W_gate h, limit), u = clamp(W_up h, +-limit): W_down (g sigmoid(1.702 g) (u + 1))."""
    g = np.minimum(linear(h, P, pre + "gate"), limit)
    u = np.clip(linear(h, P, pre + "up"), -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ f64(P[pre + "down"]).T


def route(h, P, pre, rt):
    """Sigmoid scores; the `top` largest (lowest index first among equals) -> (indices [T, top], weights = their scores)."""
    s = sigmoid(linear(h, P, pre + "router"))
    sel = np.argsort(-s, axis=-1, kind="stable")[:, :rt["top"]]
    return sel, np.take_along_axis(s, sel, -1)


def mixture_ff(h, P, pre, ml):
    """The weight multiplies an expert's INPUT: sum_k expert_k(w_k h), plus the shared expert on h itself."""
    sel, wts = route(h, P, pre, ml["router"])
    out = np.zeros_like(f64(h))
    for t in range(h.shape[0]):
        for j, w in zip(sel[t], wts[t]):
            out[t] += capped_expert(w * f64(h[t:t + 1]), P, f"{pre}e{j}.", ml["expert"]["limit"])[0]
    if ml.get("shared"):
        out += capped_expert(h, P, pre + "shared.", ml["shared"]["limit"])
    return out


# ---- the model ------------------------------------------------------------------------------------------------------
def mixer(h, P, pre, ly, eps):
    if ly["type"] == "attention":
        return differential_attention(h, P, pre, ly["mixer"], eps)
    if ly["type"] == "hgrn2":
        return hgrn2(h, P, pre, ly["mixer"], eps)
    if ly["type"] == "parallel":
        return parallel_mixer(h, P, pre, ly["mixer"], eps)
    raise ValueError(ly["type"])


def forward(cfg, P, ids, return_layers=False):
    """Logits [T, vocab] of one sequence (and the residual stream after every layer)."""
    eps, groups = cfg["norm"]["eps"], cfg["norm"].get("groups", 1)
    x = f64(P["embed"])[np.asarray(ids)]
    layers = []
    for li, ly in enumerate(cfg["layers"]):
        p = f"l{ly.get('weights_of', li)}."            # a layer may run on another layer's tensors (state of its own)
        x = x + mixer(group_norm(x, P[p + "norm1"], groups, eps), P, p + "mix.", ly, eps)
        if ly.get("mlp") is not None:
            x = x + mixture_ff(group_norm(x, P[p + "norm2"], groups, eps), P, p + "mlp.", ly["mlp"])
        layers.append(x.copy())
    logits = group_norm(x, P["final.norm"], groups, eps) @ f64(P["embed"]).T
    return (logits, np.stack(layers)) if return_layers else logits


def greedy(cfg, P, prompt, n_new):
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(np.argmax(forward(cfg, P, ids)[-1])))
    return ids[len(prompt):]
