"""Test helpers for the Gibipel decoder: small configurations, random bfloat16-exact weights, checkpoints on disk."""
import numpy as np

from tests.korupel_util import bf16_round, tokens, write_checkpoint  # noqa: F401  (shared helpers, re-exported)


def left(heads=4, kv_heads=2, dim=16, vdim=8, size=20, pool=6, scale=None, dims=None, base=10000.0, scaling="default"):
    if scaling == "default":
        scaling = dict(factor=3.0, low=1.0, high=5.0, original=64)
    rot = dict(base=base, dims=dim if dims is None else dims)
    if scaling is not None:
        rot["scaling"] = scaling
    return dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=dim ** -0.5 if scale is None else scale,
                mask=dict(size=size, pool=pool), rot=rot)


def right(heads=2, dim=8, vdim=12, gate_cap=12.0):
    return dict(heads=heads, dim=dim, vdim=vdim, gate_cap=gate_cap)


def moe(experts=5, top=2, ff=24, identity=1, groups=2, keep=1, shared=40):
    ml = dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top, identity=identity, groups=dict(count=groups, keep=keep)))
    if shared:
        ml["shared"] = dict(ff=shared)
    return ml


def layer(lf, rg, mlp, left_scale=0.8, right_scale=1.1):
    return dict(type="parallel", mixer=dict(left=lf, right=rg, left_scale=left_scale, right_scale=right_scale), mlp=mlp)


def config(layers, vocab=61, width=48, eps=2e-6, embed_scale=3.0, logit_scale=0.5):
    return dict(architecture="Gibipel", vocab=vocab, width=width, norm=dict(eps=eps), embedding=dict(scale=embed_scale),
                logit_scale=logit_scale, layers=layers)


def small_config():
    """Three layers whose sizes are neither equal to each other nor powers of two: windows of 20 / 33 / 9 with blocks of 6 / 7 / 4,
    part of a head rotating, a layer without a feed-forward, routers with and without groups, identity and shared experts."""
    return config([layer(left(heads=4, kv_heads=2, dim=16, vdim=8, size=20, pool=6, dims=12), right(heads=3, dim=8, vdim=12),
                         moe(experts=5, top=2, ff=24, identity=1, groups=2, keep=1, shared=40), 0.8, 1.1),
                   layer(left(heads=3, kv_heads=3, dim=12, vdim=20, size=33, pool=7, scale=0.3, base=500.0, scaling=None),
                         right(heads=2, dim=20, vdim=8, gate_cap=6.0), None, 1.3, 0.6),
                   layer(left(heads=6, kv_heads=2, dim=8, vdim=12, size=9, pool=4, scale=0.4), right(heads=1, dim=12, vdim=28),
                         moe(experts=4, top=3, ff=16, identity=0, groups=1, keep=1, shared=0), 0.5, 1.0)],
                  vocab=83, width=56)


def random_weights(cfg, seed=0):
    """name -> float32 array (bfloat16-exact), in the checkpoint's spelling and shapes (norm weights: one number, shape [])."""
    rs = np.random.RandomState(seed)
    W, V = cfg["width"], cfg["vocab"]
    P = {}

    def mat(name, o, i, s=None):
        P[name] = bf16_round(rs.randn(o, i) * (s if s is not None else i ** -0.5))

    def vec(name, n, s=0.1, off=0.0):
        P[name] = bf16_round(off + s * rs.randn(n))

    def one(name):
        P[name] = bf16_round(np.array([0.7 + 0.6 * rs.rand()])).reshape(())

    mat("embed", V, W, 1.0)
    for li, ly in enumerate(cfg["layers"]):
        p = f"l{li}."
        one(p + "norm1")
        a, b = ly["mixer"]["left"], ly["mixer"]["right"]
        H, G, d, e = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
        q = p + "mix.left."
        mat(q + "q", H * d, W); vec(q + "q.b", H * d, 0.3)
        mat(q + "k", G * d, W); vec(q + "k.b", G * d, 0.3)
        mat(q + "v", G * e, W); vec(q + "v.b", G * e, 0.3)
        vec(q + "q.norm", H * d, 0.2, 1.5); vec(q + "k.norm", G * d, 0.2, 1.5)
        vec(q + "sink", H, 1.0, 0.5)
        mat(q + "o", W, H * e)
        H, d, e = b["heads"], b["dim"], b["vdim"]
        q = p + "mix.right."
        mat(q + "q", H * d, W); mat(q + "k", H * d, W); mat(q + "v", H * e, W); mat(q + "g", H * e, W)
        mat(q + "i", H, W, 2.0 * W ** -0.5); vec(q + "i.b", H, 0.5)
        mat(q + "f", H, W, 2.0 * W ** -0.5); vec(q + "f.b", H, 1.0, 2.0)
        vec(q + "norm", H * e, 0.1, 1.0)
        mat(q + "o", W, H * e)
        ml = ly.get("mlp")
        if ml is not None:
            one(p + "norm2")
            ff, rt = ml["expert"]["ff"], ml["router"]
            for ex in range(rt["experts"]):
                mat(f"{p}mlp.e{ex}.gate", ff, W); mat(f"{p}mlp.e{ex}.up", ff, W); mat(f"{p}mlp.e{ex}.down", W, ff)
            outs = rt["experts"] + rt.get("identity", 0)
            mat(p + "mlp.router", outs, W, 3.0 * W ** -0.5)
            vec(p + "mlp.correction", outs, 0.05)
            if ml.get("shared"):
                sf = ml["shared"]["ff"]
                mat(p + "mlp.shared.gate", sf, W); mat(p + "mlp.shared.up", sf, W); mat(p + "mlp.shared.down", W, sf)
    one("final.norm")
    mat("head", V, W)
    return P


def planted(size, pool, heads=2, kv_heads=1, dim=16, vdim=8, alpha=8.0):
    """One layer whose attention input is a function of the token alone, with a query token QT and a key token KT: embedding
    coordinate 0 is set for KT only and feeds one key element that does not rotate, coordinate 1 likewise for QT's queries, so
    that KT's score with QT stands out whatever else is visible -- as a token of the window, and (divided by the block length,
    which the score's factor makes up for) inside the mean key of its block.  The matrix memory beside it is turned down."""
    cfg = config([layer(left(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, size=size, pool=pool, scale=max(2.0, pool / 3.0), dims=8, scaling=None),
                        right(heads=1, dim=4, vdim=4), None, 1.0, 0.05)], vocab=67, width=40, embed_scale=1.0)
    P = random_weights(cfg, 7)
    QT, KT = 65, 66
    at = dim - 3
    P["embed"][:, :2] = 0
    P["embed"][KT, 0] = 4.0
    P["embed"][QT, 1] = 4.0
    for n, shrink in (("q", 0.02), ("k", 0.25)):
        P[f"l0.mix.left.{n}"] = bf16_round(P[f"l0.mix.left.{n}"] * shrink)
        P[f"l0.mix.left.{n}.b"][:] = 0
        P[f"l0.mix.left.{n}.norm"][:] = 1.0
    for g in range(kv_heads):
        P["l0.mix.left.k"][g * dim + at] = 0
        P["l0.mix.left.k"][g * dim + at, 0] = alpha
    for hd in range(heads):
        P["l0.mix.left.q"][hd * dim + at] = 0
        P["l0.mix.left.q"][hd * dim + at, 1] = alpha
    P["l0.mix.left.sink"][:] = 0.0
    return cfg, P, QT, KT
