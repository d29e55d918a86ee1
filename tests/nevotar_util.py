"""Test helpers for the Nevotar decoder: small configurations, random bfloat16-exact weights, checkpoints on disk."""
import numpy as np

from tests.korupel_util import bf16_round, tokens, write_checkpoint  # noqa: F401  (shared helpers, re-exported)


def attn(heads=4, kv_heads=2, dim=12, vdim=20, diff=0.55, coef=0.25, every=7, scale=None):
    return dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, diff=diff, q_temp=dict(coef=coef, every=every),
                scale=dim ** -0.5 if scale is None else scale)


def hgrn(heads=3, dim=8, vdim=12):
    return dict(heads=heads, dim=dim, vdim=vdim)


def left(heads=4, kv_heads=2, dim=16, vdim=8, size=20, dims=None, base=10000.0, scale=None):
    return dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=dim ** -0.5 if scale is None else scale, mask=dict(size=size),
                rot=dict(base=base, dims=dim if dims is None else dims))


def right(heads=4, vdim=6, state=8, groups=2, conv=4, norm_groups=2):
    return dict(heads=heads, vdim=vdim, state=state, groups=groups, conv=conv, norm_groups=norm_groups)


def moe(experts=5, top=2, ff=24, limit=1.5, shared=40, shared_limit=0.75):
    ml = dict(kind="moe", expert=dict(ff=ff, limit=limit), router=dict(experts=experts, top=top))
    if shared:
        ml["shared"] = dict(ff=shared, limit=shared_limit)
    return ml


def layer(kind, mixer, mlp, weights_of=None):
    ly = dict(type=kind, mixer=mixer, mlp=mlp)
    if weights_of is not None:
        ly["weights_of"] = weights_of
    return ly


def side(lf, rg, left_scale=0.8, right_scale=1.1):
    return dict(left=lf, right=rg, left_scale=left_scale, right_scale=right_scale)


def config(layers, vocab=61, width=48, eps=2e-6, groups=3):
    return dict(architecture="Nevotar", vocab=vocab, width=width, norm=dict(eps=eps, groups=groups), layers=layers)


def small_config():
    """Every kind of layer with sizes that are neither equal to each other nor powers of two, a layer without a feed-forward, and
    two layers that run on earlier layers' tensors."""
    return config([layer("attention", attn(heads=4, kv_heads=2, dim=12, vdim=20, every=7), moe(experts=5, top=2, ff=24, shared=40)),
                   layer("hgrn2", hgrn(heads=3, dim=8, vdim=12), None),
                   layer("parallel", side(left(heads=6, kv_heads=2, dim=16, vdim=8, size=20, dims=12), right(heads=4, vdim=6, state=8, groups=2, conv=4, norm_groups=2)),
                         moe(experts=3, top=1, ff=16, limit=0.8, shared=0)),
                   layer("parallel", side(left(heads=6, kv_heads=2, dim=16, vdim=8, size=20, dims=12), right(heads=4, vdim=6, state=8, groups=2, conv=4, norm_groups=2)),
                         moe(experts=3, top=1, ff=16, limit=0.8, shared=0), weights_of=2),
                   layer("attention", attn(heads=4, kv_heads=2, dim=12, vdim=20, every=7), moe(experts=5, top=2, ff=24, shared=40), weights_of=0),
                   layer("parallel", side(left(heads=3, kv_heads=3, dim=20, vdim=12, size=33, dims=8, base=300.0, scale=0.3),
                                          right(heads=2, vdim=10, state=12, groups=1, conv=3, norm_groups=1), 1.3, 0.6), None)],
                  vocab=83, width=56, groups=4)


def random_weights(cfg, seed=0):
    """name -> float32 array (bfloat16-exact), in the checkpoint's spelling and shapes; layers with weights_of have none."""
    rs = np.random.RandomState(seed)
    W, V = cfg["width"], cfg["vocab"]
    P = {}

    def mat(name, o, i, s=None):
        P[name] = bf16_round(rs.randn(o, i) * (s if s is not None else i ** -0.5))

    def vec(name, n, s=0.1, off=0.0):
        P[name] = bf16_round(off + s * rs.randn(n))

    mat("embed", V, W, 1.0)
    for li, ly in enumerate(cfg["layers"]):
        if ly.get("weights_of") is not None:
            continue
        p = f"l{li}."
        vec(p + "norm1", W, 0.1, 1.0)
        mx = ly["mixer"]
        if ly["type"] == "attention":
            H, G, d, e = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
            q = p + "mix."
            mat(q + "q", 2 * H * d, W, 2.0 * W ** -0.5); vec(q + "q.b", 2 * H * d, 0.3)
            mat(q + "k", 2 * G * d, W, 2.0 * W ** -0.5); vec(q + "k.b", 2 * G * d, 0.3)
            mat(q + "v", G * e, W); vec(q + "v.b", G * e, 0.3)
            for n in ("lq1", "lk1", "lq2", "lk2"):
                vec(q + n, d, 0.3)
            mat(q + "o", W, H * e)
        elif ly["type"] == "hgrn2":
            H, d, e = mx["heads"], mx["dim"], mx["vdim"]
            q = p + "mix."
            mat(q + "q", H * d, W); mat(q + "f", H * d, W, 2.0 * W ** -0.5); vec(q + "f.b", H * d, 1.0, 1.0)
            P[q + "lower"] = bf16_round(0.9 * rs.rand(H * d))
            mat(q + "v", H * e, W)
            vec(q + "norm", e, 0.2, 1.0)
            mat(q + "o", W, H * e)
        else:
            a, b = mx["left"], mx["right"]
            H, G, d, e = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            q = p + "mix.left."
            mat(q + "q", H * d, W); vec(q + "q.b", H * d, 0.3)
            mat(q + "k", G * d, W); vec(q + "k.b", G * d, 0.3)
            mat(q + "v", G * e, W); vec(q + "v.b", G * e, 0.3)
            vec(q + "q.norm", d, 0.2, 1.5); vec(q + "k.norm", d, 0.2, 1.5)
            P[q + "talk"] = bf16_round(np.eye(H) + 0.4 * rs.randn(H, H))
            mat(q + "o", W, H * e)
            H, e, N, Gr, taps = b["heads"], b["vdim"], b["state"], b["groups"], b["conv"]
            inner, C = H * e, H * e + 2 * Gr * N
            q = p + "mix.right."
            mat(q + "in", 2 * inner + 2 * Gr * N + H, W)
            P[q + "conv"] = bf16_round(rs.randn(C, taps) * taps ** -0.5)
            vec(q + "conv.b", C, 0.2)
            vec(q + "dt_bias", H, 0.5, -0.5)
            vec(q + "A_log", H, 0.7, -0.5)
            vec(q + "D", H, 0.3, 1.0)
            vec(q + "norm", inner, 0.1, 1.0)
            mat(q + "o", W, inner)
        ml = ly.get("mlp")
        if ml is not None:
            vec(p + "norm2", W, 0.1, 1.0)
            ff, rt = ml["expert"]["ff"], ml["router"]
            for ex in range(rt["experts"]):
                mat(f"{p}mlp.e{ex}.gate", ff, W, 2.0 * W ** -0.5); mat(f"{p}mlp.e{ex}.up", ff, W, 2.0 * W ** -0.5); mat(f"{p}mlp.e{ex}.down", W, ff)
            mat(p + "mlp.router", rt["experts"], W, 3.0 * W ** -0.5)
            if ml.get("shared"):
                sf = ml["shared"]["ff"]
                mat(p + "mlp.shared.gate", sf, W, 2.0 * W ** -0.5); mat(p + "mlp.shared.up", sf, W, 2.0 * W ** -0.5); mat(p + "mlp.shared.down", W, sf)
    vec("final.norm", W, 0.1, 1.0)
    return P


def planted_window(size, heads=4, kv_heads=2, dim=16, vdim=8, alpha=8.0):
    """One layer whose window attention sees a query token QT and a key token KT stand out: embedding coordinate 0 is set for KT only
    and feeds one key element that does not rotate, coordinate 1 likewise for QT's queries; after the per-head norm those elements
    carry the whole head, so that KT's score with QT dominates whatever else is visible.  The mixing matrix is positive, so that
    every mixed head sees it; the state-space mixer beside it is switched off."""
    cfg = config([layer("parallel", side(left(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, size=size, dims=8, scale=1.0),
                                         right(heads=2, vdim=4, state=4, groups=1, conv=2, norm_groups=1), 1.0, 0.0), None)], vocab=67, width=40, groups=1)
    P = random_weights(cfg, 7)
    QT, KT = 65, 66
    at = dim - 3
    P["embed"][:, :2] = 0
    P["embed"][KT, 0] = 4.0
    P["embed"][QT, 1] = 4.0
    P["l0.norm1"][:] = 1.0
    for n in "qk":
        P[f"l0.mix.left.{n}"] = bf16_round(P[f"l0.mix.left.{n}"] * 0.25)
        P[f"l0.mix.left.{n}.b"][:] = 0
        P[f"l0.mix.left.{n}.norm"][:] = 1.0
    for g in range(kv_heads):
        P["l0.mix.left.k"][g * dim + at] = 0
        P["l0.mix.left.k"][g * dim + at, 0] = alpha
    for hd in range(heads):
        P["l0.mix.left.q"][hd * dim + at] = 0
        P["l0.mix.left.q"][hd * dim + at, 1] = alpha
    P["l0.mix.left.talk"] = bf16_round(np.abs(P["l0.mix.left.talk"]))
    return cfg, P, QT, KT


def planted_causal(heads=2, kv_heads=1, dim=8, vdim=8, alpha=8.0):
    """One differential-attention layer in which a key token KT far back takes nearly all of the FIRST map's weight of a query token
    QT (the second map stays spread out), among hundreds of visible keys."""
    cfg = config([layer("attention", attn(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, diff=0.3, coef=0.2, every=50, scale=1.0), None)],
                 vocab=67, width=40, groups=2)
    P = random_weights(cfg, 8)
    QT, KT = 65, 66
    P["embed"][:, :2] = 0
    P["embed"][KT, 0] = 4.0
    P["embed"][QT, 1] = 4.0
    P["l0.norm1"][:] = 1.0
    for n in "qk":
        P[f"l0.mix.{n}"] = bf16_round(P[f"l0.mix.{n}"] * 0.1)
        P[f"l0.mix.{n}.b"][:] = 0
    for g in range(kv_heads):
        P["l0.mix.k"][g * 2 * dim + 2] = 0
        P["l0.mix.k"][g * 2 * dim + 2, 0] = alpha           # element 2 of the first map
    for hd in range(heads):
        P["l0.mix.q"][hd * 2 * dim + 2] = 0
        P["l0.mix.q"][hd * 2 * dim + 2, 1] = alpha
    return cfg, P, QT, KT
