"""Named model configurations (HF ``config.json`` dictionaries).

Shapes from SURVEY.md section 8 (values tagged [external] there are the
HF-published ones).  ``tiny*`` configs are CPU-oracle-sized test models; the
first mirrors the reference's own unit-test config
(``crane-core/src/models/qwen3/modeling.rs:1386-1403``) scaled to dims the HIP
kernels accept (hidden/head_dim multiples of 64).
"""
from __future__ import annotations

import copy

_QWEN3_COMMON = dict(
    model_type="qwen3", rms_norm_eps=1e-6, rope_theta=1_000_000.0, attention_bias=False,
    use_qk_norm=True, max_position_embeddings=40960, torch_dtype="bfloat16",
)

CONFIGS = {
    "qwen3-0.6b": dict(_QWEN3_COMMON, vocab_size=151936, hidden_size=1024, intermediate_size=3072,
                       num_hidden_layers=28, num_attention_heads=16, num_key_value_heads=8,
                       head_dim=128, tie_word_embeddings=True),
    "qwen3-8b": dict(_QWEN3_COMMON, vocab_size=151936, hidden_size=4096, intermediate_size=12288,
                     num_hidden_layers=36, num_attention_heads=32, num_key_value_heads=8,
                     head_dim=128, tie_word_embeddings=False),
    # the headline geometry (every projection shape, GQA group and the 151 936-row lm_head of Qwen3-8B) at a depth the
    # CPU oracle finishes in seconds: the parity tests of the benchmarked kernel instantiations
    "qwen3-8b-2l": dict(_QWEN3_COMMON, vocab_size=151936, hidden_size=4096, intermediate_size=12288,
                        num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=8,
                        head_dim=128, tie_word_embeddings=False),
    "qwen3-0.6b-2l": dict(_QWEN3_COMMON, vocab_size=151936, hidden_size=1024, intermediate_size=3072,
                          num_hidden_layers=2, num_attention_heads=16, num_key_value_heads=8,
                          head_dim=128, tie_word_embeddings=True),
    # widths that are multiples of 2048 (what the persistent chain kernel needs), small enough for the numpy oracle
    "eng-qwen3": dict(_QWEN3_COMMON, vocab_size=2048, hidden_size=2048, intermediate_size=4096,
                      num_hidden_layers=3, num_attention_heads=32, num_key_value_heads=8,
                      head_dim=128, tie_word_embeddings=False, max_position_embeddings=8192),
    # the same with a GQA group of 2 (16 q / 8 kv heads: the text decoder of Qwen3-VL-2B, Qwen3-1.7B)
    "eng-qwen3-gqa2": dict(_QWEN3_COMMON, vocab_size=2048, hidden_size=2048, intermediate_size=6144,
                           num_hidden_layers=3, num_attention_heads=16, num_key_value_heads=8,
                           head_dim=128, tie_word_embeddings=True, max_position_embeddings=8192),
    # Qwen3-0.6B widths (hidden 1024, intermediate 3072: multiples of 1024 only -> the persistent kernel's 1024-element chunks)
    "eng-qwen3-h1024": dict(_QWEN3_COMMON, vocab_size=2048, hidden_size=1024, intermediate_size=3072,
                            num_hidden_layers=3, num_attention_heads=16, num_key_value_heads=8,
                            head_dim=128, tie_word_embeddings=True, max_position_embeddings=8192),
    # small shapes for CPU-oracle parity
    "tiny-qwen3": dict(_QWEN3_COMMON, vocab_size=512, hidden_size=256, intermediate_size=512,
                       num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
                       head_dim=128, tie_word_embeddings=True, max_position_embeddings=4096),
    "tiny-qwen3-untied": dict(_QWEN3_COMMON, vocab_size=1000, hidden_size=512, intermediate_size=1536,
                              num_hidden_layers=3, num_attention_heads=8, num_key_value_heads=2,
                              head_dim=128, tie_word_embeddings=False, max_position_embeddings=4096),
    "small-qwen3": dict(_QWEN3_COMMON, vocab_size=8192, hidden_size=1024, intermediate_size=3072,
                        num_hidden_layers=4, num_attention_heads=16, num_key_value_heads=8,
                        head_dim=128, tie_word_embeddings=True, max_position_embeddings=8192),
}


_QWEN35_COMMON = dict(
    model_type="qwen3_5_text", rms_norm_eps=1e-6, attention_bias=False, hidden_act="silu",
    linear_conv_kernel_dim=4, full_attention_interval=4, attn_output_gate=True, torch_dtype="bfloat16",
    rope_parameters=dict(rope_type="default", rope_theta=10_000_000.0, partial_rotary_factor=0.25,
                         mrope_section=[11, 11, 10], mrope_interleaved=True),
)
CONFIGS.update({
    # Qwen3.5-0.8B (values tagged [external] there)
    "qwen3.5-0.8b": dict(_QWEN35_COMMON, vocab_size=248320, hidden_size=1024, intermediate_size=3584,
                         num_hidden_layers=24, num_attention_heads=8, num_key_value_heads=2, head_dim=256,
                         linear_key_head_dim=128, linear_value_head_dim=128, linear_num_key_heads=16,
                         linear_num_value_heads=16, tie_word_embeddings=True, max_position_embeddings=262144),
    # Qwen3.5-2B: the model of the reference's only published numbers for this path (README.md:86-87,496-503: Qwen3.5-2B-Q8_0 on an
    # RX 7800 XT).  The reference does not spell its geometry out; this is the HF checkpoint's config as far as it is known here
    # (hidden 2048, 24 layers, 8 q / 2 kv heads of 256, 16 + 16 linear heads of 128): 1.88 B parameters
    "qwen3.5-2b": dict(_QWEN35_COMMON, vocab_size=248320, hidden_size=2048, intermediate_size=6144,
                       num_hidden_layers=24, num_attention_heads=8, num_key_value_heads=2, head_dim=256,
                       linear_key_head_dim=128, linear_value_head_dim=128, linear_num_key_heads=16,
                       linear_num_value_heads=16, tie_word_embeddings=True, max_position_embeddings=262144),
    # Qwen3.8-27B: fully pinned by the reference (qwen3_5/config.rs:298-324,332-364)
    "qwen3.8-27b": dict(_QWEN35_COMMON, vocab_size=248320, hidden_size=5120, intermediate_size=17408,
                        num_hidden_layers=64, num_attention_heads=24, num_key_value_heads=4, head_dim=256,
                        linear_key_head_dim=128, linear_value_head_dim=128, linear_num_key_heads=16,
                        linear_num_value_heads=48, tie_word_embeddings=False, max_position_embeddings=262144),
    # CPU-oracle sized hybrid: 3 GDN + 1 full layer, twice; value heads = 2 x key heads (interleaved pairing)
    "tiny-qwen3.5": dict(_QWEN35_COMMON, vocab_size=512, hidden_size=256, intermediate_size=512,
                         num_hidden_layers=8, num_attention_heads=4, num_key_value_heads=2, head_dim=256,
                         linear_key_head_dim=128, linear_value_head_dim=128, linear_num_key_heads=2,
                         linear_num_value_heads=4, tie_word_embeddings=False, max_position_embeddings=4096),
})


def _vl(text: dict, vision: dict, image_token_id: int) -> dict:
    t = dict(text)
    tie = t.pop("tie_word_embeddings", False)
    return dict(model_type="qwen3_5", text_config=t, vision_config=vision, tie_word_embeddings=tie,
                image_token_id=image_token_id, vision_start_token_id=image_token_id - 1,
                vision_end_token_id=image_token_id + 1, torch_dtype="bfloat16")


_VISION_COMMON = dict(model_type="qwen3_5_vision", hidden_act="gelu_pytorch_tanh", in_channels=3, patch_size=16,
                      temporal_patch_size=2, spatial_merge_size=2)
CONFIGS.update({
    # Qwen3-VL-2B-class tower ([external]): depth 24, hidden 1024, 16 heads, inter 4096, pos-emb 2304;
    # text side = the reference's LIVE VL text model (qwen3_5/vlm.rs): Qwen3.5-0.8B
    "qwen3.5-vl-0.8b": _vl(CONFIGS["qwen3.5-0.8b"],
                           dict(_VISION_COMMON, depth=24, hidden_size=1024, num_heads=16, intermediate_size=4096,
                                out_hidden_size=1024, num_position_embeddings=2304), 248056),
    "tiny-qwen3.5-vl": _vl(CONFIGS["tiny-qwen3.5"],
                           dict(_VISION_COMMON, depth=2, hidden_size=256, num_heads=4, intermediate_size=512,
                                out_hidden_size=256, num_position_embeddings=64), 500),
})


# Qwen3-VL (BASELINE configs[3]): dense Qwen3 text model with 3-axis interleaved MRoPE + the same vision tower plus DeepStack
# mergers after the listed blocks (reference: crane-core/src/models/qwen3_vl/; HF Qwen3VLConfig)
_QWEN3VL_TEXT = dict(model_type="qwen3_vl_text", rms_norm_eps=1e-6, attention_bias=False, hidden_act="silu", torch_dtype="bfloat16",
                     rope_parameters=dict(rope_type="default", rope_theta=5_000_000.0, mrope_section=[24, 20, 20], mrope_interleaved=True))


def _vl3(text: dict, vision: dict, image_token_id: int) -> dict:
    t = dict(_QWEN3VL_TEXT, **text)
    tie = t.pop("tie_word_embeddings", True)
    return dict(model_type="qwen3_vl", text_config=t, vision_config=dict(vision, model_type="qwen3_vl"), tie_word_embeddings=tie,
                image_token_id=image_token_id, video_token_id=image_token_id + 1, vision_start_token_id=image_token_id - 3,
                vision_end_token_id=image_token_id - 2, torch_dtype="bfloat16")


CONFIGS.update({
    # Qwen3-VL-2B ([external]): text 2048 / 28 layers / 16 q / 8 kv / 128 / 6144 / 151 936 tied;
    # vision depth 24, hidden 1024, 16 heads, inter 4096, patch 16, merge 2, out 2048, pos-emb 2304, deepstack [5, 11, 17]
    "qwen3-vl-2b": _vl3(dict(vocab_size=151936, hidden_size=2048, intermediate_size=6144, num_hidden_layers=28,
                             num_attention_heads=16, num_key_value_heads=8, head_dim=128, tie_word_embeddings=True,
                             max_position_embeddings=262144),
                        dict(_VISION_COMMON, depth=24, hidden_size=1024, num_heads=16, intermediate_size=4096, out_hidden_size=2048,
                             num_position_embeddings=2304, deepstack_visual_indexes=[5, 11, 17]), 151655),
    "tiny-qwen3-vl": _vl3(dict(vocab_size=512, hidden_size=256, intermediate_size=512, num_hidden_layers=3,
                               num_attention_heads=4, num_key_value_heads=2, head_dim=128, tie_word_embeddings=False,
                               max_position_embeddings=4096),
                          dict(_VISION_COMMON, depth=3, hidden_size=256, num_heads=4, intermediate_size=512, out_hidden_size=256,
                               num_position_embeddings=64, deepstack_visual_indexes=[0, 1]), 500),
})


# ---- layer-list decoders (config "architecture" + "layers"): Korupel -------------------------------------------------------
def korupel_config(vocab: int, width: int, pattern: str, heads: int, kv_heads: int, dim: int, window: int, keep_first: int,
                   lin_heads: int, lin_dim: int, lin_vdim: int, ff: int, experts: int = 0, top: int = 0, expert_ff: int = 0,
                   taps: int = 4, residual_mult: float = 0.5, eps: float = 1e-5) -> dict:
    """pattern: one letter per layer -- 'a' window attention, 'l' lightning attention; upper case: mixture of experts, lower
    case: dense feed-forward.  Lightning head h of H decays with 1 - 2^-(1 + 8 h / (H - 1)): from fast to slow."""
    layers = []
    for ch in pattern:
        if ch.lower() == "a":
            mixer = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=dim ** -0.5, mask=dict(size=window, keep_first=keep_first))
            kind = "attention"
        else:
            decay = [round(1.0 - 0.5 ** (1 + 8 * h / max(1, lin_heads - 1)), 6) for h in range(lin_heads)]
            mixer = dict(heads=lin_heads, dim=lin_dim, vdim=lin_vdim, decay=decay)
            kind = "lightning"
        mlp = (dict(kind="moe", expert=dict(ff=expert_ff), router=dict(experts=experts, top=top)) if ch.isupper()
               else dict(kind="dense", ff=ff))
        layers.append(dict(type=kind, mixer=mixer, mlp=mlp))
    return dict(architecture="Korupel", vocab=vocab, width=width, residual_mult=residual_mult, norm=dict(eps=eps),
                canon=dict(taps=taps), layers=layers)


CONFIGS.update({
    "tiny-korupel": korupel_config(320, 128, "aLlA", heads=4, kv_heads=2, dim=32, window=24, keep_first=3, lin_heads=2, lin_dim=16,
                                   lin_vdim=32, ff=192, experts=4, top=2, expert_ff=48),
    # the widths of the Qwen3.5-0.8B text decoder (1024 wide, 3584 ff, 24 layers, 3 linear : 1 softmax, vocabulary 248 320), dense
    "korupel-1b": korupel_config(248320, 1024, "llla" * 6, heads=8, kv_heads=2, dim=128, window=4096, keep_first=4, lin_heads=16,
                                 lin_dim=128, lin_vdim=128, ff=3584),
    # the same with 16 experts of 896, 4 per token (equal active width)
    "korupel-1b-moe": korupel_config(248320, 1024, "LLLA" * 6, heads=8, kv_heads=2, dim=128, window=4096, keep_first=4, lin_heads=16,
                                     lin_dim=128, lin_vdim=128, ff=3584, experts=16, top=4, expert_ff=896),
    "korupel-1b-4l": korupel_config(32768, 1024, "llla", heads=8, kv_heads=2, dim=128, window=4096, keep_first=4, lin_heads=16,
                                    lin_dim=128, lin_vdim=128, ff=3584),
})


# ---- layer-list decoders: Mononex ------------------------------------------------------------------------------------------
def mononex_config(vocab: int, width: int, pattern: str, ff: int, heads: int, kv_heads: int, dim: int, vdim: int, block: int,
                   lat_heads: int, lat_dim: int, rot_dim: int, lat_vdim: int, kv_rank: int, q_rank: int,
                   lin_heads: int, lin_dim: int, lin_vdim: int, tau: float = 8.0, rot_base: float = 10000.0,
                   yarn: "dict | None" = None, eps: float = 1e-6) -> dict:
    """pattern: one letter per layer -- 'a' softmax attention inside blocks of `block` positions, 'b' the same with the keys and
    values of the nearest 'a' before it, 'm' latent attention, 'g' gated linear attention; upper case: no feed-forward."""
    layers, last_a = [], None
    for i, ch in enumerate(pattern):
        c = ch.lower()
        if c in "ab":
            mixer = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=dim ** -0.5, mask=dict(size=block))
            if c == "b":
                if last_a is None:
                    raise ValueError("'b' needs an 'a' layer before it")
                mixer["kv_from"] = last_a
            else:
                last_a = i
            kind = "attention"
        elif c == "m":
            rot = dict(base=rot_base, dims=rot_dim)
            if yarn:
                rot["scaling"] = dict(yarn)
            mixer = dict(heads=lat_heads, dim=lat_dim, rot_dim=rot_dim, vdim=lat_vdim, kv_rank=kv_rank, q_rank=q_rank,
                         scale=(lat_dim + rot_dim) ** -0.5, rot=rot)
            kind = "latent_attention"
        elif c == "g":
            mixer = dict(heads=lin_heads, dim=lin_dim, vdim=lin_vdim, tau=tau)
            kind = "gla"
        else:
            raise ValueError(f"pattern letter {ch!r}")
        layers.append(dict(type=kind, mixer=mixer, mlp=None if ch.isupper() else dict(kind="dense", ff=ff)))
    return dict(architecture="Mononex", vocab=vocab, width=width, norm=dict(eps=eps), layers=layers)


_YARN = dict(factor=4.0, original=4096, fast=32.0, slow=1.0)
CONFIGS.update({
    "tiny-mononex": mononex_config(320, 128, "gabMg", ff=192, heads=4, kv_heads=2, dim=32, vdim=16, block=24, lat_heads=2, lat_dim=16,
                                   rot_dim=8, lat_vdim=24, kv_rank=32, q_rank=48, lin_heads=2, lin_dim=16, lin_vdim=32, tau=8.0,
                                   yarn=dict(factor=2.0, original=64, fast=8.0, slow=1.0)),
    # the widths of the Qwen3.5-0.8B text decoder (1024 wide, 3584 ff, 24 layers, vocabulary 248 320): 12 gated linear layers, 4 block
    # attention layers with keys of their own and 4 that borrow them, 4 latent attention layers
    "mononex-1b": mononex_config(248320, 1024, "ggabgm" * 4, ff=3584, heads=8, kv_heads=2, dim=128, vdim=128, block=4096, lat_heads=8,
                                 lat_dim=128, rot_dim=64, lat_vdim=128, kv_rank=512, q_rank=768, lin_heads=16, lin_dim=128, lin_vdim=128,
                                 yarn=_YARN),
    "mononex-1b-6l": mononex_config(32768, 1024, "ggabgm", ff=3584, heads=8, kv_heads=2, dim=128, vdim=128, block=4096, lat_heads=8,
                                    lat_dim=128, rot_dim=64, lat_vdim=128, kv_rank=512, q_rank=768, lin_heads=16, lin_dim=128, lin_vdim=128,
                                    yarn=_YARN),
})


# ---- layer-list decoders: Gibipel ------------------------------------------------------------------------------------------
def gibipel_config(vocab: int, width: int, n_layers: int, heads: int, kv_heads: int, dim: int, vdim: int, window: int, pool: int,
                   mem_heads: int, mem_dim: int, mem_vdim: int, experts: int, top: int, expert_ff: int, identity: int = 0,
                   groups: int = 1, keep_groups: int = 1, shared_ff: int = 0, rot_dims: "int | None" = None, rot_base: float = 10000.0,
                   scaling: "dict | None" = None, left_scale: float = 1.0, right_scale: float = 1.0, gate_cap: float = 15.0,
                   embed_scale: float = 1.0, logit_scale: float = 1.0, eps: float = 1e-5, no_ff: "tuple | list" = ()) -> dict:
    """Every layer holds both mixers side by side: window attention that sees the blocks of `pool` positions in front of its
    window through their mean key / value, and a matrix memory; a mixture-of-experts feed-forward (layers in `no_ff`: none)."""
    layers = []
    for i in range(n_layers):
        rot = dict(base=rot_base, dims=dim if rot_dims is None else rot_dims)
        if scaling:
            rot["scaling"] = dict(scaling)
        left = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=dim ** -0.5, mask=dict(size=window, pool=pool), rot=rot)
        right = dict(heads=mem_heads, dim=mem_dim, vdim=mem_vdim, gate_cap=gate_cap)
        mlp = None
        if i not in no_ff:
            mlp = dict(kind="moe", expert=dict(ff=expert_ff),
                       router=dict(experts=experts, top=top, identity=identity, groups=dict(count=groups, keep=keep_groups)))
            if shared_ff:
                mlp["shared"] = dict(ff=shared_ff)
        layers.append(dict(type="parallel", mixer=dict(left=left, right=right, left_scale=left_scale, right_scale=right_scale), mlp=mlp))
    return dict(architecture="Gibipel", vocab=vocab, width=width, norm=dict(eps=eps), embedding=dict(scale=embed_scale),
                logit_scale=logit_scale, layers=layers)


_BANDS = dict(factor=8.0, low=1.0, high=4.0, original=8192)
CONFIGS.update({
    "tiny-gibipel": gibipel_config(320, 128, 3, heads=4, kv_heads=2, dim=32, vdim=16, window=20, pool=6, mem_heads=2, mem_dim=16,
                                   mem_vdim=24, experts=6, top=2, expert_ff=48, identity=2, groups=2, keep_groups=1, shared_ff=64,
                                   rot_dims=16, scaling=dict(factor=4.0, low=1.0, high=4.0, original=64), left_scale=0.7,
                                   right_scale=1.2, embed_scale=4.0, logit_scale=0.5, no_ff=(1,)),
    # the widths of the Qwen3.5-0.8B text decoder and of korupel-1b-moe (1024 wide, 24 layers, vocabulary 248 320, 8 query / 2 key
    # heads of 128): window 1024 and blocks of 64, 8 memory heads of 64 x 128, 14 experts + 2 identity experts in 2 groups, 4 per
    # token, of 768, and a shared expert of 512 (3584 active inner columns, as the dense models)
    "gibipel-1b": gibipel_config(248320, 1024, 24, heads=8, kv_heads=2, dim=128, vdim=128, window=1024, pool=64, mem_heads=8, mem_dim=64,
                                 mem_vdim=128, experts=14, top=4, expert_ff=768, identity=2, groups=2, keep_groups=1, shared_ff=512,
                                 scaling=_BANDS, rot_base=500000.0),
    "gibipel-1b-4l": gibipel_config(32768, 1024, 4, heads=8, kv_heads=2, dim=128, vdim=128, window=1024, pool=64, mem_heads=8, mem_dim=64,
                                    mem_vdim=128, experts=14, top=4, expert_ff=768, identity=2, groups=2, keep_groups=1, shared_ff=512,
                                    scaling=_BANDS, rot_base=500000.0),
})


# ---- layer-list decoders: Nevotar ------------------------------------------------------------------------------------------
def nevotar_config(vocab: int, width: int, kinds: "list | tuple", heads: int, kv_heads: int, dim: int, vdim: int, window: int,
                   rec_heads: int, rec_dim: int, rec_vdim: int, ssm_heads: int, ssm_vdim: int, state: int, ssm_groups: int, experts: int,
                   top: int, expert_ff: int, shared_ff: int = 0, limit: float = 7.0, diff: float = 0.5, q_coef: float = 0.1, q_every: int = 1024,
                   rot_dims: "int | None" = None, rot_base: float = 1000000.0, conv: int = 4, ssm_norm_groups: int = 1, left_scale: float = 1.0,
                   right_scale: float = 1.0, norm_groups: int = 1, eps: float = 1e-6, no_ff: "tuple | list" = (), weights_of: "dict | None" = None) -> dict:
    """Pre-norm layers of the kinds named in `kinds`: "attention" (two softmax maps per head, `dim` per map), "hgrn2" (gated
    recurrence) and "parallel" (window attention with mixed heads beside a state-space mixer); mixture-of-experts feed-forwards
    (layers in `no_ff`: none); weights_of[i] = j lets layer i run on layer j's tensors."""
    made = []
    for i, kind in enumerate(kinds):
        if kind == "attention":
            mx = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, diff=diff, q_temp=dict(coef=q_coef, every=q_every), scale=dim ** -0.5)
        elif kind == "hgrn2":
            mx = dict(heads=rec_heads, dim=rec_dim, vdim=rec_vdim)
        else:
            mx = dict(left=dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=dim ** -0.5, mask=dict(size=window),
                                rot=dict(base=rot_base, dims=dim if rot_dims is None else rot_dims)),
                      right=dict(heads=ssm_heads, vdim=ssm_vdim, state=state, groups=ssm_groups, conv=conv, norm_groups=ssm_norm_groups),
                      left_scale=left_scale, right_scale=right_scale)
        mlp = None
        if i not in no_ff:
            mlp = dict(kind="moe", expert=dict(ff=expert_ff, limit=limit), router=dict(experts=experts, top=top))
            if shared_ff:
                mlp["shared"] = dict(ff=shared_ff, limit=limit)
        ly = dict(type=kind, mixer=mx, mlp=mlp)
        if weights_of and i in weights_of:
            ly = dict(copy.deepcopy(made[weights_of[i]]), weights_of=weights_of[i])
        made.append(ly)
    return dict(architecture="Nevotar", vocab=vocab, width=width, norm=dict(eps=eps, groups=norm_groups), layers=made)


_NEVOTAR_1B = dict(heads=8, kv_heads=2, dim=128, vdim=128, window=1024, rec_heads=8, rec_dim=128, rec_vdim=128, ssm_heads=16, ssm_vdim=64,
                   state=128, ssm_groups=2, experts=14, top=4, expert_ff=768, shared_ff=512, rot_dims=64, ssm_norm_groups=2, norm_groups=2)
CONFIGS.update({
    "tiny-nevotar": nevotar_config(320, 128, ["attention", "hgrn2", "parallel", "parallel", "attention"], heads=4, kv_heads=2, dim=16, vdim=24,
                                   window=20, rec_heads=2, rec_dim=16, rec_vdim=24, ssm_heads=4, ssm_vdim=8, state=16, ssm_groups=2, experts=6,
                                   top=2, expert_ff=48, shared_ff=64, limit=1.5, q_every=16, rot_dims=8, ssm_norm_groups=2, left_scale=0.7,
                                   right_scale=1.2, norm_groups=4, no_ff=(1,), weights_of={3: 2, 4: 0}),
    # the widths of korupel-1b-moe / gibipel-1b (1024 wide, 24 layers, vocabulary 248 320, 8 query / 2 key heads of 128): 6 layers of
    # two-map attention over the whole context, 6 gated recurrences of 8 heads of 128 x 128, 12 layers of window attention (1024, mixed
    # heads, half of a head rotates) beside a state-space mixer of 16 heads of 128 x 64; 14 experts of 768, 4 per token, and a shared
    # expert of 512 (3584 active inner columns, as the dense models)
    "nevotar-1b": nevotar_config(248320, 1024, ["attention", "hgrn2", "parallel", "parallel"] * 6, **_NEVOTAR_1B),
    "nevotar-1b-4l": nevotar_config(32768, 1024, ["attention", "hgrn2", "parallel", "parallel"], **_NEVOTAR_1B),
})


def get_config(name: str) -> dict:
    if name not in CONFIGS:
        raise KeyError(f"unknown config {name!r}; have {sorted(CONFIGS)}")
    return copy.deepcopy(CONFIGS[name])


def synthetic_prompt(n: int, vocab: int):
    """ids[i] = (7 i + 3) mod V  -- the pattern of qwen3_5/prefill.rs:249."""
    return [(7 * i + 3) % vocab for i in range(n)]
