// Layer-list decoders on the Model runtime (layered.h): configuration, weights, per-sequence state and the step function.
//
// What is shared with the other families: the handle and its options, the sequence table and the page allocator (Seq, ensure_pages,
// seq_alloc / seq_free / seq_fork / seq_truncate), the per-slot state pools (conv_pool: the convolution tails of every sublayer,
// state_pool: the linear-attention states), the embedding gather, the logits rows the samplers read (logitsb), the engine.
// What is new: Model::step_batch -- ONE pass over the weights for any mix of prompt portions and single decode tokens, each
// continuing its sequence from the cache and state earlier steps left; forward / prefill_multi / decode_batch / generate and the
// engine's scheduler all go through it for this family.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <map>

#include "json_min.h"
#include "model.h"
#include "safetensors.h"

namespace cm {

struct Layered {
    std::vector<LayerSpec> spec;
    std::vector<LayeredLayerW> w;
    int taps = 0;                      // 0: no convolution in front of the sublayers
    float mult = 1.f;
    // Mononex: x += mixer(shift(norm1 x)) + ff(norm2 x), no norm behind the sublayers; Korupel: one sublayer after the other,
    // a norm on each side
    bool parallel = false;
    // Gibipel: a sublayer reads the residual itself and a one-number norm sits on its output; embedding and logits are scaled
    bool post_only = false;
    float embed_scale = 1.f, logit_scale = 1.f;
    // Nevotar: x += mixer(norm1 x), x += ff(norm2 x); the norms work on norm_groups equal parts of the vector; the logits come from the
    // embedding table
    bool pre_norm = false;
    int norm_groups = 1;
    int max_conv = 0;                  // widest convolution of a state-space mixer (channels)
    float* XB = nullptr;               // [cap][max_conv] convolved and activated channels
    int max_mh = 0, max_sff = 0, max_slots = 1;   // matrix-memory heads, shared expert size, rows per token of an expert combine
    float* Z = nullptr;                // router logits [cap][most outputs]
    float *KM = nullptr, *MR = nullptr, *HS = nullptr;   // matrix memory: key factor and running maximum per token and head; shared expert's inner rows
    int max_q = 0, max_qa = 0, max_cq = 0, max_ld = 0, max_e = 0;
    bool f32 = false;                  // number format of the projections and the key cache
    float* final_norm = nullptr;
    uint16_t* head = nullptr;
    int cap = 0;                       // rows of one pass
    int max_in = 0, max_o = 0, max_ff = 0, max_top = 1, max_E = 1;
    std::vector<int> nreps;            // distinct query-heads-per-key-head values of the attention layers
    float *X = nullptr, *Hn = nullptr, *Hc = nullptr, *P = nullptr, *O = nullptr, *O2 = nullptr, *Y = nullptr, *HH = nullptr, *YS = nullptr,
          *wsel = nullptr, *Xw = nullptr;
    int32_t *sel = nullptr, *srt = nullptr, *off = nullptr;
    uint32_t *d_greedy = nullptr, *h_greedy = nullptr;
    float* h_rows = nullptr;           // pinned staging of logits rows
    int32_t *d_tab = nullptr, *h_tab = nullptr;
    size_t tab_ints = 0;
    static constexpr int LOGIT_ROWS = 256;
    // bfloat16 format, products of 32 rows or more whose shape fits (N % 128 == 0, K % 32 == 0): the matrix-core GEMM the other
    // families' prompt passes use (kernels_prefill.hip / kernels_gemm256.hip), plain bf16 activations; cm_debug_set("lay_shared_gemm", 0): never
    bool shared_gemm = true;
    bool attn_mfma = true;             // bfloat16 format, prompt passes: the matrix-core attention (cm_debug_set("lay_attn_mfma", 0): never)
    bool fused_prep = true;            // query / key norm + rotation + cache append in one launch (cm_debug_set("lay_fused_prep", 0): single operations)
    uint16_t* Abf = nullptr;           // [cap rounded up to 256][widest K] bf16 A operand
    float *G1 = nullptr, *G2 = nullptr;   // [cap][widest dense ff] the two products of a gated feed-forward
    float* U = nullptr;                // lightning attention, chunk-parallel form: [chunks of a pass][widest H d e] f32
    size_t u_stride = 0;
    float* Dch = nullptr;              // gated linear attention, chunk-parallel form: [chunks of a pass][widest H d] decay of a chunk
    float *H2 = nullptr, *Y2 = nullptr;                  // parallel layers: second norm's rows, feed-forward output
    float *CQ = nullptr, *Q = nullptr, *Qa = nullptr;    // latent attention: query latent, queries, queries against the cached latent
    float* LD = nullptr;               // gated linear attention: logarithm of the decay per token and key channel
    static constexpr int ATT_PARTS = 512;   // (query tile, key head, split) blocks of a split-key attention launch
    float *att_po = nullptr, *att_pml = nullptr;
    float* am_pv = nullptr; int* am_pi = nullptr;   // arg-max partials of the logits rows
    bool capture = false;              // cm_debug_set("lay_capture"): keep the residual stream after every layer of every pass
    std::vector<float> captured;
    ~Layered() {
        if (h_greedy) (void)hipHostFree(h_greedy);
        if (h_rows) (void)hipHostFree(h_rows);
        if (h_tab) (void)hipHostFree(h_tab);
    }
};

void LayeredDeleter::operator()(Layered* p) const { delete p; }

// one projection of a pass: the shared matrix-core GEMM where it applies, else the kernels of kernels_layered.hip
static void lay_gemm(Model& m, Layered& L, const LGemmArgs& g, int groups, hipStream_t s) {
    const bool bf = !L.f32;
    if (bf && L.shared_gemm && L.Abf && groups == 1 && !g.a_idx && !g.c_idx && !g.grp_off && !g.mul && g.M >= 32 && g.N % 128 == 0 && g.K % 32 == 0 &&
        (!g.W2 || (g.ldc == g.N && L.G1 && L.G2))) {
        launch_lay_round_rows(g.A, g.lda, L.Abf, g.M, g.K, s);
        GemmArgs a{};
        a.A_hi = L.Abf; a.A_lo = nullptr; a.W = g.W; a.bias = g.bias;
        a.C = g.W2 ? L.G1 : g.C; a.ldc = g.W2 ? g.N : g.ldc;
        a.M = g.M; a.N = g.N; a.K = g.K; a.ws = m.pWS; a.ws_floats = m.pWS ? Model::gemm_ws_floats : 0; a.ksplit = 1; a.wide256 = m.gemm256;
        bool ok = launch_gemm(a, GEPI_STORE, s);
        if (ok && g.W2) { a.W = g.W2; a.C = L.G2; ok = launch_gemm(a, GEPI_STORE, s); }
        if (ok) {
            if (g.W2) launch_lay_act_mul(L.G1, L.G2, g.C, (size_t)g.M * g.N, g.act, s, g.act_param);
            else launch_lay_act_cols(g.C, g.ldc, g.M, g.N, g.act, g.act2, g.act_split, s, g.act_param);
            return;
        }
    }
    // a wide product whose column count is no multiple of the shared GEMM's tile: the whole tiles there, the last columns here
    if (bf && L.shared_gemm && L.Abf && groups == 1 && !g.a_idx && !g.c_idx && !g.grp_off && !g.mul && !g.W2 && g.M >= 256 && g.N >= 256 &&
        g.N % 128 != 0 && g.K % 32 == 0) {
        const int n0 = g.N - g.N % 128;
        LGemmArgs g1 = g, g2 = g;
        g1.N = n0;
        g2.W = g.W + (size_t)n0 * g.K; g2.C = g.C + n0; g2.N = g.N - n0; g2.bias = g.bias ? g.bias + n0 : nullptr;
        g2.act_split = std::max(0, g.act_split - n0);
        lay_gemm(m, L, g1, 1, s);
        launch_lgemm(g2, bf, 1, s);
        return;
    }
    launch_lgemm(g, bf, groups, s);
}

static void need(bool ok, const char* what) { if (!ok) throw CmError(CM_ERR_INVALID, std::string("config.json: ") + what); }

// "mlp": null | {"kind": "dense", "ff"} | {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top"}}
static void parse_mlp(const cmjson::Value* ml, LayerSpec& sp, bool moe_ok) {
    if (!ml || ml->kind != cmjson::Value::Obj) return;
    const std::string kind = ml->string("kind", "dense");
    if (kind == "dense") {
        sp.mlp = LMLP_DENSE;
        sp.ff = (int)ml->integer("ff", 0);
    } else if (kind == "moe" && moe_ok) {
        sp.mlp = LMLP_MOE;
        const cmjson::Value* ex = ml->get("expert");
        const cmjson::Value* rt = ml->get("router");
        if (!ex || !rt) throw CmError(CM_ERR_IO, "config.json: moe without expert / router");
        sp.ff = (int)ex->integer("ff", 0);
        sp.limit = (float)ex->number("limit", 0.0);
        sp.experts = (int)rt->integer("experts", 0);
        sp.top = (int)rt->integer("top", 0);
        sp.router.identity = (int)rt->integer("identity", 0);
        if (const cmjson::Value* gr = rt->get("groups"))
            if (gr->kind == cmjson::Value::Obj) {
                sp.router.groups = (int)gr->integer("count", 1);
                sp.router.keep_groups = (int)gr->integer("keep", sp.router.groups);
            }
        const int outs = sp.experts + sp.router.identity;
        if (sp.experts <= 0 || sp.top <= 0 || sp.router.identity < 0 || sp.top > outs || outs > 4096) throw CmError(CM_ERR_INVALID, "router.experts / router.top");
        if (sp.router.groups <= 0 || outs % sp.router.groups || sp.router.keep_groups <= 0 || sp.router.keep_groups > sp.router.groups ||
            sp.top > outs / sp.router.groups * sp.router.keep_groups)
            throw CmError(CM_ERR_INVALID, "router.groups");
        if (const cmjson::Value* sh = ml->get("shared"))
            if (sh->kind == cmjson::Value::Obj) {
                sp.shared_ff = (int)sh->integer("ff", 0);
                sp.shared_limit = (float)sh->number("limit", 0.0);
                if (sp.shared_ff <= 0) throw CmError(CM_ERR_IO, "config.json: shared.ff");
            }
    } else throw CmError(CM_ERR_UNSUPPORTED, "mlp.kind '" + kind + "' not implemented");
    if (sp.ff <= 0) throw CmError(CM_ERR_IO, "config.json: ff");
}

// Korupel: "residual_mult", "canon".taps; layer types "attention" (window + kept first tokens) and "lightning"
static void parse_korupel_layer(const cmjson::Value& e, LayerSpec& sp) {
    const std::string type = e.string("type", "");
    sp.mixer = type == "attention" ? LMIX_ATTN : (type == "lightning" ? LMIX_LIGHTNING : -1);
    if (sp.mixer < 0) throw CmError(CM_ERR_UNSUPPORTED, "layer type '" + type + "' not implemented");
    const cmjson::Value* mx = e.get("mixer");
    if (!mx || mx->kind != cmjson::Value::Obj) throw CmError(CM_ERR_IO, "config.json: layer without mixer");
    sp.heads = (int)mx->integer("heads", 0);
    sp.kv_heads = (int)mx->integer("kv_heads", sp.heads);
    sp.dim = (int)mx->integer("dim", 0);
    sp.vdim = (int)mx->integer("vdim", sp.dim);
    if (sp.heads <= 0 || sp.dim <= 0 || sp.vdim <= 0) throw CmError(CM_ERR_IO, "config.json: mixer sizes");
    if (sp.mixer == LMIX_ATTN) {
        if (sp.kv_heads <= 0 || sp.heads % sp.kv_heads) throw CmError(CM_ERR_INVALID, "heads % kv_heads != 0");
        if (sp.vdim != sp.dim) throw CmError(CM_ERR_INVALID, "attention whose values are its keys needs vdim == dim");
        if (sp.dim > 256) throw CmError(CM_ERR_UNSUPPORTED, "attention head size above 256");
        sp.scale = (float)mx->number("scale", 1.0 / std::sqrt((double)sp.dim));
        sp.win = 1ll << 40; sp.keep = 0;
        if (const cmjson::Value* mk = mx->get("mask"))
            if (mk->kind == cmjson::Value::Obj) {
                sp.win = mk->integer("size", sp.win);
                sp.keep = mk->integer("keep_first", 0);
            }
        if (sp.win <= 0 || sp.keep < 0) throw CmError(CM_ERR_INVALID, "mask.size / mask.keep_first");
        sp.bias = LBIAS_LOG; sp.gate = LGATE_HEAD;
    } else {
        if (sp.dim > 256) throw CmError(CM_ERR_UNSUPPORTED, "lightning head size above 256");
        sp.kv_heads = sp.heads;
        const cmjson::Value* dc = mx->get("decay");
        if (dc && dc->kind == cmjson::Value::Arr) { for (auto& v : dc->arr) sp.decay.push_back((float)v->num); }
        else sp.decay.assign((size_t)sp.heads, (float)mx->number("decay", 1.0));
        if ((int)sp.decay.size() != sp.heads) throw CmError(CM_ERR_INVALID, "decay: one value per head");
    }
    parse_mlp(e.get("mlp"), sp, true);
}

// Mononex: layer types "attention" (position chunks, linear distance bias, sink, element-wise gate, optional "kv_from"),
// "latent_attention" ("q_rank", "kv_rank", "rot_dim", "rot": {"base", "dims", "scaling": {"factor", "original", "fast", "slow"}})
// and "gla" ("tau"); dense feed-forwards are W_down relu(W_up h)^2
static void parse_mononex_layer(const cmjson::Value& e, LayerSpec& sp, const std::vector<LayerSpec>& before) {
    const std::string type = e.string("type", "");
    sp.mixer = type == "attention" ? LMIX_ATTN : (type == "latent_attention" ? LMIX_LATENT : (type == "gla" ? LMIX_GLA : -1));
    if (sp.mixer < 0) throw CmError(CM_ERR_UNSUPPORTED, "layer type '" + type + "' not implemented");
    const cmjson::Value* mx = e.get("mixer");
    if (!mx || mx->kind != cmjson::Value::Obj) throw CmError(CM_ERR_IO, "config.json: layer without mixer");
    sp.heads = (int)mx->integer("heads", 0);
    sp.kv_heads = (int)mx->integer("kv_heads", sp.heads);
    sp.dim = (int)mx->integer("dim", 0);
    sp.vdim = (int)mx->integer("vdim", sp.dim);
    need(sp.heads > 0 && sp.dim > 0 && sp.vdim > 0, "mixer sizes");
    sp.win = 1ll << 40; sp.keep = 0;
    if (sp.mixer == LMIX_ATTN) {
        need(sp.kv_heads > 0 && sp.heads % sp.kv_heads == 0, "heads % kv_heads != 0");
        sp.scale = (float)mx->number("scale", 1.0 / std::sqrt((double)sp.dim));
        if (const cmjson::Value* mk = mx->get("mask"))
            if (mk->kind == cmjson::Value::Obj) {
                sp.chunk = mk->integer("size", 0);
                need(sp.chunk > 0, "mask.size");
            }
        sp.bias = LBIAS_LINEAR; sp.gate = LGATE_ELEM; sp.sink = true; sp.own_v = true;
        if (const cmjson::Value* kf = mx->get("kv_from"))
            if (kf->kind == cmjson::Value::Num) {
                sp.kv_from = (int)kf->num;
                need(sp.kv_from >= 0 && sp.kv_from < (int)before.size(), "kv_from names no earlier layer");
                const LayerSpec& src = before[(size_t)sp.kv_from];
                need(src.mixer == LMIX_ATTN && src.kv_from < 0 && src.kv_heads == sp.kv_heads && src.dim == sp.dim && src.vdim == sp.vdim,
                     "kv_from: the other layer's keys and values do not fit");
            }
        need(lay_attn_fits(sp.dim, sp.vdim, true), "attention head sizes too large");
    } else if (sp.mixer == LMIX_LATENT) {
        sp.q_rank = (int)mx->integer("q_rank", 0);
        sp.kv_rank = (int)mx->integer("kv_rank", 0);
        sp.rot_dim = (int)mx->integer("rot_dim", 0);
        need(sp.q_rank > 0 && sp.kv_rank > 0 && sp.rot_dim >= 0, "q_rank / kv_rank / rot_dim");
        sp.scale = (float)mx->number("scale", 1.0 / std::sqrt((double)(sp.dim + sp.rot_dim)));
        sp.kv_heads = 1;               // one cached row per token: [latent | rotated key part]
        sp.gate = LGATE_NONE;          // the gate acts on the values after their up-projection
        if (const cmjson::Value* rt = mx->get("rot"))
            if (rt->kind == cmjson::Value::Obj) {
                sp.rot.dims = (int)rt->integer("dims", sp.rot_dim);
                sp.rot.base = rt->number("base", 10000.0);
                if (const cmjson::Value* sc = rt->get("scaling"))
                    if (sc->kind == cmjson::Value::Obj) {
                        sp.rot.yarn = true;
                        sp.rot.factor = sc->number("factor", 1.0);
                        sp.rot.original = sc->number("original", 0.0);
                        sp.rot.fast = sc->number("fast", 32.0);
                        sp.rot.slow = sc->number("slow", 1.0);
                        need(sp.rot.factor > 0 && sp.rot.original > 0 && sp.rot.fast > 0 && sp.rot.slow > 0, "rot.scaling");
                    }
            }
        need(sp.rot.dims >= 0 && sp.rot.dims <= sp.rot_dim && sp.rot.dims % 2 == 0 && sp.rot.base > 1.0, "rot.dims / rot.base");
        need(lay_attn_fits(sp.kv_rank + sp.rot_dim, sp.kv_rank, false), "kv_rank + rot_dim too large");
    } else {
        sp.kv_heads = sp.heads;
        sp.tau = (float)mx->number("tau", 1.0);
        need(sp.tau > 0.f, "tau");
        if (sp.dim > 256) throw CmError(CM_ERR_UNSUPPORTED, "gla head size above 256");
    }
    parse_mlp(e.get("mlp"), sp, false);
    sp.gated_ff = false; sp.ff_act = LACT_RELU2;
}

// Gibipel: layer type "parallel" = "mixer": {"left": window attention with pooled blocks, "right": matrix memory, "left_scale",
// "right_scale"}; "mlp": mixture of experts with a softmax router ("identity", "groups": {"count", "keep"}, tensor "correction") and
// an optional "shared" expert
static void parse_gibipel_layer(const cmjson::Value& e, LayerSpec& sp) {
    const std::string type = e.string("type", "");
    if (type != "parallel") throw CmError(CM_ERR_UNSUPPORTED, "layer type '" + type + "' not implemented");
    const cmjson::Value* mx = e.get("mixer");
    const cmjson::Value* lf = mx ? mx->get("left") : nullptr;
    const cmjson::Value* rg = mx ? mx->get("right") : nullptr;
    need(lf && rg && lf->kind == cmjson::Value::Obj && rg->kind == cmjson::Value::Obj, "parallel layer without mixer.left / mixer.right");
    sp.mixer = LMIX_SIDE;
    sp.side.resize(2);
    {
        LayerSpec& a = sp.side[0];
        a.mixer = LMIX_ATTN;
        a.side_scale = (float)mx->number("left_scale", 1.0);
        a.heads = (int)lf->integer("heads", 0);
        a.kv_heads = (int)lf->integer("kv_heads", a.heads);
        a.dim = (int)lf->integer("dim", 0);
        a.vdim = (int)lf->integer("vdim", a.dim);
        need(a.heads > 0 && a.dim > 0 && a.vdim > 0 && a.kv_heads > 0 && a.heads % a.kv_heads == 0, "left mixer sizes");
        a.scale = (float)lf->number("scale", 1.0 / std::sqrt((double)a.dim));
        a.win = 1ll << 40; a.keep = 0;
        if (const cmjson::Value* mk = lf->get("mask"))
            if (mk->kind == cmjson::Value::Obj) {
                a.win = mk->integer("size", a.win);
                a.pool = mk->integer("pool", 0);
                need(a.win > 0 && a.pool >= 0, "mask.size / mask.pool");
            }
        if (const cmjson::Value* rt = lf->get("rot"))
            if (rt->kind == cmjson::Value::Obj) {
                a.rot.half = true;
                a.rot.dims = (int)rt->integer("dims", a.dim);
                a.rot.base = rt->number("base", 10000.0);
                if (const cmjson::Value* sc = rt->get("scaling"))
                    if (sc->kind == cmjson::Value::Obj) {
                        a.rot.banded = true;
                        a.rot.factor = sc->number("factor", 1.0);
                        a.rot.low = sc->number("low", 1.0);
                        a.rot.high = sc->number("high", 4.0);
                        a.rot.original = sc->number("original", 0.0);
                        need(a.rot.factor > 0 && a.rot.original > 0 && a.rot.low > 0 && a.rot.high > a.rot.low, "rot.scaling");
                    }
                need(a.rot.dims >= 0 && a.rot.dims <= a.dim && a.rot.dims % 2 == 0 && a.rot.base > 1.0, "rot.dims / rot.base");
            }
        a.bias = LBIAS_NONE; a.gate = LGATE_NONE; a.sink = true; a.own_v = true; a.qk_norm = true; a.qkv_bias = true;
        need(lay_attn_fits(a.dim, a.vdim, true), "attention head sizes too large");
    }
    {
        LayerSpec& b = sp.side[1];
        b.mixer = LMIX_MEMORY;
        b.side_scale = (float)mx->number("right_scale", 1.0);
        b.heads = (int)rg->integer("heads", 0);
        b.kv_heads = b.heads;
        b.dim = (int)rg->integer("dim", 0);
        b.vdim = (int)rg->integer("vdim", b.dim);
        b.gate_cap = (float)rg->number("gate_cap", 15.0);
        need(b.heads > 0 && b.dim > 0 && b.vdim > 0 && b.gate_cap > 0.f, "right mixer sizes");
        if (b.dim > 256) throw CmError(CM_ERR_UNSUPPORTED, "matrix memory head size above 256");
    }
    parse_mlp(e.get("mlp"), sp, true);
    sp.router.softmax = true; sp.router.correction = true; sp.router.normalise = true;
}

// softmax attention sizes shared by Nevotar's two attention kinds
static void parse_attn_sizes(const cmjson::Value& mx, LayerSpec& a) {
    a.mixer = LMIX_ATTN;
    a.heads = (int)mx.integer("heads", 0);
    a.kv_heads = (int)mx.integer("kv_heads", a.heads);
    a.dim = (int)mx.integer("dim", 0);
    a.vdim = (int)mx.integer("vdim", a.dim);
    need(a.heads > 0 && a.dim > 0 && a.vdim > 0 && a.kv_heads > 0 && a.heads % a.kv_heads == 0, "attention sizes");
    a.scale = (float)mx.number("scale", 1.0 / std::sqrt((double)a.dim));
    a.win = 1ll << 40; a.keep = 0;
    a.bias = LBIAS_NONE; a.gate = LGATE_NONE; a.sink = false; a.own_v = true; a.qkv_bias = true;
}

// Nevotar: layer types "attention" (two softmax maps per head: "diff", "q_temp": {"coef", "every"}), "hgrn2", and "parallel" =
// "mixer": {"left": window attention with "rot": {"base", "dims"}, "mask": {"size"} and mixed heads, "right": state-space mixer
// {"heads", "vdim", "state", "groups", "conv", "norm_groups"}, "left_scale", "right_scale"}; "mlp": mixture of experts whose weights
// multiply the experts' inputs ("expert": {"ff", "limit"}, "shared": {"ff", "limit"}); "weights_of": the layer whose tensors it uses
static void parse_nevotar_layer(const cmjson::Value& e, LayerSpec& sp, const std::vector<LayerSpec>& before) {
    const std::string type = e.string("type", "");
    const cmjson::Value* mx = e.get("mixer");
    need(mx && mx->kind == cmjson::Value::Obj, "layer without mixer");
    if (type == "attention") {
        parse_attn_sizes(*mx, sp);
        sp.maps = 2;
        sp.diff = (float)mx->number("diff", 0.0);
        if (const cmjson::Value* qt = mx->get("q_temp"))
            if (qt->kind == cmjson::Value::Obj) {
                sp.qt_coef = (float)qt->number("coef", 0.0);
                sp.qt_every = qt->integer("every", 1);
                need(sp.qt_every > 0 && sp.qt_every < (1ll << 30), "q_temp.every");
            }
        need(lay_attn_fits(sp.dim, sp.vdim, true), "attention head sizes too large");
        need(2 * sp.heads + 2 * sp.kv_heads <= 1024, "attention: too many heads");
    } else if (type == "hgrn2") {
        sp.mixer = LMIX_HGRN;
        sp.heads = (int)mx->integer("heads", 0);
        sp.kv_heads = sp.heads;
        sp.dim = (int)mx->integer("dim", 0);
        sp.vdim = (int)mx->integer("vdim", sp.dim);
        need(sp.heads > 0 && sp.dim > 0 && sp.vdim > 0, "mixer sizes");
        if (sp.dim > 256) throw CmError(CM_ERR_UNSUPPORTED, "hgrn2 head size above 256");
    } else if (type == "parallel") {
        const cmjson::Value* lf = mx->get("left");
        const cmjson::Value* rg = mx->get("right");
        need(lf && rg && lf->kind == cmjson::Value::Obj && rg->kind == cmjson::Value::Obj, "parallel layer without mixer.left / mixer.right");
        sp.mixer = LMIX_SIDE;
        sp.side.resize(2);
        LayerSpec& a = sp.side[0];
        parse_attn_sizes(*lf, a);
        a.side_scale = (float)mx->number("left_scale", 1.0);
        a.talk = true; a.head_norm = true;
        if (const cmjson::Value* mk = lf->get("mask"))
            if (mk->kind == cmjson::Value::Obj) {
                a.win = mk->integer("size", a.win);
                need(a.win > 0, "mask.size");
            }
        if (const cmjson::Value* rt = lf->get("rot"))
            if (rt->kind == cmjson::Value::Obj) {
                a.rot.half = true;
                a.rot.dims = (int)rt->integer("dims", a.dim);
                a.rot.base = rt->number("base", 10000.0);
                need(a.rot.dims >= 0 && a.rot.dims <= a.dim && a.rot.dims % 2 == 0 && a.rot.base > 0.0, "rot.dims / rot.base");
            }
        need(lay_attn_talk_fits(a.heads, a.kv_heads, a.dim, a.vdim), "left mixer: head count or sizes too large");
        need(a.heads + a.kv_heads <= 1024, "left mixer: too many heads");
        LayerSpec& b = sp.side[1];
        b.mixer = LMIX_SSM;
        b.side_scale = (float)mx->number("right_scale", 1.0);
        b.heads = (int)rg->integer("heads", 0);
        b.kv_heads = b.heads;
        b.vdim = (int)rg->integer("vdim", 0);
        b.state = (int)rg->integer("state", 0);
        b.dim = b.state;
        b.groups = (int)rg->integer("groups", 1);
        b.conv = (int)rg->integer("conv", 1);
        b.norm_groups = (int)rg->integer("norm_groups", 1);
        need(b.heads > 0 && b.vdim > 0 && b.state > 0 && b.groups > 0 && b.heads % b.groups == 0, "right mixer sizes");
        need(b.conv >= 1 && b.conv <= 64, "right mixer: conv");
        need(b.norm_groups > 0 && b.norm_groups <= 256 && (b.heads * b.vdim) % b.norm_groups == 0, "right mixer: norm_groups");
        if (b.state > 256) throw CmError(CM_ERR_UNSUPPORTED, "state-space state size above 256");
    } else throw CmError(CM_ERR_UNSUPPORTED, "layer type '" + type + "' not implemented");
    const cmjson::Value* ml = e.get("mlp");
    if (ml && ml->kind == cmjson::Value::Obj) {
        need(ml->string("kind", "moe") == "moe", "mlp.kind: only 'moe'");
        parse_mlp(ml, sp, true);
        sp.scale_input = true; sp.expert_act = LACT_CAPGLU;
        need(sp.limit > 0.f && (sp.shared_ff == 0 || sp.shared_limit > 0.f), "expert.limit / shared.limit");
    }
    if (const cmjson::Value* wo = e.get("weights_of"))
        if (wo->kind == cmjson::Value::Num) {
            sp.weights_of = (int)wo->num;
            need(sp.weights_of >= 0 && sp.weights_of < (int)before.size() && before[(size_t)sp.weights_of].weights_of < 0,
                 "weights_of names no earlier layer with tensors of its own");
            const LayerSpec& o = before[(size_t)sp.weights_of];
            auto same = [](const LayerSpec& x, const LayerSpec& y) {
                return x.mixer == y.mixer && x.heads == y.heads && x.kv_heads == y.kv_heads && x.dim == y.dim && x.vdim == y.vdim && x.state == y.state &&
                       x.groups == y.groups && x.conv == y.conv && x.rot.dims == y.rot.dims;
            };
            bool ok = same(sp, o) && sp.side.size() == o.side.size() && sp.mlp == o.mlp && sp.ff == o.ff && sp.experts == o.experts && sp.shared_ff == o.shared_ff;
            for (size_t k = 0; ok && k < sp.side.size(); ++k) ok = same(sp.side[k], o.side[k]);
            need(ok, "weights_of: the other layer's sizes differ");
        }
}

// config.json of a layer-list decoder: "architecture", "vocab", "width", "norm".eps and "layers": [{"type", "mixer": {...}, "mlp"}]
void Model::init_layered_config(const cmjson::Value& root) {
    const std::string arch = root.string("architecture", "");
    if (arch != "Korupel" && arch != "Mononex" && arch != "Gibipel" && arch != "Nevotar")
        throw CmError(CM_ERR_UNSUPPORTED, "architecture '" + arch + "' not implemented (Korupel, Mononex, Gibipel, Nevotar)");
    layered = true;
    lay.reset(new Layered());
    Layered& L = *lay;
    L.parallel = arch == "Mononex";
    L.post_only = arch == "Gibipel";
    L.pre_norm = arch == "Nevotar";
    cfg.model_type = L.parallel ? "mononex" : (L.post_only ? "gibipel" : (L.pre_norm ? "nevotar" : "korupel"));
    if (L.post_only) {
        if (const cmjson::Value* em = root.get("embedding")) L.embed_scale = (float)em->number("scale", 1.0);
        L.logit_scale = (float)root.number("logit_scale", 1.0);
    }
    cfg.V = (int)root.integer("vocab", 0);
    cfg.H = (int)root.integer("width", 0);
    if (const cmjson::Value* n = root.get("norm")) {
        cfg.eps = (float)n->number("eps", 1e-6);
        if (L.pre_norm) L.norm_groups = (int)n->integer("groups", 1);
    }
    if (!L.parallel && !L.post_only && !L.pre_norm) {
        if (const cmjson::Value* c = root.get("canon")) L.taps = (int)c->integer("taps", 0);
        L.mult = (float)root.number("residual_mult", 1.0);
    }
    const cmjson::Value* ls = root.get("layers");
    if (!ls || ls->kind != cmjson::Value::Arr || ls->arr.empty()) throw CmError(CM_ERR_IO, "config.json: no layers");
    if (cfg.V <= 0 || cfg.H <= 0) throw CmError(CM_ERR_IO, "config.json: vocab / width missing");
    need(L.norm_groups > 0 && L.norm_groups <= 256 && cfg.H % L.norm_groups == 0, "norm.groups");
    if (L.taps < 0 || L.taps > 64) throw CmError(CM_ERR_UNSUPPORTED, "canon.taps out of range");
    for (auto& e : ls->arr) {
        LayerSpec sp;
        if (L.parallel) parse_mononex_layer(*e, sp, L.spec);
        else if (L.post_only) parse_gibipel_layer(*e, sp);
        else if (L.pre_norm) parse_nevotar_layer(*e, sp, L.spec);
        else parse_korupel_layer(*e, sp);
        L.spec.push_back(sp);
    }
    cfg.L = (int)L.spec.size();
    // the family-wide fields of the other decoders do not exist here: neutral values for the shared set-up code
    cfg.I = 8; cfg.Hq = 1; cfg.Hkv = 1; cfg.D = 128; cfg.rot_dim = 128; cfg.max_pos = 1 << 20; cfg.tie = false; cfg.qk_norm = false;
    L.f32 = opts.compute_dtype == CM_COMPUTE_F32;
    if (opts.compute_dtype > CM_COMPUTE_F32) throw CmError(CM_ERR_INVALID, "cm_opts.compute_dtype");
    if (opts.tp_size > 1) throw CmError(CM_ERR_UNSUPPORTED, "tensor parallelism is not implemented for layer-list decoders");
    if (opts.isq != 0) throw CmError(CM_ERR_UNSUPPORTED, "in-situ quantisation is not implemented for layer-list decoders");
    // the key cache follows the number format: bfloat16 pages, or f32 pages in the float32 format
    opts.kv_dtype = L.f32 ? CM_KV_F32 : CM_KV_BF16;
}

// ---------------------------------------------------------------------------------------------------------------
// weights
// ---------------------------------------------------------------------------------------------------------------
namespace {

struct LaySource {
    virtual ~LaySource() {}
    // values of tensor `name` with exactly n elements (bf16-representable for matrices)
    virtual std::vector<float> get(const std::string& name, size_t n, float synth_scale, float synth_off) = 0;
    // first dimension of a tensor whose shape the configuration does not give (dflt: no checkpoint behind the source)
    virtual int64_t dim0(const std::string& name, int64_t dflt) = 0;
};

struct LayFileSource : LaySource {
    cmst::Checkpoint ck;
    explicit LayFileSource(const std::string& dir) : ck(dir) {}
    std::vector<float> get(const std::string& name, size_t n, float, float) override {
        const cmst::TensorView& t = ck.get(name);
        if (t.numel() != (int64_t)n) throw CmError(CM_ERR_IO, "tensor " + name + ": unexpected shape");
        std::vector<float> out(n);
        if (t.dtype == "BF16") {
            const uint16_t* p = (const uint16_t*)t.data;
            for (size_t i = 0; i < n; ++i) { const uint32_t u = (uint32_t)p[i] << 16; memcpy(&out[i], &u, 4); }
        } else if (t.dtype == "F32") {
            memcpy(out.data(), t.data, n * 4);
        } else throw CmError(CM_ERR_UNSUPPORTED, "tensor " + name + ": dtype " + t.dtype);
        return out;
    }
    int64_t dim0(const std::string& name, int64_t) override {
        const cmst::TensorView& t = ck.get(name);
        if (t.shape.empty()) throw CmError(CM_ERR_IO, "tensor " + name + ": unexpected shape");
        return t.shape[0];
    }
};

struct LaySynthSource : LaySource {
    uint64_t seed;
    explicit LaySynthSource(uint64_t s) : seed(s) {}
    int64_t dim0(const std::string&, int64_t dflt) override { return dflt; }
    std::vector<float> get(const std::string& name, size_t n, float scale, float off) override {
        uint64_t h = 1469598103934665603ull ^ seed;
        for (char c : name) { h ^= (unsigned char)c; h *= 1099511628211ull; }
        std::vector<float> out(n);
        for (size_t i = 0; i < n; ++i) {
            h ^= h << 13; h ^= h >> 7; h ^= h << 17;
            // sum of four bytes: a bell-shaped value in [-2, 2) with unit-order spread
            const int c = (int)((h & 0xFF) + ((h >> 8) & 0xFF) + ((h >> 16) & 0xFF) + ((h >> 24) & 0xFF)) - 510;
            out[i] = off + scale * (float)c / 147.8f;
        }
        return out;
    }
};

uint16_t to_bf16(float f) {
    uint32_t u; memcpy(&u, &f, 4);
    if ((u & 0x7F800000u) == 0x7F800000u) return (uint16_t)(u >> 16);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

}  // namespace

static float* up_f32(Model& m, const std::vector<float>& v) {
    float* d = m.dalloc<float>(v.size(), true);
    CM_HIP(hipMemcpy(d, v.data(), v.size() * sizeof(float), hipMemcpyHostToDevice));
    return d;
}
static uint16_t* up_bf16(Model& m, const std::vector<float>& v) {
    std::vector<uint16_t> b(v.size());
    for (size_t i = 0; i < v.size(); ++i) b[i] = to_bf16(v[i]);
    uint16_t* d = m.dalloc<uint16_t>(b.size(), true);
    CM_HIP(hipMemcpy(d, b.data(), b.size() * sizeof(uint16_t), hipMemcpyHostToDevice));
    return d;
}
static void append(std::vector<float>& dst, const std::vector<float>& src) { dst.insert(dst.end(), src.begin(), src.end()); }

// angle per position of every rotated pair: base^(-2i / dims), with the YaRN blend between the original and the stretched
// frequencies over the pair index, and the factor that goes on cos and sin
static std::vector<float> rot_frequencies(const RotSpec& r, float* mag) {
    const int half = r.dims / 2;
    std::vector<float> f((size_t)half);
    *mag = 1.f;
    double lo = 0, hi = 0;
    if (r.yarn) {
        const double two_pi = 6.283185307179586476925286766559;
        auto at = [&](double turns) { return r.dims * std::log(r.original / (two_pi * turns)) / (2.0 * std::log(r.base)); };
        lo = std::max(std::floor(at(r.fast)), 0.0);
        hi = std::min(std::ceil(at(r.slow)), (double)(r.dims - 1));
        *mag = (float)(0.1 * std::log(r.factor) + 1.0);
    }
    for (int i = 0; i < half; ++i) {
        double fi = std::pow(r.base, -2.0 * i / r.dims);
        if (r.banded) {
            const double wavelength = 6.283185307179586476925286766559 / fi;
            if (wavelength > r.original / r.low) fi /= r.factor;
            else if (wavelength >= r.original / r.high) {
                const double t = (r.original / wavelength - r.low) / (r.high - r.low);
                fi = (1.0 - t) * fi / r.factor + t * fi;
            }
        }
        if (r.yarn) {
            const double ramp = std::min(1.0, std::max(0.0, (i - lo) / std::max(hi - lo, 0.001)));
            fi = fi / r.factor * ramp + fi * (1.0 - ramp);
        }
        f[(size_t)i] = (float)fi;
    }
    return f;
}

static void build_mononex(Model& m, LaySource& src);
static void build_gibipel(Model& m, LaySource& src);
static void build_nevotar(Model& m, LaySource& src);

static void build_layered(Model& m, LaySource& src) {
    Layered& L = *m.lay;
    if (L.parallel) { build_mononex(m, src); return; }
    if (L.post_only) { build_gibipel(m, src); return; }
    if (L.pre_norm) { build_nevotar(m, src); return; }
    const size_t W = (size_t)m.cfg.H, V = (size_t)m.cfg.V;
    const float ws = 1.0f / std::sqrt((float)W);
    m.embed = up_bf16(m, src.get("embed", V * W, 1.0f, 0.f));
    L.w.resize(L.spec.size());
    int kv_idx = 0;
    for (size_t i = 0; i < L.spec.size(); ++i) {
        const LayerSpec& sp = L.spec[i];
        LayeredLayerW& w = L.w[i];
        const std::string p = "l" + std::to_string(i) + ".";
        w.norm1 = up_f32(m, src.get(p + "norm1", W, 0.1f, 1.f));
        w.norm1b = up_f32(m, src.get(p + "norm1b", W, 0.1f, 1.f));
        if (L.taps > 0) w.canon1 = up_f32(m, src.get(p + "canon1", W * L.taps, 0.3f, 0.f));
        const size_t H = (size_t)sp.heads, G = (size_t)sp.kv_heads, d = (size_t)sp.dim, e = (size_t)sp.vdim;
        std::vector<float> in, bias;
        if (sp.mixer == LMIX_ATTN) {
            w.q_off = 0; w.k_off = (int)(H * d); w.g_off = (int)(H * d + G * d); w.in_rows = (int)(H * d + G * d + H);
            append(in, src.get(p + "mix.q", H * d * W, ws, 0.f));
            append(in, src.get(p + "mix.k", G * d * W, ws, 0.f));
            append(in, src.get(p + "mix.g", H * W, ws, 0.f));
            append(bias, src.get(p + "mix.q.b", H * d, 0.1f, 0.f));
            append(bias, src.get(p + "mix.k.b", G * d, 0.1f, 0.f));
            bias.resize((size_t)w.in_rows, 0.f);
            w.in_b = up_f32(m, bias);
            w.r1 = up_f32(m, src.get(p + "mix.r1", H, 0.2f, 0.5f));
            w.r2 = up_f32(m, src.get(p + "mix.r2", H, 0.1f, 0.5f));
            w.o_w = up_bf16(m, src.get(p + "mix.o", W * H * d, 1.0f / std::sqrt((float)(H * d)), 0.f));
            w.kv_idx = kv_idx++;
        } else {
            w.q_off = 0; w.k_off = (int)(H * d); w.v_off = (int)(2 * H * d); w.g_off = (int)(2 * H * d + H * e);
            w.in_rows = (int)(2 * H * d + 2 * H * e);
            append(in, src.get(p + "mix.q", H * d * W, ws, 0.f));
            append(in, src.get(p + "mix.k", H * d * W, ws, 0.f));
            append(in, src.get(p + "mix.v", H * e * W, ws, 0.f));
            append(in, src.get(p + "mix.g", H * e * W, ws, 0.f));
            w.mix_norm = up_f32(m, src.get(p + "mix.norm", H * e, 0.1f, 1.f));
            w.o_w = up_bf16(m, src.get(p + "mix.o", W * H * e, 1.0f / std::sqrt((float)(H * e)), 0.f));
            w.decay = up_f32(m, sp.decay);
        }
        w.in_w = up_bf16(m, in);
        if (sp.mlp != LMLP_NONE) {
            w.norm2 = up_f32(m, src.get(p + "norm2", W, 0.1f, 1.f));
            w.norm2b = up_f32(m, src.get(p + "norm2b", W, 0.1f, 1.f));
            if (L.taps > 0) w.canon2 = up_f32(m, src.get(p + "canon2", W * L.taps, 0.3f, 0.f));
            const size_t ff = (size_t)sp.ff;
            const float fs = 1.0f / std::sqrt((float)ff);
            if (sp.mlp == LMLP_DENSE) {
                w.gate = up_bf16(m, src.get(p + "mlp.gate", ff * W, ws, 0.f));
                w.up = up_bf16(m, src.get(p + "mlp.up", ff * W, ws, 0.f));
                w.down = up_bf16(m, src.get(p + "mlp.down", W * ff, fs, 0.f));
            } else {
                std::vector<float> g, u, dn;
                for (int ex = 0; ex < sp.experts; ++ex) {
                    const std::string q = p + "mlp.e" + std::to_string(ex) + ".";
                    append(g, src.get(q + "gate", ff * W, ws, 0.f));
                    append(u, src.get(q + "up", ff * W, ws, 0.f));
                    append(dn, src.get(q + "down", W * ff, fs, 0.f));
                }
                w.gate = up_bf16(m, g); w.up = up_bf16(m, u); w.down = up_bf16(m, dn);
                w.router = up_bf16(m, src.get(p + "mlp.router", (size_t)sp.experts * W, ws, 0.f));
            }
        }
    }
    L.final_norm = up_f32(m, src.get("final.norm", W, 0.1f, 1.f));
    L.head = up_bf16(m, src.get("head", V * W, ws, 0.f));
    m.lm_head = L.head;
}

// norm weights stored around zero: the factor is 1 + w
static std::vector<float> plus_one(std::vector<float> v) { for (float& x : v) x += 1.f; return v; }

static void build_mononex(Model& m, LaySource& src) {
    Layered& L = *m.lay;
    const size_t W = (size_t)m.cfg.H, V = (size_t)m.cfg.V;
    const float ws = 1.0f / std::sqrt((float)W);
    m.embed = up_bf16(m, src.get("embed", V * W, 1.0f, 0.f));
    L.w.resize(L.spec.size());
    int kv_idx = 0;
    for (size_t i = 0; i < L.spec.size(); ++i) {
        LayerSpec& sp = L.spec[i];
        LayeredLayerW& w = L.w[i];
        const std::string p = "l" + std::to_string(i) + ".";
        w.norm1 = up_f32(m, plus_one(src.get(p + "norm1", W, 0.1f, 0.f)));
        {   // token shift h + (h' - h) s as the two-tap convolution h + s h' - s h
            const std::vector<float> sh = src.get(p + "shift", W, 0.25f, 0.5f);
            std::vector<float> cw(2 * W);
            for (size_t c = 0; c < W; ++c) { cw[2 * c] = sh[c]; cw[2 * c + 1] = -sh[c]; }
            w.shift = up_f32(m, cw);
        }
        const size_t H = (size_t)sp.heads, G = (size_t)sp.kv_heads, d = (size_t)sp.dim, e = (size_t)sp.vdim;
        std::vector<float> in;
        if (sp.mixer == LMIX_ATTN) {
            const bool own = sp.kv_from < 0;
            w.q_off = 0; w.k_off = (int)(H * d); w.v_off = w.k_off + (own ? (int)(G * d) : 0); w.g_off = w.v_off + (own ? (int)(G * e) : 0);
            w.in_rows = w.g_off + (int)(H * e);
            append(in, src.get(p + "mix.q", H * d * W, ws, 0.f));
            if (own) {
                append(in, src.get(p + "mix.k", G * d * W, ws, 0.f));
                append(in, src.get(p + "mix.v", G * e * W, ws, 0.f));
            }
            append(in, src.get(p + "mix.g", H * e * W, ws, 0.f));
            w.sink = up_f32(m, src.get(p + "mix.sink", H, 1.0f, 0.f));
            std::vector<float> slope(H);
            for (size_t h = 0; h < H; ++h) slope[h] = (float)std::pow(2.0, -8.0 * (double)(h + 1) / (double)H);
            w.r1 = up_f32(m, slope);
            w.o_w = up_bf16(m, src.get(p + "mix.o", W * H * e, 1.0f / std::sqrt((float)(H * e)), 0.f));
            w.kv_idx = kv_idx++;
        } else if (sp.mixer == LMIX_LATENT) {
            const size_t qr = (size_t)sp.q_rank, kr = (size_t)sp.kv_rank, r = (size_t)sp.rot_dim;
            w.q_off = 0; w.k_off = (int)qr; w.g_off = (int)(qr + kr + r); w.in_rows = w.g_off + (int)(H * e);
            append(in, src.get(p + "mix.dq", qr * W, ws, 0.f));
            append(in, src.get(p + "mix.dkv", (kr + r) * W, ws, 0.f));
            append(in, src.get(p + "mix.g", H * e * W, ws, 0.f));
            w.dq_norm = up_f32(m, src.get(p + "mix.dq.norm", qr, 0.1f, 1.f));
            w.dkv_norm = up_f32(m, src.get(p + "mix.dkv.norm", kr, 0.1f, 1.f));
            w.uq = up_bf16(m, src.get(p + "mix.uq", H * (d + r) * qr, 1.0f / std::sqrt((float)qr), 0.f));
            {   // W_uk per head, transposed: the product q_unrotated . (W_uk c) = (W_uk^T q_unrotated) . c runs against the cached latent
                const std::vector<float> uk = src.get(p + "mix.uk", H * d * kr, 1.0f / std::sqrt((float)kr), 0.f);
                std::vector<float> t(H * kr * d);
                for (size_t h = 0; h < H; ++h)
                    for (size_t a = 0; a < d; ++a)
                        for (size_t c = 0; c < kr; ++c) t[(h * kr + c) * d + a] = uk[(h * d + a) * kr + c];
                w.uk_t = up_bf16(m, t);
            }
            w.uv = up_bf16(m, src.get(p + "mix.uv", H * e * kr, 1.0f / std::sqrt((float)kr), 0.f));
            if (sp.rot.dims > 0) w.rot_freq = up_f32(m, rot_frequencies(sp.rot, &w.rot_mag));
            w.o_w = up_bf16(m, src.get(p + "mix.o", W * H * e, 1.0f / std::sqrt((float)(H * e)), 0.f));
            w.kv_idx = kv_idx++;
        } else {
            sp.a_rank = (int)src.dim0(p + "mix.a1", 16);
            if (sp.a_rank <= 0) throw CmError(CM_ERR_IO, "tensor " + p + "mix.a1: unexpected shape");
            const size_t ar = (size_t)sp.a_rank;
            w.q_off = 0; w.k_off = (int)(H * d); w.v_off = (int)(2 * H * d); w.a_off = (int)(2 * H * d + H * e);
            w.g_off = w.a_off + (int)ar; w.in_rows = w.g_off + (int)(H * e);
            append(in, src.get(p + "mix.q", H * d * W, ws, 0.f));
            append(in, src.get(p + "mix.k", H * d * W, ws, 0.f));
            append(in, src.get(p + "mix.v", H * e * W, ws, 0.f));
            append(in, src.get(p + "mix.a1", ar * W, ws, 0.f));
            append(in, src.get(p + "mix.g", H * e * W, ws, 0.f));
            w.a2 = up_bf16(m, src.get(p + "mix.a2", H * d * ar, 1.0f / std::sqrt((float)ar), 0.f));
            w.a2_b = up_f32(m, src.get(p + "mix.a2.b", H * d, 1.0f, 2.f));
            w.mix_norm = up_f32(m, src.get(p + "mix.norm", e, 0.1f, 1.f));
            w.o_w = up_bf16(m, src.get(p + "mix.o", W * H * e, 1.0f / std::sqrt((float)(H * e)), 0.f));
        }
        w.in_w = up_bf16(m, in);
        if (sp.mlp != LMLP_NONE) {
            w.norm2 = up_f32(m, plus_one(src.get(p + "norm2", W, 0.1f, 0.f)));
            const size_t ff = (size_t)sp.ff;
            w.up = up_bf16(m, src.get(p + "mlp.up", ff * W, ws, 0.f));
            w.down = up_bf16(m, src.get(p + "mlp.down", W * ff, 1.0f / std::sqrt((float)ff), 0.f));
        }
    }
    L.final_norm = up_f32(m, plus_one(src.get("final.norm", W, 0.1f, 0.f)));
    L.head = up_bf16(m, src.get("head", V * W, ws, 0.f));
    m.lm_head = L.head;
}

// experts' matrices back to back, router, correction, shared expert (the Gibipel feed-forward)
static void build_experts(Model& m, LaySource& src, const std::string& p, const LayerSpec& sp, LayeredLayerW& w) {
    const size_t W = (size_t)m.cfg.H, ff = (size_t)sp.ff;
    const float ws = 1.0f / std::sqrt((float)W), fs = 1.0f / std::sqrt((float)ff);
    std::vector<float> g, u, dn;
    for (int ex = 0; ex < sp.experts; ++ex) {
        const std::string q = p + "mlp.e" + std::to_string(ex) + ".";
        append(g, src.get(q + "gate", ff * W, ws, 0.f));
        append(u, src.get(q + "up", ff * W, ws, 0.f));
        append(dn, src.get(q + "down", W * ff, fs, 0.f));
    }
    w.gate = up_bf16(m, g); w.up = up_bf16(m, u); w.down = up_bf16(m, dn);
    const size_t outs = (size_t)(sp.experts + sp.router.identity);
    w.router = up_bf16(m, src.get(p + "mlp.router", outs * W, ws, 0.f));
    if (sp.router.correction) w.correction = up_f32(m, src.get(p + "mlp.correction", outs, 0.02f, 0.f));
    if (sp.shared_ff > 0) {
        const size_t sf = (size_t)sp.shared_ff;
        w.sh_gate = up_bf16(m, src.get(p + "mlp.shared.gate", sf * W, ws, 0.f));
        w.sh_up = up_bf16(m, src.get(p + "mlp.shared.up", sf * W, ws, 0.f));
        w.sh_down = up_bf16(m, src.get(p + "mlp.shared.down", W * sf, 1.0f / std::sqrt((float)sf), 0.f));
    }
}

static void build_gibipel(Model& m, LaySource& src) {
    Layered& L = *m.lay;
    const size_t W = (size_t)m.cfg.H, V = (size_t)m.cfg.V;
    const float ws = 1.0f / std::sqrt((float)W);
    m.embed = up_bf16(m, src.get("embed", V * W, 1.0f, 0.f));
    L.w.resize(L.spec.size());
    // a one-number norm weight as a vector, so that the norm kernels of the other families apply
    auto one_number = [&](const std::string& name, float factor) {
        const float g = src.get(name, 1, 0.1f, 1.f)[0] * factor;
        return up_f32(m, std::vector<float>(W, g));
    };
    for (size_t i = 0; i < L.spec.size(); ++i) {
        const LayerSpec& sp = L.spec[i];
        LayeredLayerW& w = L.w[i];
        const std::string p = "l" + std::to_string(i) + ".";
        w.norm1b = one_number(p + "norm1", 1.f);
        w.side.resize(2);
        const LayerSpec &sa = sp.side[0], &sb = sp.side[1];
        LayeredLayerW &wa = w.side[0], &wb = w.side[1];
        std::vector<float> in, bias;
        {   // left: q | k | v, biases on all three
            const size_t H = (size_t)sa.heads, G = (size_t)sa.kv_heads, d = (size_t)sa.dim, e = (size_t)sa.vdim;
            const std::string q = p + "mix.left.";
            wa.q_off = 0; wa.k_off = (int)(H * d); wa.v_off = wa.k_off + (int)(G * d);
            append(in, src.get(q + "q", H * d * W, ws, 0.f)); append(bias, src.get(q + "q.b", H * d, 0.1f, 0.f));
            append(in, src.get(q + "k", G * d * W, ws, 0.f)); append(bias, src.get(q + "k.b", G * d, 0.1f, 0.f));
            append(in, src.get(q + "v", G * e * W, ws, 0.f)); append(bias, src.get(q + "v.b", G * e, 0.1f, 0.f));
            wa.q_norm = up_f32(m, src.get(q + "q.norm", H * d, 0.1f, 1.f));
            wa.k_norm = up_f32(m, src.get(q + "k.norm", G * d, 0.1f, 1.f));
            wa.sink = up_f32(m, src.get(q + "sink", H, 1.0f, 0.f));
            if (sa.rot.dims > 0) wa.rot_freq = up_f32(m, rot_frequencies(sa.rot, &wa.rot_mag));
            wa.o_col = 0;
        }
        {   // right: q | k | v | input gate | forget gate | output gate; biases on the two recurrence gates
            const size_t H = (size_t)sb.heads, d = (size_t)sb.dim, e = (size_t)sb.vdim;
            const std::string q = p + "mix.right.";
            const int base = (int)(in.size() / W);
            wb.q_off = base; wb.k_off = wb.q_off + (int)(H * d); wb.v_off = wb.k_off + (int)(H * d); wb.i_off = wb.v_off + (int)(H * e);
            wb.f_off = wb.i_off + (int)H; wb.g_off = wb.f_off + (int)H;
            append(in, src.get(q + "q", H * d * W, ws, 0.f));
            append(in, src.get(q + "k", H * d * W, ws, 0.f));
            append(in, src.get(q + "v", H * e * W, ws, 0.f));
            append(in, src.get(q + "i", H * W, ws, 0.f));
            append(in, src.get(q + "f", H * W, ws, 0.f));
            append(in, src.get(q + "g", H * e * W, ws, 0.f));
            bias.resize((size_t)wb.i_off, 0.f);
            append(bias, src.get(q + "i.b", H, 0.5f, 0.f));
            append(bias, src.get(q + "f.b", H, 0.5f, 3.f));
            wb.mix_norm = up_f32(m, src.get(q + "norm", H * e, 0.1f, 1.f));
            wb.o_col = sa.heads * sa.vdim;
        }
        w.in_rows = (int)(in.size() / W);
        w.g_off = wb.g_off;
        bias.resize((size_t)w.in_rows, 0.f);
        w.in_w = up_bf16(m, in);
        w.in_b = up_f32(m, bias);
        {   // one output projection for both mixers: the input columns are [left heads | right heads]
            const size_t ka = (size_t)sa.heads * sa.vdim, kb = (size_t)sb.heads * sb.vdim, K = ka + kb;
            const std::vector<float> oa = src.get(p + "mix.left.o", W * ka, 1.0f / std::sqrt((float)ka), 0.f);
            const std::vector<float> ob = src.get(p + "mix.right.o", W * kb, 1.0f / std::sqrt((float)kb), 0.f);
            std::vector<float> o(W * K);
            for (size_t r = 0; r < W; ++r) {
                std::copy(oa.begin() + (long)(r * ka), oa.begin() + (long)((r + 1) * ka), o.begin() + (long)(r * K));
                std::copy(ob.begin() + (long)(r * kb), ob.begin() + (long)((r + 1) * kb), o.begin() + (long)(r * K + ka));
            }
            w.o_w = up_bf16(m, o);
        }
        if (sp.mlp != LMLP_NONE) {
            w.norm2b = one_number(p + "norm2", 1.f);
            if (sp.mlp == LMLP_MOE) build_experts(m, src, p, sp, w);
            else {
                const size_t ff = (size_t)sp.ff;
                w.gate = up_bf16(m, src.get(p + "mlp.gate", ff * W, ws, 0.f));
                w.up = up_bf16(m, src.get(p + "mlp.up", ff * W, ws, 0.f));
                w.down = up_bf16(m, src.get(p + "mlp.down", W * ff, 1.0f / std::sqrt((float)ff), 0.f));
            }
        }
    }
    L.final_norm = one_number("final.norm", L.logit_scale);       // the factor on the logits rides on the final norm's weight
    L.head = up_bf16(m, src.get("head", V * W, ws, 0.f));
    m.lm_head = L.head;
}

static void build_nevotar(Model& m, LaySource& src) {
    Layered& L = *m.lay;
    const size_t W = (size_t)m.cfg.H, V = (size_t)m.cfg.V;
    const float ws = 1.0f / std::sqrt((float)W);
    m.embed = up_bf16(m, src.get("embed", V * W, 1.0f, 0.f));
    L.w.resize(L.spec.size());
    for (size_t i = 0; i < L.spec.size(); ++i) {
        const LayerSpec& sp = L.spec[i];
        if (sp.weights_of >= 0) { L.w[i] = L.w[(size_t)sp.weights_of]; continue; }      // the same tensors; its place in the pools is its own
        LayeredLayerW& w = L.w[i];
        const std::string p = "l" + std::to_string(i) + ".";
        w.norm1 = up_f32(m, src.get(p + "norm1", W, 0.1f, 1.f));
        std::vector<float> in, bias;
        if (sp.mixer == LMIX_ATTN) {
            // q | k | v.  The query rows are reordered so that the two maps are heads of their own whose key head follows from the usual
            // grouping: key head (g, map m) = 2 g + m serves the query heads (2 g + m) nrep + j, j < nrep (stored: head g nrep + j, [map 1 | map 2])
            const size_t H = (size_t)sp.heads, G = (size_t)sp.kv_heads, d = (size_t)sp.dim, e = (size_t)sp.vdim, nrep = H / G;
            const std::string q = p + "mix.";
            const std::vector<float> qw = src.get(q + "q", 2 * H * d * W, ws, 0.f), qb = src.get(q + "q.b", 2 * H * d, 0.1f, 0.f);
            std::vector<float> qp(qw.size()), qbp(qb.size());
            for (size_t h = 0; h < H; ++h)
                for (size_t mp = 0; mp < 2; ++mp) {
                    const size_t from = (h * 2 + mp) * d, to = ((2 * (h / nrep) + mp) * nrep + h % nrep) * d;
                    std::copy(qw.begin() + (long)(from * W), qw.begin() + (long)((from + d) * W), qp.begin() + (long)(to * W));
                    std::copy(qb.begin() + (long)from, qb.begin() + (long)(from + d), qbp.begin() + (long)to);
                }
            w.q_off = 0; w.k_off = (int)(2 * H * d); w.v_off = w.k_off + (int)(2 * G * d);
            append(in, qp); append(bias, qbp);
            append(in, src.get(q + "k", 2 * G * d * W, ws, 0.f)); append(bias, src.get(q + "k.b", 2 * G * d, 0.1f, 0.f));
            append(in, src.get(q + "v", G * e * W, ws, 0.f)); append(bias, src.get(q + "v.b", G * e, 0.1f, 0.f));
            w.in_rows = w.v_off + (int)(G * e);
            w.g_off = w.in_rows;
            auto dot = [&](const std::string& a, const std::string& b) {
                const std::vector<float> x = src.get(q + a, d, 0.3f, 0.f), y = src.get(q + b, d, 0.3f, 0.f);
                double t = 0.0;
                for (size_t k = 0; k < d; ++k) t += (double)x[k] * (double)y[k];
                return t;
            };
            w.lambda = (float)(std::exp(dot("lq1", "lk1")) - std::exp(dot("lq2", "lk2")) + (double)sp.diff);
            w.o_w = up_bf16(m, src.get(q + "o", W * H * e, 1.0f / std::sqrt((float)(H * e)), 0.f));
        } else if (sp.mixer == LMIX_HGRN) {
            // q (SiLU) | forget gate (the key 1 - f takes its place) | v
            const size_t H = (size_t)sp.heads, d = (size_t)sp.dim, e = (size_t)sp.vdim;
            const std::string q = p + "mix.";
            w.q_off = 0; w.k_off = (int)(H * d); w.v_off = (int)(2 * H * d); w.in_rows = (int)(2 * H * d + H * e); w.g_off = (int)(H * d);
            append(in, src.get(q + "q", H * d * W, ws, 0.f));
            append(in, src.get(q + "f", H * d * W, ws, 0.f));
            append(in, src.get(q + "v", H * e * W, ws, 0.f));
            bias.assign(H * d, 0.f);
            append(bias, src.get(q + "f.b", H * d, 0.5f, 1.f));
            bias.resize((size_t)w.in_rows, 0.f);
            std::vector<float> lo = src.get(q + "lower", H * d, 0.2f, 0.4f);
            for (float& v : lo) v = std::min(std::max(v, 0.f), 0.999f);       // a bound of a gate in (0, 1); checkpoints hold such values
            w.lower = up_f32(m, lo);
            w.mix_norm = up_f32(m, src.get(q + "norm", e, 0.1f, 1.f));
            w.o_w = up_bf16(m, src.get(q + "o", W * H * e, 1.0f / std::sqrt((float)(H * e)), 0.f));
        } else {
            w.side.resize(2);
            const LayerSpec &sa = sp.side[0], &sb = sp.side[1];
            LayeredLayerW &wa = w.side[0], &wb = w.side[1];
            {   // left: q | k | v, biases on all three
                const size_t H = (size_t)sa.heads, G = (size_t)sa.kv_heads, d = (size_t)sa.dim, e = (size_t)sa.vdim;
                const std::string q = p + "mix.left.";
                wa.q_off = 0; wa.k_off = (int)(H * d); wa.v_off = wa.k_off + (int)(G * d);
                append(in, src.get(q + "q", H * d * W, ws, 0.f)); append(bias, src.get(q + "q.b", H * d, 0.1f, 0.f));
                append(in, src.get(q + "k", G * d * W, ws, 0.f)); append(bias, src.get(q + "k.b", G * d, 0.1f, 0.f));
                append(in, src.get(q + "v", G * e * W, ws, 0.f)); append(bias, src.get(q + "v.b", G * e, 0.1f, 0.f));
                wa.q_norm = up_f32(m, src.get(q + "q.norm", d, 0.1f, 1.f));
                wa.k_norm = up_f32(m, src.get(q + "k.norm", d, 0.1f, 1.f));
                wa.talk = up_f32(m, src.get(q + "talk", H * H, 0.6f / std::sqrt((float)H), 0.f));
                if (sa.rot.dims > 0) wa.rot_freq = up_f32(m, rot_frequencies(sa.rot, &wa.rot_mag));
                wa.o_col = 0;
            }
            {   // right: z | x | B | C | dt
                const size_t H = (size_t)sb.heads, e = (size_t)sb.vdim, N = (size_t)sb.state, Gr = (size_t)sb.groups, inner = H * e;
                const size_t C = inner + 2 * Gr * N, taps = (size_t)sb.conv;
                const std::string q = p + "mix.right.";
                const int base = (int)(in.size() / W);
                wb.z_off = base; wb.x_off = base + (int)inner; wb.dt_off = wb.x_off + (int)C;
                wb.v_off = 0; wb.k_off = (int)inner; wb.q_off = (int)(inner + Gr * N);       // inside the convolved channels: x | B | C
                append(in, src.get(q + "in", (2 * inner + 2 * Gr * N + H) * W, ws, 0.f));
                wb.conv_w = up_f32(m, src.get(q + "conv", C * taps, 0.5f / std::sqrt((float)taps), 0.f));
                wb.conv_b = up_f32(m, src.get(q + "conv.b", C, 0.1f, 0.f));
                wb.dt_bias = up_f32(m, src.get(q + "dt_bias", H, 0.5f, -1.f));
                std::vector<float> an = src.get(q + "A_log", H, 0.5f, 0.f);
                for (float& v : an) v = (float)(-std::exp((double)v));
                wb.a_neg = up_f32(m, an);
                wb.skip = up_f32(m, src.get(q + "D", H, 0.3f, 1.f));
                wb.mix_norm = up_f32(m, src.get(q + "norm", inner, 0.1f, 1.f));
                wb.o_col = sa.heads * sa.vdim;
            }
            w.in_rows = (int)(in.size() / W);
            w.g_off = w.in_rows;
            bias.resize((size_t)w.in_rows, 0.f);
            {   // one output projection for both mixers: the input columns are [left heads | right heads]
                const size_t ka = (size_t)sa.heads * sa.vdim, kb = (size_t)sb.heads * sb.vdim, K = ka + kb;
                const std::vector<float> oa = src.get(p + "mix.left.o", W * ka, 1.0f / std::sqrt((float)ka), 0.f);
                const std::vector<float> ob = src.get(p + "mix.right.o", W * kb, 1.0f / std::sqrt((float)kb), 0.f);
                std::vector<float> o(W * K);
                for (size_t r = 0; r < W; ++r) {
                    std::copy(oa.begin() + (long)(r * ka), oa.begin() + (long)((r + 1) * ka), o.begin() + (long)(r * K));
                    std::copy(ob.begin() + (long)(r * kb), ob.begin() + (long)((r + 1) * kb), o.begin() + (long)(r * K + ka));
                }
                w.o_w = up_bf16(m, o);
            }
        }
        w.in_w = up_bf16(m, in);
        w.in_b = up_f32(m, bias);
        if (sp.mlp == LMLP_MOE) {
            w.norm2 = up_f32(m, src.get(p + "norm2", W, 0.1f, 1.f));
            build_experts(m, src, p, sp, w);
        }
    }
    L.final_norm = up_f32(m, src.get("final.norm", W, 0.1f, 1.f));
    L.head = m.embed;                      // the logits come from the embedding table
    m.lm_head = L.head;
}

void load_layered_from_dir(Model& m, const std::string& dir) {
    try {
        LayFileSource src(dir);
        build_layered(m, src);
    } catch (const CmError&) { throw; }
    catch (const std::exception& e) { throw CmError(CM_ERR_IO, e.what()); }
}
void load_layered_synthetic(Model& m, uint64_t seed) {
    LaySynthSource src(seed);
    build_layered(m, src);
}

// ---------------------------------------------------------------------------------------------------------------
// runtime: key pages, state pools, scratch of one pass
// ---------------------------------------------------------------------------------------------------------------
void Model::alloc_runtime_layered() {
    Layered& L = *lay;
    const size_t W = (size_t)cfg.H;
    kv_mode = L.f32 ? KV_F32 : KV_BF16;
    kv_f32 = L.f32;
    kv_esize = L.f32 ? 4 : 2;
    // per-layer key pools (values are the keys: one pool per attention layer), page ids shared by all layers
    size_t pool_bytes = 0, st = 0, cv = 0;
    n_kv_layers = 0;
    kv_index.assign((size_t)cfg.L, -1);
    page_bytes = 0;
    // a mixer's share of the pools: cached rows of an attention, the state of a linear attention or matrix memory
    auto place_mixer = [&](const LayerSpec& sp, LayeredLayerW& w, size_t i) {
        if (sp.mixer == LMIX_ATTN || sp.mixer == LMIX_LATENT) {
            // cached row of a token and key head: the key (latent attention: [latent | rotated key part], one head); values that
            // are not (a part of) the keys have pages of their own
            const int dk = sp.mixer == LMIX_LATENT ? sp.kv_rank + sp.rot_dim : sp.dim;
            const int ev = sp.mixer == LMIX_LATENT ? sp.kv_rank : sp.vdim;
            if (sp.kv_from >= 0) {             // the other layer's pages
                const LayeredLayerW& o = L.w[(size_t)sp.kv_from];
                w.k_pool_off = o.k_pool_off; w.k_page_bytes = o.k_page_bytes; w.v_pool_off = o.v_pool_off; w.v_page_bytes = o.v_page_bytes;
                w.kv_idx = -1;
            } else {
                if (kv_index[i] < 0) kv_index[i] = n_kv_layers++;
                w.kv_idx = kv_index[i];
                w.k_page_bytes = (size_t)sp.kv_heads * sp.maps * page * dk * kv_esize;      // every map of a key head has rows of its own
                w.k_pool_off = pool_bytes;
                pool_bytes += (size_t)n_pages * w.k_page_bytes;
                page_bytes += w.k_page_bytes;      // all layers' share of one page (kv_bytes)
                if (sp.own_v) {
                    pool_bytes = (pool_bytes + 15) / 16 * 16;
                    w.v_page_bytes = (size_t)sp.kv_heads * page * sp.vdim * kv_esize;
                    w.v_pool_off = pool_bytes;
                    pool_bytes += (size_t)n_pages * w.v_page_bytes;
                    page_bytes += w.v_page_bytes;
                }
                if (sp.pool > 0) {             // mean rows of the position blocks that end inside a page
                    w.pool_rows = lay_pool_rows(page, sp.pool);
                    pool_bytes = (pool_bytes + 15) / 16 * 16;
                    w.pk_page_bytes = (size_t)sp.kv_heads * w.pool_rows * dk * kv_esize;
                    w.pk_pool_off = pool_bytes;
                    pool_bytes += (size_t)n_pages * w.pk_page_bytes;
                    page_bytes += w.pk_page_bytes;
                    if (sp.own_v) {
                        pool_bytes = (pool_bytes + 15) / 16 * 16;
                        w.pv_page_bytes = (size_t)sp.kv_heads * w.pool_rows * sp.vdim * kv_esize;
                        w.pv_pool_off = pool_bytes;
                        pool_bytes += (size_t)n_pages * w.pv_page_bytes;
                        page_bytes += w.pv_page_bytes;
                    }
                }
                pool_bytes = (pool_bytes + 15) / 16 * 16;
            }
            const int nrep = sp.heads / sp.kv_heads;
            if (std::find(L.nreps.begin(), L.nreps.end(), nrep) == L.nreps.end()) L.nreps.push_back(nrep);
            L.max_o = std::max(L.max_o, sp.heads * sp.maps * ev);
            L.max_e = std::max(L.max_e, ev);
            if (sp.mixer == LMIX_LATENT) {
                L.max_o = std::max(L.max_o, sp.heads * sp.vdim);
                L.max_cq = std::max(L.max_cq, sp.q_rank);
                L.max_q = std::max(L.max_q, sp.heads * (sp.dim + sp.rot_dim));
                L.max_qa = std::max(L.max_qa, sp.heads * dk);
            }
        } else if (sp.mixer == LMIX_MEMORY) {
            // [H][d][e + 1] (the last column is the normaliser vector), then the running maximum [H]
            w.st_off = st;
            st += (size_t)sp.heads * sp.dim * (sp.vdim + 1) + (size_t)sp.heads;
            L.max_o = std::max(L.max_o, sp.heads * (sp.vdim + 1));
            L.max_ld = std::max(L.max_ld, sp.heads);
            L.max_mh = std::max(L.max_mh, sp.heads);
        } else if (sp.mixer == LMIX_SSM) {
            // state [H][N][e]; the convolution's last taps - 1 inputs [taps - 1][x | B | C]
            w.st_off = st;
            st += (size_t)sp.heads * sp.state * sp.vdim;
            const int C = sp.heads * sp.vdim + 2 * sp.groups * sp.state;
            w.cv_off = cv;
            cv += (size_t)(sp.conv - 1) * C;
            L.max_conv = std::max(L.max_conv, C);
            L.max_o = std::max(L.max_o, sp.heads * sp.vdim);
            L.max_ld = std::max(L.max_ld, sp.heads);
            L.max_mh = std::max(L.max_mh, sp.heads);
        } else {
            w.st_off = st;
            st += (size_t)sp.heads * sp.dim * sp.vdim;
            L.max_o = std::max(L.max_o, sp.heads * sp.vdim);
            if (sp.mixer == LMIX_GLA || sp.mixer == LMIX_HGRN) L.max_ld = std::max(L.max_ld, sp.heads * sp.dim);
        }
    };
    for (size_t i = 0; i < L.spec.size(); ++i) {
        const LayerSpec& sp = L.spec[i];
        LayeredLayerW& w = L.w[i];
        if (sp.mixer == LMIX_SIDE) {
            int ocols = 0;
            for (size_t k = 0; k < sp.side.size(); ++k) { place_mixer(sp.side[k], w.side[k], i); ocols += sp.side[k].heads * sp.side[k].vdim; }
            L.max_o = std::max(L.max_o, ocols);
        } else place_mixer(sp, w, i);
        if (L.taps > 1) {
            w.c1_off = cv; cv += (size_t)(L.taps - 1) * W;
            if (sp.mlp != LMLP_NONE) { w.c2_off = cv; cv += (size_t)(L.taps - 1) * W; }
        }
        if (w.shift) { w.sh_off = cv; cv += W; }       // the mixer's previous input
        L.max_in = std::max(L.max_in, w.in_rows);
        if (sp.mlp != LMLP_NONE) L.max_ff = std::max(L.max_ff, sp.ff);
        if (sp.mlp == LMLP_MOE) {
            L.max_top = std::max(L.max_top, sp.top);
            L.max_E = std::max(L.max_E, sp.experts + sp.router.identity);
            L.max_slots = std::max(L.max_slots, sp.top + (sp.shared_ff > 0 ? 1 : 0));
            L.max_sff = std::max(L.max_sff, sp.shared_ff);
        }
    }
    kv_pool = (uint8_t*)dalloc<uint16_t>((pool_bytes + 1) / 2);
    free_pages.resize((size_t)n_pages);
    for (int64_t i = 0; i < n_pages; ++i) free_pages[(size_t)i] = (int32_t)(n_pages - 1 - i);
    page_ref.assign((size_t)n_pages, 0);
    conv_slot_elems = cv;
    state_slot_elems = st;
    if (cv) {
        conv_pool = dalloc<float>(cv * seqs.size());
        CM_HIP(hipMemsetAsync(conv_pool, 0, cv * seqs.size() * sizeof(float), stream));
    }
    if (st) {
        state_pool = dalloc<float>(st * seqs.size());
        CM_HIP(hipMemsetAsync(state_pool, 0, st * seqs.size() * sizeof(float), stream));
    }
    // scratch of one pass
    L.cap = opts.prefill_chunk ? (int)opts.prefill_chunk : 2048;
    L.cap = std::max(L.cap, 16);
    chunk = L.cap;
    const size_t cap = (size_t)L.cap;
    L.X = dalloc<float>(cap * W);
    L.Hn = dalloc<float>(cap * W);
    L.Hc = dalloc<float>(cap * W);
    L.Y = dalloc<float>(cap * W);
    L.P = dalloc<float>(cap * (size_t)L.max_in);
    L.O = dalloc<float>(cap * (size_t)L.max_o);
    L.O2 = dalloc<float>(cap * (size_t)L.max_o);
    if (L.max_ff) L.HH = dalloc<float>(cap * (size_t)L.max_top * (size_t)L.max_ff);
    if (L.parallel) { L.H2 = dalloc<float>(cap * W); L.Y2 = dalloc<float>(cap * W); }
    if (L.max_cq) {
        L.CQ = dalloc<float>(cap * (size_t)L.max_cq);
        L.Q = dalloc<float>(cap * (size_t)L.max_q);
        L.Qa = dalloc<float>(cap * (size_t)L.max_qa);
    }
    if (L.max_ld) L.LD = dalloc<float>(cap * (size_t)L.max_ld);
    if (L.max_mh) { L.KM = dalloc<float>(cap * (size_t)L.max_mh); L.MR = dalloc<float>(cap * (size_t)L.max_mh); }
    if (L.max_sff) L.HS = dalloc<float>(cap * (size_t)L.max_sff);
    if (L.max_conv) L.XB = dalloc<float>(cap * (size_t)L.max_conv);
    if (L.max_E > 1 || L.max_top > 1 || std::any_of(L.spec.begin(), L.spec.end(), [](const LayerSpec& s) { return s.mlp == LMLP_MOE; })) {
        L.YS = dalloc<float>(cap * (size_t)L.max_slots * W);
        L.wsel = dalloc<float>(cap * (size_t)L.max_slots);
        L.sel = dalloc<int32_t>(cap * (size_t)L.max_top);
        L.srt = dalloc<int32_t>(cap * (size_t)L.max_top);
        L.off = dalloc<int32_t>((size_t)L.max_E + 1);
        L.Z = dalloc<float>(cap * (size_t)L.max_E);
    }
    if (!L.f32) {
        int max_k = std::max({(int)W, L.max_o, L.max_ff, L.max_cq, L.max_sff}), dense_ff = L.max_sff;
        for (const LayerSpec& sp : L.spec) if (sp.mlp == LMLP_DENSE && sp.gated_ff) dense_ff = std::max(dense_ff, sp.ff);
        const size_t rows = (cap + 255) / 256 * 256;
        L.Abf = dalloc<uint16_t>(rows * (size_t)max_k);
        CM_HIP(hipMemsetAsync(L.Abf, 0, rows * (size_t)max_k * sizeof(uint16_t), stream));
        if (dense_ff) { L.G1 = dalloc<float>(cap * (size_t)dense_ff); L.G2 = dalloc<float>(cap * (size_t)dense_ff); }
        ensure_gemm_workspace();
    }
    size_t hde = 0, hd = 0;
    auto chunk_scratch = [&](const LayerSpec& sp) {
        const bool lin = sp.mixer == LMIX_LIGHTNING || sp.mixer == LMIX_GLA || sp.mixer == LMIX_HGRN || sp.mixer == LMIX_SSM;
        if (lin && sp.dim <= 128) hde = std::max(hde, (size_t)sp.heads * sp.dim * sp.vdim);
        if (lin && sp.mixer != LMIX_LIGHTNING && sp.dim <= 128) hd = std::max(hd, (size_t)sp.heads * sp.dim);
        if (sp.mixer == LMIX_MEMORY && sp.dim <= 128) {
            hde = std::max(hde, (size_t)sp.heads * sp.dim * (sp.vdim + 1));
            hd = std::max(hd, (size_t)sp.heads * sp.dim);
        }
    };
    for (const LayerSpec& sp : L.spec) {
        chunk_scratch(sp);
        for (const LayerSpec& sd : sp.side) chunk_scratch(sd);
    }
    if (hde) { L.u_stride = hde; L.U = dalloc<float>((cap / LAY_LIGHT_CHUNK + (size_t)MAXB + 1) * hde); }
    if (hd) L.Dch = dalloc<float>((cap / LAY_LIGHT_CHUNK + (size_t)MAXB + 1) * hd);
    if (L.max_e) {
        L.att_po = dalloc<float>((size_t)Layered::ATT_PARTS * 16 * L.max_e);
        L.att_pml = dalloc<float>((size_t)Layered::ATT_PARTS * 16 * 2);
    }
    L.am_pv = dalloc<float>((size_t)Layered::LOGIT_ROWS * LAY_ARGMAX_PARTS);
    L.am_pi = dalloc<int>((size_t)Layered::LOGIT_ROWS * LAY_ARGMAX_PARTS);
    L.Xw = dalloc<float>((size_t)Layered::LOGIT_ROWS * W);
    logitsb = dalloc<float>((size_t)Layered::LOGIT_ROWS * cfg.V);
    logits = dalloc<float>((size_t)cfg.V);
    V_l = cfg.V;
    CM_HIP(hipHostMalloc((void**)&h_logits, (size_t)cfg.V * sizeof(float)));
    CM_HIP(hipHostMalloc((void**)&L.h_rows, (size_t)Layered::LOGIT_ROWS * cfg.V * sizeof(float)));
    L.d_greedy = dalloc<uint32_t>(Layered::LOGIT_ROWS);
    CM_HIP(hipHostMalloc((void**)&L.h_greedy, Layered::LOGIT_ROWS * sizeof(uint32_t)));
    // one table upload per pass: ids | rowseg | wanted rows | segments | page tables | attention tiles per group size
    size_t tiles = 0;
    for (int nrep : L.nreps) tiles += 2 * (cap * (size_t)nrep / 16 + (size_t)MAXB + 1) + 2 * (cap * (size_t)nrep / LAY_ATTN_MFMA_ROWS + (size_t)MAXB + 1);
    tiles += 2 * (cap / LAY_LIGHT_CHUNK + (size_t)MAXB + 1);      // lightning chunks
    L.tab_ints = 3 * cap + (size_t)MAXB * (sizeof(LaySegDev) / 4) + (size_t)MAXB * max_pages_per_seq + tiles + 64;
    L.d_tab = dalloc<int32_t>(L.tab_ints);
    CM_HIP(hipHostMalloc((void**)&L.h_tab, L.tab_ints * sizeof(int32_t)));
    CM_HIP(hipStreamSynchronize(stream));
}

size_t Model::layered_capture(float* out, size_t n) const {
    if (!lay) throw CmError(CM_ERR_UNSUPPORTED, "not a layer-list decoder");
    const size_t k = std::min(n, lay->captured.size());
    if (out && k) memcpy(out, lay->captured.data(), k * sizeof(float));
    return lay->captured.size();
}
void Model::layered_set_shared_gemm(bool on) {
    if (!lay) throw CmError(CM_ERR_UNSUPPORTED, "not a layer-list decoder");
    lay->shared_gemm = on;
}
void Model::layered_set_attn_mfma(bool on) {
    if (!lay) throw CmError(CM_ERR_UNSUPPORTED, "not a layer-list decoder");
    lay->attn_mfma = on;
}
void Model::layered_set_fused_prep(bool on) {
    if (!lay) throw CmError(CM_ERR_UNSUPPORTED, "not a layer-list decoder");
    lay->fused_prep = on;
}
void Model::layered_set_capture(bool on) {
    if (!lay) throw CmError(CM_ERR_UNSUPPORTED, "not a layer-list decoder");
    lay->capture = on;
    lay->captured.clear();
}
void Model::layered_cow_page(int32_t oldp, int32_t newp) {
    Layered& L = *lay;
    auto copy = [&](size_t off, size_t bytes) {
        if (bytes) CM_HIP(hipMemcpyAsync(kv_pool + off + (size_t)newp * bytes, kv_pool + off + (size_t)oldp * bytes, bytes, hipMemcpyDeviceToDevice, stream));
    };
    auto one = [&](const LayeredLayerW& w) {
        if (w.kv_idx < 0) return;
        copy(w.k_pool_off, w.k_page_bytes);
        copy(w.v_pool_off, w.v_page_bytes);
        copy(w.pk_pool_off, w.pk_page_bytes);
        copy(w.pv_pool_off, w.pv_page_bytes);
    };
    for (size_t i = 0; i < L.w.size(); ++i) {
        one(L.w[i]);
        for (const LayeredLayerW& sd : L.w[i].side) one(sd);
    }
}

// ---------------------------------------------------------------------------------------------------------------
// one step: every item appends its tokens to its sequence; all items run as one batch
// ---------------------------------------------------------------------------------------------------------------
namespace {
struct PassSeg { size_t item; size_t off; int n; };
}

void Model::step_batch(const StepItem* items, size_t n_items, float* logits_out, uint32_t* greedy_out) {
    if (!layered) throw CmError(CM_ERR_UNSUPPORTED, "step_batch: not a layer-list decoder");
    if (n_items == 0 || !items) throw CmError(CM_ERR_INVALID, "empty step");
    Layered& L = *lay;
    const int W = cfg.H, V = cfg.V;
    hipStream_t s = stream;
    for (size_t i = 0; i < n_items; ++i) {
        const StepItem& it = items[i];
        if (!it.ids || it.n == 0) throw CmError(CM_ERR_INVALID, "empty input");
        Seq& q = seq(it.seq);
        for (size_t c = 0; c < i; ++c) if (items[c].seq == it.seq) throw CmError(CM_ERR_INVALID, "sequence appears twice in one step");
        if (q.len + (int64_t)it.n > (int64_t)max_seq) throw CmError(CM_ERR_RANGE, "sequence longer than max_seq_len");
        for (size_t k = 0; k < it.n; ++k) if (it.ids[k] >= (uint32_t)V) throw CmError(CM_ERR_RANGE, "token id >= vocab_size");
        for (int k = 0; k < it.n_want; ++k)
            if (it.want[k] < 0 || (size_t)it.want[k] >= it.n || (k && it.want[k] <= it.want[k - 1]))
                throw CmError(CM_ERR_INVALID, "wanted positions must ascend inside the portion");
    }
    // pages first: a step that does not fit changes nothing
    {
        size_t need = 0;
        for (size_t i = 0; i < n_items; ++i) {
            const Seq& q = seq(items[i].seq);
            const size_t want = (size_t)((q.len + (int64_t)items[i].n + page - 1) / page);
            if (want > q.pages.size()) need += want - q.pages.size();
            if ((q.len % page) != 0 && !q.pages.empty() && page_ref[(size_t)q.pages[(size_t)(q.len / page)]] > 1) ++need;
        }
        if (need > free_pages.size()) throw CmError(CM_ERR_OOM, "KV pool exhausted");
        for (size_t i = 0; i < n_items; ++i) ensure_pages(items[i].seq, seq(items[i].seq).len + (int64_t)items[i].n);
    }
    active_seq = -1; active_pages_uploaded = 0;
    size_t out_row = 0;                       // next row of logits_out / greedy_out
    size_t it_i = 0, it_off = 0;
    while (it_i < n_items) {
        // ---- cut the next pass: items in order, at most cap rows and MAXB segments
        std::vector<PassSeg> ps;
        int T = 0;
        while (it_i < n_items && T < L.cap && (int)ps.size() < MAXB) {
            const int n = (int)std::min<size_t>(items[it_i].n - it_off, (size_t)(L.cap - T));
            ps.push_back(PassSeg{it_i, it_off, n});
            T += n; it_off += (size_t)n;
            if (it_off == items[it_i].n) { ++it_i; it_off = 0; }
        }
        const int nseg = (int)ps.size();
        CM_HIP(hipStreamSynchronize(s));      // the pinned tables of the previous pass have been consumed
        int32_t* tab = L.h_tab;
        size_t o = 0;
        int32_t* t_ids = tab + o; const size_t o_ids = o; o += (size_t)T;
        int32_t* t_rowseg = tab + o; const size_t o_rowseg = o; o += (size_t)T;
        int32_t* t_wrows = tab + o; const size_t o_wrows = o; o += (size_t)T;
        LaySegDev* t_segs = (LaySegDev*)(tab + o); const size_t o_segs = o; o += (size_t)nseg * (sizeof(LaySegDev) / 4);
        int32_t* t_bt = tab + o; const size_t o_bt = o; o += (size_t)nseg * max_pages_per_seq;
        int nw = 0, row = 0, nchunks = 0, max_n = 0;
        long long max_len = 0;
        bool all_decode = true;
        for (int k = 0; k < nseg; ++k) {
            const StepItem& it = items[ps[(size_t)k].item];
            Seq& q = seq(it.seq);
            const int n = ps[(size_t)k].n;
            const int sp = (int)q.len;
            t_segs[k] = LaySegDev{row, n, sp, it.seq, k * max_pages_per_seq, nchunks, 0, 0};
            nchunks += (n + LAY_LIGHT_CHUNK - 1) / LAY_LIGHT_CHUNK;
            max_n = std::max(max_n, n);
            max_len = std::max(max_len, (long long)sp + n);
            memcpy(t_bt + (size_t)k * max_pages_per_seq, q.pages.data(), q.pages.size() * sizeof(int32_t));
            for (size_t pz = q.pages.size(); pz < (size_t)max_pages_per_seq; ++pz) t_bt[(size_t)k * max_pages_per_seq + pz] = 0;
            for (int r = 0; r < n; ++r) { t_ids[row + r] = (int32_t)it.ids[ps[(size_t)k].off + (size_t)r]; t_rowseg[row + r] = k; }
            if (it.n_want < 0) { if (ps[(size_t)k].off + (size_t)n == it.n) t_wrows[nw++] = row + n - 1; }
            else for (int j = 0; j < it.n_want; ++j) {
                const long p = (long)it.want[j] - (long)ps[(size_t)k].off;
                if (p >= 0 && p < n) t_wrows[nw++] = row + (int)p;
            }
            if (n != 1) all_decode = false;
            row += n;
            q.len += n;                        // the cache holds these positions once the pass has run
        }
        std::map<int, std::pair<size_t, int>> tiles, tiles64;      // nrep -> (offset, count): 16 / 64 query rows per tile
        for (int nrep : L.nreps) {
            if (o & 1) ++o;                    // int2 entries
            const size_t o_t = o; int cnt = 0;
            for (int k = 0; k < nseg; ++k)
                for (int q0 = 0; q0 < t_segs[k].n * nrep; q0 += 16) { tab[o++] = k; tab[o++] = q0; ++cnt; }
            tiles[nrep] = {o_t, cnt};
            const size_t o_m = o; cnt = 0;
            if (!all_decode) {
                for (int k = 0; k < nseg; ++k)
                    for (int q0 = 0; q0 < t_segs[k].n * nrep; q0 += LAY_ATTN_MFMA_ROWS) { tab[o++] = k; tab[o++] = q0; ++cnt; }
                // blocks with the longest key range first: the short ones fill the tail of the launch
                int2* tl = (int2*)(tab + o_m);
                std::stable_sort(tl, tl + cnt, [&](const int2& x, const int2& y) {
                    return t_segs[x.x].start_pos + x.y / nrep > t_segs[y.x].start_pos + y.y / nrep; });
            }
            tiles64[nrep] = {o_m, cnt};
        }
        if (o & 1) ++o;
        const size_t o_chunks = o;
        if (L.U && max_n > LAY_LIGHT_CHUNK)
            for (int k = 0; k < nseg; ++k)
                for (int t0 = 0; t0 < t_segs[k].n; t0 += LAY_LIGHT_CHUNK) { tab[o++] = k; tab[o++] = t0; }
        if (o > L.tab_ints) throw CmError(CM_ERR_INVALID, "step tables overflow");
        CM_HIP(hipMemcpyAsync(L.d_tab, tab, o * sizeof(int32_t), hipMemcpyHostToDevice, s));
        const uint32_t* d_ids = (const uint32_t*)(L.d_tab + o_ids);
        const int32_t* d_rowseg = L.d_tab + o_rowseg;
        const int32_t* d_wrows = L.d_tab + o_wrows;
        const LaySegDev* d_segs = (const LaySegDev*)(L.d_tab + o_segs);
        const int32_t* d_bt = L.d_tab + o_bt;

        if (W % 4 == 0 && L.embed_scale == 1.f) launch_embed_rows(embed, d_ids, L.X, T, W, V, s);
        else launch_lay_embed_rows(embed, d_ids, L.X, T, W, V, s, L.embed_scale);
        // the residual update of a finished sublayer waits for the next norm: decode steps run both in one launch
        struct { const float* y = nullptr; const float* w = nullptr; const float* wsel = nullptr; int top = 0; int sel_top = 0, n_real = -1; } pend;
        auto flush_post = [&]() {
            if (pend.y) {
                // identity experts: their rows are the sublayer's input, which for this update is the residual itself (a thread reads
                // an element of x before it writes it, and touches no other)
                if (pend.n_real >= 0) launch_lay_post_norm(L.X, pend.y, pend.w, L.mult, cfg.eps, T, W, pend.wsel, pend.top, s, L.sel, pend.sel_top, pend.n_real, L.X);
                else launch_lay_post_norm(L.X, pend.y, pend.w, L.mult, cfg.eps, T, W, pend.wsel, pend.top, s);
            }
            pend.y = nullptr; pend.n_real = -1;
        };
        auto post_norm = [&](const float* y, const float* w_, const float* wsel, int top) {
            flush_post();
            pend.y = y; pend.w = w_; pend.wsel = wsel; pend.top = top;
        };
        auto norm_canon = [&](const float* nw_, const float* cw, size_t coff) {
            if (pend.y && all_decode) {
                launch_lay_post_norm_canon_decode(L.X, pend.y, pend.w, L.mult, pend.wsel, pend.top, nw_, cfg.eps, L.Hc, cw, conv_pool,
                                                  conv_slot_elems, coff, d_segs, T, W, L.taps, s);
                pend.y = nullptr;
                return;
            }
            flush_post();
            if (L.taps <= 0) { launch_lay_rms_rows(L.X, nullptr, nw_, L.Hc, T, W, cfg.eps, s); return; }
            if (all_decode) {
                launch_lay_norm_canon_decode(L.X, nw_, cfg.eps, L.Hc, cw, conv_pool, conv_slot_elems, coff, d_segs, T, W, L.taps, s);
                return;
            }
            launch_lay_rms_rows(L.X, nullptr, nw_, L.Hn, T, W, cfg.eps, s);
            launch_lay_canon(L.Hn, L.Hc, cw, conv_pool, conv_slot_elems, coff, d_segs, d_rowseg, T, W, L.taps, s);
            launch_lay_canon_tail(L.Hn, conv_pool, conv_slot_elems, coff, d_segs, nseg, W, L.taps, s);
        };
        // softmax attention of one layer over the pages: queries at qsrc[row ldq + q_off + head dk], output [T][H ev] into L.O
        auto run_attention = [&](const LayerSpec& sp, const LayeredLayerW& w, const float* qsrc, int ldq, int q_off, int g_off, int dk, int ev,
                                 float* out = nullptr, int ldo = 0, float out_scale = 1.f, int v_div = 1) {
            LAttnArgs a;
            a.v_div = v_div;
            a.proj = qsrc; a.ldp = ldq; a.q_off = q_off; a.g_off = g_off;
            a.out = out ? out : L.O; a.ldo = out ? ldo : sp.heads * ev; a.out_scale = out_scale;
            if (sp.pool > 0) {
                a.pool = sp.pool; a.pool_rows = w.pool_rows; a.pk_pool = kv_pool + w.pk_pool_off;
                a.pv_pool = w.pv_page_bytes ? kv_pool + w.pv_pool_off : nullptr;
            }
            a.kpool = kv_pool + w.k_pool_off; a.bt = d_bt; a.segs = d_segs;
            a.vpool = w.v_page_bytes ? kv_pool + w.v_pool_off : nullptr; a.e = ev;
            const auto& tl = tiles[sp.heads / sp.kv_heads];
            a.tiles = (const int2*)(L.d_tab + tl.first); a.ntiles = tl.second;
            a.r1 = w.r1; a.r2 = w.r2; a.H = sp.heads; a.G = sp.kv_heads; a.d = dk; a.page = page;
            a.scale = sp.scale; a.win = sp.win; a.keep = sp.keep; a.chunk = sp.chunk;
            a.bias = sp.bias; a.gate = sp.gate; a.sink = sp.sink ? w.sink : nullptr;
            {   // few query tiles and many visible keys (decode steps): share a tile's keys among blocks
                long long seen = std::min<long long>(max_len, sp.win + sp.keep);
                if (sp.chunk > 0) seen = std::min(seen, sp.chunk);
                if (sp.pool > 0) seen = std::min<long long>(max_len, sp.win + max_len / sp.pool);
                const int kt = lay_attn_key_tile(dk, ev, a.vpool != nullptr);
                const int key_tiles = (int)((seen + kt - 1) / kt), blocks = std::max(1, a.ntiles * sp.kv_heads);
                a.nsplit = std::max(1, std::min({32, key_tiles, 256 / blocks, Layered::ATT_PARTS / blocks}));
                a.part_o = L.att_po; a.part_ml = L.att_pml;
            }
            if (L.attn_mfma && kv_mode == KV_BF16 && !all_decode && max_n >= 16 && lay_attn_mfma_fits(dk, ev, a.vpool != nullptr)) {
                const auto& tm = tiles64[sp.heads / sp.kv_heads];
                a.tiles = (const int2*)(L.d_tab + tm.first); a.ntiles = tm.second;
                launch_lay_attn_mfma(a, s);
            } else
                launch_lay_attn(a, kv_mode, s);
        };
        // lightning / gated linear attention of one layer: raw head outputs into L.O
        // ldp: width of the projection rows in L.P; kmul != null: the matrix-memory form (one decay and one key factor per head and
        // token, a constant 1 as last value column, raw outputs [T][H (e + 1)] into L.O2)
        auto run_linear = [&](const LayerSpec& sp, const LayeredLayerW& w, const float* ldec, int ldp, const float* kmul = nullptr) {
            LLightArgs a;
            a.proj = L.P; a.ldp = ldp; a.q_off = w.q_off; a.k_off = w.k_off; a.v_off = w.v_off;
            a.out = L.O; a.ldo = sp.heads * sp.vdim;
            a.state_pool = state_pool; a.slot_stride = state_slot_elems; a.st_off = w.st_off;
            a.segs = d_segs; a.nseg = nseg; a.decay = w.decay; a.H = sp.heads; a.d = sp.dim; a.e = sp.vdim;
            a.all_single = all_decode;
            if (ldec) { a.ldec = ldec; a.ldd = sp.heads * sp.dim; a.qscale = 1.0f / std::sqrt((float)sp.dim); a.D = L.Dch; }
            if (kmul) {
                a.head_decay = true; a.kmul = kmul; a.ones_col = true; a.ldd = sp.heads;
                a.e = sp.vdim + 1; a.out = L.O2; a.ldo = sp.heads * (sp.vdim + 1);
            }
            if (L.U && max_n > LAY_LIGHT_CHUNK && sp.dim <= 128) {       // a long portion in the pass: parallel over chunks
                a.U = L.U; a.chunks = (const int2*)(L.d_tab + o_chunks); a.nchunks = nchunks;
            }
            launch_lay_lightning(a, s);
        };
        // long portions in the pass: the linear-attention kernels run parallel over chunks
        auto linear_chunks = [&](LLightArgs& a) {
            if (L.U && max_n > LAY_LIGHT_CHUNK && a.d <= 128) {
                a.U = L.U; a.chunks = (const int2*)(L.d_tab + o_chunks); a.nchunks = nchunks;
                if (a.ldec) a.D = L.Dch;
            }
        };
        // pre-norm layers: the finished sublayer's rows (nsum per token, summed in order) join the residual inside the next norm's launch
        struct { const float* y = nullptr; int nsum = 1; } padd;
        auto add_gnorm = [&](const float* nw_, float* out) {
            launch_lay_add_gnorm(L.X, nullptr, padd.y, padd.nsum, nw_, out, T, W, L.norm_groups, cfg.eps, s);
            padd.y = nullptr;
        };
        const float *par_y1 = nullptr, *par_y2 = nullptr;       // parallel layers: sublayer outputs not yet added to the residual
        for (size_t li = 0; li < L.spec.size(); ++li) {
            const LayerSpec& sp = L.spec[li];
            const LayeredLayerW& w = L.w[li];
            if (L.parallel) {
                // ---- mixer and feed-forward side by side on two norms of the same residual; the mixer's rows pass the token shift
                float* h2 = sp.mlp != LMLP_NONE ? L.H2 : nullptr;
                if (all_decode) {          // one launch: the previous layer's residual update, both norms, the shift and its state
                    launch_lay_add_norm2_shift_decode(L.X, par_y1, par_y2, w.norm1, w.norm2, cfg.eps, L.Hc, h2, w.shift, conv_pool, conv_slot_elems,
                                                      w.sh_off, d_segs, T, W, s);
                    par_y1 = par_y2 = nullptr;
                } else {
                    launch_lay_rms_rows2(L.X, w.norm1, w.norm2, L.Hn, h2, T, W, cfg.eps, s);
                    launch_lay_canon(L.Hn, L.Hc, w.shift, conv_pool, conv_slot_elems, w.sh_off, d_segs, d_rowseg, T, W, 2, s);
                    launch_lay_canon_tail(L.Hn, conv_pool, conv_slot_elems, w.sh_off, d_segs, nseg, W, 2, s);
                }
                LGemmArgs g;
                g.A = L.Hc; g.lda = W; g.W = w.in_w; g.C = L.P; g.ldc = w.in_rows; g.M = T; g.N = w.in_rows; g.K = W;
                g.act_split = w.g_off; g.act = LACT_NONE; g.act2 = sp.mixer == LMIX_GLA ? LACT_SILU : LACT_SIGMOID;
                lay_gemm(*this, L, g, 1, s);
                const int H = sp.heads, ev = sp.vdim;
                const float* oa = L.O;
                if (sp.mixer == LMIX_ATTN) {
                    if (sp.kv_from < 0) {
                        launch_lay_k_append(L.P, w.in_rows, w.k_off, kv_pool + w.k_pool_off, kv_mode, d_bt, d_segs, d_rowseg, T, sp.kv_heads, sp.dim, page, s);
                        launch_lay_k_append(L.P, w.in_rows, w.v_off, kv_pool + w.v_pool_off, kv_mode, d_bt, d_segs, d_rowseg, T, sp.kv_heads, ev, page, s);
                    }
                    run_attention(sp, w, L.P, w.in_rows, w.q_off, w.g_off, sp.dim, ev);
                } else if (sp.mixer == LMIX_LATENT) {
                    const int kr = sp.kv_rank, r = sp.rot_dim, dh = sp.dim, dk = kr + r;
                    // both latents through their norms; the key latent in place, next to the shared rotated key part
                    launch_lay_rms_cols(L.P, w.in_rows, w.q_off, sp.q_rank, w.dq_norm, L.CQ, sp.q_rank, T, cfg.eps, s);
                    launch_lay_rms_cols(L.P, w.in_rows, w.k_off, kr, w.dkv_norm, L.P + w.k_off, w.in_rows, T, cfg.eps, s);
                    LGemmArgs gq;
                    gq.A = L.CQ; gq.lda = sp.q_rank; gq.W = w.uq; gq.C = L.Q; gq.ldc = H * (dh + r); gq.M = T; gq.N = H * (dh + r); gq.K = sp.q_rank;
                    lay_gemm(*this, L, gq, 1, s);
                    if (r > 0 && sp.rot.dims > 0)
                        launch_lay_rope(L.P + w.k_off + kr, w.in_rows, 0, L.P + w.k_off + kr, w.in_rows, 0, 1, r, sp.rot.dims, w.rot_freq, w.rot_mag,
                                        d_segs, d_rowseg, T, s);
                    launch_lay_k_append(L.P, w.in_rows, w.k_off, kv_pool + w.k_pool_off, kv_mode, d_bt, d_segs, d_rowseg, T, 1, dk, page, s);
                    // q_unrotated . (W_uk c) = (W_uk^T q_unrotated) . c: per head, the query moves into the latent's space
                    LGemmArgs ga;
                    ga.A = L.Q; ga.lda = H * (dh + r); ga.a_goff = (size_t)(dh + r); ga.W = w.uk_t; ga.w_stride = (size_t)kr * dh;
                    ga.C = L.Qa; ga.ldc = H * dk; ga.c_goff = (size_t)dk; ga.M = T; ga.N = kr; ga.K = dh;
                    lay_gemm(*this, L, ga, H, s);
                    if (r > 0)
                        launch_lay_rope(L.Q + dh, H * (dh + r), dh + r, L.Qa + kr, H * dk, dk, H, r, sp.rot.dims, w.rot_freq, w.rot_mag, d_segs,
                                        d_rowseg, T, s);
                    run_attention(sp, w, L.Qa, H * dk, 0, 0, dk, kr);
                    // the weighted latents become values per head, times the gate
                    LGemmArgs gv;
                    gv.A = L.O; gv.lda = H * kr; gv.a_goff = (size_t)kr; gv.W = w.uv; gv.w_stride = (size_t)ev * kr;
                    gv.C = L.O2; gv.ldc = H * ev; gv.c_goff = (size_t)ev; gv.M = T; gv.N = ev; gv.K = kr;
                    gv.mul = L.P + w.g_off; gv.ldm = w.in_rows;
                    lay_gemm(*this, L, gv, H, s);
                    oa = L.O2;
                } else {
                    // logarithm of the decay: ln(sigmoid(z)^(1 / tau)), z from the low-rank pair
                    LGemmArgs gd;
                    gd.A = L.P + w.a_off; gd.lda = w.in_rows; gd.W = w.a2; gd.bias = w.a2_b; gd.C = L.LD; gd.ldc = H * sp.dim;
                    gd.M = T; gd.N = H * sp.dim; gd.K = sp.a_rank; gd.act = LACT_LOGSIG; gd.act_split = gd.N; gd.act_param = 1.0f / sp.tau;
                    lay_gemm(*this, L, gd, 1, s);
                    run_linear(sp, w, L.LD, w.in_rows);
                    launch_lay_rms_gate(L.O, L.P + w.g_off, w.in_rows, w.mix_norm, L.O2, T, H * ev, cfg.eps, s, ev, true);
                    oa = L.O2;
                }
                LGemmArgs go;
                go.A = oa; go.lda = H * ev; go.W = w.o_w; go.C = L.Y; go.ldc = W; go.M = T; go.N = W; go.K = H * ev;
                lay_gemm(*this, L, go, 1, s);
                if (sp.mlp != LMLP_NONE) {
                    LGemmArgs gu;
                    gu.A = L.H2; gu.lda = W; gu.W = w.up; gu.C = L.HH; gu.ldc = sp.ff; gu.M = T; gu.N = sp.ff; gu.K = W;
                    gu.act = sp.ff_act; gu.act_split = sp.ff;
                    lay_gemm(*this, L, gu, 1, s);
                    LGemmArgs dn;
                    dn.A = L.HH; dn.lda = sp.ff; dn.W = w.down; dn.C = L.Y2; dn.ldc = W; dn.M = T; dn.N = W; dn.K = sp.ff;
                    lay_gemm(*this, L, dn, 1, s);
                }
                par_y1 = L.Y; par_y2 = sp.mlp != LMLP_NONE ? L.Y2 : nullptr;
                if (!all_decode || L.capture || li + 1 == L.spec.size()) {      // decode steps: inside the next layer's first launch
                    launch_lay_add_rows(L.X, par_y1, par_y2, (size_t)T * W, s);
                    par_y1 = par_y2 = nullptr;
                }
            } else if (L.pre_norm) {
                // ---- x += mixer(norm1 x), x += ff(norm2 x), norms in equal parts
                add_gnorm(w.norm1, L.Hc);
                LGemmArgs g;
                g.A = L.Hc; g.lda = W; g.W = w.in_w; g.bias = w.in_b; g.C = L.P; g.ldc = w.in_rows; g.M = T; g.N = w.in_rows; g.K = W;
                g.act_split = w.g_off; g.act = sp.mixer == LMIX_HGRN ? LACT_SILU : LACT_NONE; g.act2 = LACT_NONE;
                lay_gemm(*this, L, g, 1, s);
                const float* oa = L.O;
                int on = 0;
                if (sp.mixer == LMIX_ATTN) {
                    // two maps per head as heads of their own (2 H query heads over 2 G key heads, pairs of key heads share a value head)
                    const int H = sp.heads, G = sp.kv_heads, d = sp.dim, e = sp.vdim;
                    LQkPrepExtra ex;
                    ex.Gv = G; ex.qt_coef = sp.qt_coef; ex.qt_every = (int)sp.qt_every;
                    launch_lay_qk_prep(L.P, w.in_rows, w.q_off, w.k_off, w.v_off, 2 * H, 2 * G, d, e, nullptr, nullptr, cfg.eps, 0, false, nullptr, 1.f,
                                       kv_pool + w.k_pool_off, kv_pool + w.v_pool_off, kv_mode, d_bt, d_segs, d_rowseg, T, page, s, 0, 0, nullptr, nullptr, &ex);
                    if (L.attn_mfma && kv_mode == KV_BF16 && !all_decode && max_n >= 16 && lay_attn_talk_mfma_fits(2 * H, 2 * G, d, e, 2, false) &&
                        w.in_rows % 4 == 0 && w.q_off % 4 == 0) {
                        // prompt passes: a block of 16 positions with one wave per (head, map), all of them on the same staged tiles
                        LAttnArgs a;
                        a.proj = L.P; a.ldp = w.in_rows; a.q_off = w.q_off; a.g_off = 0;
                        a.out = L.O; a.ldo = 2 * H * e; a.out_scale = 1.f;
                        a.kpool = kv_pool + w.k_pool_off; a.vpool = kv_pool + w.v_pool_off; a.bt = d_bt; a.segs = d_segs;
                        a.tiles = nullptr; a.ntiles = 0; a.r1 = a.r2 = nullptr;
                        a.H = 2 * H; a.G = 2 * G; a.d = d; a.e = e; a.page = page; a.scale = sp.scale; a.win = sp.win; a.keep = 0;
                        a.bias = LBIAS_NONE; a.gate = LGATE_NONE; a.v_div = 2;
                        launch_lay_attn_talk_mfma(a, nullptr, nseg, max_n, s);
                    } else {
                        LayerSpec two = sp;
                        two.heads = 2 * H; two.kv_heads = 2 * G;
                        run_attention(two, w, L.P, w.in_rows, w.q_off, 0, d, e, nullptr, 0, 1.f, 2);
                    }
                    launch_lay_diff_combine(L.O, L.O2, T, H, G, e, w.lambda, 1.f - sp.diff, cfg.eps, s);
                    oa = L.O2; on = H * e;
                } else if (sp.mixer == LMIX_HGRN) {
                    const int H = sp.heads, d = sp.dim, e = sp.vdim;
                    launch_lay_hgrn_gates(L.P, w.in_rows, w.k_off, w.lower, L.LD, T, H * d, s);
                    LLightArgs a;
                    a.proj = L.P; a.ldp = w.in_rows; a.q_off = w.q_off; a.k_off = w.k_off; a.v_off = w.v_off;
                    a.out = L.O; a.ldo = H * e;
                    a.state_pool = state_pool; a.slot_stride = state_slot_elems; a.st_off = w.st_off;
                    a.segs = d_segs; a.nseg = nseg; a.decay = nullptr; a.H = H; a.d = d; a.e = e; a.all_single = all_decode;
                    a.ldec = L.LD; a.ldd = H * d;
                    linear_chunks(a);
                    launch_lay_lightning(a, s);
                    launch_lay_rms_gate(L.O, nullptr, 0, w.mix_norm, L.O2, T, H * e, cfg.eps, s, e, true);
                    oa = L.O2; on = H * e;
                } else {
                    for (const LayerSpec& sd : sp.side) on += sd.heads * sd.vdim;
                    for (size_t k = 0; k < sp.side.size(); ++k) {
                        const LayerSpec& sd = sp.side[k];
                        const LayeredLayerW& sw = w.side[k];
                        const int H = sd.heads, e = sd.vdim;
                        if (sd.mixer == LMIX_ATTN) {
                            const int G = sd.kv_heads, d = sd.dim;
                            LQkPrepExtra ex;
                            ex.head_norm = sd.head_norm;
                            launch_lay_qk_prep(L.P, w.in_rows, sw.q_off, sw.k_off, sw.v_off, H, G, d, e, sw.q_norm, sw.k_norm, cfg.eps, sd.rot.dims,
                                               sd.rot.half, sd.rot.dims > 0 ? sw.rot_freq : nullptr, sw.rot_mag, kv_pool + sw.k_pool_off,
                                               kv_pool + sw.v_pool_off, kv_mode, d_bt, d_segs, d_rowseg, T, page, s, 0, 0, nullptr, nullptr, &ex);
                            LAttnArgs a;
                            a.proj = L.P; a.ldp = w.in_rows; a.q_off = sw.q_off; a.g_off = 0;
                            a.out = L.O + sw.o_col; a.ldo = on; a.out_scale = sd.side_scale;
                            a.kpool = kv_pool + sw.k_pool_off; a.vpool = kv_pool + sw.v_pool_off; a.bt = d_bt; a.segs = d_segs;
                            a.tiles = nullptr; a.ntiles = 0; a.r1 = a.r2 = nullptr;
                            a.H = H; a.G = G; a.d = d; a.e = e; a.page = page; a.scale = sd.scale; a.win = sd.win; a.keep = 0;
                            a.bias = LBIAS_NONE; a.gate = LGATE_NONE;
                            if (all_decode) {      // few rows, many keys: the window's key tiles are dealt to several blocks
                                const long long seen = std::min<long long>(max_len, sd.win);
                                const int key_tiles = (int)((seen + 31) / 32);
                                a.nsplit = std::max(1, std::min({32, key_tiles, 256 / std::max(1, nseg), Layered::ATT_PARTS * 16 / std::max(1, nseg * H)}));
                                a.part_o = L.att_po; a.part_ml = L.att_pml;
                            }
                            if (L.attn_mfma && kv_mode == KV_BF16 && !all_decode && max_n >= 16 && lay_attn_talk_mfma_fits(H, G, d, e) && w.in_rows % 4 == 0 &&
                                sw.q_off % 4 == 0)      // (16-byte loads of the query rows)
                                launch_lay_attn_talk_mfma(a, sw.talk, nseg, max_n, s);
                            else
                                launch_lay_attn_talk(a, sw.talk, nseg, max_n, kv_mode, s);
                        } else if (sd.mixer == LMIX_SSM) {
                            const int N = sd.state, C = H * e + 2 * sd.groups * N;
                            LConvArgs c;
                            c.src = L.P; c.lds = w.in_rows; c.off = sw.x_off; c.C = C; c.dst = L.XB; c.ldd = C; c.cw = sw.conv_w; c.cb = sw.conv_b;
                            c.taps = sd.conv; c.act = LACT_SILU; c.conv_pool = conv_pool; c.slot_stride = conv_slot_elems; c.cv_off = sw.cv_off;
                            c.segs = d_segs; c.rowseg = d_rowseg;
                            c.H = H; c.dt_off = sw.dt_off; c.dt_bias = sw.dt_bias; c.a_neg = sw.a_neg; c.ldec = L.LD; c.kmul = L.KM;
                            c.tail_too = all_decode;
                            launch_lay_conv_act(c, T, s);
                            if (!all_decode) launch_lay_conv_tail(c, nseg, s);
                            LLightArgs a;
                            a.proj = L.XB; a.ldp = C; a.q_off = sw.q_off; a.k_off = sw.k_off; a.v_off = sw.v_off;
                            a.out = L.O2; a.ldo = H * e;
                            a.state_pool = state_pool; a.slot_stride = state_slot_elems; a.st_off = sw.st_off;
                            a.segs = d_segs; a.nseg = nseg; a.decay = nullptr; a.H = H; a.d = N; a.e = e; a.all_single = all_decode;
                            a.ldec = L.LD; a.ldd = H; a.head_decay = true; a.kmul = L.KM; a.qk_rep = H / sd.groups;
                            linear_chunks(a);
                            launch_lay_lightning(a, s);
                            launch_lay_ssm_out(L.O2, L.XB, C, 0, L.P, w.in_rows, sw.z_off, sw.skip, sw.mix_norm, L.O + sw.o_col, on, T, H, e,
                                               sd.norm_groups, cfg.eps, sd.side_scale, s);
                        } else throw CmError(CM_ERR_UNSUPPORTED, "side mixer kind");
                    }
                }
                LGemmArgs go;
                go.A = oa; go.lda = on; go.W = w.o_w; go.C = L.Y; go.ldc = W; go.M = T; go.N = W; go.K = on;
                lay_gemm(*this, L, go, 1, s);
                padd.y = L.Y; padd.nsum = 1;
                if (sp.mlp == LMLP_MOE) {
                    add_gnorm(w.norm2, L.Hc);
                    // an expert's weight multiplies its INPUT: the rows of the grouped product are w h, and the combine is a plain sum
                    const int slots = sp.top + (sp.shared_ff > 0 ? 1 : 0);
                    launch_lay_router(L.Hc, w.router, L.sel, L.wsel, T, W, sp.experts, sp.top, s, &sp.router, nullptr, slots, L.Z);
                    launch_lay_moe_plan(L.sel, L.off, L.srt, T * sp.top, sp.experts, s, sp.top, slots);
                    LGemmArgs gu;
                    gu.A = L.Hc; gu.lda = W; gu.a_idx = L.srt; gu.a_div = slots; gu.a_scale = sp.scale_input ? L.wsel : nullptr;
                    gu.W = w.gate; gu.W2 = w.up; gu.w_stride = (size_t)sp.ff * W;
                    gu.C = L.HH; gu.ldc = sp.ff; gu.M = T; gu.N = sp.ff; gu.K = W; gu.grp_off = L.off; gu.act = sp.expert_act; gu.act_param = sp.limit;
                    lay_gemm(*this, L, gu, sp.experts, s);
                    LGemmArgs dn;
                    dn.A = L.HH; dn.lda = sp.ff; dn.W = w.down; dn.w_stride = (size_t)W * sp.ff;
                    dn.C = L.YS; dn.ldc = W; dn.c_idx = L.srt; dn.M = T; dn.N = W; dn.K = sp.ff; dn.grp_off = L.off;
                    lay_gemm(*this, L, dn, sp.experts, s);
                    if (sp.shared_ff > 0) {        // the expert every token uses: row `top` of the token's rows
                        LGemmArgs su;
                        su.A = L.Hc; su.lda = W; su.W = w.sh_gate; su.W2 = w.sh_up; su.C = L.HS; su.ldc = sp.shared_ff; su.M = T; su.N = sp.shared_ff;
                        su.K = W; su.act = sp.expert_act; su.act_param = sp.shared_limit;
                        lay_gemm(*this, L, su, 1, s);
                        LGemmArgs sdn;
                        sdn.A = L.HS; sdn.lda = sp.shared_ff; sdn.W = w.sh_down; sdn.C = L.YS + (size_t)sp.top * W; sdn.ldc = slots * W; sdn.M = T;
                        sdn.N = W; sdn.K = sp.shared_ff;
                        lay_gemm(*this, L, sdn, 1, s);
                    }
                    padd.y = L.YS; padd.nsum = slots;
                }
                if (L.capture || li + 1 == L.spec.size()) add_gnorm(nullptr, nullptr);
            } else if (L.post_only) {
                // ---- the sublayers read the residual itself; x += g * unit(sublayer(x)).  All mixers of the layer share one input
                // projection and one output projection (their heads side by side in its input, each times its scale)
                flush_post();
                LGemmArgs g;
                g.A = L.X; g.lda = W; g.W = w.in_w; g.bias = w.in_b; g.C = L.P; g.ldc = w.in_rows; g.M = T; g.N = w.in_rows; g.K = W;
                g.act_split = w.g_off; g.act = LACT_NONE; g.act2 = LACT_SIGMOID;
                lay_gemm(*this, L, g, 1, s);
                int ocols = 0;
                for (const LayerSpec& sd : sp.side) ocols += sd.heads * sd.vdim;
                for (size_t k = 0; k < sp.side.size(); ++k) {
                    const LayerSpec& sd = sp.side[k];
                    const LayeredLayerW& sw = w.side[k];
                    const int H = sd.heads, G = sd.kv_heads, d = sd.dim, e = sd.vdim;
                    if (sd.mixer == LMIX_ATTN) {
                        if (L.fused_prep) {
                            launch_lay_qk_prep(L.P, w.in_rows, sw.q_off, sw.k_off, sw.v_off, H, G, d, e, sd.qk_norm ? sw.q_norm : nullptr,
                                               sd.qk_norm ? sw.k_norm : nullptr, cfg.eps, sd.rot.dims, sd.rot.half, sd.rot.dims > 0 ? sw.rot_freq : nullptr,
                                               sw.rot_mag, kv_pool + sw.k_pool_off, kv_pool + sw.v_pool_off, kv_mode, d_bt, d_segs, d_rowseg, T, page, s,
                                               all_decode ? (int)sd.pool : 0, sw.pool_rows, all_decode && sd.pool > 0 ? kv_pool + sw.pk_pool_off : nullptr,
                                               all_decode && sd.pool > 0 ? kv_pool + sw.pv_pool_off : nullptr);
                        } else {               // the same from the single operations
                            if (sd.qk_norm) {
                                launch_lay_rms_cols(L.P, w.in_rows, sw.q_off, H * d, sw.q_norm, L.P + sw.q_off, w.in_rows, T, cfg.eps, s);
                                launch_lay_rms_cols(L.P, w.in_rows, sw.k_off, G * d, sw.k_norm, L.P + sw.k_off, w.in_rows, T, cfg.eps, s);
                            }
                            if (sd.rot.dims > 0) {
                                launch_lay_rope(L.P + sw.q_off, w.in_rows, d, L.P + sw.q_off, w.in_rows, d, H, d, sd.rot.dims, sw.rot_freq, sw.rot_mag,
                                                d_segs, d_rowseg, T, s, sd.rot.half);
                                launch_lay_rope(L.P + sw.k_off, w.in_rows, d, L.P + sw.k_off, w.in_rows, d, G, d, sd.rot.dims, sw.rot_freq, sw.rot_mag,
                                                d_segs, d_rowseg, T, s, sd.rot.half);
                            }
                            launch_lay_k_append(L.P, w.in_rows, sw.k_off, kv_pool + sw.k_pool_off, kv_mode, d_bt, d_segs, d_rowseg, T, G, d, page, s);
                            launch_lay_k_append(L.P, w.in_rows, sw.v_off, kv_pool + sw.v_pool_off, kv_mode, d_bt, d_segs, d_rowseg, T, G, e, page, s);
                        }
                        if (sd.pool > 0 && !(L.fused_prep && all_decode))
                            launch_lay_pool_append(kv_pool + sw.k_pool_off, kv_pool + sw.pk_pool_off, d, kv_pool + sw.v_pool_off, kv_pool + sw.pv_pool_off, e,
                                                   kv_mode, d_bt, d_segs, d_rowseg, T, G, page, (int)sd.pool, sw.pool_rows, s);
                        run_attention(sd, sw, L.P, w.in_rows, sw.q_off, 0, d, e, L.O + sw.o_col, ocols, sd.side_scale);
                    } else if (sd.mixer == LMIX_MEMORY) {
                        launch_lay_memory_gates(L.P, w.in_rows, sw.i_off, sw.f_off, sd.gate_cap, L.LD, L.KM, L.MR, state_pool, state_slot_elems,
                                                sw.st_off + (size_t)H * d * (e + 1), d_segs, nseg, H, s);
                        run_linear(sd, sw, L.LD, w.in_rows, L.KM);
                        launch_lay_memory_out(L.O2, L.MR, L.P + sw.g_off, w.in_rows, sw.mix_norm, L.O + sw.o_col, ocols, T, H, e, cfg.eps,
                                              sd.side_scale, s);
                    } else throw CmError(CM_ERR_UNSUPPORTED, "side mixer kind");
                }
                LGemmArgs go;
                go.A = L.O; go.lda = ocols; go.W = w.o_w; go.C = L.Y; go.ldc = W; go.M = T; go.N = W; go.K = ocols;
                lay_gemm(*this, L, go, 1, s);
                post_norm(L.Y, w.norm1b, nullptr, 0);
                if (sp.mlp == LMLP_DENSE) {
                    flush_post();
                    LGemmArgs gu;
                    gu.A = L.X; gu.lda = W; gu.W = w.gate; gu.W2 = w.up; gu.C = L.HH; gu.ldc = sp.ff; gu.M = T; gu.N = sp.ff; gu.K = W;
                    gu.act = sp.ff_act;
                    lay_gemm(*this, L, gu, 1, s);
                    LGemmArgs dn;
                    dn.A = L.HH; dn.lda = sp.ff; dn.W = w.down; dn.C = L.Y; dn.ldc = W; dn.M = T; dn.N = W; dn.K = sp.ff;
                    lay_gemm(*this, L, dn, 1, s);
                    post_norm(L.Y, w.norm2b, nullptr, 0);
                } else if (sp.mlp == LMLP_MOE) {
                    flush_post();
                    const int outs = sp.experts + sp.router.identity, slots = sp.top + (sp.shared_ff > 0 ? 1 : 0);
                    launch_lay_router(L.X, w.router, L.sel, L.wsel, T, W, outs, sp.top, s, &sp.router, w.correction, slots, L.Z);
                    launch_lay_moe_plan(L.sel, L.off, L.srt, T * sp.top, outs, s, sp.top, slots);
                    LGemmArgs gu;
                    gu.A = L.X; gu.lda = W; gu.a_idx = L.srt; gu.a_div = slots;
                    gu.W = w.gate; gu.W2 = w.up; gu.w_stride = (size_t)sp.ff * W;
                    gu.C = L.HH; gu.ldc = sp.ff; gu.M = T; gu.N = sp.ff; gu.K = W; gu.grp_off = L.off; gu.act = LACT_SILU;
                    lay_gemm(*this, L, gu, sp.experts, s);
                    LGemmArgs dn;
                    dn.A = L.HH; dn.lda = sp.ff; dn.W = w.down; dn.w_stride = (size_t)W * sp.ff;
                    dn.C = L.YS; dn.ldc = W; dn.c_idx = L.srt; dn.M = T; dn.N = W; dn.K = sp.ff; dn.grp_off = L.off;
                    lay_gemm(*this, L, dn, sp.experts, s);
                    if (sp.shared_ff > 0) {        // the expert every token uses: row `top` of the token's rows, weight 1
                        LGemmArgs su;
                        su.A = L.X; su.lda = W; su.W = w.sh_gate; su.W2 = w.sh_up; su.C = L.HS; su.ldc = sp.shared_ff; su.M = T; su.N = sp.shared_ff;
                        su.K = W; su.act = LACT_SILU;
                        lay_gemm(*this, L, su, 1, s);
                        LGemmArgs sdn;
                        sdn.A = L.HS; sdn.lda = sp.shared_ff; sdn.W = w.sh_down; sdn.C = L.YS + (size_t)sp.top * W; sdn.ldc = slots * W; sdn.M = T;
                        sdn.N = W; sdn.K = sp.shared_ff;
                        lay_gemm(*this, L, sdn, 1, s);
                    }
                    post_norm(L.YS, w.norm2b, L.wsel, slots);
                    if (sp.router.identity > 0) { pend.sel_top = sp.top; pend.n_real = sp.experts; }      // identity rows are taken in the combine
                }
            } else {
            norm_canon(w.norm1, w.canon1, w.c1_off);
            LGemmArgs g;
            g.A = L.Hc; g.lda = W; g.W = w.in_w; g.bias = w.in_b; g.C = L.P; g.ldc = w.in_rows; g.M = T; g.N = w.in_rows; g.K = W;
            g.act_split = w.g_off; g.act2 = LACT_SIGMOID;
            g.act = sp.mixer == LMIX_ATTN ? LACT_NONE : LACT_SILU;
            lay_gemm(*this, L, g, 1, s);
            int on = 0;
            const float* oa = nullptr;
            if (sp.mixer == LMIX_ATTN) {
                launch_lay_k_append(L.P, w.in_rows, w.k_off, kv_pool + w.k_pool_off, kv_mode, d_bt, d_segs, d_rowseg, T, sp.kv_heads, sp.dim, page, s);
                run_attention(sp, w, L.P, w.in_rows, w.q_off, w.g_off, sp.dim, sp.dim);
                on = sp.heads * sp.dim; oa = L.O;
            } else {
                run_linear(sp, w, nullptr, w.in_rows);
                on = sp.heads * sp.vdim;
                launch_lay_rms_gate(L.O, L.P + w.g_off, w.in_rows, w.mix_norm, L.O2, T, on, cfg.eps, s);
                oa = L.O2;
            }
            LGemmArgs go;
            go.A = oa; go.lda = on; go.W = w.o_w; go.C = L.Y; go.ldc = W; go.M = T; go.N = W; go.K = on;
            lay_gemm(*this, L, go, 1, s);
            post_norm(L.Y, w.norm1b, nullptr, 0);
            if (sp.mlp != LMLP_NONE) {
                norm_canon(w.norm2, w.canon2, w.c2_off);
                if (sp.mlp == LMLP_DENSE) {
                    LGemmArgs gu;
                    gu.A = L.Hc; gu.lda = W; gu.W = w.gate; gu.W2 = w.up; gu.C = L.HH; gu.ldc = sp.ff; gu.M = T; gu.N = sp.ff; gu.K = W;
                    gu.act = LACT_GELU_TANH;
                    lay_gemm(*this, L, gu, 1, s);
                    LGemmArgs dn;
                    dn.A = L.HH; dn.lda = sp.ff; dn.W = w.down; dn.C = L.Y; dn.ldc = W; dn.M = T; dn.N = W; dn.K = sp.ff;
                    lay_gemm(*this, L, dn, 1, s);
                    post_norm(L.Y, w.norm2b, nullptr, 0);
                } else {
                    launch_lay_router(L.Hc, w.router, L.sel, L.wsel, T, W, sp.experts, sp.top, s, nullptr, nullptr, 0, L.Z);
                    launch_lay_moe_plan(L.sel, L.off, L.srt, T * sp.top, sp.experts, s);
                    LGemmArgs gu;
                    gu.A = L.Hc; gu.lda = W; gu.a_idx = L.srt; gu.a_div = sp.top;
                    gu.W = w.gate; gu.W2 = w.up; gu.w_stride = (size_t)sp.ff * W;
                    gu.C = L.HH; gu.ldc = sp.ff; gu.M = T; gu.N = sp.ff; gu.K = W; gu.grp_off = L.off; gu.act = LACT_SILU;
                    lay_gemm(*this, L, gu, sp.experts, s);
                    LGemmArgs dn;
                    dn.A = L.HH; dn.lda = sp.ff; dn.W = w.down; dn.w_stride = (size_t)W * sp.ff;
                    dn.C = L.YS; dn.ldc = W; dn.c_idx = L.srt; dn.M = T; dn.N = W; dn.K = sp.ff; dn.grp_off = L.off;
                    lay_gemm(*this, L, dn, sp.experts, s);
                    post_norm(L.YS, w.norm2b, L.wsel, sp.top);
                }
            }
            }
            if (L.capture || li + 1 == L.spec.size()) flush_post();
            if (L.capture) {
                const size_t at = L.captured.size();
                L.captured.resize(at + (size_t)T * W);
                CM_HIP(hipMemcpyAsync(L.captured.data() + at, L.X, (size_t)T * W * sizeof(float), hipMemcpyDeviceToHost, s));
                CM_HIP(hipStreamSynchronize(s));
            }
        }
        // ---- final norm + head over the wanted rows, LOGIT_ROWS at a time
        for (int w0 = 0; w0 < nw; w0 += Layered::LOGIT_ROWS) {
            const int nr = std::min(Layered::LOGIT_ROWS, nw - w0);
            if (L.pre_norm) launch_lay_add_gnorm(L.X, d_wrows + w0, nullptr, 0, L.final_norm, L.Xw, nr, W, L.norm_groups, cfg.eps, s);
            else launch_lay_rms_rows(L.X, d_wrows + w0, L.final_norm, L.Xw, nr, W, cfg.eps, s);
            LGemmArgs hd;
            hd.A = L.Xw; hd.lda = W; hd.W = L.head; hd.C = logitsb; hd.ldc = V; hd.M = nr; hd.N = V; hd.K = W;
            lay_gemm(*this, L, hd, 1, s);
            if (greedy_out) {
                launch_lay_argmax_rows(logitsb, V, V, L.d_greedy, nr, L.am_pv, L.am_pi, s);
                CM_HIP(hipMemcpyAsync(L.h_greedy, L.d_greedy, (size_t)nr * sizeof(uint32_t), hipMemcpyDeviceToHost, s));
            }
            if (logits_out) CM_HIP(hipMemcpyAsync(L.h_rows, logitsb, (size_t)nr * V * sizeof(float), hipMemcpyDeviceToHost, s));
            if (greedy_out || logits_out || w0 + nr < nw) CM_HIP(hipStreamSynchronize(s));
            if (greedy_out) memcpy(greedy_out + out_row, L.h_greedy, (size_t)nr * sizeof(uint32_t));
            if (logits_out) memcpy(logits_out + out_row * (size_t)V, L.h_rows, (size_t)nr * V * sizeof(float));
            out_row += (size_t)nr;
        }
    }
    logits_gathered = true;
    CM_HIP(hipStreamSynchronize(s));
}

// the entry points of the other families, for this one
void Model::layered_forward(int sq, const uint32_t* ids, size_t n, size_t start_pos, float* logits_out, uint32_t* greedy_out) {
    Seq& q = seq(sq);
    if ((int64_t)start_pos > q.len) throw CmError(CM_ERR_RANGE, "start_pos beyond cached length");
    if ((int64_t)start_pos < q.len) seq_truncate(sq, start_pos);     // only to 0: the recurrent state cannot be rewound
    StepItem it{sq, ids, n, nullptr, -1};
    uint32_t g = 0;
    step_batch(&it, 1, logits_out, &g);
    if (greedy_out) *greedy_out = g;
    // the last row's logits are also what cm_sample / cm_read_logits look at
    CM_HIP(hipMemcpyAsync(logits, logitsb, (size_t)cfg.V * sizeof(float), hipMemcpyDeviceToDevice, stream));
    CM_HIP(hipStreamSynchronize(stream));
}

uint64_t Model::layered_decode_bytes(size_t ctx) const {
    const Layered& L = *lay;
    const uint64_t W = (uint64_t)cfg.H;
    uint64_t b = 2ull * (uint64_t)cfg.V * W + 2ull * W;       // head + one embedding row
    // cached rows or state that one decode token of a mixer reads (and writes), and its own matrices besides the input projection
    auto mixer_bytes = [&](const LayerSpec& sp) {
        uint64_t n = 0;
        if (sp.mixer == LMIX_ATTN || sp.mixer == LMIX_LATENT) {
            const uint64_t H = (uint64_t)sp.heads;
            uint64_t row = (uint64_t)sp.kv_heads * sp.dim + (sp.own_v ? (uint64_t)sp.kv_heads * sp.vdim : 0);      // cached elements per token
            if (sp.mixer == LMIX_LATENT) {
                row = (uint64_t)sp.kv_rank + sp.rot_dim;
                n += 2ull * (H * (sp.dim + sp.rot_dim) * sp.q_rank + H * sp.dim * sp.kv_rank + H * sp.vdim * sp.kv_rank);
            }
            n += 2ull * W * H * sp.vdim;
            uint64_t seen = std::min<uint64_t>(ctx, (uint64_t)std::min<long long>(sp.win, 1ll << 40) + (uint64_t)sp.keep);
            if (sp.chunk > 0) seen = std::min<uint64_t>(seen, (uint64_t)sp.chunk);
            if (sp.pool > 0 && ctx > seen) seen += (ctx - seen) / (uint64_t)sp.pool;       // one mean row per block in front of the window
            n += seen * row * kv_esize;
        } else if (sp.mixer == LMIX_MEMORY) {
            n += 2ull * W * sp.heads * sp.vdim + 8ull * sp.heads * sp.dim * (sp.vdim + 1);
        } else {
            n += 2ull * W * sp.heads * sp.vdim + 8ull * sp.heads * sp.dim * sp.vdim;    // state read + write
            if (sp.mixer == LMIX_GLA) n += 2ull * sp.heads * sp.dim * sp.a_rank;
        }
        return n;
    };
    for (size_t i = 0; i < L.spec.size(); ++i) {
        const LayerSpec& sp = L.spec[i];
        b += 2ull * (uint64_t)L.w[i].in_rows * W;
        if (sp.mixer == LMIX_SIDE) { for (const LayerSpec& sd : sp.side) b += mixer_bytes(sd); }
        else b += mixer_bytes(sp);
        if (sp.mlp == LMLP_DENSE) b += (sp.gated_ff ? 6ull : 4ull) * W * sp.ff;
        else if (sp.mlp == LMLP_MOE) {
            const uint64_t real = (uint64_t)std::min(sp.top, sp.experts);
            b += 6ull * W * sp.ff * real + 2ull * W * (sp.experts + sp.router.identity) + 6ull * W * sp.shared_ff;
        }
    }
    return b;
}

}  // namespace cm
