// Layer-list decoders: a model whose config.json spells out every layer (mixer kind + sizes, feed-forward kind + sizes) instead
// of a family-wide geometry.  Members:
//   Korupel -- sandwich RMS norms with a scaled residual, a short causal convolution in front of every sublayer, softmax attention
//     over a sliding window with kept first tokens / a logarithmic distance penalty / values that are the keys / one sigmoid gate
//     per head, lightning (decayed linear) attention, dense GELU or sigmoid-routed mixture-of-experts feed-forwards;
//   Mononex -- mixer and feed-forward in parallel on two norms of the same residual (weights stored around zero), a token shift in
//     front of the mixer (the two-tap case of the short convolution), softmax attention inside position chunks with a linear
//     distance bias / a sink term in the denominator / an element-wise sigmoid gate / keys and values borrowed from an earlier
//     layer, latent attention (low-rank queries, one cached latent + one rotated key part per token, YaRN-scaled rotation), gated
//     linear attention with a data-dependent decay per key channel, dense squared-ReLU feed-forwards;
//   Gibipel -- no norm in front of a sublayer, a one-number RMS norm on its output (x += g * unit(sublayer(x))); two mixers side by
//     side on the same input, their outputs scaled and summed: softmax attention over a sliding window plus one mean key / mean
//     value per block of positions that lies wholly in front of the window (query / key RMS norm over all heads at once,
//     half-split rotation with banded frequency stretching, sink), and a matrix memory with exponential input / forget gates
//     (running-maximum stabiliser, normaliser vector); mixture-of-experts feed-forwards with a softmax router (choice by score +
//     correction inside the best groups of neighbours, identity experts, a shared expert).
//   Nevotar -- pre-norm layers (x += mixer(norm1 x), x += ff(norm2 x)) whose RMS norms work on equal consecutive parts of the
//     vector; a layer may run on an earlier layer's tensors with a cache and state of its own; the logits come from the embedding
//     table.  Mixers: differential attention (two causal softmax maps per head over the same values, the second taken off the first
//     times a learned number, unit RMS per head; the query grows with the logarithm of its position), a gated linear recurrence
//     whose forget gate also sets what is written (lower-bounded gates), and two mixers side by side: sliding-window attention with
//     per-head query / key norm, partial half-split rotation and the heads' scores mixed by a matrix before the softmax, next to a
//     state-space mixer (short causal convolution with bias and SiLU, one decay per head and token from a softplus step size, keys
//     and queries shared by groups of heads, skip term, gate before a grouped norm).  Mixture-of-experts feed-forwards whose expert
//     weight multiplies the expert's INPUT, with a capped gated activation, plus a shared expert.
// The mechanisms are kernels with their constants as arguments (kernels_layered.hip); the per-layer plumbing and the step function
// over mixed batches (prompt portions beside single decode tokens) are in model_layered.cpp.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>
#include <vector>

namespace cm {

// LMIX_SIDE: the mixers in LayerSpec::side run side by side on the layer's input; LMIX_MEMORY: matrix memory with exponential gates
// LMIX_HGRN: gated linear recurrence with k = 1 - forget gate; LMIX_SSM: state-space mixer (one decay per head and token)
enum { LMIX_ATTN = 0, LMIX_LIGHTNING = 1, LMIX_LATENT = 2, LMIX_GLA = 3, LMIX_MEMORY = 4, LMIX_SIDE = 5, LMIX_HGRN = 6, LMIX_SSM = 7 };
enum { LMLP_NONE = 0, LMLP_DENSE = 1, LMLP_MOE = 2 };
// LACT_RELU2: max(v, 0)^2;  LACT_LOGSIG: act_param * ln(sigmoid(v)) (the logarithm of a decay sigmoid(v)^act_param)
// LACT_CAPGLU (two-matrix products only): g = min(g, cap), u = clamp(u, -cap, cap): g sigmoid(1.702 g) (u + 1), cap = act_param
enum { LACT_NONE = 0, LACT_SILU = 1, LACT_SIGMOID = 2, LACT_GELU_TANH = 3, LACT_RELU2 = 4, LACT_LOGSIG = 5, LACT_CAPGLU = 6 };
// distance term taken off an attention score: none | r1 ln(1 + r2 (i - j)) | r1 (i - j)
enum { LBIAS_NONE = 0, LBIAS_LOG = 1, LBIAS_LINEAR = 2 };
// gate on the attention output: none | one value per head at g_off + head | one per element at g_off + head e + i
enum { LGATE_NONE = 0, LGATE_HEAD = 1, LGATE_ELEM = 2 };

// rotation of pairs of the first `dims` elements of a vector by the angle position * freq[i]: consecutive pairs (2i, 2i + 1), or
// (half) element i with element i + dims / 2
struct RotSpec {
    int dims = 0;
    double base = 10000.0;
    bool yarn = false;
    double factor = 1.0, original = 0.0, fast = 32.0, slow = 1.0;
    bool half = false;
    // banded stretching: wavelengths above original / low are stretched by factor, those below original / high are kept, the band
    // between blends the two frequencies linearly in original / wavelength
    bool banded = false;
    double low = 1.0, high = 4.0;
};
// how a router turns its logits into choices and weights
struct RouterSpec {
    bool softmax = false;              // scores: softmax over all outputs (false: sigmoid of each)
    bool correction = false;           // a learned vector joins the scores for the choice only
    int groups = 1, keep_groups = 1;   // outputs form `groups` equal groups of neighbours; only the keep_groups best (by their largest choice score) can be chosen
    bool normalise = false;            // weights divided by their sum
    int identity = 0;                  // the last `identity` outputs pass the input through (no matrices)
};

// one entry of config "layers"
struct LayerSpec {
    int mixer = LMIX_ATTN;
    int heads = 0, kv_heads = 0, dim = 0, vdim = 0;
    float scale = 1.f;                 // attention: score multiplier
    long long win = 0, keep = 0;       // attention: window size, kept first tokens
    std::vector<float> decay;          // lightning: per head
    long long chunk = 0;               // attention: positions see each other only inside the same block of `chunk` positions (0: off)
    int bias = LBIAS_NONE, gate = LGATE_NONE;
    bool sink = false, own_v = false;  // attention: learned sink per head in the softmax denominator; value projection of its own
    int kv_from = -1;                  // attention: keys and values of that earlier layer's cache instead of own projections
    int q_rank = 0, kv_rank = 0, rot_dim = 0;   // latent attention
    RotSpec rot;
    float tau = 1.f;                   // gated linear attention: decay = sigmoid(z)^(1 / tau)
    int a_rank = 0;                    // ... inner size of the decay's low-rank projection (from the checkpoint)
    int mlp = LMLP_NONE, ff = 0, experts = 0, top = 0;
    bool gated_ff = true;              // dense: act(gate) * up (false: act(up) alone)
    int ff_act = LACT_GELU_TANH;
    long long pool = 0;                // attention: blocks of `pool` positions wholly in front of the window are seen through their mean key / value
    bool qk_norm = false, qkv_bias = false;   // attention: RMS norm of all query (key) heads at once; biases on q, k, v
    float gate_cap = 0.f;              // matrix memory: gate pre-activations pass cap * tanh(z / cap)
    RouterSpec router;
    int shared_ff = 0;                 // mixture of experts: inner size of the expert every token uses (0: none)
    std::vector<LayerSpec> side;       // LMIX_SIDE: the mixers, each scaled by its side_scale
    float side_scale = 1.f;
    // attention: `maps` softmax maps per head over the same values (q and k hold maps * dim elements per head, map by map); two maps
    // are combined as unit_rms(a1 - lambda a2) (1 - diff)
    int maps = 1; float diff = 0.f;
    float qt_coef = 0.f; long long qt_every = 0;   // attention: q times 1 + qt_coef ln(floor((p + 1) / qt_every) + 1) at position p (0: off)
    bool talk = false;                 // attention: the heads' scores are mixed by a matrix [H][H] before mask and softmax
    bool head_norm = false;            // attention: RMS norm of every query (key) head by itself, one weight vector [dim] for all heads
    // state-space mixer: state size per head, groups of heads that share keys (B) and queries (C), convolution taps, parts of the output norm
    int state = 0, groups = 1, conv = 0, norm_groups = 1;
    bool scale_input = false;          // mixture of experts: the expert's weight multiplies its input (false: its output)
    int expert_act = LACT_SILU; float limit = 0.f, shared_limit = 0.f;    // experts: activation of the gated product and its cap
    int weights_of = -1;               // the layer runs on that earlier layer's tensors, with a cache and state of its own
};

// device-side weights of one layer (bf16 matrices [out, in], f32 vectors)
struct LayeredLayerW {
    float *norm1 = nullptr, *norm1b = nullptr, *norm2 = nullptr, *norm2b = nullptr;
    float *canon1 = nullptr, *canon2 = nullptr;      // [W][taps]
    // mixer input projection, rows concatenated so that one GEMM produces them:
    //   attention: q (H d) | k (G d) | g (H);  lightning: q (H d) | k (H d) | v (H e) | g (H e)
    uint16_t* in_w = nullptr;
    //   chunk attention: q (H d) | k (G d) | v (G e) | g (H e) (k, v absent when borrowed);  latent: dq (q_rank) | dkv (kv_rank + rot) | g (H e)
    //   gated linear attention: q (H d) | k (H d) | v (H e) | a1 (rank) | g (H e)
    float* in_b = nullptr;                           // [rows] (zeros where the checkpoint has no bias) or null
    int in_rows = 0, q_off = 0, k_off = 0, v_off = 0, g_off = 0, a_off = 0;
    float* shift = nullptr;                          // token shift as a two-tap convolution: [W][2] = {s, -s}
    float *sink = nullptr;                           // attention: [H]
    float *dq_norm = nullptr, *dkv_norm = nullptr;   // latent attention: plain norm weights of the two latents
    uint16_t *uq = nullptr, *uk_t = nullptr, *uv = nullptr;   // [H (d + rot)][q_rank]; per head [kv_rank][d] (transposed); [H e][kv_rank]
    float* rot_freq = nullptr; float rot_mag = 1.f;  // [rot.dims / 2] angle per position; factor on cos and sin
    uint16_t* a2 = nullptr; float* a2_b = nullptr;   // gated linear attention: [H d][rank], [H d]
    size_t v_pool_off = 0, v_page_bytes = 0;         // value pages (layers whose values are not their keys)
    size_t sh_off = 0;                               // the shift's previous input inside a slot of the conv pool (floats)
    uint16_t* o_w = nullptr;                         // [W][H e]
    float *r1 = nullptr, *r2 = nullptr;              // attention: per-head distance penalty
    float* decay = nullptr;                          // lightning: per head
    float* mix_norm = nullptr;                       // lightning: [H e]
    uint16_t *gate = nullptr, *up = nullptr, *down = nullptr;   // dense: [ff][W], [ff][W], [W][ff]; experts: [E] of each, back to back
    uint16_t* router = nullptr;                      // [E][W]
    int kv_idx = -1;                                 // index among the attention layers
    size_t k_pool_off = 0, k_page_bytes = 0;         // this layer's key pages inside the pool
    size_t st_off = 0;                               // lightning state offset inside a slot of the state pool (floats)
    size_t c1_off = 0, c2_off = 0;                   // convolution tails inside a slot of the conv pool (floats)
    float *q_norm = nullptr, *k_norm = nullptr;      // attention: [H d], [G d] weights of the norm over all heads
    size_t pk_pool_off = 0, pv_pool_off = 0, pk_page_bytes = 0, pv_page_bytes = 0;   // mean key / value rows of the position blocks
    int pool_rows = 0;                               // ... rows per page: the blocks whose last position lies in the page
    int i_off = 0, f_off = 0;                        // matrix memory: gate pre-activations inside the projection row
    float* correction = nullptr;                     // router: [outputs]
    uint16_t *sh_gate = nullptr, *sh_up = nullptr, *sh_down = nullptr;   // shared expert
    int o_col = 0;                                   // side mixers: first column of this mixer's heads in the joint output projection's input
    float* talk = nullptr;                           // attention: [H][H] score mixing matrix
    float lambda = 0.f;                              // two-map attention: the factor on the second map
    float* lower = nullptr;                          // gated recurrence: [H d] lower bound of the forget gate
    // state-space mixer: convolution [channels][taps] + bias, step-size bias [H], -exp(A_log) [H], skip factor [H]; columns of the
    // projection row: z_off (gate) | x_off (x | B | C: the convolution's channels) | dt_off
    float *conv_w = nullptr, *conv_b = nullptr, *dt_bias = nullptr, *a_neg = nullptr, *skip = nullptr;
    int z_off = 0, x_off = 0, dt_off = 0;
    size_t cv_off = 0;                               // the convolution's last taps - 1 inputs inside a slot of the conv pool (floats)
    std::vector<LayeredLayerW> side;
};

// rows [row0, row0 + n) of a pass are positions start_pos.. of the sequence in `slot`; its page table starts at bt_off
struct LaySegDev { int row0, n, start_pos, slot, bt_off, pad0, pad1, pad2; };

struct LGemmArgs {
    const float* A = nullptr; int lda = 0;
    const int32_t* a_idx = nullptr; int a_div = 1;   // A row of output row p: a_idx ? a_idx[p] / a_div : p
    const uint16_t* W = nullptr;                     // [N][K] bf16
    const uint16_t* W2 = nullptr;                    // second matrix: C = act(A W^T) * (A W2^T)
    size_t w_stride = 0;                             // elements between the matrices of consecutive groups
    const float* bias = nullptr;                     // [N] or null
    float* C = nullptr; int ldc = 0;
    const int32_t* c_idx = nullptr;                  // output row of p: c_idx ? c_idx[p] : p
    int M = 0, N = 0, K = 0;
    const int32_t* grp_off = nullptr;                // grouped: rows [grp_off[g], grp_off[g + 1]) use matrix g; M bounds a group's rows
    int act = LACT_NONE, act2 = LACT_NONE, act_split = 0;   // columns < act_split: act, the others act2 (W2: act on the first product)
    float act_param = 1.f;                           // LACT_LOGSIG: the factor
    // groups without grp_off (one product per head over all rows): group g reads A + g a_goff, writes C + g c_goff
    size_t a_goff = 0, c_goff = 0;
    const float* mul = nullptr; int ldm = 0;         // C[p][n] *= mul[p ldm + g c_goff + n] after the activation
    const float* a_scale = nullptr;                  // with a_idx: the A row of output row p is multiplied by a_scale[a_idx[p]] (before any rounding)
};
// bf16 = true: A rounded to bfloat16, matrix cores, f32 accumulation; false: f32 FMA throughout.  Up to 8 rows (per group): the
// streaming row kernel instead of tiles.
void launch_lgemm(const LGemmArgs& a, bool bf16, int groups, hipStream_t s);

void launch_lay_act_cols(float* C, int ldc, int M, int N, int act, int act2, int split, hipStream_t s, float param = 1.f);
void launch_lay_act_mul(const float* g, const float* u, float* out, size_t n, int act, hipStream_t s, float param = 1.f);
void launch_lay_round_rows(const float* x, int ldx, uint16_t* out, int M, int K, hipStream_t s);
void launch_lay_embed_rows(const uint16_t* emb, const uint32_t* ids, float* x, int T, int W, int V, hipStream_t s, float scale = 1.f);
void launch_lay_rms_rows(const float* x, const int32_t* rows, const float* w, float* out, int n_rows, int W, float eps, hipStream_t s);
// two norms of the same rows (one root mean square, two weights)
void launch_lay_rms_rows2(const float* x, const float* w1, const float* w2, float* out1, float* out2, int T, int W, float eps, hipStream_t s);
// RMS norm of the column range [off, off + n) of every row: dst[r ldd + c] = src[r lds + off + c] / rms * w[c] (dst may be src + off)
void launch_lay_rms_cols(const float* src, int lds, int off, int n, const float* w, float* dst, int ldd, int T, float eps, hipStream_t s);
// single-token rows only (every segment n = 1), one launch: x += y1 + y2 (when y1 is given), out1 = shift(x / rms * w1) with the
// shift's state (the previous input, in conv_pool) replaced, out2 = x / rms * w2 (when out2 is given).  cw: [W][2] = {s, -s}
void launch_lay_add_norm2_shift_decode(float* x, const float* y1, const float* y2, const float* w1, const float* w2, float eps, float* out1,
                                       float* out2, const float* cw, float* conv_pool, size_t slot_stride, size_t off, const LaySegDev* segs,
                                       int T, int W, hipStream_t s);
// x += y1 + y2 (y2 may be null)
void launch_lay_add_rows(float* x, const float* y1, const float* y2, size_t n, hipStream_t s);
// pairs (2i, 2i + 1), i < dims / 2, of `nvec` vectors per row (vector v at src + r lds + v vstride) turned by position * freq[i];
// cos and sin times mag; elements past dims are copied.  dst may be src.  half: the pairs are (i, i + dims / 2) instead.
void launch_lay_rope(const float* src, int lds, int s_vstride, float* dst, int ldd, int d_vstride, int nvec, int len, int dims,
                     const float* freq, float mag, const LaySegDev* segs, const int32_t* rowseg, int T, hipStream_t s, bool half = false);
// out = h + conv(h) over time per channel; the taps - 1 inputs before a portion come from the sequence's tail in conv_pool
void launch_lay_canon(const float* h, float* out, const float* cw, const float* conv_pool, size_t slot_stride, size_t off,
                      const LaySegDev* segs, const int32_t* rowseg, int T, int W, int taps, hipStream_t s);
void launch_lay_canon_tail(const float* h, float* conv_pool, size_t slot_stride, size_t off, const LaySegDev* segs, int nseg, int W,
                           int taps, hipStream_t s);
// single-token rows only (every segment n = 1): RMS norm, convolution and tail shift in one launch
void launch_lay_norm_canon_decode(const float* x, const float* nw, float eps, float* out, const float* cw, float* conv_pool,
                                  size_t slot_stride, size_t off, const LaySegDev* segs, int T, int W, int taps, hipStream_t s);
// single-token rows only: lay_post_norm of the finished sublayer and lay_norm_canon_decode of the next one in one launch
void launch_lay_post_norm_canon_decode(float* x, const float* y, const float* pw, float mult, const float* wsel, int top, const float* nw,
                                       float eps, float* out, const float* cw, float* conv_pool, size_t slot_stride, size_t off,
                                       const LaySegDev* segs, int T, int W, int taps, hipStream_t s);
// x += mult * RMSNorm(y) * w;  wsel != null: y[r] = sum_k wsel[r top + k] * ys[r top + k] (mixture-of-experts combine); hin given: the
// rows of choices k < sel_top with sel[r sel_top + k] >= n_real are hin[r] (identity experts)
void launch_lay_post_norm(float* x, const float* y, const float* w, float mult, float eps, int T, int W, const float* wsel, int top,
                          hipStream_t s, const int32_t* sel = nullptr, int sel_top = 0, int n_real = -1, const float* hin = nullptr);

struct LAttnArgs {
    const float* proj; int ldp, q_off, g_off;        // activated projection rows: q | k | gate
    float* out; int ldo;                             // [T][H d], gated
    const void* kpool;                               // [n_pages][G][page][d]
    const int32_t* bt; const LaySegDev* segs; const int2* tiles; int ntiles;
    const float *r1, *r2;
    int H, G, d, page;
    float scale; long long win, keep;
    long long chunk = 0;                             // > 0: only keys of the query's own block of `chunk` positions
    int bias = LBIAS_LOG, gate = LGATE_HEAD;
    const float* sink = nullptr;                     // [H]: exp(sink) joins the denominator once, with no value
    const void* vpool = nullptr; int e = 0;          // [n_pages][G][page][e]; null: the values are the first e elements of the keys
    // few query tiles, many keys (decode steps): nsplit blocks per tile share its key tiles and a merge launch follows;
    // part_o [ntiles][G][nsplit][16][d], part_ml [ntiles][G][nsplit][16][2].  nsplit <= 1 or null scratch: one block per tile
    int nsplit = 1; float* part_o = nullptr; float* part_ml = nullptr;
    // pool > 0: block b of `pool` positions is seen by position i through one mean key and one mean value when its last position
    // b pool + pool - 1 <= i - win; rows [n_pages][G][pool_rows][d] / [e] (lay_pool_append), in front of the window in the key walk
    long long pool = 0; const void* pk_pool = nullptr; const void* pv_pool = nullptr; int pool_rows = 0;
    float out_scale = 1.f;                           // factor on the output
    int v_div = 1;                                   // v_div consecutive key heads share one value head: value pages [n_pages][G / v_div][page][e]
};
void launch_lay_k_append(const float* proj, int ldp, int k_off, void* kpool, int kvt, const int32_t* bt, const LaySegDev* segs,
                         const int32_t* rowseg, int T, int G, int d, int page, hipStream_t s);
// mean key (and value) rows of the position blocks that the pass completes: block b of `pool` positions lives in the page of its
// last position, row b - (first block that ends in that page).  Reads the cached rows, so it follows lay_k_append.
// Keys [..][d] and -- vpool given -- values [..][e] in one launch.
void launch_lay_pool_append(const void* kpool, void* pk_pool, int d, const void* vpool, void* pv_pool, int e, int kvt, const int32_t* bt,
                            const LaySegDev* segs, const int32_t* rowseg, int T, int G, int page, int pool, int pool_rows, hipStream_t s);
// more of lay_qk_prep: head_norm -- every head is normed by itself with the weights qn / kn [d] (shared by the heads); Gv -- value
// heads (0: as many as key heads); qt_coef / qt_every -- the query is multiplied by 1 + qt_coef ln(floor((p + 1) / qt_every) + 1)
struct LQkPrepExtra { bool head_norm = false; int Gv = 0; float qt_coef = 0.f; int qt_every = 0; };
// queries and keys of a pass on their way into attention, one launch: RMS norm over all query heads at once and over all key heads
// at once (qn / kn: weights [H d] / [G d]; null: no norm), rotation by position (freq null: none), q back in place, keys -- and
// values, vpool given -- into the pages.  pk_pool given (only when every portion of the pass is one token): the mean rows of a block that
// the row closes, as lay_pool_append
void launch_lay_qk_prep(float* proj, int ldp, int q_off, int k_off, int v_off, int H, int G, int d, int e, const float* qn, const float* kn,
                        float eps, int dims, bool half, const float* freq, float mag, void* kpool, void* vpool, int kvt, const int32_t* bt,
                        const LaySegDev* segs, const int32_t* rowseg, int T, int page, hipStream_t s, int pool = 0, int pool_rows = 0,
                        void* pk_pool = nullptr, void* pv_pool = nullptr, const LQkPrepExtra* extra = nullptr);
inline int lay_pool_rows(int page, long long pool) { return pool >= page ? 1 : (int)((page + pool - 1) / pool); }
void launch_lay_attn(const LAttnArgs& a, int kvt, hipStream_t s);    // kvt: KV_BF16 | KV_F32
bool lay_attn_fits(int d, int e, bool own_v);                         // sizes the kernel can hold in LDS and registers
int lay_attn_key_tile(int d, int e, bool own_v);                      // keys per tile of lay_attn_kernel at these sizes (64 or 32)
// bf16 key pages, d % 16 == 0, d <= 128: the matrix-core form; a.tiles lists {segment, first query row} in steps of
// LAY_ATTN_MFMA_ROWS rows, longest key range first
constexpr int LAY_ATTN_MFMA_ROWS = 64;
void launch_lay_attn_mfma(const LAttnArgs& a, hipStream_t s);
bool lay_attn_mfma_fits(int d, int e, bool own_v);         // sizes the matrix-core form takes

struct LLightArgs {
    const float* proj; int ldp, q_off, k_off, v_off; // activated projection rows
    float* out; int ldo;                             // [T][H e] before the norm
    float* state_pool; size_t slot_stride, st_off;   // [slot] ... [H][d][e] f32
    const LaySegDev* segs; int nseg;
    const float* decay;
    int H, d, e;
    // chunk-parallel form (long portions; head size up to 128): chunk table {segment, first token}, segs[].pad0 = a segment's first
    // chunk, U = [nchunks][H][d][e] f32 scratch.  Null / 0: one block per (sequence, head, value slice) walks the portion.
    float* U = nullptr; const int2* chunks = nullptr; int nchunks = 0;
    bool all_single = false;     // every portion of the pass is one token (decode steps): the state is updated in place in HBM
    // gated form: the decay of key channel i at token t is exp(ldec[t ldd + head d + i]) instead of decay[head]
    const float* ldec = nullptr; int ldd = 0;
    float qscale = 1.f;          // q is multiplied by this
    float* D = nullptr;          // gated chunk-parallel form: [nchunks][H][d] decay of a whole chunk
    // one decay per head and token instead of one per key channel: ldec[t ldd + head] (head_decay), and a factor on the key:
    // k_t * kmul[t ldd + head].  ones_col: the last of the e value columns is the constant 1 (the projection row holds e - 1 per
    // head), so that the state's last column carries sum_s decay(s..t) k_s -- the normaliser of a matrix memory
    bool head_decay = false; const float* kmul = nullptr; bool ones_col = false;
    int qk_rep = 1;              // qk_rep consecutive heads share one query / key vector: q and k hold H / qk_rep vectors of d
};
constexpr int LAY_LIGHT_CHUNK = 32;
void launch_lay_lightning(const LLightArgs& a, hipStream_t s);
// out = o / rms(o) * w * gate (gate already activated).  The root mean square is taken over groups of `group` columns (0: the
// whole row) and group g's column c uses w[c] (weights shared by the groups) or w[g group + c] (shared_w false).
void launch_lay_rms_gate(const float* o, const float* gate, int ldg, const float* w, float* out, int T, int N, float eps, hipStream_t s,
                         int group = 0, bool shared_w = false);

// ---- kernels_layered_mix.hip ----
// x[r] += sum_(k < nsum) y[(r nsum + k) W ..] (y null: nothing is added), then out[r] = x[rows ? rows[r] : r] in `groups` equal
// consecutive parts, each over its own root mean square, times w (out null: the update alone).  rows and y exclude each other.
void launch_lay_add_gnorm(float* x, const int32_t* rows, const float* y, int nsum, const float* w, float* out, int n_rows, int W, int groups,
                          float eps, hipStream_t s);
// two-map attention: a [T][2 H e] holds the maps' outputs, key head g's heads of map m at columns ((2 g + m) nrep + j) e; out[t][h e + i] =
// unit_rms_e(a1 - lambda a2) * post
void launch_lay_diff_combine(const float* a, float* out, int T, int H, int G, int e, float lambda, float post, float eps, hipStream_t s);
// gated recurrence: z = proj[t][f_off + i] -> forget gate f = l + (1 - l) sigmoid(z); proj[t][f_off + i] <- 1 - f, ldec[t n + i] = ln f
void launch_lay_hgrn_gates(float* proj, int ldp, int f_off, const float* lower, float* ldec, int T, int n, hipStream_t s);
// causal convolution per channel with bias and activation: dst[t][c] = act(sum_j cw[c][j] src[t - taps + 1 + j][off + c] + cb[c]); inputs in
// front of a portion come from the sequence's tail in conv_pool ([taps - 1][C], oldest first).  H > 0: per head also the state-space
// step dt = softplus(src[t][dt_off + h] + dt_bias[h]) -> kmul[t H + h] = dt, ldec[t H + h] = a_neg[h] dt.  tail_too (every portion of
// the pass is one token): the thread of a channel also shifts its tail; otherwise launch_lay_conv_tail follows.
struct LConvArgs {
    const float* src; int lds, off, C; float* dst; int ldd; const float *cw, *cb; int taps, act;
    float* conv_pool; size_t slot_stride, cv_off; const LaySegDev* segs; const int32_t* rowseg;
    int H = 0, dt_off = 0; const float *dt_bias = nullptr, *a_neg = nullptr; float *ldec = nullptr, *kmul = nullptr;
    bool tail_too = false;
};
void launch_lay_conv_act(const LConvArgs& a, int T, hipStream_t s);
void launch_lay_conv_tail(const LConvArgs& a, int nseg, hipStream_t s);
// state-space output: y = (o[t][h e + i] + skip[h] x[t][x_off + h e + i]) silu(z[t][z_off + h e + i]), RMS norm in norm_groups equal
// parts, times w times out_scale -> out[t ldo + ..]
void launch_lay_ssm_out(const float* o, const float* x, int ldx, int x_off, const float* z, int ldz, int z_off, const float* skip, const float* w,
                        float* out, int ldo, int T, int H, int e, int norm_groups, float eps, float out_scale, hipStream_t s);
// softmax attention whose heads' scores are mixed before mask and softmax: score'_h = sum_g talk[h H + g] score_g.  A block owns
// some positions of one sequence with ALL heads; uses of LAttnArgs: proj / q_off, out / ldo / out_scale, kpool, vpool (needed), bt, segs,
// H, G, d, e, page, scale, win.  nseg segments, portions of up to max_n tokens; nsplit > 1 (only when max_n == 1): the keys are dealt
// to nsplit blocks and merged, part_o / part_ml hold nseg nsplit H rows.
void launch_lay_attn_talk(const LAttnArgs& a, const float* talk, int nseg, int max_n, int kvt, hipStream_t s);
bool lay_attn_talk_fits(int H, int G, int d, int e);
// bf16 key / value pages, up to 16 heads, d and e multiples of 16 up to 128: the matrix-core form for prompt passes (16 positions a block,
// one wave per head).  talk null: no mixing -- plain attention in this blocking (all heads of a position share the staged key and
// value tiles), which also takes LAttnArgs::v_div
void launch_lay_attn_talk_mfma(const LAttnArgs& a, const float* talk, int nseg, int max_n, hipStream_t s);
bool lay_attn_talk_mfma_fits(int H, int G, int d, int e, int v_div = 1, bool mixed = true);

// router: z = h . Wr^T in f32 over E outputs, scores by rs (sigmoid of each / softmax over all), the `top` largest choice scores
// (score + correction, inside the best groups; lowest index first among equals) -> sel [T top], wsel [T slots] = their scores
// (normalised when asked); slots > top: the remaining weights are 1 (rows that every token uses, e.g. a shared expert)
// zbuf [T][E] given and few rows (decode steps): the logits come from the streaming row kernel (f32 products of the unrounded rows),
// then one wave per token chooses; otherwise one block per token does both
void launch_lay_router(const float* h, const uint16_t* wr, int32_t* sel, float* wsel, int T, int W, int E, int top, hipStream_t s,
                       const RouterSpec* rs = nullptr, const float* correction = nullptr, int slots = 0, float* zbuf = nullptr);
// counting sort of the T top (token, choice) pairs by expert: off [E + 1], srt [T top] = token * slots + choice
void launch_lay_moe_plan(const int32_t* sel, int32_t* off, int32_t* srt, int n, int E, hipStream_t s, int top = 1, int slots = 1);

// matrix memory, gates: per (sequence, head) over the portion's tokens, from the pre-activations zi, zf at proj[t ldp + i_off / f_off + head]
//   li = cap tanh(zi / cap), lf = ln sigmoid(cap tanh(zf / cap)), m' = max(lf + m, li)  (m: per-sequence state at mstate, [H])
//   ldec[t H + head] = lf + m - m' (<= 0), kmul[t H + head] = exp(li - m') (<= 1), mrun[t H + head] = m'
void launch_lay_memory_gates(const float* proj, int ldp, int i_off, int f_off, float cap, float* ldec, float* kmul, float* mrun,
                             float* state_pool, size_t slot_stride, size_t m_off, const LaySegDev* segs, int nseg, int H, hipStream_t s);
// matrix memory, output: o [T][H (e + 1)] = [S^T q | n . q] -> out[t ldo + head e + c] = unit_rms_e(o_c / (max(|n . q|, exp(-m')) + 1e-6)) * w[head e + c] * gate * out_scale
void launch_lay_memory_out(const float* o, const float* mrun, const float* gate, int ldg, const float* w, float* out, int ldo, int T, int H,
                           int e, float eps, float out_scale, hipStream_t s);
constexpr int LAY_ARGMAX_PARTS = 64;
// pv / pi: [n_rows][LAY_ARGMAX_PARTS] scratch of the two-launch form for wide rows (null: one block per row)
void launch_lay_argmax_rows(const float* logits, int ld, int V, uint32_t* out, int n_rows, float* pv, int* pi, hipStream_t s);

}  // namespace cm
