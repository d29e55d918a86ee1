// More mechanisms of the layer-list decoders (layered.h), sizes and constants as arguments: RMS norm in equal parts fused with the
// residual update, the combine of a two-map (differential) attention, the gates of a recurrence whose forget gate also sets what is
// written, the short causal convolution and step sizes of a state-space mixer and its gated, grouped output norm, and softmax
// attention whose heads' scores are mixed by a matrix before mask and softmax.
// f32 in both number formats: norms, positions, scores, softmax and weighted sums, gates, logarithms of decays, step sizes.  The
// bfloat16 format only changes what the cache holds (bf16 key / value rows).
#include <hip/hip_runtime.h>

#include <algorithm>

#include "dev_common.h"
#include "layered.h"

namespace cm {

namespace {
__device__ __forceinline__ float mx_silu(float v) { return v / (1.f + expf(-v)); }
// ln(1 + e^v) without overflow
__device__ __forceinline__ float mx_softplus(float v) { return fmaxf(v, 0.f) + log1pf(expf(-fabsf(v))); }
}  // namespace

// ------------------------------------------------------------------------------------------------------------------
// residual update + RMS norm in `groups` equal consecutive parts: one block per row, one wave per part (round-robin)
// ------------------------------------------------------------------------------------------------------------------
constexpr int LGN_MAX_GROUPS = 256;
__global__ __launch_bounds__(256) void lay_add_gnorm_kernel(float* __restrict__ x, const int32_t* __restrict__ rows, const float* __restrict__ y,
                                                            int nsum, const float* __restrict__ w, float* __restrict__ out, int W, int groups,
                                                            float eps) {
    __shared__ float rs[LGN_MAX_GROUPS];
    const int r = blockIdx.x, tid = threadIdx.x;
    float* xr = x + (size_t)(rows ? rows[r] : r) * W;
    if (y) {
        for (int c = tid; c < W; c += 256) {
            float v = xr[c];
            for (int k = 0; k < nsum; ++k) v += y[((size_t)r * nsum + k) * W + c];      // fixed order: the same sum in every schedule
            xr[c] = v;
        }
        if (!out) return;
        __syncthreads();                   // the block's own writes to x are read back below
    }
    const int gw = W / groups;
    for (int g = tid >> 6; g < groups; g += 4) {
        float ss = 0.f;
        for (int c = tid & 63; c < gw; c += 64) { const float v = xr[g * gw + c]; ss += v * v; }
        ss = wave_sum(ss);
        if ((tid & 63) == 0) rs[g] = 1.f / sqrtf(ss / (float)gw + eps);
    }
    __syncthreads();
    for (int c = tid; c < W; c += 256) out[(size_t)r * W + c] = xr[c] * rs[c / gw] * w[c];
}
void launch_lay_add_gnorm(float* x, const int32_t* rows, const float* y, int nsum, const float* w, float* out, int n_rows, int W, int groups,
                          float eps, hipStream_t s) {
    if (n_rows <= 0 || (!y && !out)) return;
    if (groups <= 0 || groups > LGN_MAX_GROUPS || W % groups) groups = 1;       // the configuration reader has refused these
    hipLaunchKernelGGL(lay_add_gnorm_kernel, dim3((unsigned)n_rows), dim3(256), 0, s, x, rows, y, nsum, w, out, W, groups, eps);
}

// ------------------------------------------------------------------------------------------------------------------
// two-map attention: one wave per (row, head)
// ------------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void lay_diff_combine_kernel(const float* __restrict__ a, float* __restrict__ out, int T, int H, int G, int e,
                                                               float lambda, float post, float eps) {
    const int idx = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (idx >= T * H) return;
    const int t = idx / H, h = idx - t * H, nrep = H / G, g = h / nrep, j = h - g * nrep;
    const float* a1 = a + (size_t)t * 2 * H * e + (size_t)((2 * g) * nrep + j) * e;
    const float* a2 = a + (size_t)t * 2 * H * e + (size_t)((2 * g + 1) * nrep + j) * e;
    float ss = 0.f;
    for (int i = lane; i < e; i += 64) { const float v = a1[i] - lambda * a2[i]; ss += v * v; }
    ss = wave_sum(ss);
    const float rs = post / sqrtf(ss / (float)e + eps);
    for (int i = lane; i < e; i += 64) out[((size_t)t * H + h) * e + i] = (a1[i] - lambda * a2[i]) * rs;
}
void launch_lay_diff_combine(const float* a, float* out, int T, int H, int G, int e, float lambda, float post, float eps, hipStream_t s) {
    if (T <= 0) return;
    hipLaunchKernelGGL(lay_diff_combine_kernel, dim3((unsigned)((T * H + 3) / 4)), dim3(256), 0, s, a, out, T, H, G, e, lambda, post, eps);
}

// ------------------------------------------------------------------------------------------------------------------
// gates of the recurrence S <- diag(f) S + (1 - f) v^T: f = l + (1 - l) sigmoid(z); 1 - f = (1 - l) sigmoid(-z) keeps its digits
// ------------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void lay_hgrn_gates_kernel(float* __restrict__ proj, int ldp, int f_off, const float* __restrict__ lower,
                                                             float* __restrict__ ldec, int n) {
    const int t = blockIdx.x;
    for (int i = blockIdx.y * 256 + threadIdx.x; i < n; i += 256 * gridDim.y) {
        const float z = proj[(size_t)t * ldp + f_off + i], lo = lower[i];
        const float sg = 1.f / (1.f + expf(-z)), ng = 1.f / (1.f + expf(z));
        proj[(size_t)t * ldp + f_off + i] = (1.f - lo) * ng;
        ldec[(size_t)t * n + i] = logf(lo + (1.f - lo) * sg);
    }
}
void launch_lay_hgrn_gates(float* proj, int ldp, int f_off, const float* lower, float* ldec, int T, int n, hipStream_t s) {
    if (T <= 0 || n <= 0) return;
    hipLaunchKernelGGL(lay_hgrn_gates_kernel, dim3((unsigned)T, (unsigned)std::min(8, (n + 255) / 256)), dim3(256), 0, s, proj, ldp, f_off, lower, ldec, n);
}

// ------------------------------------------------------------------------------------------------------------------
// short causal convolution with bias and activation; the step sizes of a state-space mixer ride in the same launch
// ------------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void lay_conv_act_kernel(LConvArgs a) {
    const int r = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= a.C + a.H) return;
    if (c >= a.C) {                        // step size of head c - C
        const int h = c - a.C;
        const float dt = mx_softplus(a.src[(size_t)r * a.lds + a.dt_off + h] + a.dt_bias[h]);
        a.kmul[(size_t)r * a.H + h] = dt;
        a.ldec[(size_t)r * a.H + h] = a.a_neg[h] * dt;
        return;
    }
    const LaySegDev sg = a.segs[a.rowseg[r]];
    const int local = r - sg.row0, taps = a.taps;
    float* tail = a.conv_pool + (size_t)sg.slot * a.slot_stride + a.cv_off;
    float acc = a.cb ? a.cb[c] : 0.f;
    for (int j = 0; j < taps; ++j) {
        const int src = local - (taps - 1) + j;
        const float v = src >= 0 ? a.src[(size_t)(sg.row0 + src) * a.lds + a.off + c] : tail[(size_t)(taps - 1 + src) * a.C + c];
        acc = fmaf(a.cw[(size_t)c * taps + j], v, acc);
    }
    a.dst[(size_t)r * a.ldd + c] = a.act == LACT_SILU ? mx_silu(acc) : acc;
    if (a.tail_too) {                      // one token per sequence: this thread is the only one that touches the channel's tail
        for (int k = 0; k + 1 < taps - 1; ++k) tail[(size_t)k * a.C + c] = tail[(size_t)(k + 1) * a.C + c];
        if (taps > 1) tail[(size_t)(taps - 2) * a.C + c] = a.src[(size_t)r * a.lds + a.off + c];
    }
}
void launch_lay_conv_act(const LConvArgs& a, int T, hipStream_t s) {
    if (T <= 0) return;
    hipLaunchKernelGGL(lay_conv_act_kernel, dim3((unsigned)T, (unsigned)((a.C + a.H + 255) / 256)), dim3(256), 0, s, a);
}
// new tail = last taps - 1 entries of (old tail ++ the portion's inputs).  In place: entry k reads entry n + k > k of the old tail, and a
// thread touches its own channel only.
__global__ __launch_bounds__(256) void lay_conv_tail_kernel(LConvArgs a) {
    const LaySegDev sg = a.segs[blockIdx.x];
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= a.C) return;
    float* tail = a.conv_pool + (size_t)sg.slot * a.slot_stride + a.cv_off;
    for (int k = 0; k < a.taps - 1; ++k) {
        const int idx = sg.n + k;
        tail[(size_t)k * a.C + c] = idx < a.taps - 1 ? tail[(size_t)idx * a.C + c]
                                                      : a.src[(size_t)(sg.row0 + idx - (a.taps - 1)) * a.lds + a.off + c];
    }
}
void launch_lay_conv_tail(const LConvArgs& a, int nseg, hipStream_t s) {
    if (nseg <= 0 || a.taps <= 1) return;
    hipLaunchKernelGGL(lay_conv_tail_kernel, dim3((unsigned)nseg, (unsigned)((a.C + 255) / 256)), dim3(256), 0, s, a);
}

// ------------------------------------------------------------------------------------------------------------------
// state-space output: skip term, gate, RMS norm in parts (the gate comes BEFORE the norm), weights, scale; one block per row
// ------------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void lay_ssm_out_kernel(const float* __restrict__ o, const float* __restrict__ x, int ldx, int x_off,
                                                          const float* __restrict__ z, int ldz, int z_off, const float* __restrict__ skip,
                                                          const float* __restrict__ w, float* __restrict__ out, int ldo, int H, int e,
                                                          int norm_groups, float eps, float out_scale) {
    extern __shared__ float ys[];          // [H e] gated values, then [norm_groups] factors
    const int r = blockIdx.x, tid = threadIdx.x, n = H * e, gw = n / norm_groups;
    float* rs = ys + n;
    for (int c = tid; c < n; c += 256) {
        const float y = o[(size_t)r * n + c] + skip[c / e] * x[(size_t)r * ldx + x_off + c];
        ys[c] = y * mx_silu(z[(size_t)r * ldz + z_off + c]);
    }
    __syncthreads();
    for (int g = tid >> 6; g < norm_groups; g += 4) {
        float ss = 0.f;
        for (int c = tid & 63; c < gw; c += 64) { const float v = ys[g * gw + c]; ss += v * v; }
        ss = wave_sum(ss);
        if ((tid & 63) == 0) rs[g] = out_scale / sqrtf(ss / (float)gw + eps);
    }
    __syncthreads();
    for (int c = tid; c < n; c += 256) out[(size_t)r * ldo + c] = ys[c] * rs[c / gw] * w[c];
}
void launch_lay_ssm_out(const float* o, const float* x, int ldx, int x_off, const float* z, int ldz, int z_off, const float* skip, const float* w,
                        float* out, int ldo, int T, int H, int e, int norm_groups, float eps, float out_scale, hipStream_t s) {
    if (T <= 0) return;
    const size_t lds = (size_t)(H * e + norm_groups) * sizeof(float);
    hipLaunchKernelGGL(lay_ssm_out_kernel, dim3((unsigned)T), dim3(256), lds, s, o, x, ldx, x_off, z, ldz, z_off, skip, w, out, ldo, H, e, norm_groups,
                       eps, out_scale);
}

// ------------------------------------------------------------------------------------------------------------------
// softmax attention with mixed heads.  A block owns BQ positions of one sequence and ALL H heads: R = BQ H rows (position-major),
// row r of the tile belongs to the 16-lane group r % 16 (RPG rows per group).  Per tile of LT_KT keys: the key and value rows of
// every key head go to LDS, the raw scores (q . k) scale of all rows go to LDS, then every row mixes the H scores of its position
// and key with its line of the matrix, masks (causal, window), and runs the online softmax and the weighted sum of its value head.
// ------------------------------------------------------------------------------------------------------------------
constexpr int LT_KT = 32;
constexpr size_t LT_LDS_PLAIN = 64 * 1024, LT_LDS_MAX = 160 * 1024;
static size_t lay_talk_lds(int H, int G, int d, int e, int BQ) {
    const size_t R = (size_t)BQ * H;
    return (R * (d + 1) + (size_t)G * LT_KT * (d + 1) + (size_t)G * LT_KT * e + 2 * R * (LT_KT + 1) + (size_t)H * H) * sizeof(float);
}
template <int KVT, int RPG, int NACC>
__global__ __launch_bounds__(256) void lay_attn_talk_kernel(LAttnArgs a, const float* __restrict__ talk, int BQ) {
    extern __shared__ float lds[];
    const int d = a.d, e = a.e, H = a.H, G = a.G, nrep = H / G;
    const int ldq = d + 1, ldk = d + 1, lds_s = LT_KT + 1;
    const int R = BQ * H;
    float* qs = lds;                       // [R][d + 1]
    float* ks = qs + R * ldq;              // [G][KT][d + 1]
    float* vs = ks + G * LT_KT * ldk;      // [G][KT][e]
    float* sc = vs + G * LT_KT * e;        // [R][KT + 1] raw scores
    float* ps = sc + R * lds_s;            // [R][KT + 1] softmax weights
    float* tk = ps + R * lds_s;            // [H][H]
    const LaySegDev sg = a.segs[blockIdx.x];
    const int p0 = (int)blockIdx.y * BQ;
    if (p0 >= sg.n) return;
    const int np = min(BQ, sg.n - p0);
    const int tid = threadIdx.x, grp = tid >> 4, ln = tid & 15;
    for (int idx = tid; idx < R * d; idx += 256) {
        const int row = idx / d, i = idx - row * d, lp = row / H, h = row - lp * H;
        qs[row * ldq + i] = lp < np ? a.proj[(size_t)(sg.row0 + p0 + lp) * a.ldp + a.q_off + h * d + i] : 0.f;
    }
    for (int idx = tid; idx < H * H; idx += 256) tk[idx] = talk[idx];
    const int pmin = sg.start_pos + p0, pmax = pmin + np - 1;
    const int win = (int)min(a.win, 1ll << 30);
    const int main_lo = max(0, pmin - win + 1);
    const int total = pmax - main_lo + 1;
    float m[RPG], l[RPG], acc[RPG][NACC];
#pragma unroll
    for (int rr = 0; rr < RPG; ++rr) {
        m[rr] = -INFINITY; l[rr] = 0.f;
#pragma unroll
        for (int c = 0; c < NACC; ++c) acc[rr][c] = 0.f;
    }
    const int nsplit = (int)gridDim.z;
    constexpr int ESZ = KVT == KV_F32 ? 4 : 2;
    __syncthreads();
    for (int v0 = (int)blockIdx.z * LT_KT; v0 < total; v0 += LT_KT * nsplit) {
        __syncthreads();                   // the previous tile is fully consumed
        for (int rr = grp; rr < G * LT_KT; rr += 16) {
            const int g = rr / LT_KT, sl = rr - g * LT_KT, v = v0 + sl;
            float* kd = ks + (size_t)rr * ldk;
            float* vd = vs + (size_t)rr * e;
            if (v < total) {
                const int j = main_lo + v;
                const size_t row = ((size_t)a.bt[sg.bt_off + j / a.page] * G + g) * a.page + (size_t)(j % a.page);
                const char* ksrc = (const char*)a.kpool + row * d * ESZ;
                const char* vsrc = (const char*)a.vpool + row * e * ESZ;
                if (KVT != KV_F32 && (d & 7) == 0) {
                    for (int i = ln * 8; i < d; i += 128) {
                        const u32x4 p = *(const u32x4*)((const uint16_t*)ksrc + i);
                        kd[i] = bf16_lo(p.x); kd[i + 1] = bf16_hi(p.x); kd[i + 2] = bf16_lo(p.y); kd[i + 3] = bf16_hi(p.y);
                        kd[i + 4] = bf16_lo(p.z); kd[i + 5] = bf16_hi(p.z); kd[i + 6] = bf16_lo(p.w); kd[i + 7] = bf16_hi(p.w);
                    }
                } else
                    for (int i = ln; i < d; i += 16) kd[i] = KVT == KV_F32 ? ((const float*)ksrc)[i] : bf16_to_f32(((const uint16_t*)ksrc)[i]);
                for (int i = ln; i < e; i += 16) vd[i] = KVT == KV_F32 ? ((const float*)vsrc)[i] : bf16_to_f32(((const uint16_t*)vsrc)[i]);
            } else {
                for (int i = ln; i < d; i += 16) kd[i] = 0.f;
                for (int i = ln; i < e; i += 16) vd[i] = 0.f;
            }
        }
        __syncthreads();
#pragma unroll
        for (int rr = 0; rr < RPG; ++rr) {
            const int row = grp + 16 * rr;
            if (row < R) {
                const int h = row % H, g = h / nrep;
                const float* qrow = qs + row * ldq;
#pragma unroll
                for (int c = 0; c < LT_KT / 16; ++c) {
                    const int sl = ln + 16 * c;
                    const float* krow = ks + (size_t)(g * LT_KT + sl) * ldk;
                    float dot = 0.f;
                    for (int i = 0; i < d; ++i) dot = fmaf(qrow[i], krow[i], dot);
                    sc[row * lds_s + sl] = dot * a.scale;
                }
            }
        }
        __syncthreads();
        float corr[RPG];
#pragma unroll
        for (int rr = 0; rr < RPG; ++rr) {
            const int row = grp + 16 * rr;
            const bool rv = row < R;
            const int rw = rv ? row : 0;
            const int lp = rw / H, h = rw - lp * H, pos = pmin + lp;
            const bool qvalid = rv && lp < np;
            float s2[LT_KT / 16], tmax = -INFINITY;
#pragma unroll
            for (int c = 0; c < LT_KT / 16; ++c) {
                const int sl = ln + 16 * c, v = v0 + sl, j = main_lo + v;
                float mixed = 0.f;
                for (int g2 = 0; g2 < H; ++g2) mixed = fmaf(tk[h * H + g2], sc[(lp * H + g2) * lds_s + sl], mixed);
                const bool vis = qvalid && v < total && j <= pos && pos - j < win;
                s2[c] = vis ? mixed : -INFINITY;
                tmax = fmaxf(tmax, s2[c]);
            }
            tmax = row16_max(tmax);
            const float mn = fmaxf(m[rr], tmax);
            corr[rr] = mn == -INFINITY ? 1.f : expf(m[rr] - mn);
            float psum = 0.f;
#pragma unroll
            for (int c = 0; c < LT_KT / 16; ++c) {
                const float p = s2[c] == -INFINITY ? 0.f : expf(s2[c] - mn);
                if (rv) ps[row * lds_s + ln + 16 * c] = p;
                psum += p;
            }
            psum = row16_sum(psum);
            l[rr] = l[rr] * corr[rr] + psum;
            m[rr] = mn;
        }
        __syncthreads();
        const int kn = min(LT_KT, total - v0);
#pragma unroll
        for (int rr = 0; rr < RPG; ++rr) {
            const int row = grp + 16 * rr;
            if (row < R) {
                const int g = (row % H) / nrep;
                const float* prow = ps + row * lds_s;
                const float* vb = vs + (size_t)g * LT_KT * e;
#pragma unroll
                for (int c = 0; c < NACC; ++c) {
                    const int i = ln + 16 * c;
                    if (i < e) {
                        float o = acc[rr][c] * corr[rr];
                        for (int sl = 0; sl < kn; ++sl) o = fmaf(prow[sl], vb[sl * e + i], o);
                        acc[rr][c] = o;
                    }
                }
            }
        }
    }
#pragma unroll
    for (int rr = 0; rr < RPG; ++rr) {
        const int row = grp + 16 * rr;
        if (row >= R) continue;
        const int lp = row / H, h = row - lp * H;
        if (nsplit > 1) {                  // un-normalised partial sums + (running max, running sum) for the merge
            const size_t pr = (((size_t)blockIdx.x * gridDim.y + blockIdx.y) * nsplit + blockIdx.z) * R + row;
            if (ln == 0) { a.part_ml[pr * 2] = m[rr]; a.part_ml[pr * 2 + 1] = l[rr]; }
#pragma unroll
            for (int c = 0; c < NACC; ++c) {
                const int i = ln + 16 * c;
                if (i < e) a.part_o[pr * e + i] = acc[rr][c];
            }
        } else if (lp < np) {
            const float inv = a.out_scale / l[rr];
#pragma unroll
            for (int c = 0; c < NACC; ++c) {
                const int i = ln + 16 * c;
                if (i < e) a.out[(size_t)(sg.row0 + p0 + lp) * a.ldo + h * e + i] = acc[rr][c] * inv;
            }
        }
    }
}
// merge of the splits (single-token portions: the tile's rows are the H heads); one block of 64 threads per (sequence, head): the
// splits' factors e^(m_z - M) are formed once (one lane each, up to 64 splits), then a thread per output element sums
constexpr int LT_MAX_SPLIT = 64;
__global__ __launch_bounds__(64) void lay_attn_talk_merge_kernel(LAttnArgs a, int nsplit) {
    __shared__ float wz[LT_MAX_SPLIT];
    const LaySegDev sg = a.segs[blockIdx.x];
    const int H = a.H, e = a.e, h = blockIdx.y, lane = threadIdx.x;
    const size_t t0 = (size_t)blockIdx.x * nsplit * H + h;
    const float mz = lane < nsplit ? a.part_ml[(t0 + (size_t)lane * H) * 2] : -INFINITY;
    const float M = wave_max(mz);
    const float wgt = mz == -INFINITY ? 0.f : expf(mz - M);
    const float L = wave_sum(lane < nsplit ? a.part_ml[(t0 + (size_t)lane * H) * 2 + 1] * wgt : 0.f);
    wz[lane] = wgt;
    __syncthreads();
    const float inv = a.out_scale / L;
    for (int i = lane; i < e; i += 64) {
        float acc = 0.f;
        for (int z = 0; z < nsplit; ++z) acc = fmaf(a.part_o[(t0 + (size_t)z * H) * e + i], wz[z], acc);
        a.out[(size_t)sg.row0 * a.ldo + h * e + i] = acc * inv;
    }
}
// Matrix-core form for prompt passes in the bfloat16 format (key and value sizes multiples of 16 up to 128, up to 16 heads): a
// block owns 16 positions of one sequence, one wave per head.  Per tile of 64 keys every wave forms S_h = Q_h K^T on
// v_mfma_f32_16x16x16_bf16 from the bf16-rounded q and the cached keys of its key head and leaves it, scaled, in LDS; after a
// barrier it mixes the H raw scores of each of its (position, key) places with its line of the matrix in the accumulator's own
// layout (A[i = lane % 16][k = 4 (lane / 16) ..], B[k][j = lane % 16], D[i = 4 (lane / 16) + r][j = lane % 16]); mask, running
// max / sum and the weights are f32, the weights enter P V as a bf16 hi + lo pair (two products per tile).
// KT keys per tile (64, or 32 where that is what fits in LDS: more heads); a raw-score row holds KT + 4 floats, so that the two half-waves
// of a read hit disjoint banks
// Gv value heads (consecutive key heads may share one); mixed: the raw-score rows and the matrix are needed
static size_t lay_talk_mfma_lds(int H, int G, int Gv, int d, int e, int KT, bool mixed) {
    return (size_t)(G * KT * (d + 8) + Gv * e * (KT + 8) + 2 * H * 16 * (KT + 8)) * sizeof(uint16_t) +
           (mixed ? (size_t)(H * 16 * (KT + 4) + H * H) * sizeof(float) : 0);
}
template <int NDMAX, int NEMAX, int NT, int KT>
__global__ __launch_bounds__(NT) void lay_attn_talk_mfma_kernel(LAttnArgs a, const float* __restrict__ talk) {
    constexpr int LTM_KT = KT, LTM_LDS = KT + 4, NS = KT / 16;      // sub-tiles of 16 keys
    extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
    const int d = a.d, e = a.e, H = a.H, G = a.G, nrep = H / G, vdiv = max(a.v_div, 1), Gv = G / vdiv;
    const int ldq = d + 8, ldp = LTM_KT + 8;
    const bool mixed = talk != nullptr;                // null: every head keeps its own scores (the kernel then is plain attention, one wave per head)
    uint16_t* Ks = smem;                               // [G][KT][d + 8]
    uint16_t* Vt = Ks + G * LTM_KT * ldq;              // [Gv][e][KT + 8] the value tiles transposed (the B operand of P V: 4 keys of one element)
    uint16_t* Ph = Vt + Gv * e * ldp;                  // [H][16][KT + 8] hi
    uint16_t* Pl = Ph + H * 16 * ldp;                  // ... lo
    float* Sr = (float*)(Pl + H * 16 * ldp);           // [H][16][KT + 4] raw scores of every head
    float* tk = Sr + H * 16 * LTM_LDS;                 // [H][H]
    const LaySegDev sg = a.segs[blockIdx.x];
    const int p0 = (int)blockIdx.y * 16;
    if (p0 >= sg.n) return;
    const int np = min(16, sg.n - p0);
    const int tid = threadIdx.x, nt = 64 * H, lane = tid & 63, h = tid >> 6, lr = lane & 15, lg = lane >> 4;
    const int g = h / nrep;
    const int win = (int)min(a.win, 1ll << 30);
    if (mixed) for (int idx = tid; idx < H * H; idx += nt) tk[idx] = talk[idx];
    // this lane's part of the q fragments: position p0 + lr, elements kk 16 + 4 lg .. + 3 of head h
    const int nd = d / 16, ne = e / 16;
    bf16x4 qf[NDMAX];
#pragma unroll
    for (int kk = 0; kk < NDMAX; ++kk) {
        qf[kk] = (bf16x4){0, 0, 0, 0};
        if (kk < nd && lr < np) {
            const float4 x = *(const float4*)(a.proj + (size_t)(sg.row0 + p0 + lr) * a.ldp + a.q_off + h * d + kk * 16 + 4 * lg);
            const uint32_t lo = pack_bf16x2(x.x, x.y), hi = pack_bf16x2(x.z, x.w);
            qf[kk] = (bf16x4){(short)(lo & 0xFFFFu), (short)(lo >> 16), (short)(hi & 0xFFFFu), (short)(hi >> 16)};
        }
    }
    int qpos[4]; bool qok[4];
    float m[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY}, l[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < 4; ++r) { qok[r] = 4 * lg + r < np; qpos[r] = sg.start_pos + p0 + 4 * lg + r; }
    const int pmin = sg.start_pos + p0, pmax = pmin + np - 1;
    const int main_lo = max(0, pmin - win + 1);
    const int total = pmax - main_lo + 1;
    f32x4 O[NEMAX];
#pragma unroll
    for (int n = 0; n < NEMAX; ++n) O[n] = (f32x4){0.f, 0.f, 0.f, 0.f};
    uint16_t* ph = Ph + h * 16 * ldp;
    uint16_t* pl = Pl + h * 16 * ldp;
    const uint16_t* kg = Ks + g * LTM_KT * ldq;
    const uint16_t* vg = Vt + (g / vdiv) * e * ldp;
    float* sr = Sr + h * 16 * LTM_LDS;
    // the page of every key of a tile (-1 past the end), looked up one tile ahead so that the tile's loads do not wait for the page table
    __shared__ int rowb[2][LTM_KT];
    auto look_up = [&](int v0, int buf) {
        if (tid < LTM_KT) {
            const int v = v0 + tid, j = main_lo + v;
            rowb[buf][tid] = v < total ? a.bt[sg.bt_off + j / a.page] : -1;
        }
    };
    look_up(0, 0);
    const int nk = G * LTM_KT * (d / 8), nv = Gv * LTM_KT * (e / 8);
    for (int v0 = 0, buf = 0; v0 < total; v0 += LTM_KT, buf ^= 1) {
        __syncthreads();                   // the previous tile is consumed: keys, values and raw scores may be replaced
        look_up(v0 + LTM_KT, buf ^ 1);
        // four independent 16-byte loads in flight per thread, then their stores
        for (int base = 0; base < nk; base += 4 * nt) {
            u32x4 pk[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int idx = base + c * nt + tid;
                pk[c] = (u32x4){0u, 0u, 0u, 0u};
                if (idx < nk) {
                    const int rw = idx / (d / 8), i = (idx - rw * (d / 8)) * 8, kgi = rw / LTM_KT, sl = rw - kgi * LTM_KT, pg = rowb[buf][sl];
                    if (pg >= 0) pk[c] = *(const u32x4*)((const uint16_t*)a.kpool + (((size_t)pg * G + kgi) * a.page + (size_t)((main_lo + v0 + sl) % a.page)) * d + i);
                }
            }
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int idx = base + c * nt + tid;
                if (idx < nk) { const int rw = idx / (d / 8), i = (idx - rw * (d / 8)) * 8; *(u32x4*)&Ks[(size_t)rw * ldq + i] = pk[c]; }
            }
        }
        for (int base = 0; base < nv; base += 4 * nt) {
            u32x4 pk[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int idx = base + c * nt + tid;
                pk[c] = (u32x4){0u, 0u, 0u, 0u};
                if (idx < nv) {
                    const int rw = idx / (e / 8), i = (idx - rw * (e / 8)) * 8, kgi = rw / LTM_KT, sl = rw - kgi * LTM_KT, pg = rowb[buf][sl];
                    if (pg >= 0) pk[c] = *(const u32x4*)((const uint16_t*)a.vpool + (((size_t)pg * Gv + kgi) * a.page + (size_t)((main_lo + v0 + sl) % a.page)) * e + i);
                }
            }
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int idx = base + c * nt + tid;
                if (idx < nv) {
                    const int rw = idx / (e / 8), i = (idx - rw * (e / 8)) * 8, kgi = rw / LTM_KT, sl = rw - kgi * LTM_KT;
                    uint16_t* vt = Vt + ((size_t)kgi * e + i) * ldp + sl;
                    vt[0] = (uint16_t)(pk[c].x & 0xFFFFu); vt[ldp] = (uint16_t)(pk[c].x >> 16);
                    vt[2 * ldp] = (uint16_t)(pk[c].y & 0xFFFFu); vt[3 * ldp] = (uint16_t)(pk[c].y >> 16);
                    vt[4 * ldp] = (uint16_t)(pk[c].z & 0xFFFFu); vt[5 * ldp] = (uint16_t)(pk[c].z >> 16);
                    vt[6 * ldp] = (uint16_t)(pk[c].w & 0xFFFFu); vt[7 * ldp] = (uint16_t)(pk[c].w >> 16);
                }
            }
        }
        __syncthreads();
        f32x4 S[NS];
#pragma unroll
        for (int t = 0; t < NS; ++t) S[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < NDMAX; ++kk) {
            if (kk < nd) {
                const bf16x4 qa = qf[kk];
#pragma unroll
                for (int t = 0; t < NS; ++t) {
                    const bf16x4 kb = *(const bf16x4*)&kg[(t * 16 + lr) * ldq + kk * 16 + 4 * lg];
                    S[t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(qa, kb, S[t], 0, 0, 0);
                }
            }
        }
        if (mixed) {
#pragma unroll
            for (int t = 0; t < NS; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) sr[(4 * lg + r) * LTM_LDS + t * 16 + lr] = S[t][r] * a.scale;
            __syncthreads();               // every head's raw scores are in LDS
#pragma unroll
            for (int t = 0; t < NS; ++t) S[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
            for (int g2 = 0; g2 < H; ++g2) {
                const float w = tk[h * H + g2];
                const float* so = Sr + (size_t)g2 * 16 * LTM_LDS;
#pragma unroll
                for (int t = 0; t < NS; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r) S[t][r] = fmaf(w, so[(4 * lg + r) * LTM_LDS + t * 16 + lr], S[t][r]);
            }
        } else {
#pragma unroll
            for (int t = 0; t < NS; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) S[t][r] *= a.scale;
        }
        float corr[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float sc[NS], tmax = -INFINITY;
#pragma unroll
            for (int t = 0; t < NS; ++t) {
                const int v = v0 + t * 16 + lr, j = main_lo + v;
                const bool vis = qok[r] && v < total && j <= qpos[r] && qpos[r] - j < win;
                sc[t] = vis ? S[t][r] : -INFINITY;
                tmax = fmaxf(tmax, sc[t]);
            }
            tmax = row16_max(tmax);
            const float mn = fmaxf(m[r], tmax);
            corr[r] = mn == -INFINITY ? 1.f : __expf(m[r] - mn);
            float psum = 0.f;
#pragma unroll
            for (int t = 0; t < NS; ++t) {
                const float p = sc[t] == -INFINITY ? 0.f : __expf(sc[t] - mn);
                psum += p;
                const uint16_t hi = f32_to_bf16(p);
                ph[(4 * lg + r) * ldp + t * 16 + lr] = hi;
                pl[(4 * lg + r) * ldp + t * 16 + lr] = f32_to_bf16(p - bf16_to_f32(hi));
            }
            psum = row16_sum(psum);
            l[r] = l[r] * corr[r] + psum;
            m[r] = mn;
        }
#pragma unroll
        for (int n = 0; n < NEMAX; ++n)
#pragma unroll
            for (int r = 0; r < 4; ++r) O[n][r] *= corr[r];
        __syncthreads();                   // the wave's weights are in LDS
#pragma unroll
        for (int ks = 0; ks < NS; ++ks) {
            const bf16x4 ah = *(const bf16x4*)&ph[lr * ldp + ks * 16 + 4 * lg];
            const bf16x4 al = *(const bf16x4*)&pl[lr * ldp + ks * 16 + 4 * lg];
#pragma unroll
            for (int n = 0; n < NEMAX; ++n) {
                if (n < ne) {
                    const bf16x4 vb = *(const bf16x4*)&vg[(n * 16 + lr) * ldp + ks * 16 + 4 * lg];
                    O[n] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(ah, vb, O[n], 0, 0, 0);
                    O[n] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(al, vb, O[n], 0, 0, 0);
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        if (!qok[r]) continue;
        const float inv = a.out_scale / l[r];
#pragma unroll
        for (int n = 0; n < NEMAX; ++n)
            if (n < ne) a.out[(size_t)(sg.row0 + p0 + 4 * lg + r) * a.ldo + h * e + n * 16 + lr] = O[n][r] * inv;
    }
}
bool lay_attn_talk_mfma_fits(int H, int G, int d, int e, int v_div, bool mixed) {
    return H > 0 && H <= 16 && G > 0 && H % G == 0 && v_div > 0 && G % v_div == 0 && d > 0 && e > 0 && d % 16 == 0 && e % 16 == 0 && d <= 128 &&
           e <= 128 && lay_talk_mfma_lds(H, G, G / v_div, d, e, 32, mixed) <= LT_LDS_MAX;
}
template <int NT, int KT>
static void lay_attn_talk_mfma_go(const LAttnArgs& a, const float* talk, dim3 grid, size_t lds, hipStream_t s) {
    static bool raised = false;            // per instantiation
    if (!raised) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&lay_attn_talk_mfma_kernel<8, 8, NT, KT>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  (int)LT_LDS_MAX);
        raised = true;
    }
    hipLaunchKernelGGL((lay_attn_talk_mfma_kernel<8, 8, NT, KT>), grid, dim3((unsigned)(64 * a.H)), lds, s, a, talk);
}
void launch_lay_attn_talk_mfma(const LAttnArgs& a, const float* talk, int nseg, int max_n, hipStream_t s) {
    if (nseg <= 0 || max_n <= 0) return;
    const dim3 grid((unsigned)nseg, (unsigned)((max_n + 15) / 16));
    const int Gv = a.G / std::max(a.v_div, 1);
    const bool wide = lay_talk_mfma_lds(a.H, a.G, Gv, a.d, a.e, 64, talk != nullptr) <= LT_LDS_MAX;      // 64-key tiles where they fit
    const size_t lds = lay_talk_mfma_lds(a.H, a.G, Gv, a.d, a.e, wide ? 64 : 32, talk != nullptr);
    if (a.H <= 8) {
        if (wide) lay_attn_talk_mfma_go<512, 64>(a, talk, grid, lds, s);
        else lay_attn_talk_mfma_go<512, 32>(a, talk, grid, lds, s);
    } else {
        if (wide) lay_attn_talk_mfma_go<1024, 64>(a, talk, grid, lds, s);
        else lay_attn_talk_mfma_go<1024, 32>(a, talk, grid, lds, s);
    }
}

template <int KVT, int RPG, int NACC>
static void lay_attn_talk_go(const LAttnArgs& a, const float* talk, int BQ, dim3 grid, size_t lds, hipStream_t s) {
    if (lds > LT_LDS_PLAIN) {
        static bool raised = false;        // per instantiation
        if (!raised) {
            (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&lay_attn_talk_kernel<KVT, RPG, NACC>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)LT_LDS_MAX);
            raised = true;
        }
    }
    hipLaunchKernelGGL((lay_attn_talk_kernel<KVT, RPG, NACC>), grid, dim3(256), lds, s, a, talk, BQ);
}
template <int KVT, int RPG>
static void lay_attn_talk_e(const LAttnArgs& a, const float* talk, int BQ, dim3 grid, size_t lds, hipStream_t s) {
    if (a.e <= 64) lay_attn_talk_go<KVT, RPG, 4>(a, talk, BQ, grid, lds, s);
    else if (a.e <= 128) lay_attn_talk_go<KVT, RPG, 8>(a, talk, BQ, grid, lds, s);
    else lay_attn_talk_go<KVT, RPG, 16>(a, talk, BQ, grid, lds, s);
}
template <int KVT>
static void lay_attn_talk_r(const LAttnArgs& a, const float* talk, int rpg, int BQ, dim3 grid, size_t lds, hipStream_t s) {
    if (rpg <= 1) lay_attn_talk_e<KVT, 1>(a, talk, BQ, grid, lds, s);
    else if (rpg == 2) lay_attn_talk_e<KVT, 2>(a, talk, BQ, grid, lds, s);
    else lay_attn_talk_e<KVT, 4>(a, talk, BQ, grid, lds, s);
}
bool lay_attn_talk_fits(int H, int G, int d, int e) {
    return H > 0 && G > 0 && H % G == 0 && H <= 64 && d > 0 && e > 0 && e <= 256 && lay_talk_lds(H, G, d, e, 1) <= LT_LDS_MAX;
}
void launch_lay_attn_talk(const LAttnArgs& a0, const float* talk, int nseg, int max_n, int kvt, hipStream_t s) {
    if (nseg <= 0 || max_n <= 0) return;
    LAttnArgs a = a0;
    const int H = a.H;
    // rows per 16-lane group: what the heads of one position need, and for portions up to 4 (64 rows a block) while LDS allows
    int rpg = H <= 16 ? 1 : (H <= 32 ? 2 : 4), BQ = 1;
    if (max_n > 1) {
        for (int tr = 4; tr >= rpg; tr >>= 1) {
            const int bq = std::max(1, 16 * tr / H);
            if (lay_talk_lds(H, a.G, a.d, a.e, bq) <= LT_LDS_MAX) { rpg = tr; BQ = bq; break; }
        }
    }
    const int nsplit = (max_n == 1 && a.part_o && a.part_ml && a.nsplit > 1) ? std::min(a.nsplit, LT_MAX_SPLIT) : 1;
    const dim3 grid((unsigned)nseg, (unsigned)((max_n + BQ - 1) / BQ), (unsigned)nsplit);
    const size_t lds = lay_talk_lds(H, a.G, a.d, a.e, BQ);
    if (kvt == KV_F32) lay_attn_talk_r<KV_F32>(a, talk, rpg, BQ, grid, lds, s);
    else lay_attn_talk_r<KV_BF16>(a, talk, rpg, BQ, grid, lds, s);
    if (nsplit > 1) hipLaunchKernelGGL(lay_attn_talk_merge_kernel, dim3((unsigned)nseg, (unsigned)H), dim3(64), 0, s, a, nsplit);
}

}  // namespace cm
