// Kernels of the layer-list decoders (layered.h): every mechanism takes its sizes and constants as arguments.
// What the model's definition asks for in 32 bits is f32 here in both number formats: residual stream, norms, positions,
// attention scores and softmax, the linear-attention state and its decay powers, router logits.  The bfloat16 format rounds the
// A operand of the projections (matrix cores, f32 accumulation) and the cached keys; the float32 format rounds nothing.
#include <hip/hip_runtime.h>

#include "dev_common.h"
#include "layered.h"

namespace cm {

typedef __attribute__((ext_vector_type(16))) float f32x16;

__device__ __forceinline__ float lay_act(float v, int act, float param = 1.f) {
    switch (act) {
        case LACT_RELU2: { const float r = fmaxf(v, 0.f); return r * r; }
        case LACT_LOGSIG: return param * (fminf(v, 0.f) - log1pf(expf(-fabsf(v))));      // ln sigmoid(v), no overflow either way
        case LACT_SILU: return v / (1.f + __expf(-v));
        case LACT_SIGMOID: return 1.f / (1.f + __expf(-v));
        case LACT_GELU_TANH: {
            const float u = 0.7978845608028654f * (v + 0.044715f * v * v * v);
            return 0.5f * v * (1.f + tanhf(u));
        }
        default: return v;
    }
}
// capped gated product: g = min(g, cap), u = clamp(u, -cap, cap): g sigmoid(1.702 g) (u + 1)
__device__ __forceinline__ float lay_capglu(float g, float u, float cap) {
    g = fminf(g, cap);
    u = fminf(fmaxf(u, -cap), cap);
    return g / (1.f + expf(-1.702f * g)) * (u + 1.f);
}

// sum over the block (blockDim.x a multiple of 64, every thread calls); red: >= blockDim.x / 64 floats of LDS
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < (int)(blockDim.x >> 6); ++i) t += red[i];
    __syncthreads();
    return t;
}

// embedding rows of any width (the shared gather moves four elements at a time)
__global__ __launch_bounds__(256) void lay_embed_rows_kernel(const uint16_t* __restrict__ emb, const uint32_t* __restrict__ ids,
                                                             float* __restrict__ x, int W, int V, float scale) {
    uint32_t tok = ids[blockIdx.x];
    if (tok >= (uint32_t)V) tok = 0;
    for (int i = threadIdx.x; i < W; i += 256) x[(size_t)blockIdx.x * W + i] = bf16_to_f32(emb[(size_t)tok * W + i]) * scale;
}
void launch_lay_embed_rows(const uint16_t* emb, const uint32_t* ids, float* x, int T, int W, int V, hipStream_t s, float scale) {
    if (T <= 0) return;
    hipLaunchKernelGGL(lay_embed_rows_kernel, dim3((unsigned)T), dim3(256), 0, s, emb, ids, x, W, V, scale);
}

// ------------------------------------------------------------------------------------------------------------------
// row norms
// ------------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void lay_rms_rows_kernel(const float* __restrict__ x, const int32_t* __restrict__ rows,
                                                           const float* __restrict__ w, float* __restrict__ out, int W, float eps) {
    __shared__ float red[4];
    const int r = blockIdx.x;
    const float* xr = x + (size_t)(rows ? rows[r] : r) * W;
    float ss = 0.f;
    for (int c = threadIdx.x; c < W; c += 256) { const float v = xr[c]; ss += v * v; }
    ss = block_sum(ss, red);
    const float rs = 1.f / sqrtf(ss / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += 256) out[(size_t)r * W + c] = xr[c] * rs * w[c];
}
void launch_lay_rms_rows(const float* x, const int32_t* rows, const float* w, float* out, int n_rows, int W, float eps, hipStream_t s) {
    if (n_rows <= 0) return;
    hipLaunchKernelGGL(lay_rms_rows_kernel, dim3((unsigned)n_rows), dim3(256), 0, s, x, rows, w, out, W, eps);
}

__global__ __launch_bounds__(256) void lay_rms_rows2_kernel(const float* __restrict__ x, const float* __restrict__ w1,
                                                            const float* __restrict__ w2, float* __restrict__ out1, float* __restrict__ out2,
                                                            int W, float eps) {
    __shared__ float red[4];
    const float* xr = x + (size_t)blockIdx.x * W;
    float ss = 0.f;
    for (int c = threadIdx.x; c < W; c += 256) { const float v = xr[c]; ss += v * v; }
    ss = block_sum(ss, red);
    const float rs = 1.f / sqrtf(ss / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += 256) {
        const float v = xr[c] * rs;
        out1[(size_t)blockIdx.x * W + c] = v * w1[c];
        if (out2) out2[(size_t)blockIdx.x * W + c] = v * w2[c];
    }
}
void launch_lay_rms_rows2(const float* x, const float* w1, const float* w2, float* out1, float* out2, int T, int W, float eps, hipStream_t s) {
    if (T <= 0) return;
    hipLaunchKernelGGL(lay_rms_rows2_kernel, dim3((unsigned)T), dim3(256), 0, s, x, w1, w2, out1, out2, W, eps);
}

__global__ __launch_bounds__(256) void lay_rms_cols_kernel(const float* src, int lds, int off, int n, const float* __restrict__ w, float* dst,
                                                           int ldd, float eps) {
    __shared__ float red[4];
    const float* xr = src + (size_t)blockIdx.x * lds + off;
    float ss = 0.f;
    for (int c = threadIdx.x; c < n; c += 256) { const float v = xr[c]; ss += v * v; }
    ss = block_sum(ss, red);           // every read of the row is done behind this barrier: dst may be the same memory
    const float rs = 1.f / sqrtf(ss / (float)n + eps);
    for (int c = threadIdx.x; c < n; c += 256) dst[(size_t)blockIdx.x * ldd + c] = xr[c] * rs * w[c];
}
void launch_lay_rms_cols(const float* src, int lds, int off, int n, const float* w, float* dst, int ldd, int T, float eps, hipStream_t s) {
    if (T <= 0 || n <= 0) return;
    hipLaunchKernelGGL(lay_rms_cols_kernel, dim3((unsigned)T), dim3(256), 0, s, src, lds, off, n, w, dst, ldd, eps);
}

__global__ __launch_bounds__(256) void lay_add_rows_kernel(float* __restrict__ x, const float* __restrict__ y1, const float* __restrict__ y2,
                                                           size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) x[i] += y2 ? y1[i] + y2[i] : y1[i];
}
void launch_lay_add_rows(float* x, const float* y1, const float* y2, size_t n, hipStream_t s) {
    if (n == 0) return;
    hipLaunchKernelGGL(lay_add_rows_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, x, y1, y2, n);
}

__global__ __launch_bounds__(256) void lay_add_norm2_shift_decode_kernel(float* __restrict__ x, const float* __restrict__ y1,
                                                                         const float* __restrict__ y2, const float* __restrict__ w1,
                                                                         const float* __restrict__ w2, float eps, float* __restrict__ out1,
                                                                         float* __restrict__ out2, const float* __restrict__ cw,
                                                                         float* __restrict__ conv_pool, size_t slot_stride, size_t off,
                                                                         const LaySegDev* __restrict__ segs, int W) {
    __shared__ float red[4];
    const LaySegDev sg = segs[blockIdx.x];
    const size_t r = (size_t)sg.row0 * W;
    float ss = 0.f;
    for (int c = threadIdx.x; c < W; c += 256) {
        float v = x[r + c];
        if (y1) { v += y2 ? y1[r + c] + y2[r + c] : y1[r + c]; x[r + c] = v; }     // read back below by the same thread
        ss += v * v;
    }
    ss = block_sum(ss, red);
    const float rs = 1.f / sqrtf(ss / (float)W + eps);
    float* prev = conv_pool + (size_t)sg.slot * slot_stride + off;
    for (int c = threadIdx.x; c < W; c += 256) {
        const float v = x[r + c] * rs;
        const float h = v * w1[c];
        float acc = h;
        acc += cw[2 * c] * prev[c];
        acc += cw[2 * c + 1] * h;
        out1[r + c] = acc;
        prev[c] = h;
        if (out2) out2[r + c] = v * w2[c];
    }
}
void launch_lay_add_norm2_shift_decode(float* x, const float* y1, const float* y2, const float* w1, const float* w2, float eps, float* out1,
                                       float* out2, const float* cw, float* conv_pool, size_t slot_stride, size_t off, const LaySegDev* segs,
                                       int T, int W, hipStream_t s) {
    if (T <= 0) return;
    hipLaunchKernelGGL(lay_add_norm2_shift_decode_kernel, dim3((unsigned)T), dim3(256), 0, s, x, y1, y2, w1, w2, eps, out1, out2, cw, conv_pool,
                       slot_stride, off, segs, W);
}

// rotation by position: the angle and its sine / cosine are f32 (sincosf reduces the argument exactly)
__global__ __launch_bounds__(256) void lay_rope_kernel(const float* src, int lds, int s_vstride, float* dst, int ldd, int d_vstride, int nvec,
                                                       int len, int dims, const float* __restrict__ freq, float mag,
                                                       const LaySegDev* __restrict__ segs, const int32_t* __restrict__ rowseg, int half) {
    const int r = blockIdx.x;
    const LaySegDev sg = segs[rowseg[r]];
    const float pos = (float)(sg.start_pos + (r - sg.row0));
    const int hp = (len + 1) / 2;
    if (half) {                            // pairs (i, i + dims / 2); a thread owns both elements of its pair, so dst may be src
        const int hd = dims / 2, per = hd + (len - dims);
        for (int idx = threadIdx.x; idx < nvec * per; idx += 256) {
            const int v = idx / per, i = idx - v * per;
            const float* sp = src + (size_t)r * lds + (size_t)v * s_vstride;
            float* dp = dst + (size_t)r * ldd + (size_t)v * d_vstride;
            if (i < hd) {
                const float a = sp[i], b = sp[i + hd];
                float sn, cs;
                sincosf(pos * freq[i], &sn, &cs);
                sn *= mag; cs *= mag;
                dp[i] = a * cs - b * sn;
                dp[i + hd] = b * cs + a * sn;
            } else dp[dims + (i - hd)] = sp[dims + (i - hd)];
        }
        return;
    }
    for (int idx = threadIdx.x; idx < nvec * hp; idx += 256) {
        const int v = idx / hp, i = idx - v * hp;
        const float* sp = src + (size_t)r * lds + (size_t)v * s_vstride + 2 * i;
        float* dp = dst + (size_t)r * ldd + (size_t)v * d_vstride + 2 * i;
        const bool two = 2 * i + 1 < len;
        const float a = sp[0], b = two ? sp[1] : 0.f;
        if (2 * i + 1 < dims) {
            float sn, cs;
            sincosf(pos * freq[i], &sn, &cs);
            sn *= mag; cs *= mag;
            dp[0] = a * cs - b * sn;
            dp[1] = b * cs + a * sn;
        } else {
            dp[0] = a;
            if (two) dp[1] = b;
        }
    }
}
void launch_lay_rope(const float* src, int lds, int s_vstride, float* dst, int ldd, int d_vstride, int nvec, int len, int dims,
                     const float* freq, float mag, const LaySegDev* segs, const int32_t* rowseg, int T, hipStream_t s, bool half) {
    if (T <= 0 || nvec <= 0 || len <= 0) return;
    hipLaunchKernelGGL(lay_rope_kernel, dim3((unsigned)T), dim3(256), 0, s, src, lds, s_vstride, dst, ldd, d_vstride, nvec, len, dims, freq, mag,
                       segs, rowseg, half ? 1 : 0);
}

__global__ __launch_bounds__(256) void lay_rms_gate_kernel(const float* __restrict__ o, const float* __restrict__ gate, int ldg,
                                                           const float* __restrict__ w, float* __restrict__ out, int N, float eps) {
    __shared__ float red[4];
    const int r = blockIdx.x;
    const float* orow = o + (size_t)r * N;
    float ss = 0.f;
    for (int c = threadIdx.x; c < N; c += 256) { const float v = orow[c]; ss += v * v; }
    ss = block_sum(ss, red);
    const float rs = 1.f / sqrtf(ss / (float)N + eps);
    for (int c = threadIdx.x; c < N; c += 256) out[(size_t)r * N + c] = orow[c] * rs * w[c] * (gate ? gate[(size_t)r * ldg + c] : 1.f);
}
// the same with the root mean square over groups of `group` columns: one wave per group
__global__ __launch_bounds__(256) void lay_rms_gate_group_kernel(const float* __restrict__ o, const float* __restrict__ gate, int ldg,
                                                                 const float* __restrict__ w, float* __restrict__ out, int N, int group,
                                                                 int shared_w, float eps) {
    const int r = blockIdx.x, lane = threadIdx.x & 63;
    const int ngroups = N / group;
    for (int g = (int)blockIdx.y * 4 + (int)(threadIdx.x >> 6); g < ngroups; g += 4 * (int)gridDim.y) {
        const float* og = o + (size_t)r * N + (size_t)g * group;
        float ss = 0.f;
        for (int c = lane; c < group; c += 64) { const float v = og[c]; ss += v * v; }
        ss = wave_sum(ss);
        const float rs = 1.f / sqrtf(ss / (float)group + eps);
        for (int c = lane; c < group; c += 64)
            out[(size_t)r * N + (size_t)g * group + c] = og[c] * rs * w[shared_w ? c : g * group + c] * (gate ? gate[(size_t)r * ldg + (size_t)g * group + c] : 1.f);
    }
}
void launch_lay_rms_gate(const float* o, const float* gate, int ldg, const float* w, float* out, int T, int N, float eps, hipStream_t s,
                         int group, bool shared_w) {
    if (T <= 0) return;
    if (group > 0 && group < N) {
        const int ngroups = N / group;
        hipLaunchKernelGGL(lay_rms_gate_group_kernel, dim3((unsigned)T, (unsigned)std::min(16, (ngroups + 3) / 4)), dim3(256), 0, s, o, gate, ldg, w,
                           out, N, group, shared_w ? 1 : 0, eps);
        return;
    }
    hipLaunchKernelGGL(lay_rms_gate_kernel, dim3((unsigned)T), dim3(256), 0, s, o, gate, ldg, w, out, N, eps);
}

// the combined expert rows of token r at channel c: sum_k wsel[r top + k] * row_k, row_k = ys[(r top + k) W + c] or -- choices k < sel_top
// whose expert index is an identity expert (>= n_real) -- the sublayer's input hin[r W + c]
struct LCombine { const float* wsel; int top; const int32_t* sel; int sel_top, n_real; const float* hin; };
__device__ __forceinline__ float lay_combined(const float* __restrict__ y, const LCombine& cb, int r, int c, int W) {
    if (!cb.wsel) return y[(size_t)r * W + c];
    float v = 0.f;
    for (int k = 0; k < cb.top; ++k) {
        const bool ident = cb.sel && k < cb.sel_top && cb.sel[(size_t)r * cb.sel_top + k] >= cb.n_real;
        v += cb.wsel[(size_t)r * cb.top + k] * (ident ? cb.hin[(size_t)r * W + c] : y[((size_t)r * cb.top + k) * W + c]);
    }
    return v;
}
__global__ __launch_bounds__(256) void lay_post_norm_kernel(float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ w,
                                                            float mult, float eps, int W, LCombine cb) {
    __shared__ float red[4];
    const int r = blockIdx.x;
    float ss = 0.f;
    for (int c = threadIdx.x; c < W; c += 256) { const float v = lay_combined(y, cb, r, c, W); ss += v * v; }
    ss = block_sum(ss, red);
    const float rs = 1.f / sqrtf(ss / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += 256) x[(size_t)r * W + c] += mult * (lay_combined(y, cb, r, c, W) * rs * w[c]);
}
// rows of up to 256 EPT channels: the combined values are formed once and wait in registers for the root mean square
template <int EPT>
__global__ __launch_bounds__(256) void lay_post_norm_reg_kernel(float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ w,
                                                                float mult, float eps, int W, LCombine cb) {
    __shared__ float red[4];
    const int r = blockIdx.x;
    float yv[EPT], xv[EPT], wv[EPT];
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
        const int c = threadIdx.x + 256 * e;
        const bool ok = c < W;
        yv[e] = ok ? lay_combined(y, cb, r, c, W) : 0.f;
        xv[e] = ok ? x[(size_t)r * W + c] : 0.f;
        wv[e] = ok ? w[c] : 0.f;
        ss += yv[e] * yv[e];
    }
    ss = block_sum(ss, red);
    const float rs = 1.f / sqrtf(ss / (float)W + eps);
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
        const int c = threadIdx.x + 256 * e;
        if (c < W) x[(size_t)r * W + c] = xv[e] + mult * (yv[e] * rs * wv[e]);
    }
}
void launch_lay_post_norm(float* x, const float* y, const float* w, float mult, float eps, int T, int W, const float* wsel, int top,
                          hipStream_t s, const int32_t* sel, int sel_top, int n_real, const float* hin) {
    if (T <= 0) return;
    const LCombine cb{wsel, top, n_real >= 0 && hin ? sel : nullptr, sel_top, n_real, hin};
    if (W <= 1024) hipLaunchKernelGGL(lay_post_norm_reg_kernel<4>, dim3((unsigned)T), dim3(256), 0, s, x, y, w, mult, eps, W, cb);
    else if (W <= 4096) hipLaunchKernelGGL(lay_post_norm_reg_kernel<16>, dim3((unsigned)T), dim3(256), 0, s, x, y, w, mult, eps, W, cb);
    else hipLaunchKernelGGL(lay_post_norm_kernel, dim3((unsigned)T), dim3(256), 0, s, x, y, w, mult, eps, W, cb);
}

// ------------------------------------------------------------------------------------------------------------------
// short causal convolution in front of a sublayer: out_t = h_t + sum_j cw[:, j] h_(t - taps + 1 + j)
// tail of a sequence = its last taps - 1 inputs, oldest first: [taps - 1][W]
// ------------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void lay_canon_kernel(const float* __restrict__ h, float* __restrict__ out, const float* __restrict__ cw,
                                                        const float* __restrict__ conv_pool, size_t slot_stride, size_t off,
                                                        const LaySegDev* __restrict__ segs, const int32_t* __restrict__ rowseg, int W, int taps) {
    const int r = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= W) return;
    const LaySegDev sg = segs[rowseg[r]];
    const int local = r - sg.row0;
    const float* tail = conv_pool + (size_t)sg.slot * slot_stride + off;
    float acc = h[(size_t)r * W + c];
    for (int j = 0; j < taps; ++j) {
        const int src = local - (taps - 1) + j;
        const float v = src >= 0 ? h[(size_t)(sg.row0 + src) * W + c] : tail[(size_t)(taps - 1 + src) * W + c];
        acc += cw[(size_t)c * taps + j] * v;
    }
    out[(size_t)r * W + c] = acc;
}
void launch_lay_canon(const float* h, float* out, const float* cw, const float* conv_pool, size_t slot_stride, size_t off,
                      const LaySegDev* segs, const int32_t* rowseg, int T, int W, int taps, hipStream_t s) {
    if (T <= 0) return;
    hipLaunchKernelGGL(lay_canon_kernel, dim3((unsigned)T, (unsigned)((W + 255) / 256)), dim3(256), 0, s, h, out, cw, conv_pool, slot_stride,
                       off, segs, rowseg, W, taps);
}

// new tail = last taps - 1 entries of (old tail ++ the portion's inputs).  In place: entry k reads entry n + k > k of the old tail,
// and a thread touches its own channel only.
__global__ __launch_bounds__(256) void lay_canon_tail_kernel(const float* __restrict__ h, float* __restrict__ conv_pool, size_t slot_stride,
                                                             size_t off, const LaySegDev* __restrict__ segs, int W, int taps) {
    const LaySegDev sg = segs[blockIdx.x];
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= W) return;
    float* tail = conv_pool + (size_t)sg.slot * slot_stride + off;
    for (int k = 0; k < taps - 1; ++k) {
        const int idx = sg.n + k;
        tail[(size_t)k * W + c] = idx < taps - 1 ? tail[(size_t)idx * W + c] : h[(size_t)(sg.row0 + idx - (taps - 1)) * W + c];
    }
}
void launch_lay_canon_tail(const float* h, float* conv_pool, size_t slot_stride, size_t off, const LaySegDev* segs, int nseg, int W,
                           int taps, hipStream_t s) {
    if (nseg <= 0 || taps <= 1) return;
    hipLaunchKernelGGL(lay_canon_tail_kernel, dim3((unsigned)nseg, (unsigned)((W + 255) / 256)), dim3(256), 0, s, h, conv_pool, slot_stride,
                       off, segs, W, taps);
}

// decode rows (one token per sequence): norm, convolution and tail shift of a row by the one block that owns its sequence
__global__ __launch_bounds__(256) void lay_norm_canon_decode_kernel(const float* __restrict__ x, const float* __restrict__ nw, float eps,
                                                                    float* __restrict__ out, const float* __restrict__ cw,
                                                                    float* __restrict__ conv_pool, size_t slot_stride, size_t off,
                                                                    const LaySegDev* __restrict__ segs, int W, int taps) {
    __shared__ float red[4];
    const int r = blockIdx.x;
    const LaySegDev sg = segs[r];
    const float* xr = x + (size_t)sg.row0 * W;
    float ss = 0.f;
    for (int c = threadIdx.x; c < W; c += 256) { const float v = xr[c]; ss += v * v; }
    ss = block_sum(ss, red);
    const float rs = 1.f / sqrtf(ss / (float)W + eps);
    float* tail = conv_pool + (size_t)sg.slot * slot_stride + off;
    for (int c = threadIdx.x; c < W; c += 256) {
        const float hv = xr[c] * rs * nw[c];
        float acc = hv + cw[(size_t)c * taps + (taps - 1)] * hv;
        for (int j = 0; j < taps - 1; ++j) {
            const float tv = tail[(size_t)j * W + c];
            acc += cw[(size_t)c * taps + j] * tv;
            if (j > 0) tail[(size_t)(j - 1) * W + c] = tv;
        }
        if (taps > 1) tail[(size_t)(taps - 2) * W + c] = hv;
        out[(size_t)sg.row0 * W + c] = acc;
    }
}
// decode rows: the residual update of the sublayer that just finished AND the norm + convolution in front of the next one, one
// launch: x += mult * RMSNorm(y) * pw (y as in lay_post_norm_kernel), then as lay_norm_canon_decode_kernel on the new x
__global__ __launch_bounds__(256) void lay_post_norm_canon_decode_kernel(float* __restrict__ x, const float* __restrict__ y,
                                                                         const float* __restrict__ pw, float mult, const float* __restrict__ wsel,
                                                                         int top, const float* __restrict__ nw, float eps, float* __restrict__ out,
                                                                         const float* __restrict__ cw, float* __restrict__ conv_pool,
                                                                         size_t slot_stride, size_t off, const LaySegDev* __restrict__ segs, int W,
                                                                         int taps) {
    __shared__ float red[4];
    const LaySegDev sg = segs[blockIdx.x];
    const int r = sg.row0;
    float* xr = x + (size_t)r * W;
    float ss = 0.f;
    for (int c = threadIdx.x; c < W; c += 256) {
        float v;
        if (wsel) {
            v = 0.f;
            for (int k = 0; k < top; ++k) v += wsel[(size_t)r * top + k] * y[((size_t)r * top + k) * W + c];
        } else v = y[(size_t)r * W + c];
        ss += v * v;
    }
    ss = block_sum(ss, red);
    const float rsy = 1.f / sqrtf(ss / (float)W + eps);
    float sx = 0.f;
    for (int c = threadIdx.x; c < W; c += 256) {
        float v;
        if (wsel) {
            v = 0.f;
            for (int k = 0; k < top; ++k) v += wsel[(size_t)r * top + k] * y[((size_t)r * top + k) * W + c];
        } else v = y[(size_t)r * W + c];
        const float xn = xr[c] + mult * (v * rsy * pw[c]);
        xr[c] = xn;                        // read back below by the same thread
        sx += xn * xn;
    }
    sx = block_sum(sx, red);
    const float rs = 1.f / sqrtf(sx / (float)W + eps);
    float* tail = conv_pool + (size_t)sg.slot * slot_stride + off;
    for (int c = threadIdx.x; c < W; c += 256) {
        const float hv = xr[c] * rs * nw[c];
        float acc = hv;
        if (taps > 0) {
            acc += cw[(size_t)c * taps + (taps - 1)] * hv;
            for (int j = 0; j < taps - 1; ++j) {
                const float tv = tail[(size_t)j * W + c];
                acc += cw[(size_t)c * taps + j] * tv;
                if (j > 0) tail[(size_t)(j - 1) * W + c] = tv;
            }
            if (taps > 1) tail[(size_t)(taps - 2) * W + c] = hv;
        }
        out[(size_t)r * W + c] = acc;
    }
}
// the same for rows of up to 256 EPT channels: every operand of a channel is requested up front and lives in registers, so the
// launch costs two block reductions instead of three dependent sweeps over memory
template <int EPT>
__global__ __launch_bounds__(256) void lay_post_norm_canon_decode_reg_kernel(float* __restrict__ x, const float* __restrict__ y,
                                                                             const float* __restrict__ pw, float mult,
                                                                             const float* __restrict__ wsel, int top,
                                                                             const float* __restrict__ nw, float eps, float* __restrict__ out,
                                                                             const float* __restrict__ cw, float* __restrict__ conv_pool,
                                                                             size_t slot_stride, size_t off, const LaySegDev* __restrict__ segs,
                                                                             int W, int taps) {
    __shared__ float red[4];
    const LaySegDev sg = segs[blockIdx.x];
    const int r = sg.row0;
    float* xr = x + (size_t)r * W;
    float yv[EPT], xv[EPT], pv[EPT], nv[EPT];
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
        const int c = threadIdx.x + 256 * e;
        const bool ok = c < W;
        float v = 0.f;
        if (ok) {
            if (wsel) { for (int k = 0; k < top; ++k) v += wsel[(size_t)r * top + k] * y[((size_t)r * top + k) * W + c]; }
            else v = y[(size_t)r * W + c];
        }
        yv[e] = v;
        xv[e] = ok ? xr[c] : 0.f;
        pv[e] = ok ? pw[c] : 0.f;
        nv[e] = ok ? nw[c] : 0.f;
    }
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < EPT; ++e) ss += yv[e] * yv[e];
    ss = block_sum(ss, red);
    const float rsy = 1.f / sqrtf(ss / (float)W + eps);
    float sx = 0.f;
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
        xv[e] += mult * (yv[e] * rsy * pv[e]);
        sx += xv[e] * xv[e];
    }
    sx = block_sum(sx, red);
    const float rs = 1.f / sqrtf(sx / (float)W + eps);
    float* tail = conv_pool + (size_t)sg.slot * slot_stride + off;
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
        const int c = threadIdx.x + 256 * e;
        if (c >= W) continue;
        xr[c] = xv[e];
        const float hv = xv[e] * rs * nv[e];
        float acc = hv;
        if (taps > 0) {
            acc += cw[(size_t)c * taps + (taps - 1)] * hv;
            for (int j = 0; j < taps - 1; ++j) {
                const float tv = tail[(size_t)j * W + c];
                acc += cw[(size_t)c * taps + j] * tv;
                if (j > 0) tail[(size_t)(j - 1) * W + c] = tv;
            }
            if (taps > 1) tail[(size_t)(taps - 2) * W + c] = hv;
        }
        out[(size_t)r * W + c] = acc;
    }
}
void launch_lay_post_norm_canon_decode(float* x, const float* y, const float* pw, float mult, const float* wsel, int top, const float* nw,
                                       float eps, float* out, const float* cw, float* conv_pool, size_t slot_stride, size_t off,
                                       const LaySegDev* segs, int T, int W, int taps, hipStream_t s) {
    if (T <= 0) return;
    if (W <= 1024) {
        hipLaunchKernelGGL(lay_post_norm_canon_decode_reg_kernel<4>, dim3((unsigned)T), dim3(256), 0, s, x, y, pw, mult, wsel, top, nw, eps, out,
                           cw, conv_pool, slot_stride, off, segs, W, taps);
        return;
    }
    if (W <= 4096) {
        hipLaunchKernelGGL(lay_post_norm_canon_decode_reg_kernel<16>, dim3((unsigned)T), dim3(256), 0, s, x, y, pw, mult, wsel, top, nw, eps, out,
                           cw, conv_pool, slot_stride, off, segs, W, taps);
        return;
    }
    hipLaunchKernelGGL(lay_post_norm_canon_decode_kernel, dim3((unsigned)T), dim3(256), 0, s, x, y, pw, mult, wsel, top, nw, eps, out, cw,
                       conv_pool, slot_stride, off, segs, W, taps);
}
void launch_lay_norm_canon_decode(const float* x, const float* nw, float eps, float* out, const float* cw, float* conv_pool,
                                  size_t slot_stride, size_t off, const LaySegDev* segs, int T, int W, int taps, hipStream_t s) {
    if (T <= 0) return;
    hipLaunchKernelGGL(lay_norm_canon_decode_kernel, dim3((unsigned)T), dim3(256), 0, s, x, nw, eps, out, cw, conv_pool, slot_stride, off,
                       segs, W, taps);
}

// ------------------------------------------------------------------------------------------------------------------
// projections: C[p][n] = epilogue(sum_k A[row(p)][k] W[n][k] + bias[n])
// 64 x 64 outputs per block of 256 threads; any M, N, K (tiles are zero-filled past the edges)
// ------------------------------------------------------------------------------------------------------------------
constexpr int LG_BM = 64, LG_BN = 64;

struct LgTile { int p0, rows, n0; const uint16_t* W; const uint16_t* W2; const float* A; size_t coff; };

__device__ __forceinline__ bool lg_tile(const LGemmArgs& a, LgTile& t) {
    const int g = blockIdx.z;
    int base = 0, rows = a.M;
    if (a.grp_off) { base = a.grp_off[g]; rows = a.grp_off[g + 1] - base; }
    const int m0 = blockIdx.x * LG_BM;
    if (m0 >= rows) return false;
    t.p0 = base + m0;
    t.rows = min(LG_BM, rows - m0);
    t.n0 = blockIdx.y * LG_BN;
    t.W = a.W + (size_t)g * a.w_stride;
    t.W2 = a.W2 ? a.W2 + (size_t)g * a.w_stride : nullptr;
    t.A = a.A + (a.grp_off ? 0 : (size_t)g * a.a_goff);
    t.coff = a.grp_off ? 0 : (size_t)g * a.c_goff;
    return true;
}

__device__ __forceinline__ void lg_store(const LGemmArgs& a, size_t coff, int p, int n, float v, float v2, bool dual) {
    if (a.bias) v += a.bias[n];
    if (dual) v = a.act == LACT_CAPGLU ? lay_capglu(v, v2, a.act_param) : lay_act(v, a.act) * v2;
    else v = lay_act(v, n < a.act_split ? a.act : a.act2, a.act_param);
    if (a.mul) v *= a.mul[(size_t)p * a.ldm + coff + n];
    const size_t row = a.c_idx ? (size_t)a.c_idx[p] : (size_t)p;
    a.C[row * a.ldc + coff + n] = v;
}

// f32 FMA form: 4 x 4 outputs per thread, k in steps of 16
template <bool DUAL>
__global__ __launch_bounds__(256) void lgemm_f32_kernel(LGemmArgs a) {
    constexpr int BK = 16;
    __shared__ float As[BK][LG_BM + 4];
    __shared__ float Bs[BK][LG_BN + 4];
    __shared__ float B2s[DUAL ? BK : 1][LG_BN + 4];
    __shared__ int arow[LG_BM];
    __shared__ float ascl[LG_BM];
    LgTile t;
    if (!lg_tile(a, t)) return;
    const int tid = threadIdx.x;
    if (tid < LG_BM) {
        int ar = -1;
        float sc = 1.f;
        if (tid < t.rows) {
            const int p = t.p0 + tid;
            ar = a.a_idx ? a.a_idx[p] / a.a_div : p;
            if (a.a_scale) sc = a.a_scale[a.a_idx[p]];
        }
        arow[tid] = ar; ascl[tid] = sc;
    }
    __syncthreads();
    const int ty = tid >> 4, tx = tid & 15;
    float acc[4][4] = {}, acc2[4][4] = {};
    for (int k0 = 0; k0 < a.K; k0 += BK) {
        for (int i = 0; i < 4; ++i) {
            const int idx = tid + i * 256, r = idx >> 4, kk = idx & 15, k = k0 + kk;
            const int ar = arow[r];
            As[kk][r] = (ar >= 0 && k < a.K) ? t.A[(size_t)ar * a.lda + k] * ascl[r] : 0.f;
            const int n = t.n0 + r;
            const bool ok = n < a.N && k < a.K;
            Bs[kk][r] = ok ? bf16_to_f32(t.W[(size_t)n * a.K + k]) : 0.f;
            if (DUAL) B2s[kk][r] = ok ? bf16_to_f32(t.W2[(size_t)n * a.K + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK; ++kk) {
            float av[4], bv[4], b2[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { av[i] = As[kk][ty * 4 + i]; bv[i] = Bs[kk][tx * 4 + i]; if (DUAL) b2[i] = B2s[kk][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
                    if (DUAL) acc2[i][j] = fmaf(av[i], b2[j], acc2[i][j]);
                }
        }
        __syncthreads();
    }
    for (int i = 0; i < 4; ++i) {
        const int r = ty * 4 + i;
        if (r >= t.rows) continue;
        for (int j = 0; j < 4; ++j) {
            const int n = t.n0 + tx * 4 + j;
            if (n < a.N) lg_store(a, t.coff, t.p0 + r, n, acc[i][j], acc2[i][j], DUAL);
        }
    }
}

// bfloat16 form: A rounded to bfloat16 on its way into LDS, four waves of one 32 x 32 x 8 matrix-core tile each, k in steps of 32
template <bool DUAL>
__global__ __launch_bounds__(256) void lgemm_bf16_kernel(LGemmArgs a) {
    constexpr int BK = 32, LDS_K = BK + 8;
    __shared__ __attribute__((aligned(16))) uint16_t As[LG_BM][LDS_K];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[LG_BN][LDS_K];
    __shared__ __attribute__((aligned(16))) uint16_t B2s[DUAL ? LG_BN : 1][LDS_K];
    __shared__ int arow[LG_BM];
    __shared__ float ascl[LG_BM];
    LgTile t;
    if (!lg_tile(a, t)) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid < LG_BM) {
        int ar = -1;
        float sc = 1.f;
        if (tid < t.rows) {
            const int p = t.p0 + tid;
            ar = a.a_idx ? a.a_idx[p] / a.a_div : p;
            if (a.a_scale) sc = a.a_scale[a.a_idx[p]];
        }
        arow[tid] = ar; ascl[tid] = sc;
    }
    __syncthreads();
    const int wm = wave >> 1, wn = wave & 1;
    f32x16 acc = {}, acc2 = {};
    const int lr = tid >> 2, ks = (tid & 3) * 8;         // this thread stages 8 consecutive k of row lr
    const bool vecA = (a.lda % 4) == 0 && ((uintptr_t)t.A % 16) == 0;
    const bool vecW = (a.K % 8) == 0 && ((uintptr_t)t.W % 16) == 0 && (!DUAL || ((uintptr_t)t.W2 % 16) == 0);
    for (int k0 = 0; k0 < a.K; k0 += BK) {
        const int k = k0 + ks;
        {
            float v[8];
            const int ar = arow[lr];
            if (ar >= 0 && vecA && k + 8 <= a.K) {
                const float4 x0 = *(const float4*)(t.A + (size_t)ar * a.lda + k);
                const float4 x1 = *(const float4*)(t.A + (size_t)ar * a.lda + k + 4);
                v[0] = x0.x; v[1] = x0.y; v[2] = x0.z; v[3] = x0.w; v[4] = x1.x; v[5] = x1.y; v[6] = x1.z; v[7] = x1.w;
            } else {
                for (int i = 0; i < 8; ++i) v[i] = (ar >= 0 && k + i < a.K) ? t.A[(size_t)ar * a.lda + k + i] : 0.f;
            }
            if (a.a_scale) {
                const float sc = ascl[lr];
                for (int i = 0; i < 8; ++i) v[i] *= sc;
            }
            u32x4 pk;
            pk.x = pack_bf16x2(v[0], v[1]); pk.y = pack_bf16x2(v[2], v[3]); pk.z = pack_bf16x2(v[4], v[5]); pk.w = pack_bf16x2(v[6], v[7]);
            *(u32x4*)&As[lr][ks] = pk;
        }
        {
            const int n = t.n0 + lr;
            u32x4 pk = {0u, 0u, 0u, 0u}, pk2 = {0u, 0u, 0u, 0u};
            if (n < a.N) {
                if (vecW && k + 8 <= a.K) {
                    pk = *(const u32x4*)(t.W + (size_t)n * a.K + k);
                    if (DUAL) pk2 = *(const u32x4*)(t.W2 + (size_t)n * a.K + k);
                } else {
                    uint16_t e[8], e2[8];
                    for (int i = 0; i < 8; ++i) {
                        e[i] = k + i < a.K ? t.W[(size_t)n * a.K + k + i] : (uint16_t)0;
                        e2[i] = (DUAL && k + i < a.K) ? t.W2[(size_t)n * a.K + k + i] : (uint16_t)0;
                    }
                    pk.x = e[0] | ((uint32_t)e[1] << 16); pk.y = e[2] | ((uint32_t)e[3] << 16);
                    pk.z = e[4] | ((uint32_t)e[5] << 16); pk.w = e[6] | ((uint32_t)e[7] << 16);
                    pk2.x = e2[0] | ((uint32_t)e2[1] << 16); pk2.y = e2[2] | ((uint32_t)e2[3] << 16);
                    pk2.z = e2[4] | ((uint32_t)e2[5] << 16); pk2.w = e2[6] | ((uint32_t)e2[7] << 16);
                }
            }
            *(u32x4*)&Bs[lr][ks] = pk;
            if (DUAL) *(u32x4*)&B2s[lr][ks] = pk2;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK / 8; ++kk) {
            const int kq = kk * 8 + (lane >> 5) * 4;
            const bf16x4 av = *(const bf16x4*)&As[wm * 32 + (lane & 31)][kq];
            const bf16x4 bv = *(const bf16x4*)&Bs[wn * 32 + (lane & 31)][kq];
            acc = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(av, bv, acc, 0, 0, 0);
            if (DUAL) {
                const bf16x4 b2 = *(const bf16x4*)&B2s[wn * 32 + (lane & 31)][kq];
                acc2 = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(av, b2, acc2, 0, 0, 0);
            }
        }
        __syncthreads();
    }
    const int n = t.n0 + wn * 32 + (lane & 31);
    if (n >= a.N) return;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int r = wm * 32 + (i >> 2) * 8 + (lane >> 5) * 4 + (i & 3);
        if (r < t.rows) lg_store(a, t.coff, t.p0 + r, n, acc[i], acc2[i], DUAL);
    }
}

// few rows (decode steps): the matrix is streamed ONCE with 16-byte non-temporal loads, one wave per two output columns, every
// row of A (at most LV_MAXM, L2-resident) against each weight fragment; the wave's lanes split K.  bfloat16 format: A is rounded
// on the fly, so a row gives the same products here and in the tiled kernel.
constexpr int LV_MAXM = 8;
template <bool BF16, bool DUAL>
__global__ __launch_bounds__(256) void lgemv_kernel(LGemmArgs a) {
    const int g = blockIdx.z;
    int base = 0, rows = a.M;
    if (a.grp_off) { base = a.grp_off[g]; rows = a.grp_off[g + 1] - base; }
    if (rows <= 0) return;
    rows = min(rows, LV_MAXM);
    const uint16_t* W = a.W + (size_t)g * a.w_stride;
    const uint16_t* W2 = DUAL ? a.W2 + (size_t)g * a.w_stride : nullptr;
    const float* A = a.A + (a.grp_off ? 0 : (size_t)g * a.a_goff);
    const size_t coff = a.grp_off ? 0 : (size_t)g * a.c_goff;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n0 = (blockIdx.x * 4 + wave) * 2;
    if (n0 >= a.N) return;
    const int n1 = min(n0 + 1, a.N - 1);                 // odd N: the second column repeats the first and is not stored
    size_t ar[LV_MAXM];
    float asc[LV_MAXM];
#pragma unroll
    for (int r = 0; r < LV_MAXM; ++r) {
        const int p = base + min(r, rows - 1);
        ar[r] = (size_t)(a.a_idx ? a.a_idx[p] / a.a_div : p) * a.lda;
        asc[r] = a.a_scale ? a.a_scale[a.a_idx[p]] : 1.f;
    }
    float acc[2][LV_MAXM] = {}, acc2[2][LV_MAXM] = {};
    const int K = a.K;
    const bool vec = (K % 8) == 0 && (a.lda % 4) == 0 && ((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0 &&
                     (!DUAL || ((uintptr_t)W2 % 16) == 0);
    if (vec) {
        for (int k = lane * 8; k < K; k += 512) {
            const u32x4 w0 = ld_nt16(W + (size_t)n0 * K + k), w1 = ld_nt16(W + (size_t)n1 * K + k);
            u32x4 v0 = {0u, 0u, 0u, 0u}, v1 = {0u, 0u, 0u, 0u};
            if (DUAL) { v0 = ld_nt16(W2 + (size_t)n0 * K + k); v1 = ld_nt16(W2 + (size_t)n1 * K + k); }
#pragma unroll
            for (int r = 0; r < LV_MAXM; ++r) {
                if (r < rows) {
                    const float4 xa = *(const float4*)(A + ar[r] + k), xb = *(const float4*)(A + ar[r] + k + 4);
                    float x[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
                    if (a.a_scale) {
#pragma unroll
                        for (int i = 0; i < 8; ++i) x[i] *= asc[r];
                    }
                    if (BF16) {
#pragma unroll
                        for (int i = 0; i < 8; ++i) x[i] = bf16_round(x[i]);
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        acc[0][r] = fmaf(bf16_lo(w0[i]), x[2 * i], acc[0][r]); acc[0][r] = fmaf(bf16_hi(w0[i]), x[2 * i + 1], acc[0][r]);
                        acc[1][r] = fmaf(bf16_lo(w1[i]), x[2 * i], acc[1][r]); acc[1][r] = fmaf(bf16_hi(w1[i]), x[2 * i + 1], acc[1][r]);
                        if (DUAL) {
                            acc2[0][r] = fmaf(bf16_lo(v0[i]), x[2 * i], acc2[0][r]); acc2[0][r] = fmaf(bf16_hi(v0[i]), x[2 * i + 1], acc2[0][r]);
                            acc2[1][r] = fmaf(bf16_lo(v1[i]), x[2 * i], acc2[1][r]); acc2[1][r] = fmaf(bf16_hi(v1[i]), x[2 * i + 1], acc2[1][r]);
                        }
                    }
                }
            }
        }
    } else {
        for (int k = lane; k < K; k += 64) {
            const float w0 = bf16_to_f32(W[(size_t)n0 * K + k]), w1 = bf16_to_f32(W[(size_t)n1 * K + k]);
            const float v0 = DUAL ? bf16_to_f32(W2[(size_t)n0 * K + k]) : 0.f, v1 = DUAL ? bf16_to_f32(W2[(size_t)n1 * K + k]) : 0.f;
#pragma unroll
            for (int r = 0; r < LV_MAXM; ++r) {
                if (r < rows) {
                    float x = A[ar[r] + k] * asc[r];
                    if (BF16) x = bf16_round(x);
                    acc[0][r] = fmaf(w0, x, acc[0][r]); acc[1][r] = fmaf(w1, x, acc[1][r]);
                    if (DUAL) { acc2[0][r] = fmaf(v0, x, acc2[0][r]); acc2[1][r] = fmaf(v1, x, acc2[1][r]); }
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < LV_MAXM; ++r) {
        if (r < rows) {
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                const float v = wave_sum(acc[c][r]);
                const float v2 = DUAL ? wave_sum(acc2[c][r]) : 0.f;
                if (lane == 0 && (c == 0 || n0 + 1 < a.N)) lg_store(a, coff, base + r, n0 + c, v, v2, DUAL);
            }
        }
    }
}

// the column-range activation of a finished product, in place (products that ran on the shared GEMM kernels)
__global__ __launch_bounds__(256) void lay_act_cols_kernel(float* __restrict__ C, int ldc, int N, int act, int act2, int split, float param) {
    const int n = blockIdx.y * 256 + threadIdx.x;
    if (n >= N) return;
    float* p = C + (size_t)blockIdx.x * ldc + n;
    *p = lay_act(*p, n < split ? act : act2, param);
}
void launch_lay_act_cols(float* C, int ldc, int M, int N, int act, int act2, int split, hipStream_t s, float param) {
    if (M <= 0 || ((act == LACT_NONE || split <= 0) && (act2 == LACT_NONE || split >= N))) return;
    if (act == LACT_NONE && split > 0) { C += split; N -= split; split = 0; }       // the columns in front stay as they are: not swept
    hipLaunchKernelGGL(lay_act_cols_kernel, dim3((unsigned)M, (unsigned)((N + 255) / 256)), dim3(256), 0, s, C, ldc, N, act, act2, split, param);
}
// out = act(g) * u
__global__ __launch_bounds__(256) void lay_act_mul_kernel(const float* __restrict__ g, const float* __restrict__ u, float* __restrict__ out,
                                                          size_t n, int act, float param) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = act == LACT_CAPGLU ? lay_capglu(g[i], u[i], param) : lay_act(g[i], act) * u[i];
}
void launch_lay_act_mul(const float* g, const float* u, float* out, size_t n, int act, hipStream_t s, float param) {
    if (n == 0) return;
    hipLaunchKernelGGL(lay_act_mul_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, g, u, out, n, act, param);
}
// rows of f32 -> bfloat16 (round to nearest even): the A operand of the shared matrix-core GEMM
__global__ __launch_bounds__(256) void lay_round_rows_kernel(const float* __restrict__ x, int ldx, uint16_t* __restrict__ out, int K) {
    const float* xr = x + (size_t)blockIdx.x * ldx;
    for (int k = threadIdx.x * 2; k < K; k += 512) {
        const uint32_t pk = pack_bf16x2(xr[k], k + 1 < K ? xr[k + 1] : 0.f);
        if (k + 1 < K) *(uint32_t*)(out + (size_t)blockIdx.x * K + k) = pk;
        else out[(size_t)blockIdx.x * K + k] = (uint16_t)(pk & 0xFFFFu);
    }
}
void launch_lay_round_rows(const float* x, int ldx, uint16_t* out, int M, int K, hipStream_t s) {
    if (M <= 0) return;
    hipLaunchKernelGGL(lay_round_rows_kernel, dim3((unsigned)M), dim3(256), 0, s, x, ldx, out, K);
}

void launch_lgemm(const LGemmArgs& a, bool bf16, int groups, hipStream_t s) {
    if (a.M <= 0 || a.N <= 0 || groups <= 0) return;
    if (a.M <= LV_MAXM) {
        const dim3 gv((unsigned)((a.N + 7) / 8), 1, (unsigned)groups);
        if (bf16) {
            if (a.W2) hipLaunchKernelGGL((lgemv_kernel<true, true>), gv, dim3(256), 0, s, a);
            else hipLaunchKernelGGL((lgemv_kernel<true, false>), gv, dim3(256), 0, s, a);
        } else {
            if (a.W2) hipLaunchKernelGGL((lgemv_kernel<false, true>), gv, dim3(256), 0, s, a);
            else hipLaunchKernelGGL((lgemv_kernel<false, false>), gv, dim3(256), 0, s, a);
        }
        return;
    }
    const dim3 grid((unsigned)((a.M + LG_BM - 1) / LG_BM), (unsigned)((a.N + LG_BN - 1) / LG_BN), (unsigned)groups);
    if (bf16) {
        if (a.W2) hipLaunchKernelGGL(lgemm_bf16_kernel<true>, grid, dim3(256), 0, s, a);
        else hipLaunchKernelGGL(lgemm_bf16_kernel<false>, grid, dim3(256), 0, s, a);
    } else {
        if (a.W2) hipLaunchKernelGGL(lgemm_f32_kernel<true>, grid, dim3(256), 0, s, a);
        else hipLaunchKernelGGL(lgemm_f32_kernel<false>, grid, dim3(256), 0, s, a);
    }
}

// ------------------------------------------------------------------------------------------------------------------
// softmax attention whose values are its keys: paged key cache [n_pages][G][page][d]
// ------------------------------------------------------------------------------------------------------------------
template <int KVT>
__global__ __launch_bounds__(256) void lay_k_append_kernel(const float* __restrict__ proj, int ldp, int k_off, void* __restrict__ kpool,
                                                           const int32_t* __restrict__ bt, const LaySegDev* __restrict__ segs,
                                                           const int32_t* __restrict__ rowseg, int G, int d, int page) {
    const int r = blockIdx.x;
    const LaySegDev sg = segs[rowseg[r]];
    const int pos = sg.start_pos + (r - sg.row0);
    const int pg = bt[sg.bt_off + pos / page];
    const int n = G * d;
    for (int i = threadIdx.x; i < n; i += 256) {
        const int g = i / d, c = i - g * d;
        const size_t dst = (((size_t)pg * G + g) * page + (size_t)(pos % page)) * d + c;
        const float v = proj[(size_t)r * ldp + k_off + i];
        if (KVT == KV_F32) ((float*)kpool)[dst] = v;
        else ((uint16_t*)kpool)[dst] = f32_to_bf16(v);
    }
}
void launch_lay_k_append(const float* proj, int ldp, int k_off, void* kpool, int kvt, const int32_t* bt, const LaySegDev* segs,
                         const int32_t* rowseg, int T, int G, int d, int page, hipStream_t s) {
    if (T <= 0) return;
    if (kvt == KV_F32) hipLaunchKernelGGL(lay_k_append_kernel<KV_F32>, dim3((unsigned)T), dim3(256), 0, s, proj, ldp, k_off, kpool, bt, segs, rowseg, G, d, page);
    else hipLaunchKernelGGL(lay_k_append_kernel<KV_BF16>, dim3((unsigned)T), dim3(256), 0, s, proj, ldp, k_off, kpool, bt, segs, rowseg, G, d, page);
}

// the cached row behind entry v of a tile's key walk: [0, front) are the kept first tokens or -- pool > 0 -- the mean rows of the
// position blocks (block v lives in the page of its last position), then the window from main_lo on
struct LaRow { const char* k; const char* v; };
template <int ESZ>
__device__ __forceinline__ LaRow la_row(const LAttnArgs& a, const LaySegDev& sg, int g, int v, int front, int main_lo, int pool) {
    LaRow r;
    if (pool > 0 && v < front) {
        const int lpg = (v * pool + pool - 1) / a.page;
        const int idx = v - (int)(((long long)lpg * a.page) / pool);
        const size_t row = ((size_t)a.bt[sg.bt_off + lpg] * a.G + g) * a.pool_rows + idx;
        r.k = (const char*)a.pk_pool + row * a.d * ESZ;
        r.v = a.pv_pool ? (const char*)a.pv_pool + row * a.e * ESZ : nullptr;
    } else {
        const int j = v < front ? v : main_lo + (v - front);
        const size_t row = ((size_t)a.bt[sg.bt_off + j / a.page] * a.G + g) * a.page + (size_t)(j % a.page);
        r.k = (const char*)a.kpool + row * a.d * ESZ;
        const size_t vrow = a.v_div > 1 ? ((size_t)a.bt[sg.bt_off + j / a.page] * (a.G / a.v_div) + g / a.v_div) * a.page + (size_t)(j % a.page) : row;
        r.v = a.vpool ? (const char*)a.vpool + vrow * a.e * ESZ : nullptr;
    }
    return r;
}

// the mean row of the block of `pool` positions that ends at pos: f32 sum in position order, one rounding into the cache's format
template <int KVT>
__device__ __forceinline__ void lay_block_mean(const void* __restrict__ src, void* __restrict__ dstp, int n, const int32_t* __restrict__ bt,
                                               int bt_off, int pos, int G, int page, int pool, int pool_rows) {
    const int b = (pos + 1) / pool - 1, lpg = pos / page;
    const int idx = b - (int)(((long long)lpg * page) / pool);
    const float inv = 1.f / (float)pool;
    for (int i = threadIdx.x; i < G * n; i += 256) {
        const int g = i / n, c = i - g * n;
        float sum = 0.f;
        // page by page: one table look-up, then rows at a fixed stride, so that several loads are in flight; the sum keeps position order
        for (int j0 = b * pool; j0 <= pos;) {
            const int j1 = min(pos + 1, (j0 / page + 1) * page);
            const size_t at = (((size_t)bt[bt_off + j0 / page] * G + g) * page + (size_t)(j0 % page)) * n + c;
#pragma unroll 8
            for (int j = 0; j < j1 - j0; ++j)
                sum += KVT == KV_F32 ? ((const float*)src)[at + (size_t)j * n] : bf16_to_f32(((const uint16_t*)src)[at + (size_t)j * n]);
            j0 = j1;
        }
        const size_t dst = (((size_t)bt[bt_off + lpg] * G + g) * pool_rows + idx) * n + c;
        if (KVT == KV_F32) ((float*)dstp)[dst] = sum * inv;
        else ((uint16_t*)dstp)[dst] = f32_to_bf16(sum * inv);
    }
}
// one block per row of the pass (blockIdx.y: keys / values); a row whose position closes a block of `pool` positions writes the block's
// mean row (f32 sum in position order, then one rounding into the cache's format)
template <int KVT>
__global__ __launch_bounds__(256) void lay_pool_append_kernel(const void* __restrict__ kpool, void* __restrict__ pk_pool, int d,
                                                              const void* __restrict__ vpool, void* __restrict__ pv_pool, int e,
                                                              const int32_t* __restrict__ bt, const LaySegDev* __restrict__ segs,
                                                              const int32_t* __restrict__ rowseg, int G, int page, int pool, int pool_rows) {
    const int r = blockIdx.x;
    const LaySegDev sg = segs[rowseg[r]];
    const int pos = sg.start_pos + (r - sg.row0);
    if ((pos + 1) % pool != 0) return;
    if (blockIdx.y) lay_block_mean<KVT>(vpool, pv_pool, e, bt, sg.bt_off, pos, G, page, pool, pool_rows);
    else lay_block_mean<KVT>(kpool, pk_pool, d, bt, sg.bt_off, pos, G, page, pool, pool_rows);
}
void launch_lay_pool_append(const void* kpool, void* pk_pool, int d, const void* vpool, void* pv_pool, int e, int kvt, const int32_t* bt,
                            const LaySegDev* segs, const int32_t* rowseg, int T, int G, int page, int pool, int pool_rows, hipStream_t s) {
    if (T <= 0 || pool <= 0) return;
    const dim3 grid((unsigned)T, vpool ? 2u : 1u);
    if (kvt == KV_F32) hipLaunchKernelGGL(lay_pool_append_kernel<KV_F32>, grid, dim3(256), 0, s, kpool, pk_pool, d, vpool, pv_pool, e, bt, segs, rowseg, G, page, pool, pool_rows);
    else hipLaunchKernelGGL(lay_pool_append_kernel<KV_BF16>, grid, dim3(256), 0, s, kpool, pk_pool, d, vpool, pv_pool, e, bt, segs, rowseg, G, page, pool, pool_rows);
}

// Queries and keys on their way into attention, one block per row of the pass: RMS norm over all query heads at once and over all
// key heads at once (weights qn / kn; null: none), rotation by position (pairs (2i, 2i + 1) or (i, i + dims / 2) of the first dims
// elements of each head), q back in place, the key row -- and the value row at v_off, when vpool is given -- into the sequence's pages.
struct LQkPrepArgs {
    float* proj; int ldp, q_off, k_off, v_off;
    int H, G, d, e;
    const float *qn, *kn; float eps;
    int dims, half; const float* freq; float mag;
    void *kpool, *vpool;
    const int32_t* bt; const LaySegDev* segs; const int32_t* rowseg; int page;
    // pool > 0: every portion of the pass is ONE token, and a row that closes a block of `pool` positions also writes the block's mean
    // rows (the other positions of the block were cached by earlier passes; its own by this block)
    int pool, pool_rows; void *pk_pool, *pv_pool;
    // head_norm: every head over its own root mean square, weights [d] shared by the heads (head_rs: a place per head, H + G of them);
    // Gv value heads; qt_coef != 0: the query times 1 + qt_coef ln(floor((pos + 1) / qt_every) + 1)
    int head_norm, Gv; float qt_coef; int qt_every;
};
constexpr int LQK_MAX_HEADS = 1024;
template <int KVT>
__global__ __launch_bounds__(256) void lay_qk_prep_kernel(LQkPrepArgs a) {
    __shared__ float red[4];
    __shared__ float head_rs[LQK_MAX_HEADS];
    const int r = blockIdx.x, tid = threadIdx.x;
    const LaySegDev sg = a.segs[a.rowseg[r]];
    const int pos = sg.start_pos + (r - sg.row0);
    float* q = a.proj + (size_t)r * a.ldp + a.q_off;
    float* k = a.proj + (size_t)r * a.ldp + a.k_off;
    const int nq = a.H * a.d, nk = a.G * a.d;
    float rq = 1.f, rk = 1.f;
    if (a.head_norm) {                     // one wave per head: its own root mean square
        for (int v = tid >> 6; v < a.H + a.G; v += 4) {
            const float* x = v < a.H ? q + v * a.d : k + (v - a.H) * a.d;
            float ss = 0.f;
            for (int i = tid & 63; i < a.d; i += 64) ss += x[i] * x[i];
            ss = wave_sum(ss);
            if ((tid & 63) == 0) head_rs[v] = 1.f / sqrtf(ss / (float)a.d + a.eps);
        }
        __syncthreads();
    } else if (a.qn) {
        float ss = 0.f;
        for (int i = tid; i < nq; i += 256) { const float v = q[i]; ss += v * v; }
        rq = 1.f / sqrtf(block_sum(ss, red) / (float)nq + a.eps);
    }
    if (a.kn && !a.head_norm) {
        float ss = 0.f;
        for (int i = tid; i < nk; i += 256) { const float v = k[i]; ss += v * v; }
        rk = 1.f / sqrtf(block_sum(ss, red) / (float)nk + a.eps);
    }
    const float qt = a.qt_coef != 0.f ? 1.f + a.qt_coef * logf((float)((pos + 1) / a.qt_every) + 1.f) : 1.f;
    const int pg = a.bt[sg.bt_off + pos / a.page];
    const size_t prow = (size_t)pg * a.G * a.page + (size_t)(pos % a.page);       // + g * page: the cached row of key head g
    // a thread owns both elements of a pair (or one element past the rotated part)
    const int hd = a.dims / 2, per = hd + (a.d - a.dims);
    const float fpos = (float)pos;
    for (int idx = tid; idx < (a.H + a.G) * per; idx += 256) {
        const int v = idx / per, i = idx - v * per;
        const bool isq = v < a.H;
        const int hh = isq ? v : v - a.H;
        float* x = (isq ? q : k) + hh * a.d;
        const float* w = isq ? a.qn : a.kn;
        const float rs = (a.head_norm ? head_rs[v] : (isq ? rq : rk)) * (isq ? qt : 1.f);
        int i0, i1 = -1;
        if (i < hd) { i0 = a.half ? i : 2 * i; i1 = a.half ? i + hd : 2 * i + 1; }
        else i0 = a.dims + (i - hd);
        float x0 = x[i0] * rs, x1 = i1 >= 0 ? x[i1] * rs : 0.f;
        if (w) {
            const int wo = a.head_norm ? 0 : hh * a.d;
            x0 *= w[wo + i0];
            if (i1 >= 0) x1 *= w[wo + i1];
        }
        if (i1 >= 0) {
            float sn, cs;
            sincosf(fpos * a.freq[i], &sn, &cs);
            sn *= a.mag; cs *= a.mag;
            const float y0 = x0 * cs - x1 * sn, y1 = x1 * cs + x0 * sn;
            x0 = y0; x1 = y1;
        }
        if (isq) { x[i0] = x0; if (i1 >= 0) x[i1] = x1; }
        else {
            const size_t dst = (prow + (size_t)hh * a.page) * a.d;
            if (KVT == KV_F32) { ((float*)a.kpool)[dst + i0] = x0; if (i1 >= 0) ((float*)a.kpool)[dst + i1] = x1; }
            else { ((uint16_t*)a.kpool)[dst + i0] = f32_to_bf16(x0); if (i1 >= 0) ((uint16_t*)a.kpool)[dst + i1] = f32_to_bf16(x1); }
        }
    }
    if (a.vpool) {
        const float* vv = a.proj + (size_t)r * a.ldp + a.v_off;
        const size_t vrow = (size_t)pg * a.Gv * a.page + (size_t)(pos % a.page);
        for (int i = tid; i < a.Gv * a.e; i += 256) {
            const int g = i / a.e, c = i - g * a.e;
            const size_t dst = (vrow + (size_t)g * a.page) * a.e + c;
            if (KVT == KV_F32) ((float*)a.vpool)[dst] = vv[i];
            else ((uint16_t*)a.vpool)[dst] = f32_to_bf16(vv[i]);
        }
    }
    if (a.pool > 0 && (pos + 1) % a.pool == 0) {
        __threadfence_block();             // this block's own cached row is read back below
        __syncthreads();
        lay_block_mean<KVT>(a.kpool, a.pk_pool, a.d, a.bt, sg.bt_off, pos, a.G, a.page, a.pool, a.pool_rows);
        if (a.vpool && a.pv_pool) lay_block_mean<KVT>(a.vpool, a.pv_pool, a.e, a.bt, sg.bt_off, pos, a.G, a.page, a.pool, a.pool_rows);
    }
}
void launch_lay_qk_prep(float* proj, int ldp, int q_off, int k_off, int v_off, int H, int G, int d, int e, const float* qn, const float* kn,
                        float eps, int dims, bool half, const float* freq, float mag, void* kpool, void* vpool, int kvt, const int32_t* bt,
                        const LaySegDev* segs, const int32_t* rowseg, int T, int page, hipStream_t s, int pool, int pool_rows, void* pk_pool,
                        void* pv_pool, const LQkPrepExtra* extra) {
    if (T <= 0) return;
    const LQkPrepExtra x = extra ? *extra : LQkPrepExtra();
    LQkPrepArgs a{proj, ldp, q_off, k_off, v_off, H, G, d, e, qn, kn, eps, freq ? dims : 0, half ? 1 : 0, freq, mag, kpool, vpool, bt, segs, rowseg, page,
                  pk_pool ? pool : 0, pool_rows, pk_pool, pv_pool, x.head_norm && H + G <= LQK_MAX_HEADS ? 1 : 0, x.Gv > 0 ? x.Gv : G, x.qt_coef,
                  x.qt_every > 0 ? x.qt_every : 1};
    if (kvt == KV_F32) hipLaunchKernelGGL(lay_qk_prep_kernel<KV_F32>, dim3((unsigned)T), dim3(256), 0, s, a);
    else hipLaunchKernelGGL(lay_qk_prep_kernel<KV_BF16>, dim3((unsigned)T), dim3(256), 0, s, a);
}

// A block = 16 query rows of one sequence and one key head: row qi = (position in the portion) * nrep + (query head in the
// group), so that a single decode token fills the tile with the heads that share its keys.  16 lanes per query row.
// Keys the tile can see: the kept first tokens [0, min(keep, lo)) and the window [lo, last position], lo not before the start of
// the first query's position block when the mask is chunked; each query masks with its own position.  Values: pages of their own
// ([..][e]) or the first e elements of the key rows.  A sink adds exp(sink) to the denominator: it is the start value of the running
// (max, sum) pair of the first split.  Scores, softmax and the weighted sum are f32.
constexpr int LA_BQ = 16;
constexpr size_t LDS_PLAIN = 64 * 1024, LDS_MAX = 160 * 1024;    // without / with the kernel's dynamic-LDS attribute raised
template <int KVT, int KT, int NACC>
__global__ __launch_bounds__(256) void lay_attn_kernel(LAttnArgs a) {
    extern __shared__ float lds[];
    const int d = a.d, e = a.e, ldk = d + 1;
    const bool ownv = a.vpool != nullptr;
    const int ldq = d + 1, ldps = KT + 1;  // odd strides: the four query rows of a wave read four different banks
    float* qs = lds;                       // [16][d + 1]
    float* ks = qs + LA_BQ * ldq;          // [KT][d + 1]
    float* vs = ks + KT * ldk;             // [KT][e], own value pages only
    float* ps = vs + (ownv ? KT * e : 0);  // [16][KT + 1]
    const float* vt = ownv ? vs : ks;
    const int ldv = ownv ? e : ldk;
    const int2 tile = a.tiles[blockIdx.x];
    const LaySegDev sg = a.segs[tile.x];
    const int g = blockIdx.y, nrep = a.H / a.G;
    const int q0 = tile.y, nq = min(LA_BQ, sg.n * nrep - q0);
    const int tid = threadIdx.x, qr = tid >> 4, ln = tid & 15;
    const bool qvalid = qr < nq;
    const int qi = q0 + (qvalid ? qr : 0);
    const int lp = qi / nrep, head = g * nrep + (qi - lp * nrep);
    const int pos = sg.start_pos + lp;
    const int row = sg.row0 + lp;
    const int win = (int)min(a.win, 1ll << 30), keep = (int)min(a.keep, 1ll << 30), chunk = (int)min(a.chunk, 1ll << 30);
    for (int i = ln; i < d; i += 16) qs[qr * ldq + i] = qvalid ? a.proj[(size_t)row * a.ldp + a.q_off + head * d + i] : 0.f;
    const int pmin = sg.start_pos + q0 / nrep, pmax = sg.start_pos + (q0 + nq - 1) / nrep;
    int main_lo = max(0, pmin - win + 1);
    if (chunk > 0) main_lo = max(main_lo, pmin / chunk * chunk);
    const int clo = chunk > 0 ? pos / chunk * chunk : 0;       // first position of this query's block
    const int pool = (int)min(a.pool, 1ll << 30);
    const int sink_hi = pool > 0 ? max(0, (pmax - win + 1) / pool) : min(keep, main_lo);
    const int total = sink_hi + (pmax - main_lo + 1);
    const float r1 = a.bias != LBIAS_NONE ? a.r1[head] : 0.f, r2 = a.bias == LBIAS_LOG ? a.r2[head] : 0.f;
    float m = -INFINITY, l = 0.f, acc[NACC];
    if (a.sink && blockIdx.z == 0 && qvalid) { m = a.sink[head]; l = 1.f; }
#pragma unroll
    for (int c = 0; c < NACC; ++c) acc[c] = 0.f;
    const int nsplit = (int)gridDim.z;     // the visible keys' tiles are dealt round-robin to nsplit blocks (few queries, many keys)
    __syncthreads();                       // qs written (a split may have no tile at all)
    for (int v0 = (int)blockIdx.z * KT; v0 < total; v0 += KT * nsplit) {
        __syncthreads();                   // previous tile fully consumed
        for (int rr = 0; rr < KT / 16; ++rr) {
            const int sl = qr + 16 * rr;
            const int v = v0 + sl;
            if (v < total) {
                const LaRow cr = la_row<(KVT == KV_F32 ? 4 : 2)>(a, sg, g, v, sink_hi, main_lo, pool);
                const char* src = cr.k;
                if (KVT != KV_F32 && (d & 7) == 0) {             // 16 bytes = 8 cached keys per lane and load
                    for (int i = ln * 8; i < d; i += 128) {
                        const u32x4 p = *(const u32x4*)((const uint16_t*)src + i);
                        float* dst = ks + sl * ldk + i;
                        dst[0] = bf16_lo(p.x); dst[1] = bf16_hi(p.x); dst[2] = bf16_lo(p.y); dst[3] = bf16_hi(p.y);
                        dst[4] = bf16_lo(p.z); dst[5] = bf16_hi(p.z); dst[6] = bf16_lo(p.w); dst[7] = bf16_hi(p.w);
                    }
                } else
                for (int i = ln; i < d; i += 16)
                    ks[sl * ldk + i] = KVT == KV_F32 ? ((const float*)src)[i] : bf16_to_f32(((const uint16_t*)src)[i]);
                if (ownv) {
                    const char* vsrc = cr.v;
                    for (int i = ln; i < e; i += 16)
                        vs[sl * e + i] = KVT == KV_F32 ? ((const float*)vsrc)[i] : bf16_to_f32(((const uint16_t*)vsrc)[i]);
                }
            } else {
                for (int i = ln; i < d; i += 16) ks[sl * ldk + i] = 0.f;
                if (ownv) for (int i = ln; i < e; i += 16) vs[sl * e + i] = 0.f;
            }
        }
        __syncthreads();
        float sc[KT / 16];
        float tmax = -INFINITY;
#pragma unroll
        for (int c = 0; c < KT / 16; ++c) {
            const int sl = ln + 16 * c;
            const int v = v0 + sl;
            const int j = v < sink_hi ? v : main_lo + (v - sink_hi);
            float dot = 0.f;
            for (int i = 0; i < d; ++i) dot = fmaf(qs[qr * ldq + i], ks[sl * ldk + i], dot);
            const int dist = pos - j;
            const bool pl = pool > 0 && v < sink_hi;       // a block's mean row: seen once the whole block lies in front of the window
            const bool vis = pl ? qvalid && (v + 1) * pool <= pos - win + 1
                                : qvalid && v < total && dist >= 0 && ((dist < win && j >= clo) || j < keep);
            const float pen = pl ? 0.f : (a.bias == LBIAS_LOG ? r1 * log1pf(r2 * (float)dist) : r1 * (float)dist);
            sc[c] = vis ? dot * a.scale - pen : -INFINITY;
            tmax = fmaxf(tmax, sc[c]);
        }
        tmax = row16_max(tmax);
        const float mn = fmaxf(m, tmax);
        const float corr = mn == -INFINITY ? 1.f : expf(m - mn);     // m = -inf, mn finite: exp(-inf) = 0
        float psum = 0.f;
#pragma unroll
        for (int c = 0; c < KT / 16; ++c) {
            const float p = sc[c] == -INFINITY ? 0.f : expf(sc[c] - mn);
            ps[qr * ldps + ln + 16 * c] = p;
            psum += p;
        }
        psum = row16_sum(psum);
        l = l * corr + psum;
        m = mn;
        __syncthreads();
        const int kn = min(KT, total - v0);
#pragma unroll
        for (int c = 0; c < NACC; ++c) {
            const int i = ln + 16 * c;
            if (i < e) {
                float o = acc[c] * corr;
                for (int sl = 0; sl < kn; ++sl) o = fmaf(ps[qr * ldps + sl], vt[sl * ldv + i], o);
                acc[c] = o;
            }
        }
    }
    if (nsplit > 1) {                      // un-normalised partial sums + (running max, running sum) for the merge
        const size_t pr = (((size_t)blockIdx.x * a.G + g) * nsplit + blockIdx.z) * LA_BQ + qr;
        if (ln == 0) { a.part_ml[pr * 2] = m; a.part_ml[pr * 2 + 1] = l; }
#pragma unroll
        for (int c = 0; c < NACC; ++c) {
            const int i = ln + 16 * c;
            if (i < e) a.part_o[pr * e + i] = acc[c];
        }
        return;
    }
    if (!qvalid) return;
    const float* gp = a.proj + (size_t)row * a.ldp + a.g_off + (a.gate == LGATE_ELEM ? head * e : head);
    const float inv = (a.gate == LGATE_HEAD ? gp[0] : 1.f) / l * a.out_scale;
#pragma unroll
    for (int c = 0; c < NACC; ++c) {
        const int i = ln + 16 * c;
        if (i < e) a.out[(size_t)row * a.ldo + head * e + i] = acc[c] * inv * (a.gate == LGATE_ELEM ? gp[i] : 1.f);
    }
}
// Matrix-core form for prompt passes in the bfloat16 format (key and value sizes multiples of 16, up to 128; values from pages of
// their own or the first e elements of the keys; the same masks, distance terms, sink and gates as lay_attn_kernel): LAY_ATTN_MFMA_ROWS query rows per
// block, one wave per 16 of them, 64-key tiles (32-row blocks, two or three resident per CU, measured slower: 474 against 423 us for 2048 tokens).  S = Q K^T from the bf16-rounded q and the cached bf16 keys (exact products, f32 sums);
// mask, distance penalty, running max / sum and the weights stay f32 as in lay_attn_kernel; the weights enter P V (V = K) as a
// bf16 hi + lo pair, two products per tile, so that they keep 16 significand bits; exp and log are the hardware's (v_exp_f32 /
// v_log_f32, about 1e-6 relative: the format's own rounding is three orders above that).  Fragment layout of v_mfma_f32_16x16x16_bf16:
// A[i = lane % 16][k = 4 (lane / 16) ..], B[k = 4 (lane / 16) ..][j = lane % 16], D[i = 4 (lane / 16) + r][j = lane % 16].
constexpr int LM_BQ = LAY_ATTN_MFMA_ROWS, LM_KT = 64, LM_NT = LM_BQ * 4, LM_NW = LM_BQ / 16;    // threads, waves
// NDMAX / NEMAX: key / value size in units of 16 the registers are laid out for (q fragments, output tiles).  WIDE: long cached rows
// whose values are their own first e elements (latent attention: [latent | rotated key part]); the key tile takes the place of the
// staged queries, and the B operand of P V (4 keys of one element) is gathered from the key rows instead of a transposed copy.
template <int NDMAX, int NEMAX, bool WIDE>
__global__ __launch_bounds__(LM_NT) void lay_attn_mfma_kernel(LAttnArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
    const int d = a.d, e = a.e, ldq = d + 8, ldp = LM_KT + 8;
    const bool ownv = a.vpool != nullptr;
    uint16_t* Qs = smem;                              // [rows][d + 8] until the q fragments sit in registers, then:
    uint16_t* Kt = smem;                              // [e][72] the value tile transposed (the B operand of P V: 4 keys of one element)
    uint16_t* Ks = WIDE ? smem : smem + max(LM_BQ * ldq, e * ldp);  // [64][d + 8]
    uint16_t* Ph = Ks + LM_KT * ldq;                  // [waves][16][72] hi
    uint16_t* Pl = Ph + LM_NW * 16 * ldp;                 // ... lo
    const int2 tile = a.tiles[blockIdx.x];
    const LaySegDev sg = a.segs[tile.x];
    const int g = blockIdx.y, nrep = a.H / a.G;
    const int q0 = tile.y, nq = min(LM_BQ, sg.n * nrep - q0);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, lr = lane & 15, lg = lane >> 4;
    const int win = (int)min(a.win, 1ll << 30), keep = (int)min(a.keep, 1ll << 30), chunk = (int)min(a.chunk, 1ll << 30);
    // q rows -> bf16
    for (int idx = tid; idx < LM_BQ * (d / 4); idx += LM_NT) {
        const int qr = idx / (d / 4), i = (idx - qr * (d / 4)) * 4;
        u32x2 pk = {0u, 0u};
        if (qr < nq) {
            const int qi = q0 + qr, lp = qi / nrep, head = g * nrep + (qi - lp * nrep);
            const float* src = a.proj + (size_t)(sg.row0 + lp) * a.ldp + a.q_off + head * d + i;
            pk.x = pack_bf16x2(src[0], src[1]); pk.y = pack_bf16x2(src[2], src[3]);
        }
        *(u32x2*)&Qs[qr * ldq + i] = pk;
    }
    // this lane's four query rows (accumulator rows 4 lg + r of the wave's 16)
    int qpos[4], qhead[4], qrow[4], qclo[4]; bool qok[4]; float r1[4], r2[4];
    float m[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY}, l[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int qr = wave * 16 + 4 * lg + r;
        qok[r] = qr < nq;
        const int qi = q0 + (qok[r] ? qr : 0), lp = qi / nrep;
        qhead[r] = g * nrep + (qi - lp * nrep);
        qpos[r] = sg.start_pos + lp;
        qclo[r] = chunk > 0 ? qpos[r] / chunk * chunk : 0;
        qrow[r] = sg.row0 + lp;
        r1[r] = a.bias != LBIAS_NONE ? a.r1[qhead[r]] : 0.f; r2[r] = a.bias == LBIAS_LOG ? a.r2[qhead[r]] : 0.f;
        if (a.sink && qok[r]) { m[r] = a.sink[qhead[r]]; l[r] = 1.f; }      // exp(sink - m) with m = sink
    }
    const int pmin = sg.start_pos + q0 / nrep, pmax = sg.start_pos + (q0 + nq - 1) / nrep;
    int main_lo = max(0, pmin - win + 1);
    if (chunk > 0) main_lo = max(main_lo, pmin / chunk * chunk);
    const int pool = (int)min(a.pool, 1ll << 30);
    const int sink_hi = pool > 0 ? max(0, (pmax - win + 1) / pool) : min(keep, main_lo);
    const int total = sink_hi + (pmax - main_lo + 1);
    f32x4 O[NEMAX];
#pragma unroll
    for (int n = 0; n < NEMAX; ++n) O[n] = (f32x4){0.f, 0.f, 0.f, 0.f};
    const int nd = d / 16, ne = e / 16;
    uint16_t* ph = Ph + wave * 16 * ldp;
    uint16_t* pl = Pl + wave * 16 * ldp;
    __syncthreads();                       // Qs written
    bf16x4 qf[NDMAX];
#pragma unroll
    for (int kk = 0; kk < NDMAX; ++kk)
        qf[kk] = kk < nd ? *(const bf16x4*)&Qs[(wave * 16 + lr) * ldq + kk * 16 + 4 * lg] : (bf16x4){0, 0, 0, 0};
    // the cached rows behind the entries of a tile's key walk (null past the end), looked up one tile ahead so that the tile's loads
    // do not wait for the page table
    __shared__ LaRow rowp[2][LM_KT];
    auto look_up = [&](int v0, int buf) {
        if (tid < LM_KT) {
            const int v = v0 + tid;
            rowp[buf][tid] = v < total ? la_row<2>(a, sg, g, v, sink_hi, main_lo, pool) : LaRow{nullptr, nullptr};
        }
    };
    auto transposed = [&](const u32x4& pk, int i, int sl) {
        uint16_t* kt = Kt + i * ldp + sl;
        kt[0] = (uint16_t)(pk.x & 0xFFFFu); kt[ldp] = (uint16_t)(pk.x >> 16);
        kt[2 * ldp] = (uint16_t)(pk.y & 0xFFFFu); kt[3 * ldp] = (uint16_t)(pk.y >> 16);
        kt[4 * ldp] = (uint16_t)(pk.z & 0xFFFFu); kt[5 * ldp] = (uint16_t)(pk.z >> 16);
        kt[6 * ldp] = (uint16_t)(pk.w & 0xFFFFu); kt[7 * ldp] = (uint16_t)(pk.w >> 16);
    };
    look_up(0, 0);
    const int nkl = LM_KT * (d / 8), nvl = LM_KT * (e / 8);
    for (int v0 = 0, buf = 0; v0 < total; v0 += LM_KT, buf ^= 1) {
        __syncthreads();                   // previous tile consumed (first round: q fragments read, Qs free for Kt)
        look_up(v0 + LM_KT, buf ^ 1);
        // four independent 16-byte loads in flight per thread, then their stores
        for (int base = 0; base < nkl; base += 4 * LM_NT) {
            u32x4 pk[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int idx = base + c * LM_NT + tid;
                pk[c] = (u32x4){0u, 0u, 0u, 0u};
                if (idx < nkl) {
                    const int sl = idx / (d / 8), i = (idx - sl * (d / 8)) * 8;
                    const char* src = rowp[buf][sl].k;
                    if (src) pk[c] = *(const u32x4*)((const uint16_t*)src + i);
                }
            }
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int idx = base + c * LM_NT + tid;
                if (idx < nkl) {
                    const int sl = idx / (d / 8), i = (idx - sl * (d / 8)) * 8;
                    *(u32x4*)&Ks[sl * ldq + i] = pk[c];
                    if (!WIDE && !ownv && i < e) transposed(pk[c], i, sl);
                }
            }
        }
        if (!WIDE && ownv)
            for (int base = 0; base < nvl; base += 4 * LM_NT) {
                u32x4 pk[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const int idx = base + c * LM_NT + tid;
                    pk[c] = (u32x4){0u, 0u, 0u, 0u};
                    if (idx < nvl) {
                        const int sl = idx / (e / 8), i = (idx - sl * (e / 8)) * 8;
                        const char* src = rowp[buf][sl].v;
                        if (src) pk[c] = *(const u32x4*)((const uint16_t*)src + i);
                    }
                }
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const int idx = base + c * LM_NT + tid;
                    if (idx < nvl) { const int sl = idx / (e / 8), i = (idx - sl * (e / 8)) * 8; transposed(pk[c], i, sl); }
                }
            }
        __syncthreads();
        f32x4 S[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) S[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < NDMAX; ++kk) {
            if (kk < nd) {
                const bf16x4 qa = qf[kk];
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const bf16x4 kb = *(const bf16x4*)&Ks[(t * 16 + lr) * ldq + kk * 16 + 4 * lg];
                    S[t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(qa, kb, S[t], 0, 0, 0);
                }
            }
        }
        float corr[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float sc[4], tmax = -INFINITY;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const int v = v0 + t * 16 + lr;
                const int j = v < sink_hi ? v : main_lo + (v - sink_hi);
                const int dist = qpos[r] - j;
                const bool pl = pool > 0 && v < sink_hi;
                const bool vis = pl ? qok[r] && (v + 1) * pool <= qpos[r] - win + 1
                                    : qok[r] && v < total && dist >= 0 && ((dist < win && j >= qclo[r]) || j < keep);
                const float pen = pl ? 0.f : (a.bias == LBIAS_LOG ? r1[r] * __logf(1.f + r2[r] * (float)dist) : r1[r] * (float)dist);
                sc[t] = vis ? S[t][r] * a.scale - pen : -INFINITY;
                tmax = fmaxf(tmax, sc[t]);
            }
            tmax = row16_max(tmax);
            const float mn = fmaxf(m[r], tmax);
            corr[r] = mn == -INFINITY ? 1.f : __expf(m[r] - mn);
            float psum = 0.f;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
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
        for (int ks = 0; ks < 4; ++ks) {
            const bf16x4 ah = *(const bf16x4*)&ph[lr * ldp + ks * 16 + 4 * lg];
            const bf16x4 al = *(const bf16x4*)&pl[lr * ldp + ks * 16 + 4 * lg];
#pragma unroll
            for (int n = 0; n < NEMAX; ++n) {
                if (n < ne) {
                    bf16x4 vb;
                    if (WIDE) {
                        const uint16_t* kc = Ks + (ks * 16 + 4 * lg) * ldq + n * 16 + lr;
                        vb = (bf16x4){(short)kc[0], (short)kc[ldq], (short)kc[2 * ldq], (short)kc[3 * ldq]};
                    } else vb = *(const bf16x4*)&Kt[(n * 16 + lr) * ldp + ks * 16 + 4 * lg];
                    O[n] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(ah, vb, O[n], 0, 0, 0);
                    O[n] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(al, vb, O[n], 0, 0, 0);
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        if (!qok[r]) continue;
        const float* gp = a.proj + (size_t)qrow[r] * a.ldp + a.g_off + (a.gate == LGATE_ELEM ? qhead[r] * e : qhead[r]);
        const float inv = (a.gate == LGATE_HEAD ? gp[0] : 1.f) / l[r] * a.out_scale;
#pragma unroll
        for (int n = 0; n < NEMAX; ++n)
            if (n < ne) a.out[(size_t)qrow[r] * a.ldo + qhead[r] * e + n * 16 + lr] = O[n][r] * inv * (a.gate == LGATE_ELEM ? gp[n * 16 + lr] : 1.f);
    }
}
bool lay_attn_mfma_fits(int d, int e, bool own_v) {
    if (d <= 0 || e <= 0 || d % 16 || e % 16) return false;
    if (d <= 128 && e <= 128) return own_v || e <= d;
    return !own_v && e <= d && d <= 640 && e <= 512;      // the wide form
}
template <int NDMAX, int NEMAX, bool WIDE>
static void lay_attn_mfma_go(const LAttnArgs& a, size_t lds, hipStream_t s) {
    if (lds > LDS_PLAIN) {
        static bool raised = false;        // per instantiation
        if (!raised) {
            (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&lay_attn_mfma_kernel<NDMAX, NEMAX, WIDE>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_MAX);
            raised = true;
        }
    }
    hipLaunchKernelGGL((lay_attn_mfma_kernel<NDMAX, NEMAX, WIDE>), dim3((unsigned)a.ntiles, (unsigned)a.G), dim3(LM_NT), lds, s, a);
}
void launch_lay_attn_mfma(const LAttnArgs& a0, hipStream_t s) {
    if (a0.ntiles <= 0) return;
    LAttnArgs a = a0;
    if (a.e <= 0) a.e = a.d;
    const size_t pbytes = (size_t)2 * LM_NW * 16 * (LM_KT + 8);
    if (a.d <= 128 && a.e <= 128) {
        const size_t lds = ((size_t)std::max(LM_BQ * (a.d + 8), a.e * (LM_KT + 8)) + (size_t)LM_KT * (a.d + 8) + pbytes) * sizeof(uint16_t);
        lay_attn_mfma_go<8, 8, false>(a, lds, s);
        return;
    }
    const size_t lds = ((size_t)std::max(LM_BQ, LM_KT) * (a.d + 8) + pbytes) * sizeof(uint16_t);
    if (a.d <= 320 && a.e <= 256) lay_attn_mfma_go<20, 16, true>(a, lds, s);
    else lay_attn_mfma_go<40, 32, true>(a, lds, s);
}

// merge of the splits of a tile: out = sum_z acc_z e^(m_z - M) / sum_z l_z e^(m_z - M) * gate; one thread per (query row, element)
__global__ __launch_bounds__(256) void lay_attn_merge_kernel(LAttnArgs a, int nsplit) {
    const int2 tile = a.tiles[blockIdx.x];
    const LaySegDev sg = a.segs[tile.x];
    const int g = blockIdx.y, nrep = a.H / a.G, d = a.e;
    const int q0 = tile.y, nq = min(LA_BQ, sg.n * nrep - q0);
    const size_t t0 = ((size_t)blockIdx.x * a.G + g) * nsplit * LA_BQ;
    for (int idx = blockIdx.z * 256 + threadIdx.x; idx < nq * d; idx += 256 * gridDim.z) {
        const int qr = idx / d, i = idx - qr * d;
        const int qi = q0 + qr, lp = qi / nrep, head = g * nrep + (qi - lp * nrep), row = sg.row0 + lp;
        float M = -INFINITY;
#pragma unroll 8
        for (int z = 0; z < nsplit; ++z) M = fmaxf(M, a.part_ml[(t0 + (size_t)z * LA_BQ + qr) * 2]);
        float L = 0.f, acc = 0.f;
#pragma unroll 8
        for (int z = 0; z < nsplit; ++z) {
            const size_t pr = t0 + (size_t)z * LA_BQ + qr;
            const float mz = a.part_ml[pr * 2];
            const float w = mz == -INFINITY ? 0.f : expf(mz - M);
            L = fmaf(a.part_ml[pr * 2 + 1], w, L);
            acc = fmaf(a.part_o[pr * d + i], w, acc);
        }
        const float gate = a.gate == LGATE_NONE ? 1.f : a.proj[(size_t)row * a.ldp + a.g_off + (a.gate == LGATE_ELEM ? head * d + i : head)];
        a.out[(size_t)row * a.ldo + head * d + i] = acc * gate / L * a.out_scale;
    }
}
static size_t lay_attn_lds(int d, int e, bool own_v, int KT) {
    return (size_t)(LA_BQ * (d + 1) + KT * (d + 1) + (own_v ? KT * e : 0) + LA_BQ * (KT + 1)) * sizeof(float);
}
int lay_attn_key_tile(int d, int e, bool own_v);
bool lay_attn_fits(int d, int e, bool own_v) {
    return d > 0 && e > 0 && e <= 512 && (own_v || e <= d) && lay_attn_lds(d, e, own_v, 32) <= LDS_MAX;
}
template <int KVT, int KT, int NACC>
static void lay_attn_go(const LAttnArgs& a, dim3 grid, size_t lds, hipStream_t s) {
    if (lds > LDS_PLAIN) {
        static bool raised = false;        // per instantiation
        if (!raised) {
            (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&lay_attn_kernel<KVT, KT, NACC>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      (int)LDS_MAX);
            raised = true;
        }
    }
    hipLaunchKernelGGL((lay_attn_kernel<KVT, KT, NACC>), grid, dim3(256), lds, s, a);
}
void launch_lay_attn(const LAttnArgs& a0, int kvt, hipStream_t s) {
    if (a0.ntiles <= 0) return;
    LAttnArgs a = a0;
    if (a.e <= 0) a.e = a.d;               // values = whole key rows
    const bool own_v = a.vpool != nullptr;
    const int nsplit = (a.part_o && a.part_ml && a.nsplit > 1) ? a.nsplit : 1;
    const dim3 grid((unsigned)a.ntiles, (unsigned)a.G, (unsigned)nsplit);
    // 64-key tiles where they stay inside 64 KiB of LDS (key head sizes up to 128 without value pages of their own), else 32
    const bool narrow = lay_attn_key_tile(a.d, a.e, own_v) == 32;
    const size_t lds = lay_attn_lds(a.d, a.e, own_v, narrow ? 32 : 64);
    const bool wide = a.e > 256;           // 32 output elements per lane instead of 16
    if (kvt == KV_F32) {
        if (wide) lay_attn_go<KV_F32, 32, 32>(a, grid, lds, s);
        else if (narrow) lay_attn_go<KV_F32, 32, 16>(a, grid, lds, s);
        else lay_attn_go<KV_F32, 64, 16>(a, grid, lds, s);
    } else {
        if (wide) lay_attn_go<KV_BF16, 32, 32>(a, grid, lds, s);
        else if (narrow) lay_attn_go<KV_BF16, 32, 16>(a, grid, lds, s);
        else lay_attn_go<KV_BF16, 64, 16>(a, grid, lds, s);
    }
    // the merge: one thread per output element, blocks of 256 over a tile's 16 rows
    if (nsplit > 1)
        hipLaunchKernelGGL(lay_attn_merge_kernel, dim3((unsigned)a.ntiles, (unsigned)a.G, (unsigned)std::max(1, std::min(16, LA_BQ * a.e / 1024))),
                           dim3(256), 0, s, a, nsplit);
}
int lay_attn_key_tile(int d, int e, bool own_v) { return (d > 128 || lay_attn_lds(d, e, own_v, 64) > LDS_PLAIN) ? 32 : 64; }

// ------------------------------------------------------------------------------------------------------------------
// lightning attention: S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, per head, state [d][e] f32 per sequence.
// A block owns one (sequence, head, slice of ES value columns) and walks the portion in chunks of C tokens:
//   o_t = decay^(t+1) S0^T q_t + sum_(s <= t) decay^(t-s) (q_t . k_s) v_s,   S <- decay^n S0 + sum_s decay^(n-1-s) k_s v_s^T
// (t, s local to the chunk of n tokens).  Everything is f32.
// ------------------------------------------------------------------------------------------------------------------
constexpr int LL_ES = 32;
// GT (gated form): the decay of key channel i at token t is exp(ldec[t][head d + i]) instead of the head's constant.  With
// b_t = sum of the logarithms up to and including t (inside the chunk), all factors are exponentials of differences <= 0:
//   o_t = S0^T (q_t * e^(b_t)) + sum_(s <= t) (sum_i q_t[i] k_s[i] e^(b_t[i] - b_s[i])) v_s,   S <- diag(e^(b_(n-1))) S0 + sum_s (k_s * e^(b_(n-1) - b_s)) v_s^T
// LDS of the gated form: one more [C][d] array (the running logarithms)
// operands of the linear-attention kernels at pass row `row`: the logarithm of the decay (per key channel, or one per head), the key
// (times its per-token factor), the value column c of e (the last one the constant 1 when asked for)
__device__ __forceinline__ float ll_ldec(const LLightArgs& a, int row, int head, int i) {
    return a.head_decay ? a.ldec[(size_t)row * a.ldd + head] : a.ldec[(size_t)row * a.ldd + (size_t)head * a.d + i];
}
__device__ __forceinline__ float ll_query(const LLightArgs& a, int row, int head, int i) {
    return a.proj[(size_t)row * a.ldp + a.q_off + (size_t)(head / a.qk_rep) * a.d + i] * a.qscale;
}
__device__ __forceinline__ float ll_key(const LLightArgs& a, int row, int head, int i) {
    const float k = a.proj[(size_t)row * a.ldp + a.k_off + (size_t)(head / a.qk_rep) * a.d + i];
    return a.kmul ? k * a.kmul[(size_t)row * a.ldd + head] : k;
}
__device__ __forceinline__ float ll_val(const LLightArgs& a, int row, int head, int c) {
    if (a.ones_col) return c == a.e - 1 ? 1.f : a.proj[(size_t)row * a.ldp + a.v_off + (size_t)head * (a.e - 1) + c];
    return a.proj[(size_t)row * a.ldp + a.v_off + (size_t)head * a.e + c];
}
template <bool GT>
__device__ __forceinline__ void ll_cumsum(float* bs, int n, int d, int tid) {
    if (GT) {
        for (int i = tid; i < d; i += 256) {
            float run = 0.f;
            for (int t = 0; t < n; ++t) { run += bs[t * d + i]; bs[t * d + i] = run; }
        }
    }
}
template <bool GT>
__global__ __launch_bounds__(256) void lay_lightning_kernel(LLightArgs a, int C) {
    extern __shared__ float lds[];
    const int d = a.d, e = a.e;
    float* S = lds;                        // [d][ES]
    float* qs = S + d * LL_ES;             // [C][d]
    float* ks = qs + C * d;                // [C][d]
    float* vs = ks + C * d;                // [C][ES]
    float* As = vs + C * LL_ES;            // [C][C]
    float* pw = As + C * C;                // [C + 1] decay^n
    float* bs = pw + C + 1;                // gated: [C][d]
    const LaySegDev sg = a.segs[blockIdx.x];
    const int head = blockIdx.y, j0 = blockIdx.z * LL_ES, tid = threadIdx.x;
    const int ne = min(LL_ES, e - j0);
    const float decay = GT ? 1.f : a.decay[head];
    float* st = a.state_pool + (size_t)sg.slot * a.slot_stride + a.st_off + (size_t)head * d * e;
    for (int idx = tid; idx < d * LL_ES; idx += 256) {
        const int i = idx / LL_ES, j = idx % LL_ES;
        S[idx] = j < ne ? st[(size_t)i * e + j0 + j] : 0.f;
    }
    if (!GT && tid <= C) pw[tid] = tid == 0 ? 1.f : powf(decay, (float)tid);
    for (int t0 = 0; t0 < sg.n; t0 += C) {
        const int n = min(C, sg.n - t0);
        __syncthreads();                   // S, pw ready; the previous chunk's q / k / v no longer read
        for (int idx = tid; idx < n * d; idx += 256) {
            const int t = idx / d, i = idx - t * d;
            qs[idx] = ll_query(a, sg.row0 + t0 + t, head, i);
            ks[idx] = ll_key(a, sg.row0 + t0 + t, head, i);
            if (GT) bs[idx] = ll_ldec(a, sg.row0 + t0 + t, head, i);
        }
        for (int idx = tid; idx < n * LL_ES; idx += 256) {
            const int t = idx / LL_ES, j = idx % LL_ES;
            vs[idx] = j < ne ? ll_val(a, sg.row0 + t0 + t, head, j0 + j) : 0.f;
        }
        if (GT) { __syncthreads(); ll_cumsum<GT>(bs, n, d, tid); }
        __syncthreads();
        for (int idx = tid; idx < n * n; idx += 256) {
            const int t = idx / n, s = idx - t * n;
            float dot = 0.f;
            if (s <= t) {
                if (GT && a.head_decay) {
                    for (int i = 0; i < d; ++i) dot = fmaf(qs[t * d + i], ks[s * d + i], dot);
                    dot *= expf(bs[t * d] - bs[s * d]);
                } else if (GT) {
                    for (int i = 0; i < d; ++i) dot = fmaf(qs[t * d + i] * ks[s * d + i], expf(bs[t * d + i] - bs[s * d + i]), dot);
                } else {
                    for (int i = 0; i < d; ++i) dot = fmaf(qs[t * d + i], ks[s * d + i], dot);
                    dot *= pw[t - s];
                }
            }
            As[t * C + s] = dot;
        }
        __syncthreads();
        if (GT) {                          // q_t e^(b_t) and k_s e^(b_(n-1) - b_s) in place: what the state terms need
            for (int idx = tid; idx < n * d; idx += 256) {
                const int i = idx % d;
                qs[idx] *= expf(bs[idx]);
                ks[idx] *= expf(bs[(n - 1) * d + i] - bs[idx]);
            }
            __syncthreads();
        }
        for (int idx = tid; idx < n * LL_ES; idx += 256) {
            const int t = idx / LL_ES, j = idx % LL_ES;
            float inter = 0.f;
            for (int i = 0; i < d; ++i) inter = fmaf(S[i * LL_ES + j], qs[t * d + i], inter);
            float o = GT ? inter : inter * pw[t + 1];
            for (int s = 0; s <= t; ++s) o = fmaf(As[t * C + s], vs[s * LL_ES + j], o);
            if (j < ne) a.out[(size_t)(sg.row0 + t0 + t) * a.ldo + (size_t)head * e + j0 + j] = o;
        }
        __syncthreads();
        for (int idx = tid; idx < d * LL_ES; idx += 256) {
            const int i = idx / LL_ES, j = idx % LL_ES;
            float sv = S[idx] * (GT ? expf(bs[(n - 1) * d + i]) : pw[n]);
            if (GT) { for (int s = 0; s < n; ++s) sv = fmaf(ks[s * d + i], vs[s * LL_ES + j], sv); }
            else for (int s = 0; s < n; ++s) sv = fmaf(pw[n - 1 - s] * ks[s * d + i], vs[s * LL_ES + j], sv);
            S[idx] = sv;
        }
    }
    __syncthreads();
    for (int idx = tid; idx < d * LL_ES; idx += 256) {
        const int i = idx / LL_ES, j = idx % LL_ES;
        if (j < ne) st[(size_t)i * e + j0 + j] = S[idx];
    }
}
// Long portions: the same recurrence in three launches that are parallel over chunks of LC tokens.
//   1. every chunk's own contribution  U_c = sum_s decay^(n-1-s) k_s v_s^T                        (chunk, head, value slice)
//      (gated: also D_c = e^(b_(n-1)), the decay of the whole chunk per key channel)
//   2. the states in front of the chunks by a scan over each sequence's chunks, in place: U_c <- S_c, S_(c+1) = decay^n S_c + U_c,
//      last state back to the pool                                                              (sequence, head, state element)
//   3. o_t = decay^(t+1) S_c^T q_t + sum_(s <= t) decay^(t-s) (q_t . k_s) v_s                      (chunk, head, value slice)
// chunks[c] = {segment, first token of the chunk inside the portion}; a segment's chunks are consecutive, the first is segs[].pad0.
constexpr int LC = 32;
template <bool GT>
__global__ __launch_bounds__(256) void lay_light_chunk_kv_kernel(LLightArgs a) {
    extern __shared__ float lds[];
    const int d = a.d, e = a.e;
    float* ks = lds;                       // [LC][d]
    float* vs = ks + LC * d;               // [LC][ES]
    float* pw = vs + LC * LL_ES;           // [LC + 1]
    float* bs = pw + LC + 1;               // gated: [LC][d]
    const int2 ch = a.chunks[blockIdx.x];
    const LaySegDev sg = a.segs[ch.x];
    const int head = blockIdx.y, j0 = blockIdx.z * LL_ES, tid = threadIdx.x;
    const int ne = min(LL_ES, e - j0), n = min(LC, sg.n - ch.y);
    if (!GT) {
        const float decay = a.decay[head];
        if (tid <= LC) pw[tid] = tid == 0 ? 1.f : powf(decay, (float)tid);
    }
    for (int idx = tid; idx < n * d; idx += 256) {
        const int t = idx / d, i = idx - t * d;
        ks[idx] = ll_key(a, sg.row0 + ch.y + t, head, i);
        if (GT) bs[idx] = ll_ldec(a, sg.row0 + ch.y + t, head, i);
    }
    for (int idx = tid; idx < n * LL_ES; idx += 256) {
        const int t = idx / LL_ES, j = idx % LL_ES;
        vs[idx] = j < ne ? ll_val(a, sg.row0 + ch.y + t, head, j0 + j) : 0.f;
    }
    __syncthreads();
    if (GT) {
        ll_cumsum<GT>(bs, n, d, tid);
        __syncthreads();
        for (int idx = tid; idx < n * d; idx += 256) ks[idx] *= expf(bs[(n - 1) * d + idx % d] - bs[idx]);
        if (blockIdx.z == 0) for (int i = tid; i < d; i += 256) a.D[((size_t)blockIdx.x * a.H + head) * d + i] = expf(bs[(n - 1) * d + i]);
        __syncthreads();
    }
    float* U = a.U + ((size_t)blockIdx.x * a.H + head) * d * e;
    for (int idx = tid; idx < d * LL_ES; idx += 256) {
        const int i = idx / LL_ES, j = idx % LL_ES;
        float sv = 0.f;
        if (GT) { for (int s = 0; s < n; ++s) sv = fmaf(ks[s * d + i], vs[s * LL_ES + j], sv); }
        else for (int s = 0; s < n; ++s) sv = fmaf(pw[n - 1 - s] * ks[s * d + i], vs[s * LL_ES + j], sv);
        if (j < ne) U[(size_t)i * e + j0 + j] = sv;
    }
}
template <bool GT>
__global__ __launch_bounds__(256) void lay_light_scan_kernel(LLightArgs a) {
    const LaySegDev sg = a.segs[blockIdx.x];
    const int head = blockIdx.y, de = a.d * a.e;
    const int el = blockIdx.z * 256 + threadIdx.x;
    if (el >= de) return;
    const int nch = (sg.n + LC - 1) / LC;
    float pfull = 1.f, plast = 1.f;
    if (!GT) {
        const float decay = a.decay[head];
        pfull = powf(decay, (float)LC); plast = powf(decay, (float)(sg.n - (nch - 1) * LC));
    }
    float* st = a.state_pool + (size_t)sg.slot * a.slot_stride + a.st_off + (size_t)head * de + el;
    float S = *st;
    for (int c = 0; c < nch; ++c) {
        float* u = a.U + ((size_t)(sg.pad0 + c) * a.H + head) * de + el;
        const float own = *u;
        *u = S;
        const float dc = GT ? a.D[((size_t)(sg.pad0 + c) * a.H + head) * a.d + el / a.e] : (c == nch - 1 ? plast : pfull);
        S = fmaf(S, dc, own);
    }
    *st = S;
}
template <bool GT>
__global__ __launch_bounds__(256) void lay_light_chunk_out_kernel(LLightArgs a) {
    extern __shared__ float lds[];
    const int d = a.d, e = a.e;
    float* S = lds;                        // [d][ES] state in front of the chunk
    float* qs = S + d * LL_ES;             // [LC][d]
    const int ldk = d + 1;                 // a wave's lanes read 32 different key rows at once: odd stride, no bank conflicts
    float* ks = qs + LC * d;               // [LC][d + 1]
    float* vs = ks + LC * ldk;             // [LC][ES]
    float* As = vs + LC * LL_ES;           // [LC][LC]
    float* pw = As + LC * LC;              // [LC + 1]
    float* bs = pw + LC + 1;               // gated: [LC][d + 1]
    const int2 ch = a.chunks[blockIdx.x];
    const LaySegDev sg = a.segs[ch.x];
    const int head = blockIdx.y, tid = threadIdx.x;
    const int n = min(LC, sg.n - ch.y);
    if (!GT) {
        const float decay = a.decay[head];
        if (tid <= LC) pw[tid] = tid == 0 ? 1.f : powf(decay, (float)tid);
    }
    const float* U = a.U + ((size_t)blockIdx.x * a.H + head) * d * e;
    // value slices: the launch's z blocks take them in turn (gated form: one block may walk all of them -- the scores are its
    // expensive part and do not depend on the slice); the first slice's state and values are requested with q and k
    int j0 = blockIdx.z * LL_ES;
    auto load_slice = [&]() {
        const int ne = min(LL_ES, e - j0);
        for (int idx = tid; idx < d * LL_ES; idx += 256) {
            const int i = idx / LL_ES, j = idx % LL_ES;
            S[idx] = j < ne ? U[(size_t)i * e + j0 + j] : 0.f;
        }
        for (int idx = tid; idx < n * LL_ES; idx += 256) {
            const int t = idx / LL_ES, j = idx % LL_ES;
            vs[idx] = j < ne ? ll_val(a, sg.row0 + ch.y + t, head, j0 + j) : 0.f;
        }
    };
    load_slice();
    for (int idx = tid; idx < n * d; idx += 256) {
        const int t = idx / d, i = idx - t * d;
        qs[idx] = ll_query(a, sg.row0 + ch.y + t, head, i);
        ks[t * ldk + i] = ll_key(a, sg.row0 + ch.y + t, head, i);
        if (GT) bs[t * ldk + i] = ll_ldec(a, sg.row0 + ch.y + t, head, i);
    }
    __syncthreads();
    if (GT) {
        for (int i = tid; i < d; i += 256) {
            float run = 0.f;
            for (int t = 0; t < n; ++t) { run += bs[t * ldk + i]; bs[t * ldk + i] = run; }
        }
        __syncthreads();
    }
    for (int idx = tid; idx < n * n; idx += 256) {
        const int t = idx / n, s = idx - t * n;
        float dot = 0.f;
        if (s <= t) {
            if (GT && a.head_decay) {      // one decay for all key channels: the plain dot product, one exponential
                for (int i = 0; i < d; ++i) dot = fmaf(qs[t * d + i], ks[s * ldk + i], dot);
                dot *= expf(bs[t * ldk] - bs[s * ldk]);
            } else if (GT) {
                for (int i = 0; i < d; ++i) dot = fmaf(qs[t * d + i] * ks[s * ldk + i], expf(bs[t * ldk + i] - bs[s * ldk + i]), dot);
            } else {
                for (int i = 0; i < d; ++i) dot = fmaf(qs[t * d + i], ks[s * ldk + i], dot);
                dot *= pw[t - s];
            }
        }
        As[t * LC + s] = dot;
    }
    __syncthreads();
    if (GT) {
        for (int idx = tid; idx < n * d; idx += 256) { const int t = idx / d, i = idx - t * d; qs[idx] *= expf(bs[t * ldk + i]); }
        __syncthreads();
    }
    for (;;) {
        const int ne = min(LL_ES, e - j0);
        for (int idx = tid; idx < n * LL_ES; idx += 256) {
            const int t = idx / LL_ES, j = idx % LL_ES;
            float inter = 0.f;
            for (int i = 0; i < d; ++i) inter = fmaf(S[i * LL_ES + j], qs[t * d + i], inter);
            float o = GT ? inter : inter * pw[t + 1];
            for (int s = 0; s <= t; ++s) o = fmaf(As[t * LC + s], vs[s * LL_ES + j], o);
            if (j < ne) a.out[(size_t)(sg.row0 + ch.y + t) * a.ldo + (size_t)head * e + j0 + j] = o;
        }
        if (!GT) break;                    // every slice has its own block: straight-line code
        j0 += gridDim.z * LL_ES;
        if (j0 >= e) break;
        __syncthreads();                   // this slice's state and values are no longer read
        load_slice();
        __syncthreads();
    }
}

// single-token portions (decode steps): S <- decay S + k v^T and o = S^T q straight on the state in HBM, no staging; thread =
// (value column j, 1/8 of the key rows); the eight partial sums of a column meet in LDS
template <bool GT>
__global__ __launch_bounds__(256) void lay_light_decode_kernel(LLightArgs a) {
    __shared__ float qk[3 * 256];
    __shared__ float part[8][LL_ES];
    const int d = a.d, e = a.e;
    const LaySegDev sg = a.segs[blockIdx.x];
    const int head = blockIdx.y, j0 = blockIdx.z * LL_ES, tid = threadIdx.x;
    const int j = tid & (LL_ES - 1), rg = tid >> 5;
    const float decay = GT ? 1.f : a.decay[head];
    for (int i = tid; i < d; i += 256) {
        qk[i] = ll_query(a, sg.row0, head, i);
        qk[256 + i] = ll_key(a, sg.row0, head, i);
        if (GT) qk[512 + i] = expf(ll_ldec(a, sg.row0, head, i));
    }
    __syncthreads();
    const bool ok = j0 + j < e;
    const float v = ok ? ll_val(a, sg.row0, head, j0 + j) : 0.f;
    float* st = a.state_pool + (size_t)sg.slot * a.slot_stride + a.st_off + (size_t)head * d * e + j0 + j;
    float o = 0.f;
    if (ok)
        for (int i = rg; i < d; i += 8) {
            const float sv = fmaf(st[(size_t)i * e], GT ? qk[512 + i] : decay, qk[256 + i] * v);
            st[(size_t)i * e] = sv;
            o = fmaf(sv, qk[i], o);
        }
    part[rg][j] = o;
    __syncthreads();
    if (rg == 0 && ok) {
        float t = 0.f;
#pragma unroll
        for (int r = 0; r < 8; ++r) t += part[r][j];
        a.out[(size_t)sg.row0 * a.ldo + (size_t)head * e + j0 + j] = t;
    }
}

template <typename K>
static void ll_raise_lds(K kern, size_t lds) {
    if (lds > LDS_PLAIN) (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_MAX);
}
template <bool GT>
static void lay_lightning_go(const LLightArgs& a, hipStream_t s) {
    if (a.all_single && a.d <= 256) {
        hipLaunchKernelGGL(lay_light_decode_kernel<GT>, dim3((unsigned)a.nseg, (unsigned)a.H, (unsigned)((a.e + LL_ES - 1) / LL_ES)), dim3(256), 0, s, a);
        return;
    }
    if (a.U && a.chunks && a.nchunks > 0 && a.d <= 128 && (!GT || a.D)) {
        const dim3 gc((unsigned)a.nchunks, (unsigned)a.H, (unsigned)((a.e + LL_ES - 1) / LL_ES));
        const size_t l1 = (size_t)(LC * a.d + LC * LL_ES + LC + 1 + (GT ? LC * a.d : 0)) * sizeof(float);
        const size_t l3 = (size_t)(a.d * LL_ES + 2 * LC * a.d + LC + LC * LL_ES + LC * LC + LC + 1 + (GT ? LC * (a.d + 1) : 0)) * sizeof(float);
        ll_raise_lds(lay_light_chunk_out_kernel<GT>, l3);
        hipLaunchKernelGGL(lay_light_chunk_kv_kernel<GT>, gc, dim3(256), l1, s, a);
        hipLaunchKernelGGL(lay_light_scan_kernel<GT>, dim3((unsigned)a.nseg, (unsigned)a.H, (unsigned)((a.d * a.e + 255) / 256)), dim3(256), 0, s, a);
        // gated form: one block per (chunk, head) once the launch fills the chip without the split over value slices
        const dim3 go(gc.x, gc.y, GT && gc.x * gc.y >= 512 ? 1u : gc.z);      // the plain form keeps one block per slice
        hipLaunchKernelGGL(lay_light_chunk_out_kernel<GT>, go, dim3(256), l3, s, a);
        return;
    }
    const int C = a.d > 128 ? 8 : 16;
    const size_t lds = (size_t)(a.d * LL_ES + 2 * C * a.d + C * LL_ES + C * C + C + 1 + (GT ? C * a.d : 0)) * sizeof(float);
    hipLaunchKernelGGL(lay_lightning_kernel<GT>, dim3((unsigned)a.nseg, (unsigned)a.H, (unsigned)((a.e + LL_ES - 1) / LL_ES)), dim3(256), lds, s, a, C);
}
void launch_lay_lightning(const LLightArgs& a, hipStream_t s) {
    if (a.nseg <= 0) return;
    if (a.ldec) lay_lightning_go<true>(a, s);
    else lay_lightning_go<false>(a, s);
}

// ------------------------------------------------------------------------------------------------------------------
// matrix memory with exponential gates: S' = exp(lf + m - m') S + exp(li - m') k v^T, n' likewise with k alone, m' = max(lf + m, li),
// o = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6).  With the decay exp(lf + m - m') per head and token, the key factor exp(li - m') and a
// constant 1 as one more value column (so that the state's last column is n) this is the gated linear attention above; what is
// left are the gates with their running maximum (here) and the division, head norm and output gate (lay_memory_out).
// ------------------------------------------------------------------------------------------------------------------
// One block per (sequence, head), 256 tokens a round.  x -> max(x + lf, li) composes: after (a1, b1) then (a2, b2) it is
// x -> max(x + a1 + a2, max(b1 + a2, b2)), so the running maximum comes from a shuffle scan over each wave's 64 tokens and a
// second step over the four waves' totals; the portion's last m goes back to the state.
__global__ __launch_bounds__(256) void lay_memory_gates_kernel(const float* __restrict__ proj, int ldp, int i_off, int f_off, float cap,
                                                               float* __restrict__ ldec, float* __restrict__ kmul, float* __restrict__ mrun,
                                                               float* __restrict__ state_pool, size_t slot_stride, size_t m_off,
                                                               const LaySegDev* __restrict__ segs, int H) {
    __shared__ float wa[4], wb[4], carry;
    const LaySegDev sg = segs[blockIdx.x];
    const int head = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float* mp = state_pool + (size_t)sg.slot * slot_stride + m_off + head;
    float m = *mp;
    for (int t0 = 0; t0 < sg.n; t0 += 256) {
        const int t = t0 + tid;
        const bool ok = t < sg.n;
        float li = -INFINITY, lf = 0.f;            // past the portion: the identity x -> x
        if (ok) {
            const float* pr = proj + (size_t)(sg.row0 + t) * ldp + head;
            li = cap * tanhf(pr[i_off] / cap);
            const float u = cap * tanhf(pr[f_off] / cap);
            lf = fminf(u, 0.f) - log1pf(expf(-fabsf(u)));
        }
        float A = lf, B = li;
        for (int off = 1; off < 64; off <<= 1) {
            const float pa = __shfl_up(A, off), pb = __shfl_up(B, off);
            if (lane >= off) { B = fmaxf(pb + A, B); A = pa + A; }
        }
        if (lane == 63) { wa[wave] = A; wb[wave] = B; }
        __syncthreads();
        float mw = m;                              // the running maximum in front of this wave's tokens
        for (int w = 0; w < wave; ++w) mw = fmaxf(mw + wa[w], wb[w]);
        const float mt = fmaxf(mw + A, B);
        float mprev = __shfl_up(mt, 1);
        if (lane == 0) mprev = mw;
        if (ok) {
            const size_t o = (size_t)(sg.row0 + t) * H + head;
            ldec[o] = lf + mprev - mt;
            kmul[o] = expf(li - mt);
            mrun[o] = mt;
        }
        if (tid == 255) carry = mt;                // tokens past the portion pass the last valid m through
        __syncthreads();
        m = carry;
    }
    if (tid == 0) *mp = m;
}
void launch_lay_memory_gates(const float* proj, int ldp, int i_off, int f_off, float cap, float* ldec, float* kmul, float* mrun,
                             float* state_pool, size_t slot_stride, size_t m_off, const LaySegDev* segs, int nseg, int H, hipStream_t s) {
    if (nseg <= 0 || H <= 0) return;
    hipLaunchKernelGGL(lay_memory_gates_kernel, dim3((unsigned)nseg, (unsigned)H), dim3(256), 0, s, proj, ldp, i_off, f_off, cap, ldec, kmul, mrun,
                       state_pool, slot_stride, m_off, segs, H);
}
// one wave per (row, head)
__global__ __launch_bounds__(256) void lay_memory_out_kernel(const float* __restrict__ o, const float* __restrict__ mrun,
                                                             const float* __restrict__ gate, int ldg, const float* __restrict__ w,
                                                             float* __restrict__ out, int ldo, int H, int e, float eps, float out_scale) {
    const int r = blockIdx.x, lane = threadIdx.x & 63;
    const int head = (int)blockIdx.y * 4 + (int)(threadIdx.x >> 6);
    if (head >= H) return;
    const float* oh = o + ((size_t)r * H + head) * (e + 1);
    const float den = fmaxf(fabsf(oh[e]), expf(-mrun[(size_t)r * H + head])) + 1e-6f;
    float ss = 0.f;
    for (int c = lane; c < e; c += 64) { const float v = oh[c] / den; ss += v * v; }
    ss = wave_sum(ss);
    const float rs = 1.f / sqrtf(ss / (float)e + eps);
    for (int c = lane; c < e; c += 64)
        out[(size_t)r * ldo + head * e + c] = oh[c] / den * rs * w[head * e + c] * gate[(size_t)r * ldg + head * e + c] * out_scale;
}
void launch_lay_memory_out(const float* o, const float* mrun, const float* gate, int ldg, const float* w, float* out, int ldo, int T, int H,
                           int e, float eps, float out_scale, hipStream_t s) {
    if (T <= 0 || H <= 0) return;
    hipLaunchKernelGGL(lay_memory_out_kernel, dim3((unsigned)T, (unsigned)((H + 3) / 4)), dim3(256), 0, s, o, mrun, gate, ldg, w, out, ldo, H, e,
                       eps, out_scale);
}

// ------------------------------------------------------------------------------------------------------------------
// mixture of experts: router + counting sort
// ------------------------------------------------------------------------------------------------------------------
// One wave turns the E logits of token t in zs into choices and weights.  zs: [E] logits, then choice scores; sc = zs + E: [E] scores,
// [groups], [top].
__device__ __forceinline__ void lay_router_choose(float* zs, int t, int lane, int32_t* __restrict__ sel, float* __restrict__ wsel, int E, int top,
                                                  const RouterSpec& rs, const float* __restrict__ correction, int slots) {
    float* sc = zs + E;
    // wave 0: lane l owns outputs l, l + 64, ...; maxima, sums and the arg-max (lowest index among equals) are wave reductions
    auto arg_best = [&](bool want_max, int lo, int hi, float& bv) {      // over the live (not -inf) entries of zs[lo, hi)
        float v = 0.f; int at = 0x7fffffff;
        for (int ex = lo + lane; ex < hi; ex += 64) {
            const float z = zs[ex];
            if (z == -INFINITY) continue;
            if (at == 0x7fffffff || (want_max ? z > v : z < v)) { v = z; at = ex; }
        }
        for (int off = 32; off > 0; off >>= 1) {
            const float ov = __shfl_xor(v, off); const int oa = __shfl_xor(at, off);
            if (oa != 0x7fffffff && (at == 0x7fffffff || (want_max ? ov > v : ov < v) || (ov == v && oa < at))) { v = ov; at = oa; }
        }
        bv = v;
        return at;
    };
    // scores; the choice goes by score + correction (plain sigmoid scores: by the logits themselves, the same order)
    if (rs.softmax) {
        float mx = -INFINITY;
        for (int ex = lane; ex < E; ex += 64) mx = fmaxf(mx, zs[ex]);
        mx = wave_max(mx);
        float sum = 0.f;
        for (int ex = lane; ex < E; ex += 64) { const float p = expf(zs[ex] - mx); sc[ex] = p; sum += p; }
        sum = wave_sum(sum);
        for (int ex = lane; ex < E; ex += 64) sc[ex] /= sum;
    } else
        for (int ex = lane; ex < E; ex += 64) sc[ex] = 1.f / (1.f + expf(-zs[ex]));
    if (rs.softmax || correction)
        for (int ex = lane; ex < E; ex += 64) zs[ex] = sc[ex] + (correction ? correction[ex] : 0.f);
    __builtin_amdgcn_wave_barrier();
    if (rs.groups > 1) {                   // keep the best groups: every pass removes the worst remaining one
        const int per = E / rs.groups;
        float* gb = sc + E;                // [groups] a group's largest choice score (-inf: removed)
        for (int g = lane; g < rs.groups; g += 64) {
            float best = -INFINITY;
            for (int j = 0; j < per; ++j) best = fmaxf(best, zs[g * per + j]);
            gb[g] = best;
        }
        for (int drop = 0; drop < rs.groups - rs.keep_groups; ++drop) {
            // the worst live group, among equals the last one
            float v = 0.f; int at = -1;
            for (int g = lane; g < rs.groups; g += 64) {
                const float b = gb[g];
                if (b == -INFINITY) continue;
                if (at < 0 || b <= v) { v = b; at = g; }
            }
            for (int off = 32; off > 0; off >>= 1) {
                const float ov = __shfl_xor(v, off); const int oa = __shfl_xor(at, off);
                if (oa >= 0 && (at < 0 || ov < v || (ov == v && oa > at))) { v = ov; at = oa; }
            }
            if (at < 0) break;
            if (lane == 0) gb[at] = -INFINITY;
            for (int j = lane; j < per; j += 64) zs[at * per + j] = -INFINITY;
            __builtin_amdgcn_wave_barrier();      // LDS accesses of one wave complete in order; this keeps the compiler from moving them
        }
    }
    float* wl = sc + E + rs.groups;        // [top] the chosen scores
    float wsum = 0.f;
    for (int k = 0; k < top; ++k) {
        float bz;
        int best = arg_best(true, 0, E, bz);
        if (best == 0x7fffffff) best = 0;
        const float w = sc[best];
        wsum += w;
        if (lane == 0) {
            sel[(size_t)t * top + k] = best;
            wl[k] = w;
            zs[best] = -INFINITY;
        }
        __builtin_amdgcn_wave_barrier();
    }
    for (int k = lane; k < top; k += 64) wsel[(size_t)t * slots + k] = rs.normalise ? wl[k] / (wsum + 1e-20f) : wl[k];
    for (int k = top + lane; k < slots; k += 64) wsel[(size_t)t * slots + k] = 1.f;
}
// logits and choice in one launch, one block per token
__global__ __launch_bounds__(256) void lay_router_kernel(const float* __restrict__ h, const uint16_t* __restrict__ wr, int32_t* __restrict__ sel,
                                                         float* __restrict__ wsel, int W, int E, int top, RouterSpec rs,
                                                         const float* __restrict__ correction, int slots) {
    extern __shared__ float zs[];
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float* hr = h + (size_t)t * W;
    for (int ex = wave; ex < E; ex += 4) {
        float s = 0.f;
        for (int i = lane; i < W; i += 64) s = fmaf(hr[i], bf16_to_f32(wr[(size_t)ex * W + i]), s);
        s = wave_sum(s);
        if (lane == 0) zs[ex] = s;
    }
    __syncthreads();
    if (wave == 0) lay_router_choose(zs, t, lane, sel, wsel, E, top, rs, correction, slots);
}
// the choice from logits z [T][E] that a projection left: one wave per token
__global__ __launch_bounds__(256) void lay_router_choose_kernel(const float* __restrict__ z, int32_t* __restrict__ sel, float* __restrict__ wsel, int T,
                                                                int E, int top, RouterSpec rs, const float* __restrict__ correction, int slots,
                                                                int per_wave) {
    extern __shared__ float zs[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int t = blockIdx.x * 4 + wave;
    if (t >= T) return;
    float* mine = zs + (size_t)wave * per_wave;
    for (int ex = lane; ex < E; ex += 64) mine[ex] = z[(size_t)t * E + ex];
    __builtin_amdgcn_wave_barrier();
    lay_router_choose(mine, t, lane, sel, wsel, E, top, rs, correction, slots);
}
void launch_lay_router(const float* h, const uint16_t* wr, int32_t* sel, float* wsel, int T, int W, int E, int top, hipStream_t s,
                       const RouterSpec* rs, const float* correction, int slots, float* zbuf) {
    if (T <= 0) return;
    const RouterSpec r = rs ? *rs : RouterSpec();
    if (zbuf && T <= LV_MAXM) {            // decode steps: logits by the streaming row kernel in f32 (every wave busy), then the choice
        LGemmArgs g;
        g.A = h; g.lda = W; g.W = wr; g.C = zbuf; g.ldc = E; g.M = T; g.N = E; g.K = W;
        launch_lgemm(g, false, 1, s);
        const int per_wave = 2 * E + r.groups + top;
        hipLaunchKernelGGL(lay_router_choose_kernel, dim3((unsigned)((T + 3) / 4)), dim3(256), (size_t)4 * per_wave * sizeof(float), s, zbuf, sel, wsel,
                           T, E, top, r, r.correction ? correction : nullptr, slots > top ? slots : top, per_wave);
        return;
    }
    hipLaunchKernelGGL(lay_router_kernel, dim3((unsigned)T), dim3(256), (size_t)(2 * E + r.groups + top) * sizeof(float), s, h, wr, sel, wsel, W, E, top, r,
                       r.correction ? correction : nullptr, slots > top ? slots : top);
}

__global__ __launch_bounds__(1024) void lay_moe_plan_kernel(const int32_t* __restrict__ sel, int32_t* __restrict__ off, int32_t* __restrict__ srt,
                                                            int n, int E, int top, int slots) {
    extern __shared__ int cnt[];           // [E] counts, then cursors
    for (int i = threadIdx.x; i < E; i += 1024) cnt[i] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < n; p += 1024) atomicAdd(&cnt[sel[p]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int run = 0;
        for (int i = 0; i < E; ++i) { const int c = cnt[i]; off[i] = run; cnt[i] = run; run += c; }
        off[E] = run;
    }
    __syncthreads();
    for (int p = threadIdx.x; p < n; p += 1024) srt[atomicAdd(&cnt[sel[p]], 1)] = (p / top) * slots + p % top;
}
void launch_lay_moe_plan(const int32_t* sel, int32_t* off, int32_t* srt, int n, int E, hipStream_t s, int top, int slots) {
    hipLaunchKernelGGL(lay_moe_plan_kernel, dim3(1), dim3(1024), (size_t)E * sizeof(int), s, sel, off, srt, n, E, top, slots);
}

// arg-max of every row, lowest index among equals
__global__ __launch_bounds__(256) void lay_argmax_rows_kernel(const float* __restrict__ logits, int ld, int V, uint32_t* __restrict__ out) {
    __shared__ float bv[256];
    __shared__ int bi[256];
    const float* lr = logits + (size_t)blockIdx.x * ld;
    float best = -INFINITY; int idx = 0x7fffffff;
    for (int i = threadIdx.x; i < V; i += 256) { const float v = lr[i]; if (v > best) { best = v; idx = i; } }
    bv[threadIdx.x] = best; bi[threadIdx.x] = idx;
    __syncthreads();
    for (int st = 128; st > 0; st >>= 1) {
        if ((int)threadIdx.x < st) {
            const float ov = bv[threadIdx.x + st]; const int oi = bi[threadIdx.x + st];
            if (ov > bv[threadIdx.x] || (ov == bv[threadIdx.x] && oi < bi[threadIdx.x])) { bv[threadIdx.x] = ov; bi[threadIdx.x] = oi; }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) out[blockIdx.x] = (uint32_t)(bi[0] == 0x7fffffff ? 0 : bi[0]);
}
// wide rows: LAY_ARGMAX_PARTS blocks per row leave (value, index) partials, one block per row picks among them
__global__ __launch_bounds__(256) void lay_argmax_part_kernel(const float* __restrict__ logits, int ld, int V, float* __restrict__ pv,
                                                              int* __restrict__ pi) {
    __shared__ float bv[256];
    __shared__ int bi[256];
    const float* lr = logits + (size_t)blockIdx.x * ld;
    const int per = (V + (int)gridDim.y - 1) / (int)gridDim.y, lo = blockIdx.y * per, hi = min(V, lo + per);
    float best = -INFINITY; int idx = 0x7fffffff;
    for (int i = lo + threadIdx.x; i < hi; i += 256) { const float v = lr[i]; if (v > best) { best = v; idx = i; } }
    bv[threadIdx.x] = best; bi[threadIdx.x] = idx;
    __syncthreads();
    for (int st = 128; st > 0; st >>= 1) {
        if ((int)threadIdx.x < st) {
            const float ov = bv[threadIdx.x + st]; const int oi = bi[threadIdx.x + st];
            if (ov > bv[threadIdx.x] || (ov == bv[threadIdx.x] && oi < bi[threadIdx.x])) { bv[threadIdx.x] = ov; bi[threadIdx.x] = oi; }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) { pv[blockIdx.x * gridDim.y + blockIdx.y] = bv[0]; pi[blockIdx.x * gridDim.y + blockIdx.y] = bi[0]; }
}
__global__ __launch_bounds__(64) void lay_argmax_final_kernel(const float* __restrict__ pv, const int* __restrict__ pi, int parts,
                                                              uint32_t* __restrict__ out) {
    if (threadIdx.x != 0) return;
    float best = -INFINITY; int idx = 0x7fffffff;
    for (int p = 0; p < parts; ++p) {
        const float v = pv[blockIdx.x * parts + p]; const int i = pi[blockIdx.x * parts + p];
        if (v > best || (v == best && i < idx)) { best = v; idx = i; }
    }
    out[blockIdx.x] = (uint32_t)(idx == 0x7fffffff ? 0 : idx);
}
void launch_lay_argmax_rows(const float* logits, int ld, int V, uint32_t* out, int n_rows, float* pv, int* pi, hipStream_t s) {
    if (n_rows <= 0) return;
    if (pv && pi && V >= 8192) {
        hipLaunchKernelGGL(lay_argmax_part_kernel, dim3((unsigned)n_rows, LAY_ARGMAX_PARTS), dim3(256), 0, s, logits, ld, V, pv, pi);
        hipLaunchKernelGGL(lay_argmax_final_kernel, dim3((unsigned)n_rows), dim3(64), 0, s, pv, pi, LAY_ARGMAX_PARTS, out);
        return;
    }
    hipLaunchKernelGGL(lay_argmax_rows_kernel, dim3((unsigned)n_rows), dim3(256), 0, s, logits, ld, V, out);
}

}  // namespace cm
