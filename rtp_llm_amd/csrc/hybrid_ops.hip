// Kernels of the hybrid decoder family: layers x <- x + m * (g1 * mixer(norm1 x) + g2 * ffn(norm2 x)) over an fp32 residual stream (g: optional
// per-channel sigmoid gates), whose token mixer is paged attention (chunk-local or plain causal mask, optional sink logit in the softmax
// denominator, optionally unit-normed values that are rotated by their position and turned back at the query's position; or low-rank latent
// attention over one cached row per token that serves as key and, with its leading channels, as value) or a linear recurrence
// S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t with its state in fp32 slots (HGRN2, gated-linear-attention and fixed-decay retention
// parametrisations of a, k, q; or the generalized delta rule S_t = diag(w_t) S_(t-1) - (a_t * u_t)(u_t^T S_(t-1)) + k_t v_t^T); feed-forward
// helpers: PolyNorm, and routing / sorting / weighted sum of a mixture of experts.  Options of the attention kernels: sliding window, tanh
// cap on the scores, per-head sigmoid gate on the output, normed queries and keys, scaled rotary magnitude, a query temperature.  For members
// whose sublayers follow each other: the layer's end as residual update + weighted average over the results of all earlier layers + norm,
// and a hashed bigram row beside the token embedding.
//
// One ragged batch of rows serves prefill portions and decode tokens alike: every row carries its position and the index of its
// sequence; a sequence carries its block-table row, its state slot and the range of its rows.  What the model states as 32-bit is fp32
// here whatever the activation type T (bf16 or float): positions and angles, scores and softmax, norms, gates, decays, states, residual.
#include "common.h"
#include "../../include/mi355_hybrid.h"

namespace {

template <typename T> __device__ __forceinline__ void hy_load8(const T* p, float (&o)[8]);
template <> __device__ __forceinline__ void hy_load8<bf16>(const bf16* p, float (&o)[8]) { act_unpack8<true>(*(const u32x4*)p, o); }
template <> __device__ __forceinline__ void hy_load8<float>(const float* p, float (&o)[8]) {
    const f32x4 a = *(const f32x4*)p, b = *(const f32x4*)(p + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) { o[i] = a[i]; o[4 + i] = b[i]; }
}

// eight consecutive cache elements as loaded (16 bytes of bf16, 32 of fp32), widened only where they are used: more loads fit in flight
template <typename T> struct HyRaw8;
template <> struct HyRaw8<bf16> {
    u32x4 r;
    __device__ __forceinline__ void load(const bf16* p) { r = *(const u32x4*)p; }
    __device__ __forceinline__ void zero() { r = u32x4{0u, 0u, 0u, 0u}; }
    __device__ __forceinline__ void get(float (&o)[8]) const { act_unpack8<true>(r, o); }
};
template <> struct HyRaw8<float> {
    f32x4 a, b;
    __device__ __forceinline__ void load(const float* p) { a = *(const f32x4*)p; b = *(const f32x4*)(p + 4); }
    __device__ __forceinline__ void zero() { a = b = f32x4{0.f, 0.f, 0.f, 0.f}; }
    __device__ __forceinline__ void get(float (&o)[8]) const {
#pragma unroll
        for (int i = 0; i < 4; ++i) { o[i] = a[i]; o[4 + i] = b[i]; }
    }
};

__device__ __forceinline__ float hy_wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float hy_wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ float hy_sigmoid(float z) { return 1.f / (1.f + expf(-z)); }
__device__ __forceinline__ float hy_silu(float z) { return z / (1.f + expf(-z)); }

// channel indices of rotation pair i under a layout: 0 = interleaved (2i, 2i+1), 1 = halves (i, i + n/2)
__device__ __forceinline__ void hy_pair(int layout, int i, int n, int& c0, int& c1) {
    if (layout == 0) { c0 = 2 * i; c1 = 2 * i + 1; } else { c0 = i; c1 = i + n / 2; }
}

// ------------------------------------------------------------------------------------------------ embedding -> fp32 stream
// bigram non-null: the row also takes the table row ((previous token * mul_prev + token * mul_cur) mod buckets), or row `buckets` for a
// sequence's first token (prev < 0); the sum is formed in fp32.  out2 non-null: a second copy of the rows.
template <typename T>
__global__ __launch_bounds__(256) void hy_embed_kernel(const int32_t* ids, const T* table, int W, int vocab, float* out, const int32_t* prev, const T* bigram,
                                                       int buckets, unsigned long long mul_prev, unsigned long long mul_cur, float* out2) {
    const int r = blockIdx.x;
    int id = ids[r];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    size_t br = 0;
    if (bigram) {
        const int pv = prev[r];
        br = pv < 0 ? (size_t)buckets : (size_t)(((unsigned long long)pv * mul_prev + (unsigned long long)id * mul_cur) % (unsigned long long)buckets);
    }
    for (int c = threadIdx.x; c < W; c += 256) {
        float v = (float)table[(size_t)id * W + c];
        if (bigram) v += (float)bigram[br * W + c];
        out[(size_t)r * W + c] = v;
        if (out2) out2[(size_t)r * W + c] = v;
    }
}

// ------------------------------------------------------------------------------------------------ residual update + one or two norms
template <typename T> __device__ __forceinline__ void hy_load4(const T* p, float (&o)[4]);
template <> __device__ __forceinline__ void hy_load4<float>(const float* p, float (&o)[4]) { const f32x4 v = *(const f32x4*)p; o[0] = v[0]; o[1] = v[1]; o[2] = v[2]; o[3] = v[3]; }
template <> __device__ __forceinline__ void hy_load4<bf16>(const bf16* p, float (&o)[4]) {
    const u32x2 v = *(const u32x2*)p;
    o[0] = act_lo<true>(v[0]); o[1] = act_hi<true>(v[0]); o[2] = act_lo<true>(v[1]); o[3] = act_hi<true>(v[1]);
}
template <typename T> __device__ __forceinline__ void hy_store4(T* p, const float (&o)[4]);
template <> __device__ __forceinline__ void hy_store4<float>(float* p, const float (&o)[4]) { *(f32x4*)p = f32x4{o[0], o[1], o[2], o[3]}; }
template <> __device__ __forceinline__ void hy_store4<bf16>(bf16* p, const float (&o)[4]) { *(u32x2*)p = u32x2{act_pack<true>(o[0], o[1]), act_pack<true>(o[2], o[3])}; }

// x[src] <- x[src] + mult * (ga * a[src] + gb * b[src]) (written back unless rows are gathered), then h1 = norm(x) * (off + w1), h2 likewise.
// gate null: ga = gb = 1; else ga = sigmoid(gate[src, c]) and gb = sigmoid(gate[src, W + c]) (fp32 pre-activations, row stride ldg).
// ms.y non-null: the second branch is a mixture's weighted sum formed here, b[src] (if any) + sum_k ms.wts[src, k] * ms.y[ms.place[src, k]].
// VEC: W % 4 == 0, four channels per thread and trip (16-byte accesses on the fp32 stream).
struct MoeSum { const float* y; const int32_t* place; const float* wts; int top; };

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void hy_residual_norm_kernel(float* x, const float* a, const float* b, MoeSum ms, const float* gate, int ldg, float mult,
                                                               const int32_t* rows, const T* w1, const T* w2, float off, float eps, int W, T* h1, T* h2) {
    extern __shared__ __attribute__((aligned(16))) float hy_xs[];
    __shared__ float red[4];
    const int r = blockIdx.x, src = rows ? rows[r] : r;
    constexpr int V = VEC ? 4 : 1;
    float ss = 0.f;
    for (int c = threadIdx.x * V; c < W; c += 256 * V) {
        const size_t i = (size_t)src * W + c;
        float v[4], ya[4] = {0.f, 0.f, 0.f, 0.f}, yb[4] = {0.f, 0.f, 0.f, 0.f};
        if (VEC) { hy_load4<float>(x + i, v); if (a) hy_load4<float>(a + i, ya); if (b) hy_load4<float>(b + i, yb); }
        else     { v[0] = x[i]; if (a) ya[0] = a[i]; if (b) yb[0] = b[i]; }
        const bool has_b = b || ms.y;
        if (ms.y) {         // the chosen experts' outputs in choice order, then the shared expert's
            float sum[4] = {0.f, 0.f, 0.f, 0.f};
            for (int k = 0; k < ms.top; ++k) {
                const float wk = ms.wts[(size_t)src * ms.top + k];
                const float* yr = ms.y + (size_t)ms.place[(size_t)src * ms.top + k] * W + c;
                float t[4] = {0.f, 0.f, 0.f, 0.f};
                if (VEC) hy_load4<float>(yr, t); else t[0] = yr[0];
#pragma unroll
                for (int e = 0; e < V; ++e) sum[e] = __builtin_fmaf(wk, t[e], sum[e]);
            }
#pragma unroll
            for (int e = 0; e < V; ++e) yb[e] = sum[e] + yb[e];
        }
        if (gate && (a || has_b)) {
            float ga[4] = {0.f, 0.f, 0.f, 0.f}, gb[4] = {0.f, 0.f, 0.f, 0.f};
            const float* gp = gate + (size_t)src * ldg + c;
            if (VEC) { if (a) hy_load4<float>(gp, ga); if (has_b) hy_load4<float>(gp + W, gb); }
            else     { if (a) ga[0] = gp[0]; if (has_b) gb[0] = gp[W]; }
#pragma unroll
            for (int e = 0; e < V; ++e) { ya[e] *= hy_sigmoid(ga[e]); yb[e] *= hy_sigmoid(gb[e]); }
        }
        if (a || has_b) {
#pragma unroll
            for (int e = 0; e < V; ++e) v[e] = v[e] + mult * (ya[e] + yb[e]);
            if (!rows) { if (VEC) hy_store4<float>(x + i, v); else x[i] = v[0]; }
        }
#pragma unroll
        for (int e = 0; e < V; ++e) { hy_xs[c + e] = v[e]; ss = __builtin_fmaf(v[e], v[e], ss); }
    }
    ss = hy_wave_sum(ss);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float inv = 1.f / sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)W + eps);
    for (int c = threadIdx.x * V; c < W; c += 256 * V) {
        float u[4], g1[4], g2[4], o1[4], o2[4];
#pragma unroll
        for (int e = 0; e < V; ++e) u[e] = hy_xs[c + e] * inv;
        if (h1) {
            if (VEC) hy_load4<T>(w1 + c, g1); else g1[0] = (float)w1[c];
#pragma unroll
            for (int e = 0; e < V; ++e) o1[e] = u[e] * (off + g1[e]);
            if (VEC) hy_store4<T>(h1 + (size_t)r * W + c, o1); else h1[(size_t)r * W + c] = (T)o1[0];
        }
        if (h2) {
            if (VEC) hy_load4<T>(w2 + c, g2); else g2[0] = (float)w2[c];
#pragma unroll
            for (int e = 0; e < V; ++e) o2[e] = u[e] * (off + g2[e]);
            if (VEC) hy_store4<T>(h2 + (size_t)r * W + c, o2); else h2[(size_t)r * W + c] = (T)o2[0];
        }
    }
}

// ------------------------------------------------------------------------------------------------ scaled embedding; norm on a sublayer's OUTPUT
// out[r] = table[ids[r]] * scale (fp32 stream); outh (null: none): the same rows rounded to the activation type, the input of the first sublayer of a
// stack whose sublayers read the stream itself.
template <typename T>
__global__ __launch_bounds__(256) void hy_embed_scaled_kernel(const int32_t* ids, const T* table, int W, int vocab, float scale, float* out, T* outh) {
    const int r = blockIdx.x;
    int id = ids[r];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    for (int c = threadIdx.x; c < W; c += 256) {
        const float v = (float)table[(size_t)id * W + c] * scale;
        out[(size_t)r * W + c] = v;
        if (outh) outh[(size_t)r * W + c] = (T)v;
    }
}

__device__ __forceinline__ float hy_block_sum(float v, float* red) {       // red: 4 floats of LDS; every thread of the 256 calls it
    v = hy_wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}

// A stack that norms what a sublayer RETURNS and lets the sublayers read the stream itself:  x[r] <- x[r] + N(y[r]) * w,  h[r] = x[r] rounded to
// the activation type (the next sublayer's input; null: not written), with the sublayer's result
//     y = ca * a + cb * b + sum_k ms.wts[r, k] * ms.y[ms.place[r, k]] + sigmoid(sg[r * ldsg]) * sh          (every term optional)
// and N the layer norm (center: (y - mean) / sqrt(mean of squared deviations + eps)) or the RMS norm (y / sqrt(mean y^2 + eps)).
// self_rows non-null: nothing is added; out row r is N(x[self_rows[r]]) * w in the activation type (the model's last norm on the asked rows).
// Mean and variance are taken in two passes over the row kept in LDS; everything is fp32.
struct BranchTerms { const float* a; float ca; const float* b; float cb; const float* sh; const float* sg; int ldsg; };

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void hy_branch_norm_kernel(float* x, BranchTerms bt, MoeSum ms, const int32_t* self_rows, const T* w, int center, float eps,
                                                             int W, T* h) {
    extern __shared__ __attribute__((aligned(16))) float hy_xs[];
    __shared__ float red[4];
    constexpr int V = VEC ? 4 : 1, KMAX = 8;
    const int r = blockIdx.x, src = self_rows ? self_rows[r] : r;
    const size_t base = (size_t)src * W;
    const float gsh = (bt.sh && bt.sg) ? hy_sigmoid(bt.sg[(size_t)src * bt.ldsg]) : 1.f;
    // the row's mixture weights and places, read once (the first KMAX choices; more are read in the loop)
    float mw[KMAX];
    const float* my[KMAX];
    if (ms.y) {
#pragma unroll
        for (int k = 0; k < KMAX; ++k)
            if (k < ms.top) { mw[k] = ms.wts[(size_t)src * ms.top + k]; my[k] = ms.y + (size_t)ms.place[(size_t)src * ms.top + k] * W; }
    }
    float s1 = 0.f;
    for (int c = threadIdx.x * V; c < W; c += 256 * V) {
        float y[4] = {0.f, 0.f, 0.f, 0.f}, t[4] = {0.f, 0.f, 0.f, 0.f};
        if (self_rows) { if (VEC) hy_load4<float>(x + base + c, y); else y[0] = x[base + c]; }
        else {
            if (bt.a) {
                if (VEC) hy_load4<float>(bt.a + base + c, t); else t[0] = bt.a[base + c];
#pragma unroll
                for (int e = 0; e < V; ++e) y[e] = bt.ca * t[e];
            }
            if (bt.b) {
                if (VEC) hy_load4<float>(bt.b + base + c, t); else t[0] = bt.b[base + c];
#pragma unroll
                for (int e = 0; e < V; ++e) y[e] = __builtin_fmaf(bt.cb, t[e], y[e]);
            }
            if (ms.y) {                    // the chosen experts in choice order
                float sum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int k = 0; k < KMAX; ++k) {
                    if (k >= ms.top) break;
                    if (VEC) hy_load4<float>(my[k] + c, t); else t[0] = my[k][c];
#pragma unroll
                    for (int e = 0; e < V; ++e) sum[e] = __builtin_fmaf(mw[k], t[e], sum[e]);
                }
                for (int k = KMAX; k < ms.top; ++k) {
                    const float wk = ms.wts[(size_t)src * ms.top + k];
                    const float* yr = ms.y + (size_t)ms.place[(size_t)src * ms.top + k] * W + c;
                    if (VEC) hy_load4<float>(yr, t); else t[0] = yr[0];
#pragma unroll
                    for (int e = 0; e < V; ++e) sum[e] = __builtin_fmaf(wk, t[e], sum[e]);
                }
#pragma unroll
                for (int e = 0; e < V; ++e) y[e] += sum[e];
            }
            if (bt.sh) {
                if (VEC) hy_load4<float>(bt.sh + base + c, t); else t[0] = bt.sh[base + c];
#pragma unroll
                for (int e = 0; e < V; ++e) y[e] = __builtin_fmaf(gsh, t[e], y[e]);
            }
        }
#pragma unroll
        for (int e = 0; e < V; ++e) { hy_xs[c + e] = y[e]; s1 += y[e]; }
    }
    const float mean = center ? hy_block_sum(s1, red) / (float)W : 0.f;
    float ss = 0.f;
    for (int c = threadIdx.x * V; c < W; c += 256 * V) {
#pragma unroll
        for (int e = 0; e < V; ++e) { const float d = hy_xs[c + e] - mean; ss = __builtin_fmaf(d, d, ss); }
    }
    const float inv = 1.f / sqrtf(hy_block_sum(ss, red) / (float)W + eps);
    for (int c = threadIdx.x * V; c < W; c += 256 * V) {
        float g[4], n[4], v[4] = {0.f, 0.f, 0.f, 0.f};
        if (VEC) hy_load4<T>(w + c, g); else g[0] = (float)w[c];
#pragma unroll
        for (int e = 0; e < V; ++e) n[e] = (hy_xs[c + e] - mean) * inv * g[e];
        if (self_rows) {
            if (VEC) hy_store4<T>(h + (size_t)r * W + c, n); else h[(size_t)r * W + c] = (T)n[0];
            continue;
        }
        if (VEC) hy_load4<float>(x + base + c, v); else v[0] = x[base + c];
#pragma unroll
        for (int e = 0; e < V; ++e) v[e] = v[e] + n[e];
        if (VEC) hy_store4<float>(x + base + c, v); else x[base + c] = v[0];
        if (h) { if (VEC) hy_store4<T>(h + base + c, v); else h[base + c] = (T)v[0]; }
    }
}

// ------------------------------------------------------------------------------------------------ residual update + weighted average over depth + norm
// A layer's own result X_n = x + a (a: the layer's last branch, may be null) joins the per-step stack of earlier results (stack[j] = X_j, planes
// of `plane` floats; X_0 is the embedding output), and what the next layer reads is x <- sum_{j <= n} coef[j] X_j, summed in the order j = 0 .. n in
// fp32; then h1 = x / rms(x) * (off + w1).  With `rows` only the listed rows are formed and neither x nor the stack is written (the final norm of
// the rows whose logits are asked for).
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void hy_depth_mix_norm_kernel(float* x, const float* a, float* stack, size_t plane, int n, const float* coef,
                                                                const int32_t* rows, const T* w1, float off, float eps, int W, T* h1) {
    extern __shared__ __attribute__((aligned(16))) float hy_xs[];
    __shared__ float red[4];
    const int r = blockIdx.x, src = rows ? rows[r] : r;
    constexpr int V = VEC ? 4 : 1;
    float ss = 0.f;
    for (int c = threadIdx.x * V; c < W; c += 256 * V) {
        const size_t i = (size_t)src * W + c;
        float v[4], ya[4] = {0.f, 0.f, 0.f, 0.f}, acc[4] = {0.f, 0.f, 0.f, 0.f};
        if (VEC) { hy_load4<float>(x + i, v); if (a) hy_load4<float>(a + i, ya); }
        else     { v[0] = x[i]; if (a) ya[0] = a[i]; }
#pragma unroll
        for (int e = 0; e < V; ++e) v[e] = v[e] + ya[e];
        if (!rows) { if (VEC) hy_store4<float>(stack + (size_t)n * plane + i, v); else stack[(size_t)n * plane + i] = v[0]; }
        for (int j = 0; j < n; ++j) {
            const float cj = coef[j];
            float t[4] = {0.f, 0.f, 0.f, 0.f};
            if (VEC) hy_load4<float>(stack + (size_t)j * plane + i, t); else t[0] = stack[(size_t)j * plane + i];
#pragma unroll
            for (int e = 0; e < V; ++e) acc[e] = __builtin_fmaf(cj, t[e], acc[e]);
        }
        const float cn = coef[n];
#pragma unroll
        for (int e = 0; e < V; ++e) acc[e] = __builtin_fmaf(cn, v[e], acc[e]);
        if (!rows) { if (VEC) hy_store4<float>(x + i, acc); else x[i] = acc[0]; }
#pragma unroll
        for (int e = 0; e < V; ++e) { hy_xs[c + e] = acc[e]; ss = __builtin_fmaf(acc[e], acc[e], ss); }
    }
    ss = hy_wave_sum(ss);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    if (!h1) return;
    const float inv = 1.f / sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)W + eps);
    for (int c = threadIdx.x * V; c < W; c += 256 * V) {
        float g1[4], o1[4];
        if (VEC) hy_load4<T>(w1 + c, g1); else g1[0] = (float)w1[c];
#pragma unroll
        for (int e = 0; e < V; ++e) o1[e] = hy_xs[c + e] * inv * (off + g1[e]);
        if (VEC) hy_store4<T>(h1 + (size_t)r * W + c, o1); else h1[(size_t)r * W + c] = (T)o1[0];
    }
}

// ------------------------------------------------------------------------------------------------ attention: rotate q in place, write K / V pages
struct AttnGeom {
    int H, G, dim, vdim;
    int rot_dims, rot_layout;     // rotary span of q / k heads (0 = none) and its pair layout
    int v_layout;                 // pair layout of the value rotation
    int page, max_blocks, num_pages;
    int v_ld;                     // row stride of the value cache in elements (vdim, or wider when the value rows are a part of wider rows)
};

// Optional steps around the rotation (AttnPrepExtra): a per-head RMS norm of queries and keys under weights shared by the heads (before the
// rotation), a magnitude on cos and sin, and a position-dependent temperature on the queries, q *= 1 + coef ln(floor((p + 1) / every) + 1).
// norm_whole: the norm runs over ALL query heads of the row at once (and over all key heads), under weights [H * dim] / [G * dim].
struct AttnPrepExtra { const void* qnorm; const void* knorm; float mag; float qt_coef; int qt_every; int norm_whole; };

template <typename T>
__global__ __launch_bounds__(256) void hy_attn_prep_kernel(float* qkv, int ld, int koff, int voff, AttnGeom g, const float* kfreq, const float* vfreq,
                                                           int v_norm, float eps, const int32_t* pos, const int32_t* seq, const int32_t* block_table,
                                                           T* kcache, T* vcache, AttnPrepExtra ex) {
    const int r = blockIdx.x, tid = threadIdx.x;
    const int p = pos[r];
    float* row = qkv + (size_t)r * ld;
    const bool has_kv = kcache != nullptr;
    if (ex.norm_whole && (ex.qnorm || (ex.knorm && has_kv))) {   // unit RMS over the whole projection (every head), times a weight per channel
        __shared__ float redq[4], redk[4];
        const int nq_ = ex.qnorm ? g.H * g.dim : 0, nk_ = (ex.knorm && has_kv) ? g.G * g.dim : 0;
        float sq = 0.f, sk = 0.f;
        for (int i = tid; i < nq_; i += 256) sq = __builtin_fmaf(row[i], row[i], sq);
        for (int i = tid; i < nk_; i += 256) sk = __builtin_fmaf(row[koff + i], row[koff + i], sk);
        sq = hy_wave_sum(sq); sk = hy_wave_sum(sk);
        if ((tid & 63) == 0) { redq[tid >> 6] = sq; redk[tid >> 6] = sk; }
        __syncthreads();
        if (nq_) {
            const float inv = 1.f / sqrtf(((redq[0] + redq[1]) + (redq[2] + redq[3])) / (float)nq_ + eps);
            for (int i = tid; i < nq_; i += 256) row[i] = row[i] * inv * (float)((const T*)ex.qnorm)[i];
        }
        if (nk_) {
            const float inv = 1.f / sqrtf(((redk[0] + redk[1]) + (redk[2] + redk[3])) / (float)nk_ + eps);
            for (int i = tid; i < nk_; i += 256) row[koff + i] = row[koff + i] * inv * (float)((const T*)ex.knorm)[i];
        }
        __syncthreads();
    } else if (ex.qnorm || (ex.knorm && has_kv)) {           // one wave per head: unit RMS over the head's channels, times the shared weight
        const int nqh = ex.qnorm ? g.H : 0, nkh = (ex.knorm && has_kv) ? g.G : 0;
        for (int j = tid >> 6; j < nqh + nkh; j += 4) {
            const bool isq = j < nqh;
            float* hd = row + (isq ? j * g.dim : koff + (j - nqh) * g.dim);
            const T* wn = (const T*)(isq ? ex.qnorm : ex.knorm);
            float ss = 0.f;
            for (int c = tid & 63; c < g.dim; c += 64) ss = __builtin_fmaf(hd[c], hd[c], ss);
            const float inv = 1.f / sqrtf(hy_wave_sum(ss) / (float)g.dim + eps);
            for (int c = tid & 63; c < g.dim; c += 64) hd[c] = hd[c] * inv * (float)wn[c];
        }
        __syncthreads();
    }
    size_t slot = 0;
    bool slot_ok = false;
    if (has_kv && p >= 0 && p / g.page < g.max_blocks) {
        const int pg = block_table[(size_t)seq[r] * g.max_blocks + p / g.page];
        slot_ok = pg >= 0 && pg < g.num_pages;
        slot = (size_t)pg * g.G * g.page + (p % g.page);           // + kv head * page
    }
    const float fp = (float)p;
    const int hp = g.rot_dims / 2, nq = g.H * hp, nk = has_kv ? g.G * hp : 0;
    for (int i = tid; i < nq + nk; i += 256) {
        const bool isq = i < nq;
        const int j = isq ? i : i - nq, head = j / hp, pr = j % hp;
        int c0, c1;
        hy_pair(g.rot_layout, pr, g.rot_dims, c0, c1);
        float sn, cs;
        sincosf(fp * kfreq[pr], &sn, &cs);
        sn *= ex.mag; cs *= ex.mag;
        float* base = row + (isq ? 0 : koff) + head * g.dim;
        const float u = base[c0], v = base[c1];
        const float ru = u * cs - v * sn, rv = v * cs + u * sn;
        if (isq) { base[c0] = ru; base[c1] = rv; }
        else if (slot_ok) {
            T* kd = kcache + (slot + (size_t)head * g.page) * g.dim;
            kd[c0] = (T)ru; kd[c1] = (T)rv;
        }
    }
    if (ex.qt_coef != 0.f) {                           // the temperature follows the rotation: every channel of every query head
        __syncthreads();
        const float temp = 1.f + ex.qt_coef * logf((float)((p + 1) / ex.qt_every) + 1.f);
        for (int i = tid; i < g.H * g.dim; i += 256) row[i] *= temp;
    }
    if (!has_kv || !slot_ok) return;
    const int pass = g.dim - g.rot_dims;                             // key channels beyond the rotary span
    for (int i = tid; i < g.G * pass; i += 256) {
        const int head = i / pass, c = g.rot_dims + i % pass;
        kcache[(slot + (size_t)head * g.page) * g.dim + c] = (T)row[koff + head * g.dim + c];
    }
    const int lane = tid & 63, wave = tid >> 6;
    for (int head = wave; head < g.G; head += 4) {
        const float* v = row + voff + head * g.vdim;
        T* vd = vcache + (slot + (size_t)head * g.page) * g.v_ld;
        float inv = 1.f;
        if (v_norm) {
            float ss = 0.f;
            for (int c = lane; c < g.vdim; c += 64) ss = __builtin_fmaf(v[c], v[c], ss);
            inv = 1.f / sqrtf(hy_wave_sum(ss) / (float)g.vdim + eps);
        }
        if (vfreq) {
            for (int m = lane; m < g.vdim / 2; m += 64) {
                int c0, c1;
                hy_pair(g.v_layout, m, g.vdim, c0, c1);
                float sn, cs;
                sincosf(fp * vfreq[m], &sn, &cs);
                const float a = v[c0] * inv, b = v[c1] * inv;
                vd[c0] = (T)(a * cs - b * sn); vd[c1] = (T)(b * cs + a * sn);
            }
        } else {
            for (int c = lane; c < g.vdim; c += 64) vd[c] = (T)(v[c] * inv);
        }
    }
}

// ------------------------------------------------------------------------------------------------ attention over the paged cache
constexpr int HY_MAX_DIM = 512, HY_MAX_VDIM = 512;

// Four or sixteen waves per (row, head): wave w takes the 64-key tiles w, w + NW, ... of the row's visible range with its own running maximum,
// denominator and value sum; they are merged at the end.  Inside a tile a lane owns one key; the scores are computed by groups of lanes that
// share a key row (whole rows per load instruction: the address unit sees each cache line once), the weights and page rows then travel by
// lane broadcast, and groups of lanes accumulate the value channels of whole value rows in the same way.
__device__ __forceinline__ float hy_lane_f(float v, int j) { return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), j)); }

// Optional parts of the mask, the scores and the output (AttnExtra): window > 0: a row at position i sees keys j with 0 <= i - j < window;
// softcap > 0: score <- softcap tanh(score / softcap) after the scale; ogate non-null: head h of row r is multiplied by
// sigmoid(ogate[r * ldg + h]) (fp32 pre-activations, one number per head).
struct AttnExtra { int window; float softcap; const float* ogate; int ldg; };
__device__ __forceinline__ int hy_first_visible(int p, int chunk, int window) {
    return chunk > 0 ? (p / chunk) * chunk : (window > 0 ? max(0, p - window + 1) : 0);
}

template <typename T>
__global__ __launch_bounds__(1024) void hy_attn_rows_kernel(const float* q, int ldq, float scale, AttnGeom g, int chunk, const float* sink, const float* vfreq,
                                                           const int32_t* pos, const int32_t* seq, const int32_t* block_table,
                                                           const T* kcache, const T* vcache, T* out, float* parts, AttnExtra ex) {
    constexpr int NV = HY_MAX_VDIM / 64;
    __shared__ __attribute__((aligned(16))) float q_s[HY_MAX_DIM];
    __shared__ float m_s[16], l_s[16];
    __shared__ float acc_s[16][HY_MAX_VDIM];
    __shared__ float o_s[HY_MAX_VDIM];
    const int r = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, NW = blockDim.x >> 6, NT = blockDim.x;
    const int S = gridDim.z, sp = blockIdx.z;             // the row's key tiles are dealt over S blocks; with S > 1 they leave partial sums
    const int p = __builtin_amdgcn_readfirstlane(pos[r]), kvh = h / (g.H / g.G);
    const int32_t* bt = block_table + (size_t)seq[r] * g.max_blocks;
    for (int d = tid; d < g.dim; d += NT) q_s[d] = q[(size_t)r * ldq + h * g.dim + d];
    __syncthreads();
    const int lo = hy_first_visible(p, chunk, ex.window);
    // the sink is a key of (unscaled) score sink[h] that carries no value: wave 0 starts from m = sink[h], l = 1
    float m = (sink && wave == 0 && sp == 0) ? sink[h] : -INFINITY, l = (sink && wave == 0 && sp == 0) ? 1.f : 0.f;
    float acc[NV], facc[8];
#pragma unroll
    for (int i = 0; i < NV; ++i) acc[i] = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) facc[i] = 0.f;
    const bool fast = g.vdim % 8 == 0 && g.v_ld % 8 == 0;
    const int LPK = fast ? g.vdim / 8 : 1, KPI = fast ? 64 / LPK : 1;      // lanes per key, keys per load instruction (vdim <= 512: KPI >= 1)
    const int grp = lane / LPK, cl = (lane % LPK) * 8;
    const bool gok = grp < KPI;
    // the same for the keys: LK lanes per key row (a power of two >= dim / 8), KK keys per load instruction
    const bool coop = g.dim % 8 == 0;
    int LK = 1;
    while (LK * 8 < g.dim) LK <<= 1;
    const int KK = 64 / LK, kg = lane / LK, kl = lane % LK;
    const bool kl_ok = kl * 8 < g.dim;
    float qv[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) qv[i] = (coop && kl_ok) ? q_s[kl * 8 + i] : 0.f;
    for (int t0 = lo + (sp * NW + wave) * 64; t0 <= p; t0 += 64 * NW * S) {
        const int kj = t0 + lane;
        const bool valid = kj <= p;
        float s = -INFINITY;
        int rowi = 0;                                              // row of the key inside the cache tensors: (page * G + kv head) * page size + offset
        if (valid) rowi = (bt[kj / g.page] * g.G + kvh) * g.page + (kj % g.page);
        if (coop) {
            // LK lanes share a key row (8 channels = one 16- or 32-byte piece each), so a load instruction reads KK whole rows instead of one
            // piece of 64 rows; the partial products are summed over the LK lanes and handed to the lane that owns the key
            const int nk = min(64, p - t0 + 1);
            float sc = 0.f;
            constexpr int UB = 8;                                  // load instructions in flight
            for (int it0 = 0; it0 * KK < nk; it0 += UB) {
                HyRaw8<T> kr[UB];
#pragma unroll
                for (int u = 0; u < UB; ++u) {
                    const int key = (it0 + u) * KK + kg;
                    const int rk = __shfl(rowi, key & 63, 64);
                    if (kl_ok && key < nk) kr[u].load(kcache + (size_t)rk * g.dim + kl * 8);
                    else kr[u].zero();
                }
#pragma unroll
                for (int u = 0; u < UB; ++u) {
                    float kv[8], part = 0.f;
                    kr[u].get(kv);
#pragma unroll
                    for (int i = 0; i < 8; ++i) part = __builtin_fmaf(qv[i], kv[i], part);
                    for (int o = LK >> 1; o > 0; o >>= 1) part += __shfl_xor(part, o, 64);
                    const float got = __shfl(part, (lane % KK) * LK, 64);
                    if (lane / KK == it0 + u) sc = got;
                }
            }
            if (valid) s = sc * scale;
            if (valid && ex.softcap > 0.f) s = ex.softcap * tanhf(s / ex.softcap);
        } else if (valid) {
            const T* kp = kcache + (size_t)rowi * g.dim;
            float d0 = 0.f;
            for (int d = 0; d < g.dim; ++d) d0 = __builtin_fmaf(q_s[d], (float)kp[d], d0);
            s = d0 * scale;
            if (ex.softcap > 0.f) s = ex.softcap * tanhf(s / ex.softcap);
        }
        const float mn = fmaxf(m, hy_wave_max(s));
        const float pj = valid ? expf(s - mn) : 0.f;
        const float corr = (m == -INFINITY) ? 0.f : expf(m - mn);
        l = l * corr + hy_wave_sum(pj);
        m = mn;
        const int nv = min(64, p - t0 + 1);
        if (fast) {
            // LPK lanes share one key's value row (8 channels = 16 bytes each), so one load instruction covers KPI keys
#pragma unroll
            for (int i = 0; i < 8; ++i) facc[i] *= corr;
            constexpr int VF = sizeof(T) == 2 ? 8 : 4;             // value pieces in flight per lane
            for (int j = 0; j < nv; j += VF * KPI) {
                float pw[VF];
                HyRaw8<T> vr[VF];
#pragma unroll
                for (int u = 0; u < VF; ++u) {
                    const int kk = j + u * KPI + grp;
                    const bool ok = gok && kk < nv;
                    const float pk = __shfl(pj, kk & 63, 64);
                    const int rk = __shfl(rowi, kk & 63, 64);
                    pw[u] = ok ? pk : 0.f;
                    if (ok) vr[u].load(vcache + (size_t)rk * g.v_ld + cl);
                    else vr[u].zero();
                }
#pragma unroll
                for (int u = 0; u < VF; ++u) {
                    float vv[8];
                    vr[u].get(vv);
#pragma unroll
                    for (int i = 0; i < 8; ++i) facc[i] = __builtin_fmaf(pw[u], vv[i], facc[i]);
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int c = lane + 64 * i;
                if (64 * i >= g.vdim) break;
                const bool cok = c < g.vdim;
                float a = acc[i] * corr;
                for (int j = 0; j < nv; ++j) {
                    const float pw = hy_lane_f(pj, j);
                    const size_t vr = (size_t)__builtin_amdgcn_readlane(rowi, j) * g.v_ld;
                    a = __builtin_fmaf(pw, cok ? (float)vcache[vr + c] : 0.f, a);
                }
                acc[i] = a;
            }
        }
    }
    if (fast) {       // sum the KPI partial rows of this wave (lanes j, j + LPK, ...) into acc_s[wave]
        float tot[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) tot[i] = facc[i];
        for (int k = 1; k < KPI; ++k) {
#pragma unroll
            for (int i = 0; i < 8; ++i) tot[i] += __shfl(facc[i], (lane + k * LPK) & 63, 64);
        }
        if (lane < LPK) {
#pragma unroll
            for (int i = 0; i < 8; ++i) acc_s[wave][lane * 8 + i] = tot[i];
        }
    } else {
#pragma unroll
        for (int i = 0; i < NV; ++i) { const int c = lane + 64 * i; if (c < g.vdim) acc_s[wave][c] = acc[i]; }
    }
    if (lane == 0) { m_s[wave] = m; l_s[wave] = l; }
    __syncthreads();
    float mm = m_s[0];
    for (int w = 1; w < NW; ++w) mm = fmaxf(mm, m_s[w]);
    float lt = 0.f;
    for (int w = 0; w < NW; ++w) lt = __builtin_fmaf(l_s[w], (m_s[w] == -INFINITY) ? 0.f : expf(m_s[w] - mm), lt);
    float invl = S > 1 ? 1.f : (lt > 0.f ? 1.f / lt : 0.f);
    if (S == 1 && ex.ogate) invl *= hy_sigmoid(ex.ogate[(size_t)r * ex.ldg + h]);
    for (int c = tid; c < g.vdim; c += NT) {
        float a = 0.f;
        for (int w = 0; w < NW; ++w) a = __builtin_fmaf(acc_s[w][c], (m_s[w] == -INFINITY) ? 0.f : expf(m_s[w] - mm), a);
        o_s[c] = a * invl;
    }
    __syncthreads();
    if (S > 1) {        // partial of this block: {running maximum, denominator, value sums}; hy_attn_merge_kernel finishes the row
        float* pd = parts + (((size_t)r * g.H + h) * S + sp) * (g.vdim + 2);
        if (tid == 0) { pd[0] = mm; pd[1] = lt; }
        for (int c = tid; c < g.vdim; c += NT) pd[2 + c] = o_s[c];
        return;
    }
    T* od = out + ((size_t)r * g.H + h) * g.vdim;
    if (vfreq) {     // turn the summed values back by the query's own position
        const float fp = (float)p;
        for (int mi = tid; mi < g.vdim / 2; mi += NT) {
            int c0, c1;
            hy_pair(g.v_layout, mi, g.vdim, c0, c1);
            float sn, cs;
            sincosf(fp * vfreq[mi], &sn, &cs);
            const float a = o_s[c0], b = o_s[c1];
            od[c0] = (T)(a * cs + b * sn); od[c1] = (T)(b * cs - a * sn);
        }
    } else {
        for (int c = tid; c < g.vdim; c += NT) od[c] = (T)o_s[c];
    }
}

// The S partials of a (row, head) -> the head's output: common maximum, summed denominators, value sums rescaled, then the turn back.
template <typename T>
__global__ __launch_bounds__(256) void hy_attn_merge_kernel(const float* parts, int S, AttnGeom g, const float* vfreq, const int32_t* pos, T* out, AttnExtra ex) {
    __shared__ float o_s[HY_MAX_VDIM];
    const int r = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const float* pd = parts + ((size_t)r * g.H + h) * S * (g.vdim + 2);
    float mm = -INFINITY;
    for (int s_ = 0; s_ < S; ++s_) mm = fmaxf(mm, pd[(size_t)s_ * (g.vdim + 2)]);
    float lt = 0.f;
    for (int s_ = 0; s_ < S; ++s_) {
        const float ms = pd[(size_t)s_ * (g.vdim + 2)];
        lt = __builtin_fmaf(pd[(size_t)s_ * (g.vdim + 2) + 1], (ms == -INFINITY) ? 0.f : expf(ms - mm), lt);
    }
    float invl = lt > 0.f ? 1.f / lt : 0.f;
    if (ex.ogate) invl *= hy_sigmoid(ex.ogate[(size_t)r * ex.ldg + h]);
    for (int c = tid; c < g.vdim; c += 256) {
        float a = 0.f;
        for (int s_ = 0; s_ < S; ++s_) {
            const float ms = pd[(size_t)s_ * (g.vdim + 2)];
            a = __builtin_fmaf(pd[(size_t)s_ * (g.vdim + 2) + 2 + c], (ms == -INFINITY) ? 0.f : expf(ms - mm), a);
        }
        o_s[c] = a * invl;
    }
    __syncthreads();
    T* od = out + ((size_t)r * g.H + h) * g.vdim;
    if (vfreq) {
        const float fp = (float)pos[r];
        for (int mi = tid; mi < g.vdim / 2; mi += 256) {
            int c0, c1;
            hy_pair(g.v_layout, mi, g.vdim, c0, c1);
            float sn, cs;
            sincosf(fp * vfreq[mi], &sn, &cs);
            const float a = o_s[c0], b = o_s[c1];
            od[c0] = (T)(a * cs + b * sn); od[c1] = (T)(b * cs - a * sn);
        }
    } else {
        for (int c = tid; c < g.vdim; c += 256) od[c] = (T)o_s[c];
    }
}

// ------------------------------------------------------------------------------------------------ attention for prompt portions: MFMA tiles (bf16 cache)
// One wave per (tile of up to 16 consecutive rows of one sequence, head); up to four heads of one key/value head form a block.  Keys go by 32: S = Q K^T with v_mfma_f32_16x16x32_bf16 (K fragments
// straight from the cache: 8 consecutive channels per lane), mask and online softmax on the fp32 accumulator fragments, then O += P V with P
// passed through LDS into the A layout and the 32 value rows transposed through LDS into the B layout.  Scores and weights stay 32-bit: the
// fp32 queries (scaled) and the fp32 weights enter the matrix unit as an exact sum of two bf16 terms (high part + remainder), the cached
// keys and values are bf16 as stored, every accumulation is fp32.
__device__ __forceinline__ void hy_split_bf16(float x, bf16& hi, bf16& lo) { hi = (bf16)x; lo = (bf16)(x - (float)hi); }
// reductions over the 16 lanes of a DPP row (the lanes that hold one fragment row): quad swaps, then the half-row and row mirrors
template <int CTRL> __device__ __forceinline__ float hy_dpp(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float hy_max16(float v) {
    v = fmaxf(v, hy_dpp<0xB1>(v));      // quad_perm [1,0,3,2]
    v = fmaxf(v, hy_dpp<0x4E>(v));      // quad_perm [2,3,0,1]
    v = fmaxf(v, hy_dpp<0x141>(v));     // row_half_mirror
    return fmaxf(v, hy_dpp<0x140>(v));  // row_mirror
}
__device__ __forceinline__ float hy_sum16(float v) {
    v += hy_dpp<0xB1>(v);
    v += hy_dpp<0x4E>(v);
    v += hy_dpp<0x141>(v);
    return v + hy_dpp<0x140>(v);
}

constexpr int AT_LD = 40;     // LDS row stride (elements) of the 32-key tiles: 80 bytes, 16-byte aligned

template <int DKM, int NCBM, int NWV>     // most 32-channel steps of a key row / 16-channel fragments of a value row the instance holds; waves per block
__global__ __launch_bounds__(256) void hy_attn_tiles_kernel(const float* q, int ldq, float scale, AttnGeom g, int chunk, const float* sink, const float* vfreq,
                                                           const int32_t* pos, const int32_t* seq, const int32_t* block_table,
                                                           const int32_t* tile_row0, const int32_t* tile_n, int ntiles, const bf16* kcache, const bf16* vcache,
                                                           bf16* out, AttnExtra ex) {
    __shared__ __attribute__((aligned(16))) bf16 Ph_all[4][16 * AT_LD];
    __shared__ __attribute__((aligned(16))) bf16 Pl_all[4][16 * AT_LD];
    __shared__ __attribute__((aligned(16))) bf16 Vt[NCBM * 16 * AT_LD];
    // the waves of a block are query heads that share one key/value head: they walk the same keys and share the transposed value tile
    const int wave = threadIdx.x >> 6;
    constexpr int VEM = NCBM / NWV;                           // 32 VP pieces of 16 bytes over 64 NWV threads: at most NCBM / NWV per thread
    const int h = blockIdx.y * NWV + wave, lane = threadIdx.x & 63, lr = lane & 15, lq = lane >> 4;
    bf16* Ph = Ph_all[wave];
    bf16* Pl = Pl_all[wave];
    // a block takes tile b and then tile ntiles - 1 - b: under a causal mask an early (short) tile of a prompt and a late (long) one, so that
    // the blocks of one prompt walk about the same number of keys
    for (int pass = 0; pass < 2; ++pass) {
    const int tile = pass == 0 ? (int)blockIdx.x : ntiles - 1 - (int)blockIdx.x;
    if (pass == 1 && tile <= (int)blockIdx.x) break;
    const int r0 = tile_row0[tile], n = tile_n[tile];
    const int p0 = pos[r0], kvh = h / (g.H / g.G);
    const int32_t* bt = block_table + (size_t)seq[r0] * g.max_blocks;
    const int DK = g.dim / 32, NCB = g.vdim / 16, VP = g.vdim / 8;
    const int psh = (g.page & (g.page - 1)) == 0 ? __builtin_ctz(g.page) : -1;       // page size a power of two: shifts instead of divisions
    auto cache_row = [&](int kc) {
        const int pi = psh >= 0 ? kc >> psh : kc / g.page, po = psh >= 0 ? kc & (g.page - 1) : kc % g.page;
        return (size_t)(bt[pi] * g.G + kvh) * g.page + po;
    };
    // scores are kept times log2(e): the weights are then 2^(s - m), one v_exp_f32 each; the sink (score 0) and the ratios are unchanged
    // (with a cap the products come out in natural units, are capped, and only then go to the log2 scale)
    const float scale2 = ex.softcap > 0.f ? scale : scale * 1.44269504088896340736f;
    const float cap2 = ex.softcap * 1.44269504088896340736f, icap2 = ex.softcap > 0.f ? 2.f * 1.44269504088896340736f / ex.softcap : 0.f;
    bf16x8 qh[DKM], ql[DKM];
#pragma unroll
    for (int ks = 0; ks < DKM; ++ks) {
        if (ks >= DK) continue;
        const float* qp = q + (size_t)(r0 + min(lr, n - 1)) * ldq + h * g.dim + ks * 32 + lq * 8;
#pragma unroll
        for (int i = 0; i < 8; ++i) { bf16 a, b; hy_split_bf16(qp[i] * scale2, a, b); qh[ks][i] = a; ql[ks][i] = b; }
    }
    float m[4], l[4];
    f32x4 o[NCBM];
#pragma unroll
    for (int e = 0; e < 4; ++e) { m[e] = sink ? sink[h] * 1.44269504088896340736f : -INFINITY; l[e] = (sink && lr == 0) ? 1.f : 0.f; }   // l: per-lane share of the row's denominator
#pragma unroll
    for (int cb = 0; cb < NCBM; ++cb) o[cb] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int plast = p0 + n - 1;
    const int rlo_last = hy_first_visible(plast, chunk, ex.window);
    int rlo4[4];                                              // first visible position of the lane's four rows
#pragma unroll
    for (int e = 0; e < 4; ++e) rlo4[e] = hy_first_visible(p0 + lq * 4 + e, chunk, ex.window);
    const int kstart = hy_first_visible(p0, chunk, ex.window) & ~31;
    // the key fragments and raw value rows of the next 32 keys are fetched while the current 32 are worked on
    bf16x8 kn[2][DKM];
    u32x4 vn[VEM];
    auto fetch = [&](int t0) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            const int kc = min(t0 + kb * 16 + lr, plast);
            const bf16* kp = kcache + cache_row(kc) * g.dim + lq * 8;
#pragma unroll
            for (int ks = 0; ks < DKM; ++ks) if (ks < DK) kn[kb][ks] = *(const bf16x8*)(kp + ks * 32);
        }
#pragma unroll
        for (int e = 0; e < VEM; ++e) {
            const int i = threadIdx.x + e * 64 * NWV;
            if (i < 32 * VP) {
                const int kc = min(t0 + (i & 31), plast);
                vn[e] = *(const u32x4*)(vcache + cache_row(kc) * g.v_ld + (i >> 5) * 8);
            }
        }
    };
    fetch(kstart);
    for (int t0 = kstart; t0 <= plast; t0 += 32) {
        f32x4 s[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < DKM; ++ks)
                if (ks < DK) {
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qh[ks], kn[kb][ks], acc, 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ql[ks], kn[kb][ks], acc, 0, 0, 0);
                }
            if (ex.softcap > 0.f) {       // cap tanh(s / cap) = cap (t - 1) / (t + 1), t = 2^(2 s log2(e) / cap), the exponent kept inside fp32's range
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float t = __builtin_amdgcn_exp2f(fminf(fmaxf(acc[e] * icap2, -60.f), 60.f));
                    acc[e] = cap2 * ((t - 1.f) / (t + 1.f));
                }
            }
            s[kb] = acc;
        }
        // the 32 value rows, transposed: Vt[channel][key]; neighbouring lanes write neighbouring keys of one channel row
#pragma unroll
        for (int e = 0; e < VEM; ++e) {
            const int i = threadIdx.x + e * 64 * NWV;
            if (i < 32 * VP) {
                const int key = i & 31, c8 = (i >> 5) * 8;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    *(uint16_t*)&Vt[(c8 + 2 * j) * AT_LD + key] = (uint16_t)(vn[e][j] & 0xFFFFu);
                    *(uint16_t*)&Vt[(c8 + 2 * j + 1) * AT_LD + key] = (uint16_t)(vn[e][j] >> 16);
                }
            }
        }
        if (t0 + 32 <= plast) fetch(t0 + 32);                  // in flight during the softmax and the second product
        // a step whose 32 keys are visible to every row of the tile (behind the first row, inside the last row's block) needs no mask
        const bool interior = t0 + 31 <= p0 && t0 >= rlo_last;
        // mask, running maximum, weights; fragment element e is row 4 lq + e, the lane's key columns are kb * 16 + lr
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = lq * 4 + e, rpos = p0 + row;
            const int rlo = rlo4[e];
            float sv[2];
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                const int kpos = t0 + kb * 16 + lr;
                sv[kb] = (interior || (row < n && kpos <= rpos && kpos >= rlo)) ? s[kb][e] : -INFINITY;
            }
            const float mn = fmaxf(m[e], hy_max16(fmaxf(sv[0], sv[1])));
            float pw[2] = {0.f, 0.f}, corr = 1.f;
            if (mn != -INFINITY) {
                corr = (m[e] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m[e] - mn);
#pragma unroll
                for (int kb = 0; kb < 2; ++kb) pw[kb] = (sv[kb] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(sv[kb] - mn);
            }
            l[e] = l[e] * corr + pw[0] + pw[1];
            m[e] = mn;
#pragma unroll
            for (int cb = 0; cb < NCBM; ++cb) if (cb < NCB) o[cb][e] *= corr;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                bf16 a, b;
                hy_split_bf16(pw[kb], a, b);
                Ph[row * AT_LD + kb * 16 + lr] = a; Pl[row * AT_LD + kb * 16 + lr] = b;
            }
        }
        __syncthreads();
        const bf16x8 ph = *(const bf16x8*)&Ph[lr * AT_LD + lq * 8], pl = *(const bf16x8*)&Pl[lr * AT_LD + lq * 8];
#pragma unroll
        for (int cb = 0; cb < NCBM; ++cb)
            if (cb < NCB) {
                const bf16x8 vf = *(const bf16x8*)&Vt[(cb * 16 + lr) * AT_LD + lq * 8];
                o[cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ph, vf, o[cb], 0, 0, 0);
                o[cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pl, vf, o[cb], 0, 0, 0);
            }
        __syncthreads();
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int row = lq * 4 + e;
        const float lt = hy_sum16(l[e]);
        float inv = lt > 0.f ? 1.f / lt : 0.f;
        if (ex.ogate && row < n) inv *= hy_sigmoid(ex.ogate[(size_t)(r0 + row) * ex.ldg + h]);
        const float fp = (float)(p0 + row);
        bf16* od = out + ((size_t)(r0 + row) * g.H + h) * g.vdim;
#pragma unroll
        for (int cb = 0; cb < NCBM; ++cb) {
            if (cb >= NCB) continue;
            const int c = cb * 16 + lr;
            float v = o[cb][e] * inv;
            if (vfreq) {          // turn back by the row's position; the partner channel sits in the next lane (interleaved) or NCB / 2 fragments away (halves)
                float other, sn, cs;
                bool first;
                int mi;
                if (g.v_layout == 0) { other = __shfl_xor(v, 1, 64); first = (c & 1) == 0; mi = c >> 1; }
                else {
                    const int half = NCB / 2;
                    first = cb < half; mi = first ? c : c - g.vdim / 2;
                    float t = 0.f;
#pragma unroll
                    for (int k = 0; k < NCBM; ++k) if (k == (first ? cb + half : cb - half)) t = o[k][e] * inv;
                    other = t;
                }
                sincosf(fp * vfreq[mi], &sn, &cs);
                v = first ? (v * cs + other * sn) : (v * cs - other * sn);
            }
            if (row < n) od[c] = (bf16)v;
        }
    }
    }   // pass
}

// decay^n for a constant decay in [0, 1] and n >= 0 (n = 0: 1, also for a decay of 0)
__device__ __forceinline__ float hy_decay_pow(float a, int n) { return n == 0 ? 1.f : exp2f((float)n * log2f(a)); }

// ------------------------------------------------------------------------------------------------ fixed-decay recurrence over long prompts: chunks
// A recurrence with a constant decay per head, S_t = a S_(t-1) + k_t v_t^T, splits into chunks of C tokens that are walked side by side:
//   1. every chunk is walked from a ZERO state (hy_scan_kernel over the chunks as if they were sequences): its outputs lack the part that comes
//      from the state at its start, and what it leaves is its own contribution L_c = sum_j a^(n - 1 - j) k_j v_j^T;
//   2. hy_chunk_prefix_kernel runs over a sequence's chunks in order: the state at the start of chunk c is S_c, S_(c+1) = a^(n_c) S_c + L_c; the
//      S_c replace the L_c in the scratch buffer, the last one goes to the sequence's slot;
//   3. hy_scan_kernel with `apply`: out_t += a^(t + 1) S_c^T q_t for token t of chunk c.
// The sums are those of the token-by-token walk in another order (fp32 throughout).  The plan: chunk i covers rows cs[i] .. cs[i + 1] - 1 (unused
// trailing chunks are empty), sequence s owns chunks sc[s] .. sc[s + 1] - 1.
__global__ __launch_bounds__(256) void hy_chunk_plan_kernel(const int32_t* row_start, int nseq, int C, int max_chunks, int32_t* cs, int32_t* sc, int32_t* ids,
                                                            int32_t* zeros, int32_t* ones) {
    __shared__ int total;
    if (threadIdx.x == 0) {
        int a = 0;
        for (int s_ = 0; s_ < nseq; ++s_) { sc[s_] = a; a += (row_start[s_ + 1] - row_start[s_] + C - 1) / C; }
        sc[nseq] = a; total = a;
    }
    __syncthreads();
    const int T = row_start[nseq];
    for (int s_ = 0; s_ < nseq; ++s_) {
        const int r0 = row_start[s_], c0 = sc[s_], n = sc[s_ + 1] - c0;
        for (int i = threadIdx.x; i < n; i += 256) cs[c0 + i] = r0 + i * C;
    }
    for (int i = total + threadIdx.x; i <= max_chunks; i += 256) cs[i] = T;
    for (int i = threadIdx.x; i < max_chunks; i += 256) { ids[i] = i; zeros[i] = 0; ones[i] = 1; }
}

__global__ __launch_bounds__(256) void hy_chunk_prefix_kernel(const int32_t* cs, const int32_t* sc, const int32_t* slot, const int32_t* first_pos, const float* decay,
                                                              int H, int per_head, float* chunk_state, float* state) {
    const int sq = blockIdx.x, h = blockIdx.y, e = blockIdx.z * 256 + threadIdx.x;
    if (e >= per_head) return;
    const float a = decay[h];
    float* st = state + ((size_t)slot[sq] * H + h) * per_head + e;
    float S = first_pos[sq] == 0 ? 0.f : *st;
    for (int c = sc[sq]; c < sc[sq + 1]; ++c) {
        float* cp = chunk_state + ((size_t)c * H + h) * per_head + e;
        const float L = *cp;
        *cp = S;
        S = __builtin_fmaf(hy_decay_pow(a, cs[c + 1] - cs[c]), S, L);
    }
    *st = S;
}

// ------------------------------------------------------------------------------------------------ gated linear recurrence
// Block = 64 value columns x DS groups of RD key rows: thread (c, ds) keeps S[ds * RD .. + RD - 1][c] in registers.  Tokens are staged `tok`
// at a time: all threads compute the gates of the staged tokens once into LDS, then every thread walks the tokens in order (its RD rows:
// decay, rank-one update, partial q . S), and the DS partial outputs per token are summed from LDS.  Short RD keeps the dependent chain per
// token short; the walk itself is the sequential part of the recurrence.
enum { SCAN_HGRN2 = 0, SCAN_GLA = 1, SCAN_FIXED = 2, SCAN_FIXED_SILU = 3 };

struct ScanParams {
    const float* proj; int ld; int qo, ko, vo;     // fp32 projections [rows, ld]: q, k (GLA) or forget pre-activation (HGRN2), v at these columns
    const float* z; int ldz;                        // GLA: decay pre-activation [rows, H * dim]
    const void* lower; const void* fbias;           // HGRN2: lower bound and bias of the forget gate [H * dim], activation type
    float tau, qscale;
    int mode, H, dim, vdim;
    const int32_t* row_start; const int32_t* slot; const int32_t* first_pos;
    float* state;                                   // [slots, H, dim, vdim]
    float* out;                                     // [rows, H * vdim]
    int tok;                                        // tokens staged per pass
    int apply;                                      // fixed-decay modes: the state is only read: out[t] += decay^(t - first row + 1) * (S^T q_t), nothing is written back
};

template <typename T, int RD>
__global__ __launch_bounds__(1024) void hy_scan_kernel(ScanParams p) {
    extern __shared__ __attribute__((aligned(16))) float hy_sm[];
    const int DS = blockDim.x >> 6, dpad = DS * RD, TOK = p.tok;
    float* q_s = hy_sm;                          // [TOK][dpad]
    float* k_s = q_s + TOK * dpad;
    float* a_s = k_s + TOK * dpad;
    float* v_s = a_s + TOK * dpad;               // [TOK][64]
    float* part_s = v_s + TOK * 64;              // [TOK][DS][64]
    const int sq = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * 64;
    const int tid = threadIdx.x, c = tid & 63, ds = tid >> 6;
    const int r0 = p.row_start[sq], r1 = p.row_start[sq + 1];
    const bool vok = v0 + c < p.vdim;
    float* st = p.state + (((size_t)p.slot[sq] * p.H + h) * p.dim) * p.vdim + v0 + c;
    float s[RD];
    const bool fresh = p.first_pos[sq] == 0;
#pragma unroll
    for (int j = 0; j < RD; ++j) {
        const int d = ds * RD + j;
        s[j] = (!fresh && vok && d < p.dim) ? st[(size_t)d * p.vdim] : 0.f;
    }
    // raw projections of the next pass are fetched into registers while the current pass is walked: element i of the staged (token, row)
    // grid belongs to thread i % blockDim, at most RD / 4 per thread (16 tokens x DS x RD rows over 64 DS threads), value columns likewise
    constexpr int EL = RD / 4;
    constexpr int VE = 4;                       // value elements fetched ahead per thread; a block of fewer than four waves reads the rest late
    float rq[EL], rk[EL], rz[EL], rv[VE];
    auto fetch = [&](int t0) {
        const int nt = min(TOK, r1 - t0);
#pragma unroll
        for (int e = 0; e < EL; ++e) {
            const int i = tid + e * blockDim.x, t = i / dpad, d = i % dpad;
            rq[e] = rk[e] = rz[e] = 0.f;
            if (i < nt * dpad && d < p.dim) {
                const float* row = p.proj + (size_t)(t0 + t) * p.ld;
                const int hd = h * p.dim + d;
                rq[e] = row[p.qo + hd]; rk[e] = row[p.ko + hd];
                if (p.mode == SCAN_GLA) rz[e] = p.z[(size_t)(t0 + t) * p.ldz + hd];
            }
        }
#pragma unroll
        for (int e = 0; e < VE; ++e) {
            const int i = tid + e * blockDim.x;
            rv[e] = 0.f;
            if (i < nt * 64 && v0 + (i & 63) < p.vdim) rv[e] = p.proj[(size_t)(t0 + (i >> 6)) * p.ld + p.vo + h * p.vdim + v0 + (i & 63)];
        }
    };
    if (r0 < r1) fetch(r0);
    for (int t0 = r0; t0 < r1; t0 += TOK) {
        const int nt = min(TOK, r1 - t0);
#pragma unroll
        for (int e = 0; e < EL; ++e) {
            const int i = tid + e * blockDim.x, d = i % dpad;
            if (i >= nt * dpad) continue;
            float qv = 0.f, kv = 0.f, av = 1.f;
            if (d < p.dim) {
                const int hd = h * p.dim + d;
                if (p.mode == SCAN_FIXED) {          // one decay per head (fp32 [H] behind `lower`), q and k as given
                    qv = rq[e]; kv = rk[e]; av = ((const float*)p.lower)[h];
                } else if (p.mode == SCAN_FIXED_SILU) {   // the same decay; q, k (and v below) pass through silu first
                    qv = hy_silu(rq[e]); kv = hy_silu(rk[e]); av = ((const float*)p.lower)[h];
                } else if (p.mode == SCAN_HGRN2) {
                    const float lw = (float)((const T*)p.lower)[hd];
                    const float f = lw + (1.f - lw) * hy_sigmoid(rk[e] + (float)((const T*)p.fbias)[hd]);
                    qv = hy_silu(rq[e]); av = f; kv = 1.f - f;
                } else {
                    const float zz = rz[e];
                    const float ls = fminf(zz, 0.f) - log1pf(expf(-fabsf(zz)));       // log sigmoid(z)
                    qv = rq[e] * p.qscale; kv = rk[e]; av = expf(ls / p.tau);
                }
            }
            q_s[i] = qv; k_s[i] = kv; a_s[i] = av;
        }
#pragma unroll
        for (int e = 0; e < VE; ++e) {
            const int i = tid + e * blockDim.x;
            if (i < nt * 64) v_s[i] = p.mode == SCAN_FIXED_SILU ? hy_silu(rv[e]) : rv[e];
        }
        for (int i = tid + VE * blockDim.x; i < nt * 64; i += blockDim.x) {
            const float vv = (v0 + (i & 63) < p.vdim) ? p.proj[(size_t)(t0 + (i >> 6)) * p.ld + p.vo + h * p.vdim + v0 + (i & 63)] : 0.f;
            v_s[i] = p.mode == SCAN_FIXED_SILU ? hy_silu(vv) : vv;
        }
        __syncthreads();
        if (t0 + TOK < r1) fetch(t0 + TOK);
        for (int t = 0; t < nt; ++t) {
            const float vt = v_s[t * 64 + c];
            const f32x4* qq = (const f32x4*)(q_s + t * dpad + ds * RD);
            const f32x4* kk = (const f32x4*)(k_s + t * dpad + ds * RD);
            const f32x4* aa = (const f32x4*)(a_s + t * dpad + ds * RD);
            float o[4] = {0.f, 0.f, 0.f, 0.f};
            if (p.apply) {
#pragma unroll
                for (int j4 = 0; j4 < RD / 4; ++j4) {
                    const f32x4 q4 = qq[j4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[e] = __builtin_fmaf(s[j4 * 4 + e], q4[e], o[e]);
                }
            } else {
#pragma unroll
                for (int j4 = 0; j4 < RD / 4; ++j4) {
                    const f32x4 a4 = aa[j4], k4 = kk[j4], q4 = qq[j4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int j = j4 * 4 + e;
                        s[j] = __builtin_fmaf(a4[e], s[j], k4[e] * vt);
                        o[e] = __builtin_fmaf(s[j], q4[e], o[e]);
                    }
                }
            }
            part_s[(t * DS + ds) * 64 + c] = (o[0] + o[1]) + (o[2] + o[3]);
        }
        __syncthreads();
        for (int i = tid; i < nt * 64; i += blockDim.x) {
            const int t = i >> 6, cc = i & 63;
            if (v0 + cc >= p.vdim) continue;
            float o = 0.f;
            for (int k = 0; k < DS; ++k) o += part_s[(t * DS + k) * 64 + cc];
            float* dst = p.out + (size_t)(t0 + t) * p.H * p.vdim + h * p.vdim + v0 + cc;
            if (p.apply) *dst += o * hy_decay_pow(((const float*)p.lower)[h], t0 + t - r0 + 1);
            else *dst = o;
        }
    }
    if (vok && !p.apply) {
#pragma unroll
        for (int j = 0; j < RD; ++j) {
            const int d = ds * RD + j;
            if (d < p.dim) st[(size_t)d * p.vdim] = s[j];
        }
    }
}

// ------------------------------------------------------------------------------------------------ generalized delta rule
// S_t = diag(w_t) S_(t-1) - (a_t * u_t)(u_t^T S_(t-1)) + k_t v_t^T, o_t = S_t^T r_t per head, S [dim (key channel), vdim] in an fp32 slot; both the
// decayed and the removed term read the old state.  w = exp(-decay_mult * sigmoid(z)), a = sigmoid(removal pre-activation), u = k / sqrt(|k|^2 +
// unit_eps) over the head's key channels: all in fp32.  A group of neighbouring lanes owns one value column, each lane some of its key rows.  Per
// token the only exchange is the group's sum of u^T S (and of the output) by DPP steps; the gates of a pass of tokens are computed once into LDS by
// the whole block.  The walk over a sequence's tokens is the same arithmetic however the tokens were cut into steps.
struct DeltaParams {
    const float* proj; int ld; int ro, ko, vo, ao;   // fp32 projections [rows, ld]: r, k, v heads and the removal pre-activation at these columns
    const float* z; int ldz;                          // decay pre-activation [rows, H * dim]
    float decay_mult, unit_eps;
    int H, dim, vdim;
    const int32_t* row_start; const int32_t* slot; const int32_t* first_pos;
    float* state;                                     // [slots, H, dim, vdim]
    float* out;                                       // [rows, H * vdim]
};

template <int LPC> __device__ __forceinline__ float hy_lanes_sum(float v);
template <> __device__ __forceinline__ float hy_lanes_sum<4>(float v) {
    v += hy_dpp<0xB1>(v);        // quad_perm [1,0,3,2]
    return v + hy_dpp<0x4E>(v);  // quad_perm [2,3,0,1]
}
template <> __device__ __forceinline__ float hy_lanes_sum<16>(float v) { return hy_sum16(v); }

// LPC lanes (4 or 16, neighbours inside a DPP row) own one value column, each RD key rows of it (dim <= LPC * RD); a wave owns 64 / LPC columns and a
// block of four waves CW = 256 / LPC.  Sixteen lanes per column keep the per-token chain short (RD multiply-adds, four DPP steps), which is what a
// single sequence's walk is bound by; TOK tokens are staged per pass, and the raw projections of the next pass are fetched during the walk.
template <int RD, int LPC>
__global__ __launch_bounds__(256) void hy_delta_kernel(DeltaParams p) {
    constexpr int dpad = LPC * RD, CW = 256 / LPC, TOK = dpad <= 128 ? 16 : 8;
    constexpr int EL = (TOK * dpad + 255) / 256, VE = (TOK * CW + 255) / 256;
    __shared__ __attribute__((aligned(16))) float w_s[TOK * dpad], b_s[TOK * dpad], u_s[TOK * dpad], k_s[TOK * dpad], r_s[TOK * dpad];
    __shared__ float v_s[TOK * CW], o_s[TOK * CW], inv_s[TOK];
    const int sq = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * CW;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, rg = lane % LPC, col = wave * (64 / LPC) + lane / LPC;
    const int r0 = p.row_start[sq], r1 = p.row_start[sq + 1];
    const bool vok = v0 + col < p.vdim;
    float* st = p.state + (((size_t)p.slot[sq] * p.H + h) * p.dim) * p.vdim + v0 + col;
    const bool fresh = p.first_pos[sq] == 0;
    float S[RD];
#pragma unroll
    for (int j = 0; j < RD; ++j) {
        const int d = rg * RD + j;
        S[j] = (!fresh && vok && d < p.dim) ? st[(size_t)d * p.vdim] : 0.f;
    }
    float fr[EL], fk[EL], fa[EL], fz[EL], fv[VE];
    auto fetch = [&](int t0) {
        const int nt = min(TOK, r1 - t0);
#pragma unroll
        for (int e = 0; e < EL; ++e) {
            const int i = tid + e * 256, t = i / dpad, d = i % dpad;
            fr[e] = fk[e] = fa[e] = fz[e] = 0.f;
            if (i < nt * dpad && d < p.dim) {
                const float* row = p.proj + (size_t)(t0 + t) * p.ld;
                const int hd = h * p.dim + d;
                fr[e] = row[p.ro + hd]; fk[e] = row[p.ko + hd]; fa[e] = row[p.ao + hd];
                fz[e] = p.z[(size_t)(t0 + t) * p.ldz + hd];
            }
        }
#pragma unroll
        for (int e = 0; e < VE; ++e) {
            const int i = tid + e * 256, cc = i % CW;
            fv[e] = (i < nt * CW && v0 + cc < p.vdim) ? p.proj[(size_t)(t0 + i / CW) * p.ld + p.vo + h * p.vdim + v0 + cc] : 0.f;
        }
    };
    if (r0 < r1) fetch(r0);
    for (int t0 = r0; t0 < r1; t0 += TOK) {
        const int nt = min(TOK, r1 - t0);
#pragma unroll
        for (int e = 0; e < EL; ++e) {
            const int i = tid + e * 256, d = i % dpad;
            if (i >= nt * dpad) continue;
            const bool in = d < p.dim;                  // rows beyond the key size: zero keys, no removal, state stays zero
            r_s[i] = fr[e]; k_s[i] = fk[e];
            b_s[i] = in ? hy_sigmoid(fa[e]) : 0.f;
            w_s[i] = in ? expf(-p.decay_mult * hy_sigmoid(fz[e])) : 1.f;
        }
#pragma unroll
        for (int e = 0; e < VE; ++e) {
            const int i = tid + e * 256;
            if (i < nt * CW) v_s[i] = fv[e];
        }
        __syncthreads();
        {                                             // |k|^2 of a token's head: sixteen neighbouring lanes per token (TOK <= 16 tokens, 256 threads)
            const int t = tid >> 4, l = tid & 15;
            float ss = 0.f;
            if (t < nt)
                for (int d = l; d < dpad; d += 16) ss = __builtin_fmaf(k_s[t * dpad + d], k_s[t * dpad + d], ss);
            ss = hy_sum16(ss);
            if (t < nt && l == 0) inv_s[t] = 1.f / sqrtf(ss + p.unit_eps);
        }
        __syncthreads();
#pragma unroll
        for (int e = 0; e < EL; ++e) {
            const int i = tid + e * 256;
            if (i >= nt * dpad) continue;
            const float u = k_s[i] * inv_s[i / dpad];
            u_s[i] = u; b_s[i] = b_s[i] * u;
        }
        __syncthreads();
        if (t0 + TOK < r1) fetch(t0 + TOK);          // in flight during the walk
        // the gates of token t + 1 are read from LDS while token t is worked on (two register sets, taken in turns)
        struct Gates { f32x4 u[RD / 4], w[RD / 4], b[RD / 4], k[RD / 4], r[RD / 4]; float v; };
        auto load = [&](int t, Gates& g) {
            const int o = t * dpad + rg * RD;
#pragma unroll
            for (int j4 = 0; j4 < RD / 4; ++j4) {
                g.u[j4] = *(const f32x4*)(u_s + o + j4 * 4); g.w[j4] = *(const f32x4*)(w_s + o + j4 * 4); g.b[j4] = *(const f32x4*)(b_s + o + j4 * 4);
                g.k[j4] = *(const f32x4*)(k_s + o + j4 * 4); g.r[j4] = *(const f32x4*)(r_s + o + j4 * 4);
            }
            g.v = v_s[t * CW + col];
        };
        auto step = [&](int t, const Gates& g) {
            float sp[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j4 = 0; j4 < RD / 4; ++j4) {
#pragma unroll
                for (int e = 0; e < 4; ++e) sp[e] = __builtin_fmaf(g.u[j4][e], S[j4 * 4 + e], sp[e]);
            }
            const float sb = hy_lanes_sum<LPC>((sp[0] + sp[1]) + (sp[2] + sp[3]));      // (u^T S_old)[column]
            float op[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j4 = 0; j4 < RD / 4; ++j4) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int j = j4 * 4 + e;
                    S[j] = __builtin_fmaf(g.w[j4][e], S[j], __builtin_fmaf(-g.b[j4][e], sb, g.k[j4][e] * g.v));
                    op[e] = __builtin_fmaf(g.r[j4][e], S[j], op[e]);
                }
            }
            const float o = hy_lanes_sum<LPC>((op[0] + op[1]) + (op[2] + op[3]));
            if (rg == 0) o_s[t * CW + col] = o;
        };
        Gates ga, gb;
        load(0, ga);
        for (int t = 0; t < nt; t += 2) {
            load(min(t + 1, nt - 1), gb);
            step(t, ga);
            if (t + 1 < nt) {
                load(min(t + 2, nt - 1), ga);
                step(t + 1, gb);
            }
        }
        __syncthreads();
        for (int i = tid; i < nt * CW; i += 256) {
            const int cc = i % CW;
            if (v0 + cc < p.vdim) p.out[(size_t)(t0 + i / CW) * p.H * p.vdim + h * p.vdim + v0 + cc] = o_s[i];
        }
    }
    if (vok) {
#pragma unroll
        for (int j = 0; j < RD; ++j) {
            const int d = rg * RD + j;
            if (d < p.dim) st[(size_t)d * p.vdim] = S[j];
        }
    }
}

// per-head RMS norm over vdim with a plain weight (null: none; shared by the heads, or w_heads: one per head and channel, [H * vdim]), optional
// gate (silu, or gate_sigmoid: sigmoid): one block per (row, head), a single wave for heads of up to 256 channels and a wave per 256 channels
// beyond, up to sixteen (one "head" that spans all heads of a row: a norm over the whole concatenation)
template <typename T>
__global__ __launch_bounds__(1024) void hy_head_norm_kernel(const float* o, int H, int vdim, const T* w, float eps, const float* gate, int ldg, int goff, T* out,
                                                           int w_heads, int gate_sigmoid) {
    __shared__ float red[16];
    const int r = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, NT = blockDim.x;
    const float* src = o + ((size_t)r * H + h) * vdim;
    float ss = 0.f;
    for (int c = tid; c < vdim; c += NT) ss = __builtin_fmaf(src[c], src[c], ss);
    ss = hy_wave_sum(ss);
    if (NT > 64) {
        if ((tid & 63) == 0) red[tid >> 6] = ss;
        __syncthreads();
        ss = 0.f;
        for (int i = 0; i < (NT >> 6); ++i) ss += red[i];
    }
    const float inv = 1.f / sqrtf(ss / (float)vdim + eps);
    for (int c = tid; c < vdim; c += NT) {
        float v = src[c] * inv;
        if (w) v *= (float)w[w_heads ? h * vdim + c : c];
        if (gate) { const float gz = gate[(size_t)r * ldg + goff + h * vdim + c]; v *= gate_sigmoid ? hy_sigmoid(gz) : hy_silu(gz); }
        out[((size_t)r * H + h) * vdim + c] = (T)v;
    }
}


// ------------------------------------------------------------------------------------------------ latent attention: normed latent + shared rotated key -> page; queries split
// A token caches ONE row [c (R) | rotated shared key part (dr) | zeros up to dpad] for all heads: c = unit-RMS(first R outputs of the down
// projection) * w, the key part is the remaining dr outputs with their first `rdims` channels turned by the position (interleaved pairs,
// cos and sin times `mag`).  Values are the first R channels of the same row.  Per query head the un-rotated part goes to qn (activation
// type, input of the per-head product with the key up-projection) and the rotated part to columns R.. of the head's absorbed query row
// (fp32, dpad wide, zeros behind).
struct LatentGeom { int H, dim, dr, R, dpad, rdims, page, max_blocks, num_pages; };

template <typename T>
__global__ __launch_bounds__(256) void hy_latent_prep_kernel(const float* proj, int ld, int doff, LatentGeom g, const float* freq, float mag, const T* cw, float eps,
                                                             const int32_t* pos, const int32_t* seq, const int32_t* block_table, T* qn, float* qabs, T* cache) {
    __shared__ float red[4];
    const int r = blockIdx.x, tid = threadIdx.x;
    const int p = pos[r];
    const float fp = (float)p;
    const float* row = proj + (size_t)r * ld;
    const int hd = g.dim + g.dr, hp = g.rdims / 2;
    // queries
    for (int i = tid; i < g.H * g.dim; i += 256) qn[(size_t)r * g.H * g.dim + i] = (T)row[(i / g.dim) * hd + i % g.dim];
    const int tail = g.dpad - g.R;                                   // rotated part + padding of an absorbed query row
    for (int i = tid; i < g.H * tail; i += 256) {
        const int h = i / tail, j = i % tail;
        float v = 0.f;
        if (j < g.dr) {
            const float* qr = row + h * hd + g.dim;
            if (j < g.rdims) {
                const int pr = j >> 1;
                float sn, cs;
                sincosf(fp * freq[pr], &sn, &cs);
                sn *= mag; cs *= mag;
                const float u = qr[2 * pr], w = qr[2 * pr + 1];
                v = (j & 1) ? (w * cs + u * sn) : (u * cs - w * sn);
            } else v = qr[j];
        }
        qabs[((size_t)r * g.H + h) * g.dpad + g.R + j] = v;
    }
    (void)hp;
    // cache row
    bool ok = p >= 0 && p / g.page < g.max_blocks;
    int pg = 0;
    if (ok) { pg = block_table[(size_t)seq[r] * g.max_blocks + p / g.page]; ok = pg >= 0 && pg < g.num_pages; }
    const float* dk = row + doff;
    float ss = 0.f;
    for (int c = tid; c < g.R; c += 256) ss = __builtin_fmaf(dk[c], dk[c], ss);
    ss = hy_wave_sum(ss);
    if ((tid & 63) == 0) red[tid >> 6] = ss;
    __syncthreads();
    if (!ok) return;
    const float inv = 1.f / sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)g.R + eps);
    T* dst = cache + ((size_t)pg * g.page + (p % g.page)) * g.dpad;
    for (int c = tid; c < g.dpad; c += 256) {
        float v = 0.f;
        if (c < g.R) v = dk[c] * inv * (float)cw[c];
        else if (c < g.R + g.dr) {
            const int j = c - g.R;
            if (j < g.rdims) {
                const int pr = j >> 1;
                float sn, cs;
                sincosf(fp * freq[pr], &sn, &cs);
                sn *= mag; cs *= mag;
                const float u = dk[g.R + 2 * pr], w = dk[g.R + 2 * pr + 1];
                v = (j & 1) ? (w * cs + u * sn) : (u * cs - w * sn);
            } else v = dk[c];
        }
        dst[c] = (T)v;
    }
}

// ------------------------------------------------------------------------------------------------ rotary on fp32 projections, in place
// Up to two segments of heads in one buffer (queries and keys): the first `rdims` channels of every head are turned by position * freq
// (pair layout 0 / 1 as hy_pair), cos and sin times `mag`; then the whole head is multiplied by the segment's scale.
struct RotSeg { int off, heads, dim; float scale; };

__global__ __launch_bounds__(256) void hy_rotary_kernel(float* buf, int ld, RotSeg s0, RotSeg s1, int rdims, int layout, const float* freq, float mag,
                                                        const int32_t* pos) {
    const int r = blockIdx.x, tid = threadIdx.x;
    const float fp = (float)pos[r];
    float* row = buf + (size_t)r * ld;
    const int hp = rdims / 2;
    for (int sg = 0; sg < 2; ++sg) {
        const RotSeg s = sg ? s1 : s0;
        for (int i = tid; i < s.heads * hp; i += 256) {
            const int head = i / hp, pr = i % hp;
            int c0, c1;
            hy_pair(layout, pr, rdims, c0, c1);
            float sn, cs;
            sincosf(fp * freq[pr], &sn, &cs);
            sn *= mag; cs *= mag;
            float* b = row + s.off + head * s.dim;
            const float u = b[c0], v = b[c1];
            b[c0] = (u * cs - v * sn) * s.scale; b[c1] = (v * cs + u * sn) * s.scale;
        }
        if (s.scale != 1.f)
            for (int i = tid; i < s.heads * (s.dim - rdims); i += 256) {
                float* b = row + s.off + (i / (s.dim - rdims)) * s.dim + rdims + i % (s.dim - rdims);
                *b *= s.scale;
            }
    }
}

// ------------------------------------------------------------------------------------------------ PolyNorm activation
// out = a N(z) + b N(z^2) + c N(z^3) + e per row, N(u) = u / sqrt(mean(u^2) + eps) over the row's n channels; z fp32 [rows, ld].
__device__ __forceinline__ float hy_block_sum3(float& a, float& b, float& c, float (*red)[4]) {
    a = hy_wave_sum(a); b = hy_wave_sum(b); c = hy_wave_sum(c);
    if ((threadIdx.x & 63) == 0) { red[0][threadIdx.x >> 6] = a; red[1][threadIdx.x >> 6] = b; red[2][threadIdx.x >> 6] = c; }
    __syncthreads();
    a = (red[0][0] + red[0][1]) + (red[0][2] + red[0][3]);
    b = (red[1][0] + red[1][1]) + (red[1][2] + red[1][3]);
    c = (red[2][0] + red[2][1]) + (red[2][2] + red[2][3]);
    return a;
}

template <typename T>
__global__ __launch_bounds__(256) void hy_polynorm_kernel(const float* z, int ld, int n, float ca, float cb, float cc, float ce, float eps, T* out, int ldo) {
    __shared__ float red[3][4];
    const int r = blockIdx.x;
    const float* zr = z + (size_t)r * ld;
    float s1 = 0.f, s2 = 0.f, s3 = 0.f;
    for (int c = threadIdx.x; c < n; c += 256) {
        const float v = zr[c], v2 = v * v, v3 = v2 * v;
        s1 = __builtin_fmaf(v, v, s1); s2 = __builtin_fmaf(v2, v2, s2); s3 = __builtin_fmaf(v3, v3, s3);
    }
    hy_block_sum3(s1, s2, s3, red);
    const float i1 = ca / sqrtf(s1 / (float)n + eps), i2 = cb / sqrtf(s2 / (float)n + eps), i3 = cc / sqrtf(s3 / (float)n + eps);
    for (int c = threadIdx.x; c < n; c += 256) {
        const float v = zr[c], v2 = v * v;
        out[(size_t)r * ldo + c] = (T)(((v * i1 + v2 * i2) + v2 * v * i3) + ce);
    }
}

// ------------------------------------------------------------------------------------------------ mixture of experts: routing, sorting by expert, weighted sum
// One wave per token: scores from the E router logits (fp32; softmax, or a sigmoid each); experts come in `groups` runs of E / groups neighbours, a
// group scores as its best expert (or as the sum of its two best) and only the `keep` best groups stay eligible; the `top` eligible experts with
// the largest scores are chosen, ties to the lower index; the weights are their scores as they are, times a constant.
__device__ __forceinline__ void hy_wave_argmax(float& v, int& i) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(v, o, 64);
        const int oi = __shfl_xor(i, o, 64);
        if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
    }
}

// How a router scores: softmax over the logits or a sigmoid of each (sigmoid != 0); a group's score is its best expert's or the sum of its two
// best (group_top = 1 | 2); the chosen experts weigh score * wscale.
struct RouteMode { int sigmoid; int group_top; float wscale; };

// The routing of one token by one wave; sc [E] and gb [groups] are the wave's scratch in LDS.  Every thread of the block calls it the same
// number of times (it holds block barriers); a wave without a token passes active = false.
__device__ __forceinline__ void hy_route_token(bool active, const float* zr, float* sc, float* gb, int E, int groups, int keep, int top, int32_t* ids,
                                               float* wts, int lane, RouteMode rm) {
    if (rm.sigmoid) {
        if (active) for (int e = lane; e < E; e += 64) sc[e] = hy_sigmoid(zr[e]);
    } else {
        float m = -INFINITY;
        if (active) for (int e = lane; e < E; e += 64) m = fmaxf(m, zr[e]);
        m = hy_wave_max(m);
        float sum = 0.f;
        if (active) for (int e = lane; e < E; e += 64) { const float x = expf(zr[e] - m); sc[e] = x; sum += x; }
        sum = hy_wave_sum(sum);
        if (active) for (int e = lane; e < E; e += 64) sc[e] = sc[e] / sum;
    }
    __syncthreads();
    const int per = E / groups;
    if (groups > 1 && keep < groups) {
        if (active)
            for (int g = lane; g < groups; g += 64) {
                float b1 = -1.f, b2 = -1.f;                       // the group's two largest scores (scores are >= 0)
                for (int j = 0; j < per; ++j) {
                    const float v = sc[g * per + j];
                    if (v > b1) { b2 = b1; b1 = v; } else if (v > b2) b2 = v;
                }
                gb[g] = (rm.group_top >= 2 && per >= 2) ? b1 + b2 : b1;
            }
        __syncthreads();
        for (int k = 0; k < keep; ++k) {          // a kept group is marked by an infinite score, the others stay finite
            float bv = -2.f; int bi = 0x7fffffff;
            if (active) for (int g = lane; g < groups; g += 64) { const float v = gb[g]; if (v < INFINITY && (v > bv || (v == bv && g < bi))) { bv = v; bi = g; } }
            hy_wave_argmax(bv, bi);
            if (active && lane == 0) gb[bi] = INFINITY;
            __syncthreads();
        }
    } else {
        if (active) for (int g = lane; g < groups; g += 64) gb[g] = INFINITY;
        __syncthreads();
    }
    // sigmoid scores are ranked by their logits (the same order, and it survives where the fp32 sigmoid rounds to one)
    for (int k = 0; k < top; ++k) {
        float bv = -INFINITY; int bi = 0x7fffffff;
        if (active)
            for (int e = lane; e < E; e += 64) {
                const float v = rm.sigmoid ? zr[e] : sc[e];
                if (sc[e] >= 0.f && gb[e / per] == INFINITY && (bi == 0x7fffffff || v > bv || (v == bv && e < bi))) { bv = v; bi = e; }
            }
        hy_wave_argmax(bv, bi);
        if (active && lane == 0) { ids[k] = bi; wts[k] = sc[bi] * rm.wscale; sc[bi] = -1.f; }     // taken
        __syncthreads();
    }
}

__global__ __launch_bounds__(64) void hy_moe_route_kernel(const float* z, int ld, int E, int groups, int keep, int top, int32_t* ids, float* wts, RouteMode rm) {
    extern __shared__ float hy_rs[];            // scores [E], group best [groups]
    const int t = blockIdx.x;
    hy_route_token(true, z + (size_t)t * ld, hy_rs, hy_rs + E, E, groups, keep, top, ids + (size_t)t * top, wts + (size_t)t * top, threadIdx.x, rm);
}

// Counting sort of the n = tokens * top (token, choice) pairs by expert, one block: offs [E + 1], src_row[sorted place] = token,
// place_of[pair] = sorted place, tiles = {count, (expert, first row) x count}: the 64-row tiles of the sorted list that hold rows.  The order
// inside an expert is arbitrary (rows are independent of each other).
__device__ __forceinline__ void hy_align_pairs(const int32_t* ids, int n, int top, int E, int* cnt, int* cur, int32_t* offs, int32_t* src_row,
                                               int32_t* place_of, int32_t* tiles) {
    for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += blockDim.x) atomicAdd(&cnt[ids[i]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int a = 0, nt = 0;
        for (int e = 0; e < E; ++e) {
            cur[e] = a; offs[e] = a;
            for (int m = 0; m < cnt[e]; m += 64) { tiles[1 + 2 * nt] = e; tiles[2 + 2 * nt] = a + m; ++nt; }
            a += cnt[e];
        }
        offs[E] = a; tiles[0] = nt;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const int at = atomicAdd(&cur[ids[i]], 1);
        src_row[at] = i / top;
        place_of[i] = at;
    }
}

__global__ __launch_bounds__(1024) void hy_moe_align_kernel(const int32_t* ids, int n, int top, int E, int32_t* offs, int32_t* src_row, int32_t* place_of,
                                                            int32_t* tiles) {
    extern __shared__ int hy_cnt[];             // counts [E], cursors [E]
    hy_align_pairs(ids, n, top, E, hy_cnt, hy_cnt + E, offs, src_row, place_of, tiles);
}

// Routing and sorting of a few tokens (a decode step) in ONE block: its sixteen waves route a token each per trip, then the block sorts the pairs.
__global__ __launch_bounds__(1024) void hy_moe_route_align_kernel(const float* z, int ld, int T, int E, int groups, int keep, int top, int32_t* ids, float* wts,
                                                                  int32_t* offs, int32_t* src_row, int32_t* place_of, int32_t* tiles, RouteMode rm) {
    extern __shared__ float hy_ra[];            // per wave: scores [E], group best [groups]; then counts [E], cursors [E]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float* sc = hy_ra + (size_t)wave * (E + groups);
    for (int t0 = 0; t0 < T; t0 += 16) {
        const int t = t0 + wave;
        const bool active = t < T;
        hy_route_token(active, z + (size_t)(active ? t : 0) * ld, sc, sc + E, E, groups, keep, top, ids + (size_t)(active ? t : 0) * top,
                       wts + (size_t)(active ? t : 0) * top, lane, rm);
    }
    __threadfence_block();
    __syncthreads();
    int* cnt = (int*)(hy_ra + (size_t)16 * (E + groups));
    hy_align_pairs(ids, T * top, top, E, cnt, cnt + E, offs, src_row, place_of, tiles);
}

// out[t] = sum_k wts[t, k] * y[place_of[t * top + k]] (+ extra[t]): fp32 [tokens, W], the choices added in order k = 0 .. top - 1
__global__ __launch_bounds__(256) void hy_moe_combine_kernel(const float* y, int W, const int32_t* place_of, const float* wts, int top, const float* extra, float* out) {
    const int t = blockIdx.x;
    for (int c = threadIdx.x; c < W; c += 256) {
        float a = 0.f;
        for (int k = 0; k < top; ++k) a = __builtin_fmaf(wts[(size_t)t * top + k], y[(size_t)place_of[(size_t)t * top + k] * W + c], a);
        if (extra) a += extra[(size_t)t * W + c];
        out[(size_t)t * W + c] = a;
    }
}

int hy_geom_ok(const AttnGeom& g) {
    MI355_CHECK_ARG(g.H > 0 && g.G > 0 && g.H % g.G == 0, "hybrid attention: heads=%d kv_heads=%d", g.H, g.G);
    MI355_CHECK_ARG(g.dim > 0 && g.dim <= HY_MAX_DIM, "hybrid attention: head size %d (<= %d)", g.dim, HY_MAX_DIM);
    MI355_CHECK_ARG(g.vdim > 0 && g.vdim <= HY_MAX_VDIM, "hybrid attention: value size %d (<= %d)", g.vdim, HY_MAX_VDIM);
    MI355_CHECK_ARG(g.rot_dims >= 0 && g.rot_dims <= g.dim && g.rot_dims % 2 == 0, "hybrid attention: rotary span %d of %d", g.rot_dims, g.dim);
    MI355_CHECK_ARG(g.page > 0 && g.max_blocks > 0 && g.num_pages > 0, "hybrid attention: page=%d max_blocks=%d pages=%d", g.page, g.max_blocks, g.num_pages);
    MI355_CHECK_ARG(g.v_ld >= g.vdim, "hybrid attention: value row stride %d under the value size %d", g.v_ld, g.vdim);
    MI355_CHECK_ARG((long long)g.num_pages * g.G * g.page < (1ll << 31), "hybrid attention: %d pages x %d heads x %d tokens overflow a 32-bit row index", g.num_pages, g.G, g.page);
    return MI355_OK;
}

#define HY_DISPATCH(dt, ...)                                                          \
    do {                                                                              \
        if ((dt) == MI355_ACT_BF16) { using T = bf16; __VA_ARGS__; }                  \
        else if ((dt) == MI355_ACT_F32) { using T = float; __VA_ARGS__; }             \
        else { mi355_set_error("hybrid op: act_dtype=%d (bf16 or fp32)", (int)(dt)); return MI355_ERR_ARG; } \
    } while (0)

} // namespace

extern "C" int mi355_hy_embed(const int32_t* ids, int32_t rows, const void* table, int32_t W, int32_t vocab, float* out, int32_t act_dtype,
                              mi355_stream_t stream) {
    return mi355_hy_embed_bigram(ids, rows, table, W, vocab, out, nullptr, nullptr, 0, 0, 0, nullptr, act_dtype, stream);
}

// out[r] = table[ids[r]] (+ bigram[row(prev[r], ids[r])]): fp32 [rows, W]; bigram [buckets + 1, W] of act_dtype with prev int32 [rows] (the token
// before each row in its sequence, < 0 for a first token: row `buckets`), row = (prev * mul_prev + id * mul_cur) mod buckets in 64-bit arithmetic.
// out2: null, or a second fp32 [rows, W] that receives the same rows.
extern "C" int mi355_hy_embed_bigram(const int32_t* ids, int32_t rows, const void* table, int32_t W, int32_t vocab, float* out, const int32_t* prev,
                                     const void* bigram, int32_t buckets, int64_t mul_prev, int64_t mul_cur, float* out2, int32_t act_dtype,
                                     mi355_stream_t stream) {
    MI355_CHECK_ARG(ids && table && out && rows > 0 && W > 0 && vocab > 0, "hy_embed: rows=%d W=%d", rows, W);
    MI355_CHECK_ARG(!bigram || (prev && buckets > 0 && mul_prev >= 0 && mul_cur >= 0), "hy_embed: bigram table of %d buckets", buckets);
    HY_DISPATCH(act_dtype, hipLaunchKernelGGL(hy_embed_kernel<T>, dim3(rows), dim3(256), 0, (hipStream_t)stream, ids, (const T*)table, W, vocab, out, prev,
                                              (const T*)bigram, buckets, (unsigned long long)mul_prev, (unsigned long long)mul_cur, out2));
    MI355_CHECK_LAUNCH("hy_embed_kernel");
    return MI355_OK;
}

// x [*, W] fp32 stream; a, b [*, W] fp32 branch outputs (either may be null); rows: null, or `n` source rows to gather (x is then read only).
// h1 / h2 [n, W] of act_dtype: x / rms(x) * (weight_offset + w).  w2 / h2 may be null.
// gate: null, or fp32 [*, ldg] pre-activations of per-channel branch gates: a is scaled by sigmoid(gate[:, 0:W]), b by sigmoid(gate[:, W:2W]).
// moe_y non-null: the second branch is b (may be null) + sum_k moe_wts[r, k] * moe_y[moe_place[r, k]] (fp32 [pairs, W], int32 [*, top], fp32 [*, top]):
// the weighted sum of a mixture's chosen experts, formed here instead of by mi355_hy_moe_combine.
extern "C" int mi355_hy_gated_residual_norm(float* x, const float* a, const float* b, const float* gate, int32_t ldg, float mult, const int32_t* rows,
                                            int32_t n, int32_t W, const void* w1, const void* w2, float weight_offset, float eps, void* h1, void* h2,
                                            const float* moe_y, const int32_t* moe_place, const float* moe_wts, int32_t moe_top, int32_t act_dtype,
                                            mi355_stream_t stream) {
    MI355_CHECK_ARG(!moe_y || (moe_place && moe_wts && moe_top > 0), "hy_residual_norm: a mixture's sum needs its places and weights");
    const MoeSum ms{moe_y, moe_place, moe_wts, moe_top};
    MI355_CHECK_ARG(x && n > 0 && W > 0 && (!h1 || w1) && (!h2 || w2), "hy_residual_norm: n=%d W=%d", n, W);
    MI355_CHECK_ARG((size_t)W * 4 <= 64 * 1024, "hy_residual_norm: W=%d too wide for one block", W);
    MI355_CHECK_ARG(!gate || ldg >= 2 * W, "hy_residual_norm: gate row stride %d for two gates of %d", ldg, W);
    auto al = [](const void* p_) { return ((uintptr_t)p_ & 15) == 0; };
    if (W % 4 == 0 && ldg % 4 == 0 && al(x) && al(a) && al(b) && al(gate) && al(w1) && al(w2) && al(h1) && al(h2) && al(moe_y))
        HY_DISPATCH(act_dtype, hipLaunchKernelGGL((hy_residual_norm_kernel<T, true>), dim3(n), dim3(256), (size_t)W * 4, (hipStream_t)stream, x, a, b, ms, gate, ldg,
                                                  mult, rows, (const T*)w1, (const T*)w2, weight_offset, eps, W, (T*)h1, (T*)h2));
    else
        HY_DISPATCH(act_dtype, hipLaunchKernelGGL((hy_residual_norm_kernel<T, false>), dim3(n), dim3(256), (size_t)W * 4, (hipStream_t)stream, x, a, b, ms, gate, ldg,
                                                  mult, rows, (const T*)w1, (const T*)w2, weight_offset, eps, W, (T*)h1, (T*)h2));
    MI355_CHECK_LAUNCH("hy_residual_norm_kernel");
    return MI355_OK;
}

extern "C" int mi355_hy_residual_norm(float* x, const float* a, const float* b, float mult, const int32_t* rows, int32_t n, int32_t W,
                                      const void* w1, const void* w2, float weight_offset, float eps, void* h1, void* h2, int32_t act_dtype,
                                      mi355_stream_t stream) {
    return mi355_hy_gated_residual_norm(x, a, b, nullptr, 0, mult, rows, n, W, w1, w2, weight_offset, eps, h1, h2, nullptr, nullptr, nullptr, 0, act_dtype, stream);
}

// out fp32 [rows, W] = table[ids] * scale; outh (act_dtype [rows, W], or null): the same rows in the activation type.
extern "C" int mi355_hy_embed_scaled(const int32_t* ids, int32_t rows, const void* table, int32_t W, int32_t vocab, float scale, float* out, void* outh,
                                     int32_t act_dtype, mi355_stream_t stream) {
    MI355_CHECK_ARG(ids && table && out && rows > 0 && W > 0 && vocab > 0, "hy_embed_scaled: rows=%d W=%d", rows, W);
    HY_DISPATCH(act_dtype, hipLaunchKernelGGL(hy_embed_scaled_kernel<T>, dim3(rows), dim3(256), 0, (hipStream_t)stream, ids, (const T*)table, W, vocab, scale, out,
                                              (T*)outh));
    MI355_CHECK_LAUNCH("hy_embed_scaled_kernel");
    return MI355_OK;
}

// The end of a sublayer whose OUTPUT is normed: x [n, W] fp32 stream <- x + N(y) * w with y = ca * a + cb * b + (mixture sum) + sigmoid(sg) * sh, h [n, W]
// (act_dtype, or null) = the new x.  a, b, sh: fp32 [n, W] or null; sg: fp32, one pre-activation per row at stride ldsg (null: sh is added as it is);
// moe_*: as in mi355_hy_gated_residual_norm.  center != 0: layer norm (mean removed, variance of the deviations); 0: RMS norm.  w [W] of act_dtype.
// self_rows (int32 [n]) non-null: no branch is read and x is not written; h [n, W] = N(x[self_rows]) * w.
extern "C" int mi355_hy_branch_norm(float* x, const float* a, float ca, const float* b, float cb, const float* sh, const float* sg, int32_t ldsg,
                                    const float* moe_y, const int32_t* moe_place, const float* moe_wts, int32_t moe_top, const int32_t* self_rows, int32_t n,
                                    int32_t W, const void* w, int32_t center, float eps, void* h, int32_t act_dtype, mi355_stream_t stream) {
    MI355_CHECK_ARG(x && w && n > 0 && W > 0, "hy_branch_norm: n=%d W=%d", n, W);
    MI355_CHECK_ARG(!moe_y || (moe_place && moe_wts && moe_top > 0), "hy_branch_norm: a mixture's sum needs its places and weights");
    MI355_CHECK_ARG(self_rows ? h != nullptr : (a || b || sh || moe_y), "hy_branch_norm: nothing to norm");
    MI355_CHECK_ARG(!sg || (sh && ldsg > 0), "hy_branch_norm: a gate without its branch (stride %d)", ldsg);
    MI355_CHECK_ARG((size_t)W * 4 <= 64 * 1024, "hy_branch_norm: W=%d too wide for one block", W);
    const BranchTerms bt{a, ca, b, cb, sh, sg, ldsg};
    const MoeSum ms{moe_y, moe_place, moe_wts, moe_top};
    auto al = [](const void* p_) { return ((uintptr_t)p_ & 15) == 0; };
    if (W % 4 == 0 && al(x) && al(a) && al(b) && al(sh) && al(moe_y) && al(w) && al(h))
        HY_DISPATCH(act_dtype, hipLaunchKernelGGL((hy_branch_norm_kernel<T, true>), dim3(n), dim3(256), (size_t)W * 4, (hipStream_t)stream, x, bt, ms, self_rows,
                                                  (const T*)w, center, eps, W, (T*)h));
    else
        HY_DISPATCH(act_dtype, hipLaunchKernelGGL((hy_branch_norm_kernel<T, false>), dim3(n), dim3(256), (size_t)W * 4, (hipStream_t)stream, x, bt, ms, self_rows,
                                                  (const T*)w, center, eps, W, (T*)h));
    MI355_CHECK_LAUNCH("hy_branch_norm_kernel");
    return MI355_OK;
}

// x fp32 [T, W] stream (the layer's input plus its earlier branches), a fp32 [T, W] or null; stack fp32 [>= n + 1, T, W] with planes 0 .. n - 1 filled;
// coef fp32 [n + 1] on the device.  Writes stack[n] = x + a, x = sum_j coef[j] stack[j], h1 [rows_n, W] of act_dtype (null: no norm).  rows: null
// (rows_n = T rows, in place), or rows_n row indices to form without writing x or the stack.
extern "C" int mi355_hy_depth_mix_norm(float* x, const float* a, float* stack, int64_t plane, int32_t n, const float* coef, const int32_t* rows,
                                       int32_t rows_n, int32_t W, const void* w1, float weight_offset, float eps, void* h1, int32_t act_dtype,
                                       mi355_stream_t stream) {
    MI355_CHECK_ARG(x && stack && coef && rows_n > 0 && W > 0 && n >= 0 && plane >= W && (!h1 || w1), "hy_depth_mix_norm: rows=%d W=%d n=%d", rows_n, W, n);
    MI355_CHECK_ARG((size_t)W * 4 <= 64 * 1024, "hy_depth_mix_norm: W=%d too wide for one block", W);
    auto al = [](const void* p_) { return ((uintptr_t)p_ & 15) == 0; };
    if (W % 4 == 0 && plane % 4 == 0 && al(x) && al(a) && al(stack) && al(w1) && al(h1))
        HY_DISPATCH(act_dtype, hipLaunchKernelGGL((hy_depth_mix_norm_kernel<T, true>), dim3(rows_n), dim3(256), (size_t)W * 4, (hipStream_t)stream, x, a, stack,
                                                  (size_t)plane, n, coef, rows, (const T*)w1, weight_offset, eps, W, (T*)h1));
    else
        HY_DISPATCH(act_dtype, hipLaunchKernelGGL((hy_depth_mix_norm_kernel<T, false>), dim3(rows_n), dim3(256), (size_t)W * 4, (hipStream_t)stream, x, a, stack,
                                                  (size_t)plane, n, coef, rows, (const T*)w1, weight_offset, eps, W, (T*)h1));
    MI355_CHECK_LAUNCH("hy_depth_mix_norm_kernel");
    return MI355_OK;
}

// geom: {H, G, dim, vdim, rot_dims, rot_layout, v_layout, page, max_blocks, num_pages}.  qkv fp32 [rows, ld]: q heads at column 0 (rotated in
// place), k heads at koff, v heads at voff.  kcache [pages, G, page, dim], vcache [pages, G, page, vdim] of act_dtype; null kcache: queries only
// (a layer that reads another layer's cache).  kfreq [rot_dims / 2], vfreq [vdim / 2] fp32 angular steps (vfreq null: values are not rotated).
extern "C" int mi355_hy_attn_prep(float* qkv, int32_t ld, int32_t koff, int32_t voff, const int32_t* geom, const float* kfreq, const float* vfreq,
                                  int32_t v_norm, float eps, const int32_t* pos, const int32_t* seq, const int32_t* block_table, int32_t rows,
                                  void* kcache, void* vcache, int32_t act_dtype, mi355_stream_t stream) {
    return mi355_hy_attn_prep_ex(qkv, ld, koff, voff, geom, kfreq, vfreq, v_norm, eps, pos, seq, block_table, rows, kcache, vcache, nullptr, nullptr, 1.f, 0.f, 1,
                                 act_dtype, stream);
}

// The same with the optional steps: qnorm / knorm (act_dtype [dim], or null): queries / keys are brought to unit RMS per head (eps) and multiplied
// by the weight before the rotation; mag multiplies cos and sin; qt_coef != 0: queries are multiplied by 1 + qt_coef ln(floor((p + 1) / qt_every) + 1)
// after the rotation.
extern "C" int mi355_hy_attn_prep_ex(float* qkv, int32_t ld, int32_t koff, int32_t voff, const int32_t* geom, const float* kfreq, const float* vfreq,
                                     int32_t v_norm, float eps, const int32_t* pos, const int32_t* seq, const int32_t* block_table, int32_t rows,
                                     void* kcache, void* vcache, const void* qnorm, const void* knorm, float mag, float qt_coef, int32_t qt_every,
                                     int32_t act_dtype, mi355_stream_t stream) {
    return mi355_hy_attn_prep_ex2(qkv, ld, koff, voff, geom, kfreq, vfreq, v_norm, eps, pos, seq, block_table, rows, kcache, vcache, qnorm, knorm, 0, mag, qt_coef,
                                  qt_every, act_dtype, stream);
}

// norm_whole != 0: qnorm is [H * dim] and knorm [G * dim]; the queries of a row are brought to unit RMS over all their heads at once (the keys likewise)
// and multiplied by a weight per channel, before the rotation.
extern "C" int mi355_hy_attn_prep_ex2(float* qkv, int32_t ld, int32_t koff, int32_t voff, const int32_t* geom, const float* kfreq, const float* vfreq,
                                      int32_t v_norm, float eps, const int32_t* pos, const int32_t* seq, const int32_t* block_table, int32_t rows,
                                      void* kcache, void* vcache, const void* qnorm, const void* knorm, int32_t norm_whole, float mag, float qt_coef,
                                      int32_t qt_every, int32_t act_dtype, mi355_stream_t stream) {
    MI355_CHECK_ARG(qkv && geom && pos && seq && rows > 0, "hy_attn_prep: null argument");
    MI355_CHECK_ARG(qt_coef == 0.f || qt_every > 0, "hy_attn_prep: query temperature every %d positions", qt_every);
    const AttnPrepExtra ex{qnorm, knorm, mag, qt_coef, qt_every, norm_whole};
    const AttnGeom g{geom[0], geom[1], geom[2], geom[3], geom[4], geom[5], geom[6], geom[7], geom[8], geom[9], geom[10] > 0 ? geom[10] : geom[3]};
    if (int e = hy_geom_ok(g)) return e;
    MI355_CHECK_ARG((g.rot_dims == 0 || kfreq) && (!kcache || (vcache && block_table)), "hy_attn_prep: missing table or cache");
    MI355_CHECK_ARG(!vfreq || g.vdim % 2 == 0, "hy_attn_prep: rotated values need an even value size (%d)", g.vdim);
    HY_DISPATCH(act_dtype, hipLaunchKernelGGL(hy_attn_prep_kernel<T>, dim3(rows), dim3(256), 0, (hipStream_t)stream, qkv, ld, koff, voff, g, kfreq, vfreq,
                                              v_norm, eps, pos, seq, block_table, (T*)kcache, (T*)vcache, ex));
    MI355_CHECK_LAUNCH("hy_attn_prep_kernel");
    return MI355_OK;
}

// out [rows, H * vdim] of act_dtype.  chunk > 0: row at position i sees keys j <= i of its own block of `chunk` positions; 0: all j <= i.
// splits > 1 (few rows with long contexts): the key tiles of a row are dealt over `splits` blocks that leave partial sums in parts
// (fp32 [rows, H, splits, vdim + 2]) and a second launch merges them; splits == 1 needs no parts.
// sink: null, or fp32 [H]: exp(sink[h]) is added to head h's softmax denominator (a key of that unscaled score without a value).  vfreq non-null: the head output is turned back by the row's position.
extern "C" int mi355_hy_attn_rows(const float* q, int32_t ldq, float scale, const int32_t* geom, int32_t chunk, const float* sink, const float* vfreq,
                                  const int32_t* pos, const int32_t* seq, const int32_t* block_table, int32_t rows, const void* kcache,
                                  const void* vcache, void* out, int32_t splits, float* parts, int32_t act_dtype, mi355_stream_t stream) {
    return mi355_hy_attn_rows_ex(q, ldq, scale, geom, chunk, sink, vfreq, pos, seq, block_table, rows, kcache, vcache, out, splits, parts, 0, 0.f, nullptr, 0,
                                 act_dtype, stream);
}

// The same with a sliding window (window > 0, chunk must be 0: keys j with 0 <= i - j < window), a tanh cap on the scaled scores (softcap > 0) and a
// sigmoid gate per (row, head) on the output (ogate fp32 [rows, ldg], column h; null: none).
extern "C" int mi355_hy_attn_rows_ex(const float* q, int32_t ldq, float scale, const int32_t* geom, int32_t chunk, const float* sink, const float* vfreq,
                                     const int32_t* pos, const int32_t* seq, const int32_t* block_table, int32_t rows, const void* kcache,
                                     const void* vcache, void* out, int32_t splits, float* parts, int32_t window, float softcap, const float* ogate,
                                     int32_t ldg, int32_t act_dtype, mi355_stream_t stream) {
    MI355_CHECK_ARG(window >= 0 && (window == 0 || chunk == 0) && softcap >= 0.f && (!ogate || ldg >= geom[0]), "hy_attn_rows: window=%d chunk=%d ldg=%d", window, chunk, ldg);
    const AttnExtra ex{window, softcap, ogate, ldg};
    MI355_CHECK_ARG(q && geom && pos && seq && block_table && kcache && vcache && out && rows > 0 && chunk >= 0, "hy_attn_rows: bad argument");
    MI355_CHECK_ARG(splits >= 1 && splits <= 64 && (splits == 1 || parts), "hy_attn_rows: %d splits", splits);
    MI355_CHECK_ARG(!vfreq || geom[3] % 2 == 0, "hy_attn_rows: rotated values need an even value size (%d)", geom[3]);
    const AttnGeom g{geom[0], geom[1], geom[2], geom[3], geom[4], geom[5], geom[6], geom[7], geom[8], geom[9], geom[10] > 0 ? geom[10] : geom[3]};
    if (int e = hy_geom_ok(g)) return e;
    const int threads = rows * g.H <= 2048 ? 1024 : 256;     // few (decode) rows: sixteen waves share a row's keys
    HY_DISPATCH(act_dtype, hipLaunchKernelGGL(hy_attn_rows_kernel<T>, dim3(rows, g.H, splits), dim3(threads), 0, (hipStream_t)stream, q, ldq, scale, g, chunk, sink, vfreq,
                                              pos, seq, block_table, (const T*)kcache, (const T*)vcache, (T*)out, parts, ex));
    MI355_CHECK_LAUNCH("hy_attn_rows_kernel");
    if (splits > 1) {
        HY_DISPATCH(act_dtype, hipLaunchKernelGGL(hy_attn_merge_kernel<T>, dim3(rows, g.H), dim3(256), 0, (hipStream_t)stream, parts, splits, g, vfreq, pos, (T*)out, ex));
        MI355_CHECK_LAUNCH("hy_attn_merge_kernel");
    }
    return MI355_OK;
}

// The same attention for prompt portions (bf16 cache): tile t covers rows tile_row0[t] .. + tile_n[t] - 1 (<= 16, consecutive positions of one
// sequence).  Needs dim % 32 == 0 and vdim % 16 == 0 (% 32 under the halves layout), both <= 256: MI355_ERR_UNSUPPORTED otherwise.
extern "C" int mi355_hy_attn_tiles(const float* q, int32_t ldq, float scale, const int32_t* geom, int32_t chunk, const float* sink, const float* vfreq,
                                   const int32_t* pos, const int32_t* seq, const int32_t* block_table, const int32_t* tile_row0,
                                   const int32_t* tile_n, int32_t tiles, const void* kcache, const void* vcache, void* out, int32_t act_dtype,
                                   mi355_stream_t stream) {
    return mi355_hy_attn_tiles_ex(q, ldq, scale, geom, chunk, sink, vfreq, pos, seq, block_table, tile_row0, tile_n, tiles, kcache, vcache, out, 0, 0.f, nullptr, 0,
                                  act_dtype, stream);
}

extern "C" int mi355_hy_attn_tiles_ex(const float* q, int32_t ldq, float scale, const int32_t* geom, int32_t chunk, const float* sink, const float* vfreq,
                                      const int32_t* pos, const int32_t* seq, const int32_t* block_table, const int32_t* tile_row0,
                                      const int32_t* tile_n, int32_t tiles, const void* kcache, const void* vcache, void* out, int32_t window, float softcap,
                                      const float* ogate, int32_t ldg, int32_t act_dtype, mi355_stream_t stream) {
    MI355_CHECK_ARG(window >= 0 && (window == 0 || chunk == 0) && softcap >= 0.f && (!ogate || ldg >= geom[0]), "hy_attn_tiles: window=%d chunk=%d ldg=%d", window, chunk, ldg);
    const AttnExtra ex{window, softcap, ogate, ldg};
    MI355_CHECK_ARG(q && geom && pos && seq && block_table && tile_row0 && tile_n && kcache && vcache && out && tiles > 0 && chunk >= 0, "hy_attn_tiles: bad argument");
    const AttnGeom g{geom[0], geom[1], geom[2], geom[3], geom[4], geom[5], geom[6], geom[7], geom[8], geom[9], geom[10] > 0 ? geom[10] : geom[3]};
    if (int e = hy_geom_ok(g)) return e;
    if (act_dtype != MI355_ACT_BF16 || g.dim % 32 || g.dim > 256 || g.vdim % 16 || g.vdim > 256 || g.v_ld % 8 || (vfreq && g.v_layout != 0 && g.vdim % 32)) {
        mi355_set_error("hy_attn_tiles: bf16, dim %% 32 == 0, vdim %% 16 == 0 only (dim=%d vdim=%d dtype=%d)", g.dim, g.vdim, act_dtype);
        return MI355_ERR_UNSUPPORTED;
    }
    const int gq = g.H / g.G, nwv = gq % 4 == 0 ? 4 : gq % 2 == 0 ? 2 : 1;       // query heads of one key/value head per block
#define HY_TILES(DKM_, NCBM_, NWV_)                                                                                                            \
    hipLaunchKernelGGL((hy_attn_tiles_kernel<DKM_, NCBM_, NWV_>), dim3((tiles + 1) / 2, g.H / NWV_), dim3(64 * NWV_), 0, (hipStream_t)stream, q, ldq, scale, g, chunk, \
                       sink, vfreq, pos, seq, block_table, tile_row0, tile_n, tiles, (const bf16*)kcache, (const bf16*)vcache, (bf16*)out, ex)
    if (g.dim <= 128 && g.vdim <= 128) { if (nwv == 4) HY_TILES(4, 8, 4); else if (nwv == 2) HY_TILES(4, 8, 2); else HY_TILES(4, 8, 1); }
    else                               { if (nwv == 4) HY_TILES(8, 16, 4); else if (nwv == 2) HY_TILES(8, 16, 2); else HY_TILES(8, 16, 1); }
#undef HY_TILES
    MI355_CHECK_LAUNCH("hy_attn_tiles_kernel");
    return MI355_OK;
}

// mode 0 (HGRN2): q = silu(proj q), f = lower + (1 - lower) sigmoid(proj k + fbias), a = f, k = 1 - f.
// mode 1 (GLA):   q = proj q * qscale, k = proj k, a = sigmoid(z)^(1 / tau).
// mode 2 (fixed): q = proj q, k = proj k, a = lower[h] (fp32 [H], one decay per head whatever act_dtype is).
// mode 3 (fixed, silu): q = silu(proj q), k = silu(proj k), v = silu(proj v), a = lower[h] as in mode 2.
// mode 6 / 7: modes 2 / 3 as the third pass of the chunked form: the states are only read, out[t] += a^(t - first row + 1) S^T q_t.
// Sequence s owns rows row_start[s] .. row_start[s + 1] - 1 in order, continues the state in slot[s] (starts from zero when first_pos[s] == 0)
// and leaves the new state there.  out fp32 [rows, H * vdim].
extern "C" int mi355_hy_scan(int32_t mode, const float* proj, int32_t ld, int32_t qo, int32_t ko, int32_t vo, const float* z, int32_t ldz,
                             const void* lower, const void* fbias, float tau, float qscale, int32_t H, int32_t dim, int32_t vdim,
                             const int32_t* row_start, const int32_t* slot, const int32_t* first_pos, int32_t nseq, float* state, float* out,
                             int32_t act_dtype, mi355_stream_t stream) {
    MI355_CHECK_ARG(proj && row_start && slot && first_pos && state && out && nseq > 0 && H > 0 && dim > 0 && vdim > 0, "hy_scan: bad argument");
    const int apply = mode & 4;                                   // mode + 4 (fixed-decay modes only): the read-only pass over chunk-start states
    mode &= 3;
    MI355_CHECK_ARG(mode == SCAN_HGRN2 ? (lower && fbias) : (mode == SCAN_FIXED || mode == SCAN_FIXED_SILU) ? lower != nullptr : (mode == SCAN_GLA && z && tau > 0.f),
                    "hy_scan: mode %d lacks its gate inputs", mode);
    MI355_CHECK_ARG(!apply || mode == SCAN_FIXED || mode == SCAN_FIXED_SILU, "hy_scan: the read-only pass belongs to the fixed-decay modes (mode %d)", mode);
    mode |= apply;
    MI355_CHECK_ARG(dim <= 512, "hy_scan: key size %d > 512", dim);
    const int RD = dim <= 128 ? 8 : dim <= 256 ? 16 : 32;       // rows per thread: at most 16 groups of RD rows (1024 threads)
    const int DS = (dim + RD - 1) / RD;
    int tok = 16;                                                // staged tokens: keep the LDS buffers under 60 KiB
    auto lds_of = [&](int t) { return (size_t)(3 * t * DS * RD + t * 64 + t * DS * 64) * 4; };
    while (tok > 1 && lds_of(tok) > 60 * 1024) tok >>= 1;
    ScanParams p{proj, ld, qo, ko, vo, z, ldz, lower, fbias, tau, qscale, mode & 3, H, dim, vdim, row_start, slot, first_pos, state, out, tok, (mode & 4) ? 1 : 0};
    const size_t lds = lds_of(tok);
    const dim3 grid(nseq, H, (vdim + 63) / 64);
    if (RD == 8)       HY_DISPATCH(act_dtype, hipLaunchKernelGGL((hy_scan_kernel<T, 8>), grid, dim3(64 * DS), lds, (hipStream_t)stream, p));
    else if (RD == 16) HY_DISPATCH(act_dtype, hipLaunchKernelGGL((hy_scan_kernel<T, 16>), grid, dim3(64 * DS), lds, (hipStream_t)stream, p));
    else               HY_DISPATCH(act_dtype, hipLaunchKernelGGL((hy_scan_kernel<T, 32>), grid, dim3(64 * DS), lds, (hipStream_t)stream, p));
    MI355_CHECK_LAUNCH("hy_scan_kernel");
    return MI355_OK;
}

// The plan of the chunked form for the sequences row_start[0 .. nseq]: chunks of C rows, at most max_chunks (>= rows / C + nseq).  cs int32 [max_chunks + 1],
// sc int32 [nseq + 1]; ids / zeros / ones int32 [max_chunks]: 0, 1, 2 .. / all 0 / all 1 (slot and first_pos arrays of the chunk passes).
extern "C" int mi355_hy_chunk_plan(const int32_t* row_start, int32_t nseq, int32_t C, int32_t max_chunks, int32_t* cs, int32_t* sc, int32_t* ids, int32_t* zeros,
                                   int32_t* ones, mi355_stream_t stream) {
    MI355_CHECK_ARG(row_start && cs && sc && ids && zeros && ones && nseq > 0 && C > 0 && max_chunks > 0, "hy_chunk_plan: nseq=%d C=%d chunks=%d", nseq, C, max_chunks);
    hipLaunchKernelGGL(hy_chunk_plan_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, row_start, nseq, C, max_chunks, cs, sc, ids, zeros, ones);
    MI355_CHECK_LAUNCH("hy_chunk_plan_kernel");
    return MI355_OK;
}

// Pass 2 of the chunked form: chunk_state fp32 [chunks, H, dim * vdim] holds the chunks' own contributions and receives the states at their starts;
// state [slots, H, dim * vdim] is continued (from zero where first_pos is 0) and receives the sequences' final states.  decay fp32 [H].
extern "C" int mi355_hy_chunk_prefix(const int32_t* cs, const int32_t* sc, const int32_t* slot, const int32_t* first_pos, int32_t nseq, const float* decay, int32_t H,
                                     int32_t per_head, float* chunk_state, float* state, mi355_stream_t stream) {
    MI355_CHECK_ARG(cs && sc && slot && first_pos && decay && chunk_state && state && nseq > 0 && H > 0 && per_head > 0, "hy_chunk_prefix: nseq=%d H=%d", nseq, H);
    hipLaunchKernelGGL(hy_chunk_prefix_kernel, dim3(nseq, H, (per_head + 255) / 256), dim3(256), 0, (hipStream_t)stream, cs, sc, slot, first_pos, decay, H, per_head,
                       chunk_state, state);
    MI355_CHECK_LAUNCH("hy_chunk_prefix_kernel");
    return MI355_OK;
}

// proj fp32 [rows, ld]: receptance r, key k (H heads of dim) at columns ro, ko, value v (H heads of vdim) at vo, removal pre-activation (H heads of dim,
// bias included) at ao; z fp32 [rows, ldz]: decay pre-activation (H heads of dim, bias included).  w = exp(-decay_mult sigmoid(z)), a = sigmoid(.),
// u = k / sqrt(|k|^2 + unit_eps).  Sequences, slots and the state [slots, H, dim, vdim] as in mi355_hy_scan.  out fp32 [rows, H * vdim].  dim <= 256.
extern "C" int mi355_hy_delta_scan(const float* proj, int32_t ld, int32_t ro, int32_t ko, int32_t vo, int32_t ao, const float* z, int32_t ldz,
                                   float decay_mult, float unit_eps, int32_t H, int32_t dim, int32_t vdim, const int32_t* row_start, const int32_t* slot,
                                   const int32_t* first_pos, int32_t nseq, float* state, float* out, mi355_stream_t stream) {
    MI355_CHECK_ARG(proj && z && row_start && slot && first_pos && state && out && nseq > 0 && H > 0 && dim > 0 && vdim > 0, "hy_delta_scan: bad argument");
    MI355_CHECK_ARG(dim <= 256, "hy_delta_scan: key size %d > 256", dim);
    MI355_CHECK_ARG(ld >= H * dim && ldz >= H * dim && unit_eps >= 0.f, "hy_delta_scan: ld=%d ldz=%d", ld, ldz);
    DeltaParams p{proj, ld, ro, ko, vo, ao, z, ldz, decay_mult, unit_eps, H, dim, vdim, row_start, slot, first_pos, state, out};
    hipStream_t st = (hipStream_t)stream;
    // sixteen lanes per value column (16 columns per block) for heads of more than 32 key channels, four (64 columns per block) below
    const dim3 g16(nseq, H, (vdim + 15) / 16), g4(nseq, H, (vdim + 63) / 64);
    if (dim <= 16)       hipLaunchKernelGGL((hy_delta_kernel<4, 4>), g4, dim3(256), 0, st, p);
    else if (dim <= 32)  hipLaunchKernelGGL((hy_delta_kernel<8, 4>), g4, dim3(256), 0, st, p);
    else if (dim <= 64)  hipLaunchKernelGGL((hy_delta_kernel<4, 16>), g16, dim3(256), 0, st, p);
    else if (dim <= 128) hipLaunchKernelGGL((hy_delta_kernel<8, 16>), g16, dim3(256), 0, st, p);
    else if (dim <= 192) hipLaunchKernelGGL((hy_delta_kernel<12, 16>), g16, dim3(256), 0, st, p);
    else                 hipLaunchKernelGGL((hy_delta_kernel<16, 16>), g16, dim3(256), 0, st, p);
    MI355_CHECK_LAUNCH("hy_delta_kernel");
    return MI355_OK;
}

extern "C" int mi355_hy_head_norm(const float* o, int32_t rows, int32_t H, int32_t vdim, const void* w, float eps, const float* gate, int32_t ldg,
                                  int32_t goff, void* out, int32_t act_dtype, mi355_stream_t stream) {
    return mi355_hy_head_norm_ex(o, rows, H, vdim, w, eps, gate, ldg, goff, out, 0, 0, act_dtype, stream);
}

// w_heads: w is [H * vdim] (a weight per head and channel) instead of [vdim]; gate_sigmoid: the gate is sigmoid(gate) instead of silu(gate).
extern "C" int mi355_hy_head_norm_ex(const float* o, int32_t rows, int32_t H, int32_t vdim, const void* w, float eps, const float* gate, int32_t ldg,
                                     int32_t goff, void* out, int32_t w_heads, int32_t gate_sigmoid, int32_t act_dtype, mi355_stream_t stream) {
    MI355_CHECK_ARG(o && out && rows > 0 && H > 0 && vdim > 0, "hy_head_norm: bad argument");
    HY_DISPATCH(act_dtype, hipLaunchKernelGGL(hy_head_norm_kernel<T>, dim3(rows, H), dim3(vdim > 256 ? std::min(1024, (vdim + 255) / 256 * 64) : 64), 0, (hipStream_t)stream, o, H, vdim, (const T*)w, eps,
                                              gate, ldg, goff, (T*)out, w_heads, gate_sigmoid));
    MI355_CHECK_LAUNCH("hy_head_norm_kernel");
    return MI355_OK;
}

// geom: {H, dim, dr, R, dpad, rdims, page, max_blocks, num_pages}.  proj fp32 [rows, ld]: H query heads of dim + dr channels from column 0, the down
// projection (R + dr channels) from column doff.  freq [rdims / 2] fp32, mag multiplies cos and sin; cw [R] norm weight of act_dtype.
// qn [rows, H * dim] act_dtype, qabs fp32 [rows, H * dpad] (columns R .. dpad - 1 of every head are written), cache [pages, page, dpad] act_dtype.
extern "C" int mi355_hy_latent_prep(const float* proj, int32_t ld, int32_t doff, const int32_t* geom, const float* freq, float mag, const void* cw, float eps,
                                    const int32_t* pos, const int32_t* seq, const int32_t* block_table, int32_t rows, void* qn, float* qabs, void* cache,
                                    int32_t act_dtype, mi355_stream_t stream) {
    MI355_CHECK_ARG(proj && geom && cw && pos && seq && block_table && qn && qabs && cache && rows > 0, "hy_latent_prep: null argument");
    const LatentGeom g{geom[0], geom[1], geom[2], geom[3], geom[4], geom[5], geom[6], geom[7], geom[8]};
    MI355_CHECK_ARG(g.H > 0 && g.dim > 0 && g.dr >= 0 && g.R > 0 && g.dpad >= g.R + g.dr && g.rdims >= 0 && g.rdims <= g.dr && g.rdims % 2 == 0 && (g.rdims == 0 || freq),
                    "hy_latent_prep: heads=%d dim=%d rot=%d rank=%d padded=%d span=%d", g.H, g.dim, g.dr, g.R, g.dpad, g.rdims);
    MI355_CHECK_ARG(g.page > 0 && g.max_blocks > 0 && g.num_pages > 0 && ld >= doff + g.R + g.dr && doff >= g.H * (g.dim + g.dr), "hy_latent_prep: ld=%d doff=%d", ld, doff);
    HY_DISPATCH(act_dtype, hipLaunchKernelGGL(hy_latent_prep_kernel<T>, dim3(rows), dim3(256), 0, (hipStream_t)stream, proj, ld, doff, g, freq, mag, (const T*)cw, eps,
                                              pos, seq, block_table, (T*)qn, qabs, (T*)cache));
    MI355_CHECK_LAUNCH("hy_latent_prep_kernel");
    return MI355_OK;
}

// buf fp32 [rows, ld]; segment i: heads_i heads of dim_i channels from column off_i, multiplied by scale_i after the turn (heads1 = 0: one segment).
extern "C" int mi355_hy_rotary(float* buf, int32_t ld, int32_t rows, int32_t off0, int32_t heads0, int32_t dim0, float scale0, int32_t off1, int32_t heads1,
                               int32_t dim1, float scale1, int32_t rdims, int32_t layout, const float* freq, float mag, const int32_t* pos, mi355_stream_t stream) {
    MI355_CHECK_ARG(buf && pos && rows > 0 && rdims >= 0 && rdims % 2 == 0 && (rdims == 0 || freq) && (layout == 0 || layout == 1), "hy_rotary: bad argument");
    MI355_CHECK_ARG(heads0 >= 0 && heads1 >= 0 && (heads0 == 0 || rdims <= dim0) && (heads1 == 0 || rdims <= dim1), "hy_rotary: span %d of heads of %d / %d", rdims, dim0, dim1);
    MI355_CHECK_ARG(off0 + heads0 * dim0 <= ld && off1 + heads1 * dim1 <= ld, "hy_rotary: segments past the row (ld=%d)", ld);
    hipLaunchKernelGGL(hy_rotary_kernel, dim3(rows), dim3(256), 0, (hipStream_t)stream, buf, ld, RotSeg{off0, heads0, dim0, scale0}, RotSeg{off1, heads1, dim1, scale1},
                       rdims, layout, freq, mag, pos);
    MI355_CHECK_LAUNCH("hy_rotary_kernel");
    return MI355_OK;
}

extern "C" int mi355_hy_polynorm(const float* z, int32_t ld, int32_t rows, int32_t n, float ca, float cb, float cc, float ce, float eps, void* out, int32_t ldo,
                                 int32_t act_dtype, mi355_stream_t stream) {
    MI355_CHECK_ARG(z && out && rows > 0 && n > 0 && ld >= n && ldo >= n, "hy_polynorm: rows=%d n=%d", rows, n);
    HY_DISPATCH(act_dtype, hipLaunchKernelGGL(hy_polynorm_kernel<T>, dim3(rows), dim3(256), 0, (hipStream_t)stream, z, ld, n, ca, cb, cc, ce, eps, (T*)out, ldo));
    MI355_CHECK_LAUNCH("hy_polynorm_kernel");
    return MI355_OK;
}

// z fp32 [tokens, ld] router logits -> ids int32 [tokens, top], wts fp32 [tokens, top]
extern "C" int mi355_hy_moe_route(const float* z, int32_t ld, int32_t tokens, int32_t E, int32_t groups, int32_t keep, int32_t top, int32_t* ids, float* wts,
                                  mi355_stream_t stream) {
    return mi355_hy_moe_route_ex(z, ld, tokens, E, groups, keep, top, ids, wts, 0, 1, 1.f, stream);
}

// The same with the router's form as arguments: score_sigmoid (scores are sigmoids of the logits instead of their softmax), group_top (1: a group
// scores as its best expert; 2: as the sum of its two best), wscale (the chosen experts weigh score * wscale).
extern "C" int mi355_hy_moe_route_ex(const float* z, int32_t ld, int32_t tokens, int32_t E, int32_t groups, int32_t keep, int32_t top, int32_t* ids, float* wts,
                                     int32_t score_sigmoid, int32_t group_top, float wscale, mi355_stream_t stream) {
    MI355_CHECK_ARG(group_top == 1 || group_top == 2, "hy_moe_route: a group scores by its best %d experts (1 or 2)", group_top);
    const RouteMode rm{score_sigmoid, group_top, wscale};
    MI355_CHECK_ARG(z && ids && wts && tokens > 0 && E > 0 && ld >= E, "hy_moe_route: tokens=%d experts=%d", tokens, E);
    MI355_CHECK_ARG(groups >= 1 && E % groups == 0 && keep >= 1 && keep <= groups && top >= 1 && top <= (E / groups) * keep, "hy_moe_route: %d experts in %d groups, keep %d, top %d",
                    E, groups, keep, top);
    MI355_CHECK_ARG((size_t)(E + groups) * 4 <= 48 * 1024, "hy_moe_route: %d experts do not fit the block's scratch", E);
    hipLaunchKernelGGL(hy_moe_route_kernel, dim3(tokens), dim3(64), (size_t)(E + groups) * 4, (hipStream_t)stream, z, ld, E, groups, keep, top, ids, wts, rm);
    MI355_CHECK_LAUNCH("hy_moe_route_kernel");
    return MI355_OK;
}

// tiles: int32 [1 + 2 * (n / 64 + E)] (at most n / 64 + E tiles hold rows)
extern "C" int mi355_hy_moe_align(const int32_t* ids, int32_t n, int32_t top, int32_t E, int32_t* offs, int32_t* src_row, int32_t* place_of, int32_t* tiles,
                                  mi355_stream_t stream) {
    MI355_CHECK_ARG(ids && offs && src_row && place_of && tiles && n > 0 && top > 0 && E > 0 && (size_t)E * 8 <= 48 * 1024, "hy_moe_align: n=%d experts=%d", n, E);
    hipLaunchKernelGGL(hy_moe_align_kernel, dim3(1), dim3(1024), (size_t)E * 8, (hipStream_t)stream, ids, n, top, E, offs, src_row, place_of, tiles);
    MI355_CHECK_LAUNCH("hy_moe_align_kernel");
    return MI355_OK;
}

// Both in one launch for a few tokens (tokens <= 64 and the scratch of sixteen waves fits: MI355_ERR_UNSUPPORTED otherwise).
extern "C" int mi355_hy_moe_route_align(const float* z, int32_t ld, int32_t tokens, int32_t E, int32_t groups, int32_t keep, int32_t top, int32_t* ids, float* wts,
                                        int32_t* offs, int32_t* src_row, int32_t* place_of, int32_t* tiles, mi355_stream_t stream) {
    return mi355_hy_moe_route_align_ex(z, ld, tokens, E, groups, keep, top, ids, wts, offs, src_row, place_of, tiles, 0, 1, 1.f, stream);
}

extern "C" int mi355_hy_moe_route_align_ex(const float* z, int32_t ld, int32_t tokens, int32_t E, int32_t groups, int32_t keep, int32_t top, int32_t* ids,
                                           float* wts, int32_t* offs, int32_t* src_row, int32_t* place_of, int32_t* tiles, int32_t score_sigmoid,
                                           int32_t group_top, float wscale, mi355_stream_t stream) {
    MI355_CHECK_ARG(group_top == 1 || group_top == 2, "hy_moe_route_align: a group scores by its best %d experts (1 or 2)", group_top);
    const RouteMode rm{score_sigmoid, group_top, wscale};
    MI355_CHECK_ARG(z && ids && wts && offs && src_row && place_of && tiles && tokens > 0 && E > 0 && ld >= E, "hy_moe_route_align: tokens=%d experts=%d", tokens, E);
    MI355_CHECK_ARG(groups >= 1 && E % groups == 0 && keep >= 1 && keep <= groups && top >= 1 && top <= (E / groups) * keep, "hy_moe_route_align: %d experts in %d groups, keep %d, top %d",
                    E, groups, keep, top);
    const size_t lds = (size_t)16 * (E + groups) * 4 + (size_t)E * 8;
    if (tokens > 64 || lds > 48 * 1024) {
        mi355_set_error("hy_moe_route_align: %d tokens, %d experts: use the two launches", tokens, E);
        return MI355_ERR_UNSUPPORTED;
    }
    hipLaunchKernelGGL(hy_moe_route_align_kernel, dim3(1), dim3(1024), lds, (hipStream_t)stream, z, ld, tokens, E, groups, keep, top, ids, wts, offs, src_row, place_of, tiles, rm);
    MI355_CHECK_LAUNCH("hy_moe_route_align_kernel");
    return MI355_OK;
}

extern "C" int mi355_hy_moe_combine(const float* y, int32_t tokens, int32_t W, const int32_t* place_of, const float* wts, int32_t top, const float* extra, float* out,
                                    mi355_stream_t stream) {
    MI355_CHECK_ARG(y && place_of && wts && out && tokens > 0 && W > 0 && top > 0, "hy_moe_combine: tokens=%d W=%d", tokens, W);
    hipLaunchKernelGGL(hy_moe_combine_kernel, dim3(tokens), dim3(256), 0, (hipStream_t)stream, y, W, place_of, wts, top, extra, out);
    MI355_CHECK_LAUNCH("hy_moe_combine_kernel");
    return MI355_OK;
}
