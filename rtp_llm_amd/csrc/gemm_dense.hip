// Dense linear layers on weights kept in checkpoint layout: y[M, N] = x[M, K] . W[N, K]^T with W row-major [out, in].
//
// Both operands are contiguous along K, which is the layout v_mfma_f32_16x16x32_bf16 wants for its A and B fragments (8 consecutive k per
// lane), so no weight image is built: a model whose layers have many small, differently shaped projections (recurrent gates, low-rank
// decays, shared-KV attention) loads its tensors as they are.  Three kernels, all with fp32 accumulation and an fp32 epilogue:
//   * tile kernel, bf16:  64 x 128 block tile, 4 waves of 32 x 64, K staged through LDS 64 at a time, MFMA 16x16x32;
//   * tile kernel, fp32:  64 x 64 block tile, 4 x 4 register micro-tiles, true fp32 FMAs (no reduced-precision matrix mode);
//   * skinny kernel, bf16, 2 <= M <= 16: one block per 16 outputs, its waves split K, MFMA fragments loaded straight from memory;
//   * row kernel (M = 1; fp32 up to M = 16): a wave per output column streams its weight row once, 16-byte loads, wave reduction at the end.
//   * grouped forms of the tile kernels (per-head weights over column slices, or rows sorted by expert with a gather and a tile list) and
//     of the row kernel (the few rows of a decode step, each with its own expert's weight): mi355_dense_grouped.
// Epilogues: bias, gated activation act(gate) * up (weight rows grouped [32 gate | 32 up], so one lane holds both; also the clamped form
// min(g, L) sigmoid(1.702 min(g, L)) (clamp(u, -L, L) + 1)), tanh soft cap.
// Output is fp32 or the activation type.  A result row depends only on its own input row: the k order of the accumulation is fixed by
// the kernel, never by M or by the row's place in the batch.
#include "common.h"
#include "../../include/mi355_hybrid.h"

namespace {

constexpr int DN_ACT_NONE = 0, DN_ACT_RELU = 1, DN_ACT_SILU = 2, DN_ACT_GELU_TANH = 3, DN_ACT_TANH = 4, DN_ACT_SWIGLU_CLAMP = 5;

struct DenseParams {
    const void* x; const void* w; const void* bias; void* y;
    int M, N, K, ldx, ldy;
    int gated;       // 0: N outputs; 1: rows of w are [32 gate | 32 up] groups, N / 2 outputs
    int act;         // DN_ACT_* applied to the gate
    float act_param; // DN_ACT_SWIGLU_CLAMP: the limit of the gate (from above) and of the up value (both sides)
    int out_f32;
    float softcap;   // > 0: y = cap * tanh(y / cap)
    int vec;         // 16-byte loads allowed (alignment and K % 8 == 0 checked on the host)
    // groups (tile kernels, blockIdx.z): group g multiplies its rows by the weight w + g * ws (bias + g * N) and writes columns ys * g + ...
    // of y; it reads x from column xs * g on.  Its rows are all M rows, or rows offs[g] .. offs[g + 1] - 1 of a list sorted by group, whose
    // entry r reads x row gather[r] (identity without gather) and writes y row r.  tiles (with offs): {count, (group, first row) x count}, the
    // 64-row tiles that hold rows; blockIdx.y indexes this list instead of (blockIdx.z, row tile), so no block is spent on a tile without rows.
    int G;
    long long xs, ws, ys;
    const int32_t* offs; const int32_t* gather; const int32_t* tiles;
    // y[row, col] is multiplied by sigmoid(egate[row * ldg + goff + col]) before it is stored (fp32 pre-activations; null: no gate)
    const float* egate; int ldg, goff;
};

// first row and end of the rows of the block's tile in its group, and the group's operand bases
struct DnGroup { int m0, rend; long long xo, wo, yo; int bo; };
__device__ __forceinline__ DnGroup dn_group(const DenseParams& p, int tile_rows) {
    int g = blockIdx.z;
    DnGroup r;
    if (p.tiles) {
        const int i = blockIdx.y;
        if (i >= p.tiles[0]) { r.m0 = r.rend = 0; return r; }
        g = p.tiles[1 + 2 * i]; r.m0 = p.tiles[2 + 2 * i]; r.rend = p.offs[g + 1];
    } else {
        r.m0 = (p.offs ? p.offs[g] : 0) + blockIdx.y * tile_rows; r.rend = p.offs ? p.offs[g + 1] : p.M;
    }
    r.xo = p.xs * g; r.wo = p.ws * g; r.yo = p.ys * g; r.bo = g * p.N;
    return r;
}

__device__ __forceinline__ float dn_act(float g, int act) {
    if (act == DN_ACT_RELU) return g > 0.f ? g : 0.f;
    if (act == DN_ACT_SILU) return g / (1.f + __expf(-g));
    if (act == DN_ACT_GELU_TANH) return 0.5f * g * (1.f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
    if (act == DN_ACT_TANH) return tanhf(g);
    return g;
}

// act(gate) * up of a gated pair.  DN_ACT_SWIGLU_CLAMP: g' = min(g, L), u' = clamp(u, -L, L), g' sigmoid(1.702 g') (u' + 1).
__device__ __forceinline__ float dn_gated(float g, float u, int act, float lim) {
    if (act == DN_ACT_SWIGLU_CLAMP) {
        g = fminf(g, lim); u = fminf(fmaxf(u, -lim), lim);
        return g / (1.f + expf(-1.702f * g)) * (u + 1.f);
    }
    return dn_act(g, act) * u;
}

template <typename T> __device__ __forceinline__ float dn_ld(const T* p) { return (float)*p; }

template <typename T>
__device__ __forceinline__ void dn_store(const DenseParams& p, int row, int col, float v) {
    if (p.softcap > 0.f) v = p.softcap * tanhf(v / p.softcap);
    if (p.egate) v *= 1.f / (1.f + expf(-p.egate[(size_t)row * p.ldg + p.goff + col]));
    if (p.out_f32) ((float*)p.y)[(size_t)row * p.ldy + col] = v;
    else           ((T*)p.y)[(size_t)row * p.ldy + col] = (T)v;
}

// ------------------------------------------------------------------------------------------------ bf16 tile kernel
constexpr int TB_M = 64, TB_N = 128, TB_K = 64, TB_LD = TB_K + 8;   // LDS row stride in elements (144 bytes: 16-byte aligned)

__device__ __forceinline__ u32x4 dn_chunk_bf16(const bf16* base, int row, int rows, int k, int K, int ld, int vec) {
    u32x4 z = {0u, 0u, 0u, 0u};
    if (row >= rows || k >= K) return z;     // row 0x7fffffff: no row
    const bf16* p = base + (size_t)row * ld + k;
    if (vec) return *(const u32x4*)p;
    uint16_t e[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) e[i] = (k + i < K) ? __builtin_bit_cast(uint16_t, p[i]) : (uint16_t)0;
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = (uint32_t)e[2 * i] | ((uint32_t)e[2 * i + 1] << 16);
    return r;
}

__global__ __launch_bounds__(256) void dense_tile_bf16_kernel(DenseParams p) {
    __shared__ __attribute__((aligned(16))) bf16 As[TB_M * TB_LD];
    __shared__ __attribute__((aligned(16))) bf16 Bs[TB_N * TB_LD];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave & 1, wn = wave >> 1;                       // wave tile: rows wm*32.., cols wn*64..
    const DnGroup gr = dn_group(p, TB_M);
    const int m0 = gr.m0, n0 = blockIdx.x * TB_N;
    if (m0 >= gr.rend) return;
    const bf16* X = (const bf16*)p.x + gr.xo;
    const bf16* W = (const bf16*)p.w + gr.wo;
    const bf16* Bi = p.bias ? (const bf16*)p.bias + gr.bo : nullptr;
    int arow[2];                                                   // x rows this thread stages (past the group's end: none)
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int r = m0 + ((tid + i * 256) >> 3);
        arow[i] = r < gr.rend ? (p.gather ? p.gather[r] : r) : 0x7fffffff;
    }
    f32x4 acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    // staging: chunk c of 8 elements; A has 64 x 8 chunks (2 per thread), B 128 x 8 (4 per thread)
    u32x4 ra[2], rb[4];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 2; ++i) { const int c = tid + i * 256; ra[i] = dn_chunk_bf16(X, arow[i], 0x7fffffff, k0 + (c & 7) * 8, p.K, p.ldx, p.vec); }
#pragma unroll
        for (int i = 0; i < 4; ++i) { const int c = tid + i * 256; rb[i] = dn_chunk_bf16(W, n0 + (c >> 3), p.N, k0 + (c & 7) * 8, p.K, p.K, p.vec); }
    };
    fetch(0);
    for (int k0 = 0; k0 < p.K; k0 += TB_K) {
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 2; ++i) { const int c = tid + i * 256; *(u32x4*)&As[(c >> 3) * TB_LD + (c & 7) * 8] = ra[i]; }
#pragma unroll
        for (int i = 0; i < 4; ++i) { const int c = tid + i * 256; *(u32x4*)&Bs[(c >> 3) * TB_LD + (c & 7) * 8] = rb[i]; }
        __syncthreads();
        if (k0 + TB_K < p.K) fetch(k0 + TB_K);
#pragma unroll
        for (int ks = 0; ks < TB_K; ks += 32) {
            const int kk = ks + (lane >> 4) * 8, r = lane & 15;
            bf16x8 a[2], b[4];
#pragma unroll
            for (int i = 0; i < 2; ++i) a[i] = *(const bf16x8*)&As[(wm * 32 + i * 16 + r) * TB_LD + kk];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = *(const bf16x8*)&Bs[(wn * 64 + j * 16 + r) * TB_LD + kk];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
    }
    // C fragment: lane holds column (lane & 15), rows 4 * (lane >> 4) + e
    const int cl = lane & 15, rq = (lane >> 4) * 4;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = m0 + wm * 32 + i * 16 + rq + e;
            if (row >= gr.rend) continue;
            if (p.gated) {
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int ng = n0 + wn * 64 + j * 16 + cl;         // weight row of the gate; its up row is ng + 32
                    if (ng + 32 >= p.N) continue;
                    float g = acc[i][j][e], u = acc[i][j + 2][e];
                    if (Bi) { g += dn_ld(Bi + ng); u += dn_ld(Bi + ng + 32); }
                    dn_store<bf16>(p, row, (int)gr.yo + (ng >> 6) * 32 + (ng & 31), dn_gated(g, u, p.act, p.act_param));
                }
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int n = n0 + wn * 64 + j * 16 + cl;
                    if (n >= p.N) continue;
                    float v = acc[i][j][e];
                    if (Bi) v += dn_ld(Bi + n);
                    dn_store<bf16>(p, row, (int)gr.yo + n, dn_act(v, p.act));
                }
            }
        }
}

// ------------------------------------------------------------------------------------------------ fp32 tile kernel
constexpr int TF_M = 64, TF_N = 64, TF_K = 16, TF_LD = 68;

__device__ __forceinline__ f32x4 dn_chunk_f32(const float* base, int row, int rows, int k, int K, int ld, int vec) {
    f32x4 r = {0.f, 0.f, 0.f, 0.f};
    if (row >= rows || k >= K) return r;
    const float* p = base + (size_t)row * ld + k;
    if (vec) return *(const f32x4*)p;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = (k + i < K) ? p[i] : 0.f;
    return r;
}

__global__ __launch_bounds__(256) void dense_tile_f32_kernel(DenseParams p) {
    __shared__ __attribute__((aligned(16))) float As[TF_K * TF_LD];   // [k][m]
    __shared__ __attribute__((aligned(16))) float Bs[TF_K * TF_LD];   // [k][n]
    const int tid = threadIdx.x, ty = tid >> 4, tx = tid & 15;
    const DnGroup gr = dn_group(p, TF_M);
    const int m0 = gr.m0, n0 = blockIdx.x * TF_N;
    if (m0 >= gr.rend) return;
    const float* X = (const float*)p.x + gr.xo;
    const float* W = (const float*)p.w + gr.wo;
    const float* Bi = p.bias ? (const float*)p.bias + gr.bo : nullptr;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
    const int lr = tid >> 2, lk = (tid & 3) * 4;          // staging: row lr, k offset lk
    const int arow = m0 + lr < gr.rend ? (p.gather ? p.gather[m0 + lr] : m0 + lr) : 0x7fffffff;
    f32x4 ra = dn_chunk_f32(X, arow, 0x7fffffff, lk, p.K, p.ldx, p.vec);
    f32x4 rb = dn_chunk_f32(W, n0 + lr, p.N, lk, p.K, p.K, p.vec);
    for (int k0 = 0; k0 < p.K; k0 += TF_K) {
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 4; ++i) { As[(lk + i) * TF_LD + lr] = ra[i]; Bs[(lk + i) * TF_LD + lr] = rb[i]; }
        __syncthreads();
        if (k0 + TF_K < p.K) {
            ra = dn_chunk_f32(X, arow, 0x7fffffff, k0 + TF_K + lk, p.K, p.ldx, p.vec);
            rb = dn_chunk_f32(W, n0 + lr, p.N, k0 + TF_K + lk, p.K, p.K, p.vec);
        }
#pragma unroll
        for (int k = 0; k < TF_K; ++k) {
            const f32x4 a = *(const f32x4*)&As[k * TF_LD + ty * 4];
            const float b0 = Bs[k * TF_LD + 2 * tx], b1 = Bs[k * TF_LD + 2 * tx + 1];
            const float b2 = Bs[k * TF_LD + 32 + 2 * tx], b3 = Bs[k * TF_LD + 32 + 2 * tx + 1];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc[i][0] = __builtin_fmaf(a[i], b0, acc[i][0]); acc[i][1] = __builtin_fmaf(a[i], b1, acc[i][1]);
                acc[i][2] = __builtin_fmaf(a[i], b2, acc[i][2]); acc[i][3] = __builtin_fmaf(a[i], b3, acc[i][3]);
            }
        }
    }
    // thread columns: {2 tx, 2 tx + 1} of the first 32 and the same of the second 32 (gate / up of one channel under `gated`)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = m0 + ty * 4 + i;
        if (row >= gr.rend) continue;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int n = n0 + 2 * tx + j;
            if (p.gated) {
                if (n + 32 >= p.N) continue;
                float g = acc[i][j], u = acc[i][j + 2];
                if (Bi) { g += Bi[n]; u += Bi[n + 32]; }
                dn_store<float>(p, row, (int)gr.yo + (n >> 6) * 32 + (n & 31), dn_gated(g, u, p.act, p.act_param));
            } else {
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int nn = n + 32 * h;
                    if (nn >= p.N) continue;
                    float v = acc[i][j + 2 * h];
                    if (Bi) v += Bi[nn];
                    dn_store<float>(p, row, (int)gr.yo + nn, dn_act(v, p.act));
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------ row kernel (small M)
template <typename T> struct DnVec;
template <> struct DnVec<bf16> {
    static constexpr int W = 8;
    static __device__ __forceinline__ void load(const bf16* p, int n, int vec, float (&o)[8]) {
        if (vec && n >= 8) { act_unpack8<true>(*(const u32x4*)p, o); return; }
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = i < n ? (float)p[i] : 0.f;
    }
};
template <> struct DnVec<float> {
    static constexpr int W = 8;
    static __device__ __forceinline__ void load(const float* p, int n, int vec, float (&o)[8]) {
        if (vec && n >= 8) {
            const f32x4 a = *(const f32x4*)p, b = *(const f32x4*)(p + 4);
#pragma unroll
            for (int i = 0; i < 4; ++i) { o[i] = a[i]; o[4 + i] = b[i]; }
            return;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = i < n ? p[i] : 0.f;
    }
};

__device__ __forceinline__ float dn_wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// One wave per NC outputs: plain columns, or under GATED channels (a gate row and an up row each).  MR rows of x per pass: every 16-byte
// piece of x is loaded once per wave and meets NC (2 NC) weight pieces, so the wave streams its weight rows with few loads of x between.
template <typename T, int MR, int NC, bool GATED>
__global__ __launch_bounds__(256) void dense_rows_kernel(DenseParams p, int mbase) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int o0 = (blockIdx.x * 4 + wave) * NC;
    const int nout = GATED ? p.N / 2 : p.N;
    if (o0 >= nout) return;
    const T* X = (const T*)p.x;
    const T* W0[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int o = min(o0 + c, nout - 1);                       // a column past the end repeats the last one and is not stored
        W0[c] = (const T*)p.w + (size_t)(GATED ? (o >> 5) * 64 + (o & 31) : o) * p.K;
    }
    const int rows = min(MR, p.M - mbase);
    float a0[MR][NC], a1[GATED ? MR : 1][NC];
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int c = 0; c < NC; ++c) { a0[m][c] = 0.f; if (GATED) a1[m][c] = 0.f; }
    for (int k = lane * 8; k < p.K; k += 64 * 8) {
        float w0[NC][8], w1[GATED ? NC : 1][8], xv[8];
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            DnVec<T>::load(W0[c] + k, p.K - k, p.vec, w0[c]);
            if (GATED) DnVec<T>::load(W0[c] + (size_t)32 * p.K + k, p.K - k, p.vec, w1[c]);
        }
#pragma unroll
        for (int m = 0; m < MR; ++m) {
            if (m >= rows) break;
            DnVec<T>::load(X + (size_t)(mbase + m) * p.ldx + k, p.K - k, p.vec, xv);
#pragma unroll
            for (int c = 0; c < NC; ++c) {
#pragma unroll
                for (int i = 0; i < 8; ++i) a0[m][c] = __builtin_fmaf(xv[i], w0[c][i], a0[m][c]);
                if (GATED) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) a1[m][c] = __builtin_fmaf(xv[i], w1[c][i], a1[m][c]);
                }
            }
        }
    }
#pragma unroll
    for (int m = 0; m < MR; ++m) {
        if (m >= rows) break;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            float g = dn_wave_sum(a0[m][c]);
            float u = GATED ? dn_wave_sum(a1[m][c]) : 0.f;
            const int o = o0 + c;
            if (lane != 0 || o >= nout) continue;
            const int n0 = GATED ? (o >> 5) * 64 + (o & 31) : o;
            if (p.bias) { g += dn_ld((const T*)p.bias + n0); if (GATED) u += dn_ld((const T*)p.bias + n0 + 32); }
            dn_store<T>(p, mbase + m, o, GATED ? dn_gated(g, u, p.act, p.act_param) : dn_act(g, p.act));
        }
    }
}

// The same for a few rows that each belong to a group of their own (the experts of a decode step): blockIdx.y is the sorted row, its group is
// found in offs, a wave streams the weight row(s) of NC outputs of that group's weight once.
template <typename T, int NC, bool GATED>
__global__ __launch_bounds__(256) void dense_rows_grouped_kernel(DenseParams p) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int o0 = (blockIdx.x * 4 + wave) * NC, r = blockIdx.y;
    const int nout = GATED ? p.N / 2 : p.N;
    if (o0 >= nout || r >= p.offs[p.G]) return;
    int g = 0;
    while (g + 1 < p.G && p.offs[g + 1] <= r) ++g;
    const T* X = (const T*)p.x + (size_t)(p.gather ? p.gather[r] : r) * p.ldx + p.xs * g;
    const T* W0[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int o = min(o0 + c, nout - 1);
        W0[c] = (const T*)p.w + p.ws * g + (size_t)(GATED ? (o >> 5) * 64 + (o & 31) : o) * p.K;
    }
    float a0[NC], a1[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) a0[c] = a1[c] = 0.f;
    for (int k = lane * 8; k < p.K; k += 64 * 8) {
        float w0[NC][8], w1[GATED ? NC : 1][8], xv[8];
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            DnVec<T>::load(W0[c] + k, p.K - k, p.vec, w0[c]);
            if (GATED) DnVec<T>::load(W0[c] + (size_t)32 * p.K + k, p.K - k, p.vec, w1[c]);
        }
        DnVec<T>::load(X + k, p.K - k, p.vec, xv);
#pragma unroll
        for (int c = 0; c < NC; ++c) {
#pragma unroll
            for (int i = 0; i < 8; ++i) a0[c] = __builtin_fmaf(xv[i], w0[c][i], a0[c]);
            if (GATED) {
#pragma unroll
                for (int i = 0; i < 8; ++i) a1[c] = __builtin_fmaf(xv[i], w1[c][i], a1[c]);
            }
        }
    }
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        float gsum = dn_wave_sum(a0[c]);
        const float u = GATED ? dn_wave_sum(a1[c]) : 0.f;
        const int o = o0 + c;
        if (lane != 0 || o >= nout) continue;
        dn_store<T>(p, r, (int)(p.ys * g) + o, GATED ? dn_gated(gsum, u, p.act, p.act_param) : dn_act(gsum, p.act));
    }
}

template <typename T, bool GATED>
void launch_rows(const DenseParams& p, hipStream_t st) {
    const int nout = GATED ? p.N / 2 : p.N;
    for (int mb = 0; mb < p.M; mb += 16) {
        const int r = p.M - mb;
        // few rows: one output per wave keeps the most waves streaming; more rows: several outputs per wave share the loads of x
        if (r <= 2)      hipLaunchKernelGGL((dense_rows_kernel<T, 2, 1, GATED>), dim3((nout + 3) / 4), dim3(256), 0, st, p, mb);
        else if (r <= 4) hipLaunchKernelGGL((dense_rows_kernel<T, 4, 2, GATED>), dim3((nout + 7) / 8), dim3(256), 0, st, p, mb);
        else if (r <= 8) hipLaunchKernelGGL((dense_rows_kernel<T, 8, GATED ? 2 : 4, GATED>), dim3((nout + (GATED ? 7 : 15)) / (GATED ? 8 : 16)), dim3(256), 0, st, p, mb);
        else             hipLaunchKernelGGL((dense_rows_kernel<T, 16, GATED ? 2 : 4, GATED>), dim3((nout + (GATED ? 7 : 15)) / (GATED ? 8 : 16)), dim3(256), 0, st, p, mb);
    }
}

// ------------------------------------------------------------------------------------------------ skinny kernel (bf16, M <= 16)
// One block per 16 outputs; its NW waves split K in interleaved steps of 32 and each wave runs MFMA 16x16x32 with the (up to) 16 rows of x as
// the A operand and 16 weight rows as B, both fragments loaded straight from memory (8 consecutive k per lane, no LDS staging).  The weight
// stream is read once whatever M is; the waves' partial tiles are summed through LDS.  Under GATED a tile is 16 channels: their gate rows and
// their up rows share the A fragments.
template <bool GATED>
__global__ __launch_bounds__(512) void dense_skinny_bf16_kernel(DenseParams p, int mbase) {
    __shared__ f32x4 red[8][2][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, NW = blockDim.x >> 6;
    const int nout = GATED ? p.N / 2 : p.N;
    const int r = lane & 15, kq = (lane >> 4) * 8;
    const int o = min((int)blockIdx.x * 16 + r, nout - 1);
    const int n = GATED ? (o >> 5) * 64 + (o & 31) : o;
    const bf16* wg = (const bf16*)p.w + (size_t)n * p.K + kq;
    const bf16* wu = wg + (size_t)32 * p.K;
    const bf16* xr = (const bf16*)p.x + (size_t)min(mbase + r, p.M - 1) * p.ldx + kq;
    f32x4 ag = {0.f, 0.f, 0.f, 0.f}, au = {0.f, 0.f, 0.f, 0.f};
    const bf16x8 zero = {};
    const int stride = NW * 32;
    for (int k0 = wave * 32; k0 < p.K; k0 += 4 * stride) {
        bf16x8 a[4], b[4], c[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int k = k0 + u * stride;
            const bool ok = k + kq < p.K;
            a[u] = ok ? *(const bf16x8*)(xr + k) : zero;
            b[u] = ok ? *(const bf16x8*)(wg + k) : zero;
            if (GATED) c[u] = ok ? *(const bf16x8*)(wu + k) : zero;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            ag = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], b[u], ag, 0, 0, 0);
            if (GATED) au = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], c[u], au, 0, 0, 0);
        }
    }
    red[wave][0][lane] = ag;
    if (GATED) red[wave][1][lane] = au;
    __syncthreads();
    if (wave != 0) return;
    for (int w = 1; w < NW; ++w) {
        ag += red[w][0][lane];
        if (GATED) au += red[w][1][lane];
    }
    // C fragment: lane holds output (lane & 15), rows 4 * (lane >> 4) + e
    const int oc = blockIdx.x * 16 + r;
    if (oc >= nout) return;
    const int nb = GATED ? (oc >> 5) * 64 + (oc & 31) : oc;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int row = mbase + (lane >> 4) * 4 + e;
        if (row >= p.M) continue;
        float g = ag[e], u = au[e];
        if (p.bias) { g += dn_ld((const bf16*)p.bias + nb); if (GATED) u += dn_ld((const bf16*)p.bias + nb + 32); }
        dn_store<bf16>(p, row, oc, GATED ? dn_gated(g, u, p.act, p.act_param) : dn_act(g, p.act));
    }
}

} // namespace

// x [M, K] (row stride ldx) and w [N, K] of act_dtype (MI355_ACT_BF16 or MI355_ACT_F32); bias [N] of act_dtype or null;
// y [M, N or N / 2] fp32 (out_f32) or act_dtype, row stride ldy.  gated: the N weight rows are groups of 64 = 32 gate rows followed by
// the 32 up rows of the same channels (N % 64 == 0); y[m, c] = act(gate_c) * up_c.  act: 0 none, 1 relu, 2 silu, 3 gelu (tanh form), 4 tanh (on the gate,
// or on the plain output).  softcap > 0: y <- softcap * tanh(y / softcap).
extern "C" int mi355_dense_linear(const void* x, int32_t ldx, int32_t M, const void* w, int32_t N, int32_t K, const void* bias,
                                  void* y, int32_t ldy, int32_t out_f32, int32_t gated, int32_t act, float softcap,
                                  int32_t act_dtype, mi355_stream_t stream) {
    return mi355_dense_linear_ex(x, ldx, M, w, N, K, bias, y, ldy, out_f32, gated, act, 0.f, softcap, act_dtype, stream);
}

// The same with a parameter for the activation.  act 5 (gated only): with L = act_param > 0, g' = min(gate, L), u' = clamp(up, -L, L) and
// y = g' sigmoid(1.702 g') (u' + 1).
extern "C" int mi355_dense_linear_ex(const void* x, int32_t ldx, int32_t M, const void* w, int32_t N, int32_t K, const void* bias,
                                     void* y, int32_t ldy, int32_t out_f32, int32_t gated, int32_t act, float act_param, float softcap,
                                     int32_t act_dtype, mi355_stream_t stream) {
    MI355_CHECK_ARG(x && w && y && M > 0 && N > 0 && K > 0 && ldx >= K, "dense_linear: M=%d N=%d K=%d ldx=%d", M, N, K, ldx);
    MI355_CHECK_ARG(act_dtype == MI355_ACT_BF16 || act_dtype == MI355_ACT_F32, "dense_linear: act_dtype=%d (bf16 or fp32)", act_dtype);
    MI355_CHECK_ARG(!gated || N % 64 == 0, "dense_linear: gated needs N %% 64 == 0 (N=%d)", N);
    MI355_CHECK_ARG(act >= 0 && act <= 5 && (act != DN_ACT_SWIGLU_CLAMP || (gated && act_param > 0.f)), "dense_linear: act=%d (gated=%d, parameter %g)", act, gated, (double)act_param);
    MI355_CHECK_ARG(ldy >= (gated ? N / 2 : N), "dense_linear: ldy=%d", ldy);
    const bool bf = act_dtype == MI355_ACT_BF16;
    const size_t es = bf ? 2 : 4;
    DenseParams p;
    p.x = x; p.w = w; p.bias = bias; p.y = y; p.M = M; p.N = N; p.K = K; p.ldx = ldx; p.ldy = ldy;
    p.gated = gated; p.act = act; p.act_param = act_param; p.out_f32 = bf ? out_f32 : 1; p.softcap = softcap;
    p.vec = (K % 8 == 0) && (ldx % 8 == 0) && ((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0);
    p.G = 1; p.xs = p.ws = p.ys = 0; p.offs = nullptr; p.gather = nullptr; p.tiles = nullptr; p.egate = nullptr; p.ldg = p.goff = 0;
    (void)es;
    hipStream_t st = (hipStream_t)stream;
    if (bf && M > 1 && M <= 16 && p.vec) {
        const int tiles = ((gated ? N / 2 : N) + 15) / 16;
        const int nw = (tiles >= 1024 || K < 1024) ? 4 : 8;        // narrow outputs: more waves per tile keep the memory system busy
        if (gated) hipLaunchKernelGGL(dense_skinny_bf16_kernel<true>, dim3(tiles), dim3(64 * nw), 0, st, p, 0);
        else       hipLaunchKernelGGL(dense_skinny_bf16_kernel<false>, dim3(tiles), dim3(64 * nw), 0, st, p, 0);
        MI355_CHECK_LAUNCH("dense_skinny_bf16_kernel");
        return MI355_OK;
    }
    if (M <= 16) {
        if (bf) { if (gated) launch_rows<bf16, true>(p, st); else launch_rows<bf16, false>(p, st); }
        else    { if (gated) launch_rows<float, true>(p, st); else launch_rows<float, false>(p, st); }
        MI355_CHECK_LAUNCH("dense_rows_kernel");
        return MI355_OK;
    }
    if (bf) {
        const dim3 grid((N + TB_N - 1) / TB_N, (M + TB_M - 1) / TB_M);
        hipLaunchKernelGGL(dense_tile_bf16_kernel, grid, dim3(256), 0, st, p);
        MI355_CHECK_LAUNCH("dense_tile_bf16_kernel");
    } else {
        const dim3 grid((N + TF_N - 1) / TF_N, (M + TF_M - 1) / TF_M);
        hipLaunchKernelGGL(dense_tile_f32_kernel, grid, dim3(256), 0, st, p);
        MI355_CHECK_LAUNCH("dense_tile_f32_kernel");
    }
    return MI355_OK;
}

// The same product for G groups in one launch (tile kernels at every M): group g uses the weight w + g * N * K ([G, N, K] contiguous) and
// bias + g * N, reads x from column xs * g on and writes y from column ys * g on.  offs null: every group takes all M rows (per-head
// projections: xs, ys = the head's column step).  offs [G + 1] (device): M rows are sorted by group, group g owns rows offs[g] .. offs[g + 1] - 1;
// sorted row r reads x row gather[r] (device, or null for r itself) and writes y row r (experts of a mixture: xs = ys = 0).  A row's result
// depends on its own input and its group's weight only.  tiles (device, with offs; null: every group is given ceil(M / 64) row tiles, most of
// them empty): {n, (group, first row) x n}, the 64-row tiles that hold rows, at most max_tiles of them (mi355_hy_moe_align writes the list).
// egate (fp32 [M, ldg], or null): y[m, c] is multiplied by sigmoid(egate[m, goff + c]), c counted over the whole output row.
extern "C" int mi355_dense_grouped(const void* x, int32_t ldx, int32_t M, const void* w, int32_t N, int32_t K, const void* bias, void* y,
                                   int32_t ldy, int32_t out_f32, int32_t gated, int32_t act, int32_t act_dtype, int32_t G, int64_t xs,
                                   int64_t ys, const int32_t* offs, const int32_t* gather, const int32_t* tiles, int32_t max_tiles,
                                   const float* egate, int32_t ldg, int32_t goff, mi355_stream_t stream) {
    return mi355_dense_grouped_ex(x, ldx, M, w, N, K, bias, y, ldy, out_f32, gated, act, 0.f, act_dtype, G, xs, ys, offs, gather, tiles, max_tiles, egate, ldg,
                                  goff, stream);
}

// The same with the activation's parameter (act 5 as in mi355_dense_linear_ex).
extern "C" int mi355_dense_grouped_ex(const void* x, int32_t ldx, int32_t M, const void* w, int32_t N, int32_t K, const void* bias, void* y,
                                      int32_t ldy, int32_t out_f32, int32_t gated, int32_t act, float act_param, int32_t act_dtype, int32_t G,
                                      int64_t xs, int64_t ys, const int32_t* offs, const int32_t* gather, const int32_t* tiles, int32_t max_tiles,
                                      const float* egate, int32_t ldg, int32_t goff, mi355_stream_t stream) {
    MI355_CHECK_ARG(x && w && y && M > 0 && N > 0 && K > 0 && G > 0 && xs >= 0 && ys >= 0, "dense_grouped: M=%d N=%d K=%d G=%d", M, N, K, G);
    MI355_CHECK_ARG(ldx >= xs * (G - 1) + K, "dense_grouped: ldx=%d for %d groups of K=%d at step %lld", ldx, G, K, (long long)xs);
    MI355_CHECK_ARG(act_dtype == MI355_ACT_BF16 || act_dtype == MI355_ACT_F32, "dense_grouped: act_dtype=%d (bf16 or fp32)", act_dtype);
    MI355_CHECK_ARG(!gated || N % 64 == 0, "dense_grouped: gated needs N %% 64 == 0 (N=%d)", N);
    MI355_CHECK_ARG(act >= 0 && act <= 5 && (act != DN_ACT_SWIGLU_CLAMP || (gated && act_param > 0.f)), "dense_grouped: act=%d (gated=%d, parameter %g)", act, gated, (double)act_param);
    MI355_CHECK_ARG(ldy >= ys * (G - 1) + (gated ? N / 2 : N), "dense_grouped: ldy=%d", ldy);
    MI355_CHECK_ARG(G <= 65535 && (!gather || offs) && (!tiles || (offs && max_tiles > 0)), "dense_grouped: G=%d, gather and tiles need offs", G);
    const bool bf = act_dtype == MI355_ACT_BF16;
    DenseParams p;
    p.x = x; p.w = w; p.bias = bias; p.y = y; p.M = M; p.N = N; p.K = K; p.ldx = ldx; p.ldy = ldy;
    p.gated = gated; p.act = act; p.act_param = act_param; p.out_f32 = bf ? out_f32 : 1; p.softcap = 0.f;
    p.vec = (K % 8 == 0) && (ldx % 8 == 0) && (xs % 8 == 0) && ((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0);
    p.G = G; p.xs = xs; p.ws = (long long)N * K; p.ys = ys; p.offs = offs; p.gather = gather; p.tiles = tiles;
    p.egate = egate; p.ldg = ldg; p.goff = goff;
    MI355_CHECK_ARG(!egate || (goff >= 0 && ldg >= goff + (offs ? 0 : ys * (G - 1)) + (gated ? N / 2 : N)), "dense_grouped: gate row stride %d", ldg);
    static_assert(TB_M == 64 && TF_M == 64, "the tile list is made of 64-row tiles");
    hipStream_t st = (hipStream_t)stream;
    const int gy = tiles ? max_tiles : (M + 63) / 64, gz = tiles ? 1 : G;
    if (offs && M <= 16 && !bias) {            // a decode step's few rows: each streams its own group's weight
        const int nout = gated ? N / 2 : N, nc = gated ? 1 : 2;
        const dim3 grid((nout + 4 * nc - 1) / (4 * nc), M);
        if (bf) { if (gated) hipLaunchKernelGGL((dense_rows_grouped_kernel<bf16, 1, true>), grid, dim3(256), 0, st, p);
                  else       hipLaunchKernelGGL((dense_rows_grouped_kernel<bf16, 2, false>), grid, dim3(256), 0, st, p); }
        else    { if (gated) hipLaunchKernelGGL((dense_rows_grouped_kernel<float, 1, true>), grid, dim3(256), 0, st, p);
                  else       hipLaunchKernelGGL((dense_rows_grouped_kernel<float, 2, false>), grid, dim3(256), 0, st, p); }
        MI355_CHECK_LAUNCH("dense_rows_grouped_kernel");
        return MI355_OK;
    }
    if (bf) {
        const dim3 grid((N + TB_N - 1) / TB_N, gy, gz);
        hipLaunchKernelGGL(dense_tile_bf16_kernel, grid, dim3(256), 0, st, p);
        MI355_CHECK_LAUNCH("dense_tile_bf16_kernel");
    } else {
        const dim3 grid((N + TF_N - 1) / TF_N, gy, gz);
        hipLaunchKernelGGL(dense_tile_f32_kernel, grid, dim3(256), 0, st, p);
        MI355_CHECK_LAUNCH("dense_tile_f32_kernel");
    }
    return MI355_OK;
}
