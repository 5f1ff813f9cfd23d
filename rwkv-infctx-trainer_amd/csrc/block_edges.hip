// The element-wise passes on either side of the WKV operator inside a block:
//   * token shift + mixing of the block input (RWKV-v5/src/module/TimeMix.py:292-298, ChannelMix.py:44-47;
//     RWKV-v6/src/module/TimeMix.py:262-276, ChannelMix.py:31-35), forward and backward, any number of mixed
//     copies of x from one read of x;
//   * ln_x (GroupNorm, one group per head) times the SiLU gate on the operator's output
//     (RWKV-v5/src/module/TimeMix.py:301,317-320; RWKV-v6/src/module/TimeMix.py:278,296-298), forward and backward;
//   * the two activations of the channel mix (RWKV-v5/src/module/ChannelMix.py:48-49): relu(k)^2 and
//     sigmoid(r) * kv, forward and backward;
//   * the backward of L2Wrap (RWKV-v5/src/model.py:140-148): row maximum and its position.
// All of them are bound by HBM bandwidth: every tensor is read once and written once, eight channels per lane
// (16 bytes of bf16), rows walked by the same lane so that the previous token comes from registers.  Sums over
// tokens (parameter gradients) go through per-workgroup partial sums that a second kernel adds in a fixed order,
// so two runs give the same bits.
#include "common.h"

namespace wkv {
namespace edges {

constexpr int CH_LANES = 64, ROW_LANES = 4, VEC = 8, ROWS_PER_LANE = 8;
constexpr int TILE_C = CH_LANES * VEC;                   // channels per workgroup
constexpr int TILE_R = ROW_LANES * ROWS_PER_LANE;        // rows (tokens) per workgroup
constexpr int MAX_MIX = 5;

template <class T> __device__ __forceinline__ void load8(const T *p, float (&o)[8]) {
    float a[4], b[4];
    load4(p, a); load4(p + 4, b);
#pragma unroll
    for (int e = 0; e < 4; e++) { o[e] = a[e]; o[4 + e] = b[e]; }
}
template <class T> __device__ __forceinline__ void store8(T *p, const float (&o)[8]) {
    const float a[4] = {o[0], o[1], o[2], o[3]}, b[4] = {o[4], o[5], o[6], o[7]};
    store4(p, a); store4(p + 4, b);
}

// The same for a result that this pass does not read again: stored with the non-temporal hint, so that a tensor being
// written does not push the tensors being read out of the last-level cache (5 to 25 % on these passes taken alone,
// most at sizes near the cache's 256 MB).  The two channel-mix activations keep the plain store: their results are the
// very next matrix product's operand, and a layer measured as a whole is 1 % slower when they bypass the cache.
__device__ __forceinline__ void stream8(float *p, const float (&o)[8]) {
    typedef float f4_ __attribute__((ext_vector_type(4)));
    __builtin_nontemporal_store(f4_{o[0], o[1], o[2], o[3]}, reinterpret_cast<f4_ *>(p));
    __builtin_nontemporal_store(f4_{o[4], o[5], o[6], o[7]}, reinterpret_cast<f4_ *>(p + 4));
}
__device__ __forceinline__ void stream8(bf16 *p, const float (&o)[8]) {
    typedef unsigned int u4_ __attribute__((ext_vector_type(4)));
    __builtin_nontemporal_store(u4_{bf16_pack2(o[0], o[1]), bf16_pack2(o[2], o[3]), bf16_pack2(o[4], o[5]), bf16_pack2(o[6], o[7])},
                                reinterpret_cast<u4_ *>(p));
}
__device__ __forceinline__ void stream8(f16 *p, const float (&o)[8]) {
    typedef _Float16 h8_ __attribute__((ext_vector_type(8)));
    const h8_ x = {(_Float16)o[0], (_Float16)o[1], (_Float16)o[2], (_Float16)o[3], (_Float16)o[4], (_Float16)o[5], (_Float16)o[6], (_Float16)o[7]};
    __builtin_nontemporal_store(x, reinterpret_cast<h8_ *>(p));
}

template <int N> struct Ptrs { void *p[N]; };
template <int N> struct ConstPtrs { const void *p[N]; };

// out_j[t] = x[t] + (x[t-1] - x[t]) * d_j[t],  x[-1] = shift.
// lerp != 0: coef_j is the reference's time_mix_j (weight of x itself), d_j = 1 - coef_j;
// lerp == 0: coef_j is time_maa_j (weight of the difference), d_j = coef_j (+ dyn_j[t] for the data-dependent mix).
template <class T, int N, bool DYN>
__global__ __launch_bounds__(256) void shift_mix_forward(int Tlen, int C, int lerp, const T *__restrict__ x,
        const T *__restrict__ shift, const float *__restrict__ coef, const T *__restrict__ dyn, Ptrs<N> out)
{
    const int cl = threadIdx.x & (CH_LANES - 1), tl = threadIdx.x / CH_LANES;
    const int c = blockIdx.x * TILE_C + cl * VEC, b = blockIdx.z;
    const int t0 = blockIdx.y * TILE_R + tl * ROWS_PER_LANE;
    if (c >= C || t0 >= Tlen) return;
    float cd[N][8];
#pragma unroll
    for (int j = 0; j < N; j++) {
        load8(coef + (size_t)j * C + c, cd[j]);
        if (lerp) {
#pragma unroll
            for (int e = 0; e < 8; e++) cd[j][e] = 1.f - cd[j][e];
        }
    }
    const size_t base = (size_t)b * Tlen * C + c, plane = (size_t)gridDim.z * Tlen * C;
    float row[ROWS_PER_LANE + 1][8];
    if (t0 == 0) load8(shift + (size_t)b * C + c, row[0]);
    else load8(x + base + (size_t)(t0 - 1) * C, row[0]);
#pragma unroll
    for (int i = 0; i < ROWS_PER_LANE; i++)
        if (t0 + i < Tlen) load8(x + base + (size_t)(t0 + i) * C, row[i + 1]);
#pragma unroll
    for (int i = 0; i < ROWS_PER_LANE; i++) {
        if (t0 + i >= Tlen) break;
        const size_t off = base + (size_t)(t0 + i) * C;
#pragma unroll
        for (int j = 0; j < N; j++) {
            float d[8], o[8];
            if (DYN) load8(dyn + (size_t)j * plane + off, d);
#pragma unroll
            for (int e = 0; e < 8; e++)
                o[e] = fmaf(row[i][e] - row[i + 1][e], DYN ? cd[j][e] + d[e] : cd[j][e], row[i + 1][e]);
            stream8((T *)out.p[j] + off, o);
        }
    }
}

// Backward of the above.  With g_j the gradients of the N outputs and d_j as in the forward:
//   gx[t]    = sum_j g_j[t] (1 - d_j[t]) + sum_j g_j[t+1] d_j[t+1]
//   gshift   = sum_j g_j[0] d_j[0]
//   gdyn_j[t] = g_j[t] (x[t-1] - x[t])
//   gcoef_j  = +-sum_{b,t} g_j[t] (x[t-1] - x[t])       (minus for lerp), left as one partial row per workgroup.
template <class T, int N, bool DYN>
__global__ __launch_bounds__(256) void shift_mix_backward(int Tlen, int C, int lerp, const T *__restrict__ x,
        const T *__restrict__ shift, const float *__restrict__ coef, const T *__restrict__ dyn, ConstPtrs<N> gout,
        T *__restrict__ gx, T *__restrict__ gshift, float *__restrict__ partial, T *__restrict__ gdyn)
{
    __shared__ float red[ROW_LANES][N][TILE_C];
    const int cl = threadIdx.x & (CH_LANES - 1), tl = threadIdx.x / CH_LANES;
    const int c = blockIdx.x * TILE_C + cl * VEC, b = blockIdx.z;
    const int t0 = blockIdx.y * TILE_R + tl * ROWS_PER_LANE;
    float acc[N][8];
#pragma unroll
    for (int j = 0; j < N; j++)
#pragma unroll
        for (int e = 0; e < 8; e++) acc[j][e] = 0.f;
    if (c < C && t0 < Tlen) {
        float cd[N][8];
#pragma unroll
        for (int j = 0; j < N; j++) {
            load8(coef + (size_t)j * C + c, cd[j]);
            if (lerp) {
#pragma unroll
                for (int e = 0; e < 8; e++) cd[j][e] = 1.f - cd[j][e];
            }
        }
        const size_t base = (size_t)b * Tlen * C + c, plane = (size_t)gridDim.z * Tlen * C;
        float row[ROWS_PER_LANE + 1][8];
        if (t0 == 0) load8(shift + (size_t)b * C + c, row[0]);
        else load8(x + base + (size_t)(t0 - 1) * C, row[0]);
#pragma unroll
        for (int i = 0; i < ROWS_PER_LANE; i++)
            if (t0 + i < Tlen) load8(x + base + (size_t)(t0 + i) * C, row[i + 1]);
        // what the first token after this lane's rows sends back to the lane's last row
        float carry[8];
#pragma unroll
        for (int e = 0; e < 8; e++) carry[e] = 0.f;
        if (t0 + ROWS_PER_LANE < Tlen) {
            const size_t off = base + (size_t)(t0 + ROWS_PER_LANE) * C;
#pragma unroll
            for (int j = 0; j < N; j++) {
                float g[8], d[8];
                load8((const T *)gout.p[j] + off, g);
                if (DYN) load8(dyn + (size_t)j * plane + off, d);
#pragma unroll
                for (int e = 0; e < 8; e++) carry[e] = fmaf(g[e], DYN ? cd[j][e] + d[e] : cd[j][e], carry[e]);
            }
        }
#pragma unroll
        for (int i = ROWS_PER_LANE - 1; i >= 0; i--) {
            if (t0 + i >= Tlen) continue;
            const size_t off = base + (size_t)(t0 + i) * C;
            float own[8], next[8], dx[8];
#pragma unroll
            for (int e = 0; e < 8; e++) { own[e] = carry[e]; next[e] = 0.f; dx[e] = row[i][e] - row[i + 1][e]; }
#pragma unroll
            for (int j = 0; j < N; j++) {
                float g[8], d[8];
                load8((const T *)gout.p[j] + off, g);
                if (DYN) load8(dyn + (size_t)j * plane + off, d);
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const float w = DYN ? cd[j][e] + d[e] : cd[j][e];
                    own[e] = fmaf(g[e], 1.f - w, own[e]);
                    next[e] = fmaf(g[e], w, next[e]);
                    d[e] = g[e] * dx[e];
                    acc[j][e] += d[e];
                }
                if (DYN) stream8(gdyn + (size_t)j * plane + off, d);
            }
            stream8(gx + off, own);
#pragma unroll
            for (int e = 0; e < 8; e++) carry[e] = next[e];
        }
        if (t0 == 0) store8(gshift + (size_t)b * C + c, carry);
    }
#pragma unroll
    for (int j = 0; j < N; j++)
#pragma unroll
        for (int e = 0; e < 8; e++) red[tl][j][cl * VEC + e] = acc[j][e];
    __syncthreads();
    const size_t tile = (size_t)b * gridDim.y + blockIdx.y;
    for (int i = threadIdx.x; i < N * TILE_C; i += 256) {
        const int j = i / TILE_C, col = i % TILE_C;
        if (blockIdx.x * TILE_C + col >= C) continue;
        float s = 0.f;
#pragma unroll
        for (int r = 0; r < ROW_LANES; r++) s += red[r][j][col];
        partial[(tile * N + j) * C + blockIdx.x * TILE_C + col] = lerp ? -s : s;
    }
}

// out[n] = sum over rows of in[row][n], rows added in a fixed order: 32 columns x 8 row groups per workgroup, each
// group four interleaved running sums over its rows, the groups added in order at the end
__global__ __launch_bounds__(256) void sum_rows(int rows, int n, const float *__restrict__ in, float *__restrict__ out) {
    __shared__ float red[8][32];
    const int lane = threadIdx.x & 31, rg = threadIdx.x >> 5;
    const int i = blockIdx.x * 32 + lane;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    if (i < n) {
        int r = rg;
        for (; r + 24 < rows; r += 32) {
            s0 += in[(size_t)r * n + i];
            s1 += in[(size_t)(r + 8) * n + i];
            s2 += in[(size_t)(r + 16) * n + i];
            s3 += in[(size_t)(r + 24) * n + i];
        }
        for (; r < rows; r += 8) s0 += in[(size_t)r * n + i];
    }
    red[rg][lane] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    if (rg == 0 && i < n) {
        float s = red[0][lane];
#pragma unroll
        for (int g = 1; g < 8; g++) s += red[g][lane];
        out[i] = s;
    }
}

// ---- ln_x * gate
__device__ __forceinline__ float head_sum(float v) {          // over the 8 lanes that hold one head's 64 channels
    v += __shfl_xor(v, 1);
    v += __shfl_xor(v, 2);
    v += __shfl_xor(v, 4);
    return v;
}
// 1 / (1 + e^-x) on the hardware exp2 and reciprocal (1 ulp each): a full-precision division per element would make
// these passes bound by vector instructions instead of by memory
__device__ __forceinline__ float sigmoid_f(float x) { return __builtin_amdgcn_rcpf(1.f + exp2_fast(-LOG2E * x)); }

constexpr int ROW_BATCH = 4;       // rows whose loads are issued together before any of them is used

// out = (GroupNorm_head(y * scale) * weight + bias) * silu(gate); gate == nullptr: no gate
template <class T>
__global__ __launch_bounds__(256) void ln_gate_forward(int rows, int C, float scale, float eps, const T *__restrict__ y,
        const T *__restrict__ gate, const float *__restrict__ weight, const float *__restrict__ bias, T *__restrict__ out)
{
    const int cl = threadIdx.x & (CH_LANES - 1), tl = threadIdx.x / CH_LANES;
    const int c = blockIdx.x * TILE_C + cl * VEC;
    const int r0 = blockIdx.y * TILE_R + tl * ROWS_PER_LANE;
    const bool live = c < C;                    // a head never straddles the edge: C is a multiple of 64
    float w[8], bs[8];
    if (live) { load8(weight + c, w); load8(bias + c, bs); }
#pragma unroll
    for (int i0 = 0; i0 < ROWS_PER_LANE; i0 += ROW_BATCH) {
        float v[ROW_BATCH][8], g[ROW_BATCH][8];
#pragma unroll
        for (int i = 0; i < ROW_BATCH; i++) {
            const int r = r0 + i0 + i;
#pragma unroll
            for (int e = 0; e < 8; e++) { v[i][e] = 0.f; g[i][e] = 0.f; }
            if (live && r < rows) {
                load8(y + (size_t)r * C + c, v[i]);
                if (gate) load8(gate + (size_t)r * C + c, g[i]);
            }
        }
#pragma unroll
        for (int i = 0; i < ROW_BATCH; i++) {
            const int r = r0 + i0 + i;
            float s = 0.f;
#pragma unroll
            for (int e = 0; e < 8; e++) { v[i][e] *= scale; s += v[i][e]; }
            const float mean = head_sum(s) * (1.f / HEAD);
            float q = 0.f;
#pragma unroll
            for (int e = 0; e < 8; e++) { v[i][e] -= mean; q = fmaf(v[i][e], v[i][e], q); }
            const float rstd = rsqrtf(head_sum(q) * (1.f / HEAD) + eps);
            if (!live || r >= rows) continue;
            float o[8];
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float n = fmaf(v[i][e] * rstd, w[e], bs[e]);
                o[e] = gate ? n * g[i][e] * sigmoid_f(g[i][e]) : n;
            }
            stream8(out + (size_t)r * C + c, o);
        }
    }
}

template <class T>
__global__ __launch_bounds__(256) void ln_gate_backward(int rows, int C, float scale, float eps, const T *__restrict__ y,
        const T *__restrict__ gate, const float *__restrict__ weight, const float *__restrict__ bias,
        const T *__restrict__ gout, T *__restrict__ gy, T *__restrict__ ggate, float *__restrict__ partial)
{
    __shared__ float red[ROW_LANES][2][TILE_C];
    const int cl = threadIdx.x & (CH_LANES - 1), tl = threadIdx.x / CH_LANES;
    const int c = blockIdx.x * TILE_C + cl * VEC;
    const int r0 = blockIdx.y * TILE_R + tl * ROWS_PER_LANE;
    const bool live = c < C;
    float w[8], bs[8], aw[8], ab[8];
#pragma unroll
    for (int e = 0; e < 8; e++) { aw[e] = 0.f; ab[e] = 0.f; w[e] = 0.f; bs[e] = 0.f; }
    if (live) { load8(weight + c, w); load8(bias + c, bs); }
#pragma unroll
    for (int i0 = 0; i0 < ROWS_PER_LANE; i0 += ROW_BATCH) {
        float vv[ROW_BATCH][8], gg_[ROW_BATCH][8], go_[ROW_BATCH][8];
#pragma unroll
        for (int i = 0; i < ROW_BATCH; i++) {
            const int r = r0 + i0 + i;
#pragma unroll
            for (int e = 0; e < 8; e++) { vv[i][e] = 0.f; gg_[i][e] = 0.f; go_[i][e] = 0.f; }
            if (live && r < rows) {
                const size_t off = (size_t)r * C + c;
                load8(y + off, vv[i]);
                load8(gout + off, go_[i]);
                if (gate) load8(gate + off, gg_[i]);
            }
        }
#pragma unroll
        for (int i = 0; i < ROW_BATCH; i++) {
            const int r = r0 + i0 + i;
            float (&v)[8] = vv[i], (&g)[8] = gg_[i], (&go)[8] = go_[i];
            float s = 0.f;
#pragma unroll
            for (int e = 0; e < 8; e++) { v[e] *= scale; s += v[e]; }
            const float mean = head_sum(s) * (1.f / HEAD);
            float q = 0.f;
#pragma unroll
            for (int e = 0; e < 8; e++) { v[e] -= mean; q = fmaf(v[e], v[e], q); }
            const float rstd = rsqrtf(head_sum(q) * (1.f / HEAD) + eps);
            float gg[8], m1 = 0.f, m2 = 0.f;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                v[e] *= rstd;                                       // normalised value
                float gn = go[e];
                if (gate) {
                    const float sg = sigmoid_f(g[e]), n = fmaf(v[e], w[e], bs[e]);
                    gg[e] = go[e] * n * sg * (1.f + g[e] * (1.f - sg));
                    gn = go[e] * g[e] * sg;
                }
                aw[e] = fmaf(gn, v[e], aw[e]);                      // rows past the end carry zeros
                ab[e] += gn;
                go[e] = gn * w[e];                                  // gradient of the normalised value
                m1 += go[e];
                m2 = fmaf(go[e], v[e], m2);
            }
            m1 = head_sum(m1) * (1.f / HEAD);
            m2 = head_sum(m2) * (1.f / HEAD);
            if (!live || r >= rows) continue;
            const size_t off = (size_t)r * C + c;
            float o[8];
#pragma unroll
            for (int e = 0; e < 8; e++) o[e] = scale * rstd * (go[e] - m1 - v[e] * m2);
            stream8(gy + off, o);
            if (gate) stream8(ggate + off, gg);
        }
    }
#pragma unroll
    for (int e = 0; e < 8; e++) { red[tl][0][cl * VEC + e] = aw[e]; red[tl][1][cl * VEC + e] = ab[e]; }
    __syncthreads();
    for (int i = threadIdx.x; i < 2 * TILE_C; i += 256) {
        const int j = i / TILE_C, col = i % TILE_C;
        if (blockIdx.x * TILE_C + col >= C) continue;
        float s = 0.f;
#pragma unroll
        for (int r = 0; r < ROW_LANES; r++) s += red[r][j][col];
        partial[((size_t)blockIdx.y * 2 + j) * C + blockIdx.x * TILE_C + col] = s;
    }
}

// ---- channel-mix activations (n elements, n a multiple of 8)
template <class T> __global__ __launch_bounds__(256) void relu_square_forward(size_t n, const T *__restrict__ k, T *__restrict__ out) {
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * VEC;
    if (i >= n) return;
    float v[8];
    load8(k + i, v);
#pragma unroll
    for (int e = 0; e < 8; e++) { const float p = fmaxf(v[e], 0.f); v[e] = p * p; }
    store8(out + i, v);
}
template <class T> __global__ __launch_bounds__(256) void relu_square_backward(size_t n, const T *__restrict__ k,
        const T *__restrict__ gout, T *__restrict__ gk) {
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * VEC;
    if (i >= n) return;
    float v[8], g[8];
    load8(k + i, v); load8(gout + i, g);
#pragma unroll
    for (int e = 0; e < 8; e++) v[e] = 2.f * fmaxf(v[e], 0.f) * g[e];
    store8(gk + i, v);
}
template <class T> __global__ __launch_bounds__(256) void sigmoid_mul_forward(size_t n, const T *__restrict__ r,
        const T *__restrict__ kv, T *__restrict__ out) {
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * VEC;
    if (i >= n) return;
    float a[8], b[8];
    load8(r + i, a); load8(kv + i, b);
#pragma unroll
    for (int e = 0; e < 8; e++) a[e] = sigmoid_f(a[e]) * b[e];
    store8(out + i, a);
}
template <class T> __global__ __launch_bounds__(256) void sigmoid_mul_backward(size_t n, const T *__restrict__ r,
        const T *__restrict__ kv, const T *__restrict__ gout, T *__restrict__ gr, T *__restrict__ gkv) {
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * VEC;
    if (i >= n) return;
    float a[8], b[8], g[8];
    load8(r + i, a); load8(kv + i, b); load8(gout + i, g);
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const float s = sigmoid_f(a[e]);
        a[e] = g[e] * b[e] * s * (1.f - s);
        b[e] = g[e] * s;
    }
    store8(gr + i, a); store8(gkv + i, b);
}

// ---- L2Wrap backward: gy[row] = 0 except factor * mask[row] * max(y[row]) at the (first) position of the maximum
template <class T>
__global__ __launch_bounds__(256) void l2wrap_backward(int V, float factor, const T *__restrict__ y,
        const float *__restrict__ mask, T *__restrict__ gy)
{
    __shared__ float best_v[4];
    __shared__ int best_i[4];
    const size_t base = (size_t)blockIdx.x * V;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    const bool vec = (V % VEC) == 0;
    if (vec) {
        for (int i = threadIdx.x * VEC; i < V; i += 256 * VEC) {
            float v[8];
            load8(y + base + i, v);
#pragma unroll
            for (int e = 0; e < 8; e++)
                if (v[e] > bv) { bv = v[e]; bi = i + e; }        // strict: keeps the first of equal values
        }
    } else {
        for (int i = threadIdx.x; i < V; i += 256) {
            const float v = to_float(y[base + i]);
            if (v > bv) { bv = v; bi = i; }
        }
    }
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) {
        const float ov = __shfl_xor(bv, m);
        const int oi = __shfl_xor(bi, m);
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if ((threadIdx.x & 63) == 0) { best_v[threadIdx.x >> 6] = bv; best_i[threadIdx.x >> 6] = bi; }
    __syncthreads();
    bv = best_v[0]; bi = best_i[0];
#pragma unroll
    for (int wv = 1; wv < 4; wv++)
        if (best_v[wv] > bv || (best_v[wv] == bv && best_i[wv] < bi)) { bv = best_v[wv]; bi = best_i[wv]; }
    const float val = bv * factor * (mask ? mask[blockIdx.x] : 1.f);
    if (vec) {
        for (int i = threadIdx.x * VEC; i < V; i += 256 * VEC) {
            float o[8];
#pragma unroll
            for (int e = 0; e < 8; e++) o[e] = (i + e == bi) ? val : 0.f;
            stream8(gy + base + i, o);
        }
    } else {
        for (int i = threadIdx.x; i < V; i += 256) gy[base + i] = from_float<T>(i == bi ? val : 0.f);
    }
}

// ---- launchers
inline dim3 tile_grid(int rows, int C, int B) { return dim3((C + TILE_C - 1) / TILE_C, (rows + TILE_R - 1) / TILE_R, B); }
inline size_t row_tiles(int rows) { return (size_t)(rows + TILE_R - 1) / TILE_R; }

inline size_t shift_mix_backward_workspace(int B, int Tlen, int C, int n) {
    return (size_t)B * row_tiles(Tlen) * n * C * sizeof(float);
}
inline size_t ln_gate_backward_workspace(int rows, int C) { return row_tiles(rows) * 2 * C * sizeof(float); }

template <class T, int N, bool DYN>
hipError_t shift_mix_forward_n(hipStream_t s, int B, int Tlen, int C, int lerp, const void *x, const void *shift,
                               const float *coef, const void *dyn, void *const *out) {
    Ptrs<N> po;
    for (int j = 0; j < N; j++) po.p[j] = out[j];
    hipLaunchKernelGGL((shift_mix_forward<T, N, DYN>), tile_grid(Tlen, C, B), dim3(256), 0, s, Tlen, C, lerp, (const T *)x,
                       (const T *)shift, coef, (const T *)dyn, po);
    return hipGetLastError();
}
template <class T>
hipError_t shift_mix_forward_t(hipStream_t s, int B, int Tlen, int C, int n, int lerp, const void *x, const void *shift,
                               const float *coef, const void *dyn, void *const *out) {
    if (dyn) {
        switch (n) {
        case 1: return shift_mix_forward_n<T, 1, true>(s, B, Tlen, C, lerp, x, shift, coef, dyn, out);
        case 2: return shift_mix_forward_n<T, 2, true>(s, B, Tlen, C, lerp, x, shift, coef, dyn, out);
        case 3: return shift_mix_forward_n<T, 3, true>(s, B, Tlen, C, lerp, x, shift, coef, dyn, out);
        case 4: return shift_mix_forward_n<T, 4, true>(s, B, Tlen, C, lerp, x, shift, coef, dyn, out);
        case 5: return shift_mix_forward_n<T, 5, true>(s, B, Tlen, C, lerp, x, shift, coef, dyn, out);
        }
    } else {
        switch (n) {
        case 1: return shift_mix_forward_n<T, 1, false>(s, B, Tlen, C, lerp, x, shift, coef, dyn, out);
        case 2: return shift_mix_forward_n<T, 2, false>(s, B, Tlen, C, lerp, x, shift, coef, dyn, out);
        case 3: return shift_mix_forward_n<T, 3, false>(s, B, Tlen, C, lerp, x, shift, coef, dyn, out);
        case 4: return shift_mix_forward_n<T, 4, false>(s, B, Tlen, C, lerp, x, shift, coef, dyn, out);
        case 5: return shift_mix_forward_n<T, 5, false>(s, B, Tlen, C, lerp, x, shift, coef, dyn, out);
        }
    }
    return hipErrorInvalidValue;
}

template <class T, int N, bool DYN>
hipError_t shift_mix_backward_n(hipStream_t s, int B, int Tlen, int C, int lerp, const void *x, const void *shift,
                                const float *coef, const void *dyn, const void *const *gout, void *gx, void *gshift,
                                float *gcoef, void *gdyn, float *partial) {
    ConstPtrs<N> pg;
    for (int j = 0; j < N; j++) pg.p[j] = gout[j];
    hipLaunchKernelGGL((shift_mix_backward<T, N, DYN>), tile_grid(Tlen, C, B), dim3(256), 0, s, Tlen, C, lerp, (const T *)x,
                       (const T *)shift, coef, (const T *)dyn, pg, (T *)gx, (T *)gshift, partial, (T *)gdyn);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(sum_rows, dim3((N * C + 31) / 32), dim3(256), 0, s, (int)(B * row_tiles(Tlen)), N * C, partial, gcoef);
    return hipGetLastError();
}
template <class T>
hipError_t shift_mix_backward_t(hipStream_t s, int B, int Tlen, int C, int n, int lerp, const void *x, const void *shift,
                                const float *coef, const void *dyn, const void *const *gout, void *gx, void *gshift,
                                float *gcoef, void *gdyn, float *partial) {
#define WKV_EDGE_CASE(N_, D_) \
    return shift_mix_backward_n<T, N_, D_>(s, B, Tlen, C, lerp, x, shift, coef, dyn, gout, gx, gshift, gcoef, gdyn, partial)
    if (dyn) {
        switch (n) {
        case 1: WKV_EDGE_CASE(1, true);
        case 2: WKV_EDGE_CASE(2, true);
        case 3: WKV_EDGE_CASE(3, true);
        case 4: WKV_EDGE_CASE(4, true);
        case 5: WKV_EDGE_CASE(5, true);
        }
    } else {
        switch (n) {
        case 1: WKV_EDGE_CASE(1, false);
        case 2: WKV_EDGE_CASE(2, false);
        case 3: WKV_EDGE_CASE(3, false);
        case 4: WKV_EDGE_CASE(4, false);
        case 5: WKV_EDGE_CASE(5, false);
        }
    }
#undef WKV_EDGE_CASE
    return hipErrorInvalidValue;
}

template <class T>
hipError_t ln_gate_forward_t(hipStream_t s, int rows, int C, float scale, float eps, const void *y, const void *gate,
                             const float *weight, const float *bias, void *out) {
    hipLaunchKernelGGL(ln_gate_forward<T>, tile_grid(rows, C, 1), dim3(256), 0, s, rows, C, scale, eps, (const T *)y,
                       (const T *)gate, weight, bias, (T *)out);
    return hipGetLastError();
}
template <class T>
hipError_t ln_gate_backward_t(hipStream_t s, int rows, int C, float scale, float eps, const void *y, const void *gate,
                              const float *weight, const float *bias, const void *gout, void *gy, void *ggate,
                              float *gweight_gbias, float *partial) {
    hipLaunchKernelGGL(ln_gate_backward<T>, tile_grid(rows, C, 1), dim3(256), 0, s, rows, C, scale, eps, (const T *)y,
                       (const T *)gate, weight, bias, (const T *)gout, (T *)gy, (T *)ggate, partial);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(sum_rows, dim3((2 * C + 31) / 32), dim3(256), 0, s, (int)row_tiles(rows), 2 * C, partial, gweight_gbias);
    return hipGetLastError();
}

inline dim3 flat_grid(size_t n) { return dim3((unsigned)((n / VEC + 255) / 256)); }

template <class T> hipError_t relu_square_forward_t(hipStream_t s, size_t n, const void *k, void *out) {
    hipLaunchKernelGGL(relu_square_forward<T>, flat_grid(n), dim3(256), 0, s, n, (const T *)k, (T *)out);
    return hipGetLastError();
}
template <class T> hipError_t relu_square_backward_t(hipStream_t s, size_t n, const void *k, const void *gout, void *gk) {
    hipLaunchKernelGGL(relu_square_backward<T>, flat_grid(n), dim3(256), 0, s, n, (const T *)k, (const T *)gout, (T *)gk);
    return hipGetLastError();
}
template <class T> hipError_t sigmoid_mul_forward_t(hipStream_t s, size_t n, const void *r, const void *kv, void *out) {
    hipLaunchKernelGGL(sigmoid_mul_forward<T>, flat_grid(n), dim3(256), 0, s, n, (const T *)r, (const T *)kv, (T *)out);
    return hipGetLastError();
}
template <class T> hipError_t sigmoid_mul_backward_t(hipStream_t s, size_t n, const void *r, const void *kv, const void *gout,
                                                     void *gr, void *gkv) {
    hipLaunchKernelGGL(sigmoid_mul_backward<T>, flat_grid(n), dim3(256), 0, s, n, (const T *)r, (const T *)kv, (const T *)gout,
                       (T *)gr, (T *)gkv);
    return hipGetLastError();
}
template <class T> hipError_t l2wrap_backward_t(hipStream_t s, int rows, int V, float factor, const void *y, const float *mask,
                                                void *gy) {
    hipLaunchKernelGGL(l2wrap_backward<T>, dim3(rows), dim3(256), 0, s, V, factor, (const T *)y, mask, (T *)gy);
    return hipGetLastError();
}

}  // namespace edges
}  // namespace wkv
