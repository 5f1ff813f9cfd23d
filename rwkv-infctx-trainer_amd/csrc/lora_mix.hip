// The data-dependent token mix of the v6 TimeMix (RWKV-v6/src/module/TimeMix.py:264-276) with its second LoRA
// product inside the pass:
//
//     dyn_j[t][c] = sum_{i<32} act[t][j][i] w2[j][i][c]          (torch.bmm(xxx, time_maa_w2), :265)
//     out_j[t][c] = x[t][c] + (x[t-1][c] - x[t][c]) (maa_j[c] + dyn_j[t][c]),   j = w, k, v, r, g     (:269-273)
//
// with act = tanh(xxx @ time_maa_w1) as (B*T, 5, 32).  The five (B,T,C) tensors dyn_j (the reference's mw..mg) are
// never written: a wavefront forms the 16-token x 16V-channel tile of each of them with V 16x16x32 MFMAs (the
// 32-deep product is exactly one instruction deep) and uses it from the accumulators.  The tokens are the MFMA rows
// and the channels its columns, column n of the V MFMAs being the channels Vn..Vn+V-1: a lane ends up with V
// consecutive channels of four tokens, and the sixteen lanes of a row with 32V consecutive bytes of a token's row
// (V = 8 forward: 256 bytes; V = 4 backward, which keeps four times the values per channel in registers: 128 bytes),
// so x, the gradients and the outputs move in full row segments.  The factors of a workgroup's channels wait in
// LDS in the order the lanes read them.
//
// The backward pass forms dyn_j again the same way and leaves the gradients of dyn_j in memory (bf16, as the
// reference's autograd has them): the two reductions that follow from them (over the channels for act, over the
// tokens for w2) are library GEMMs.
//
// bf16 only (the operands of the MFMA); C a multiple of 8.
#include "common.h"

namespace wkv {
namespace edges {

constexpr int LORA = 32;                 // inner size of the mix's LoRA (TIME_MIX_EXTRA_DIM, TimeMix.py:150)
constexpr int LM_N = 5;                  // mixes
constexpr int LM_WAVES = 4;              // wavefronts per workgroup: the same channels, consecutive token ranges
constexpr int LM_TOK = 16;               // tokens of a wavefront's tile
constexpr int LM_TILES = 4;              // tiles a wavefront walks: 256 tokens per workgroup
constexpr int LM_WG_TOK = LM_WAVES * LM_TILES * LM_TOK;
constexpr int LM_V_FWD = 8, LM_V_BWD = 4;       // channels per lane

typedef __bf16 lm_b8 __attribute__((ext_vector_type(8)));
typedef float lm_f4 __attribute__((ext_vector_type(4)));

template <int V> struct LmShared {
    uint4 w2[LM_N][V][64];       // [mix][tau][lane (g, n)]: w2[j][8g..8g+7][c0 + Vn + tau], the lane's B operand
    float coef[LM_N][16 * V];
    float red[LM_WAVES][LM_N][16 * V];      // backward: the wavefronts' sums over their tokens
};
template <int V> struct LmRow;           // V consecutive bf16
template <> struct LmRow<8> { typedef uint4 type; };
template <> struct LmRow<4> { typedef uint2 type; };

// w2t: time_maa_w2 with its last two dimensions exchanged, (5, C, 32): the 32 factors of a channel are 64 bytes
template <int V>
__device__ __forceinline__ void lm_stage(LmShared<V> &sm, int C, int c0, const float *__restrict__ coef, const bf16 *__restrict__ w2t) {
    for (int s = threadIdx.x; s < LM_N * V * 64; s += 64 * LM_WAVES) {
        const int n = s & 15, g = (s >> 4) & 3, tau = (s >> 6) % V, j = (s >> 6) / V;
        const int ch = c0 + V * n + tau;
        uint4 v = make_uint4(0u, 0u, 0u, 0u);
        if (ch < C) v = *reinterpret_cast<const uint4 *>(w2t + ((size_t)j * C + ch) * LORA + 8 * g);
        sm.w2[j][tau][s & 63] = v;
    }
    for (int s = threadIdx.x; s < LM_N * 16 * V; s += 64 * LM_WAVES) {
        const int j = s / (16 * V), c = s % (16 * V);
        sm.coef[j][c] = c0 + c < C ? coef[(size_t)j * C + c0 + c] : 0.f;
    }
    __syncthreads();
}
// dyn_j of the tile: d[tau][e] = dyn_j[token 4g+e][channel Vn+tau]
template <int V>
__device__ __forceinline__ void lm_dyn(const LmShared<V> &sm, int j, int lane, lm_b8 actv, lm_f4 (&d)[V]) {
    const lm_f4 z = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int tau = 0; tau < V; tau++)
        d[tau] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(actv, __builtin_bit_cast(lm_b8, sm.w2[j][tau][lane]), z, 0, 0, 0);
}
__device__ __forceinline__ void lm_unpack(uint4 p, float (&o)[8]) {
    o[0] = __uint_as_float(p.x << 16); o[1] = __uint_as_float(p.x & 0xffff0000u);
    o[2] = __uint_as_float(p.y << 16); o[3] = __uint_as_float(p.y & 0xffff0000u);
    o[4] = __uint_as_float(p.z << 16); o[5] = __uint_as_float(p.z & 0xffff0000u);
    o[6] = __uint_as_float(p.w << 16); o[7] = __uint_as_float(p.w & 0xffff0000u);
}
__device__ __forceinline__ void lm_unpack(uint2 p, float (&o)[4]) {
    o[0] = __uint_as_float(p.x << 16); o[1] = __uint_as_float(p.x & 0xffff0000u);
    o[2] = __uint_as_float(p.y << 16); o[3] = __uint_as_float(p.y & 0xffff0000u);
}
__device__ __forceinline__ uint4 lm_pack(const float (&o)[8]) {
    return make_uint4(bf16_pack2(o[0], o[1]), bf16_pack2(o[2], o[3]), bf16_pack2(o[4], o[5]), bf16_pack2(o[6], o[7]));
}
__device__ __forceinline__ uint2 lm_pack(const float (&o)[4]) { return make_uint2(bf16_pack2(o[0], o[1]), bf16_pack2(o[2], o[3])); }
__device__ __forceinline__ void lm_store_nt(bf16 *p, uint4 v) {
    typedef unsigned int u4 __attribute__((ext_vector_type(4)));
    __builtin_nontemporal_store(u4{v.x, v.y, v.z, v.w}, reinterpret_cast<u4 *>(p));
}
__device__ __forceinline__ void lm_store_nt(bf16 *p, uint2 v) {
    typedef unsigned int u2 __attribute__((ext_vector_type(2)));
    __builtin_nontemporal_store(u2{v.x, v.y}, reinterpret_cast<u2 *>(p));
}
template <int V> __device__ __forceinline__ void lm_load_f(const float *p, float (&o)[V]) {
#pragma unroll
    for (int i = 0; i < V; i += 4) {
        const float4 v = *reinterpret_cast<const float4 *>(p + i);
        o[i] = v.x; o[i + 1] = v.y; o[i + 2] = v.z; o[i + 3] = v.w;
    }
}
template <int V> __device__ __forceinline__ void lm_store_f(float *p, const float (&o)[V]) {
#pragma unroll
    for (int i = 0; i < V; i += 4) *reinterpret_cast<float4 *>(p + i) = make_float4(o[i], o[i + 1], o[i + 2], o[i + 3]);
}
// the five rows of x a lane needs for its four tokens tfirst .. tfirst+3: those and the one before (rows[0]); the
// token before the first of the sequence is the shift state; tokens past the end repeat the last one (never used)
template <int V>
__device__ __forceinline__ void lm_load_x(const bf16 *__restrict__ x, const bf16 *__restrict__ shift, int b, int Tlen, int C,
                                          int cl, int tfirst, typename LmRow<V>::type (&rows)[5]) {
#pragma unroll
    for (int e = -1; e < 4; e++) {
        const int t = tfirst + e;
        const bf16 *p = t < 0 ? shift + (size_t)b * C + cl : x + ((size_t)b * Tlen + min(t, Tlen - 1)) * C + cl;
        rows[e + 1] = *reinterpret_cast<const typename LmRow<V>::type *>(p);
    }
}

// The lane-dependent indices, re-derived inside a tile's step from an opaque copy of the lane id: hoisted out of the
// loop, the address arithmetic of every tensor would live in registers across the whole kernel (several hundred).
#define LM_LOCAL_LANE                                                                              \
    int lane_v_ = lane0;                                                                           \
    asm volatile("" : "+v"(lane_v_));                                                              \
    const int lane = lane_v_, g = lane >> 4, n = lane & 15;                                        \
    const int cl = min(c0 + V * n, C - V);   /* the lane's first channel (lanes past the width repeat the last: not stored) */ \
    const bool cok = c0 + V * n < C;

template <int V>
__global__ __launch_bounds__(64 * LM_WAVES) void lora_mix_forward(int Tlen, int C, const bf16 *__restrict__ x,
        const bf16 *__restrict__ shift, const float *__restrict__ coef, const bf16 *__restrict__ act,
        const bf16 *__restrict__ w2t, Ptrs<LM_N> out)
{
    typedef typename LmRow<V>::type row_t;
    __shared__ LmShared<V> sm;
    const int wv = threadIdx.x >> 6, lane0 = threadIdx.x & 63;
    const int c0 = blockIdx.x * (16 * V), b = blockIdx.z;
    lm_stage<V>(sm, C, c0, coef, w2t);
    const int t_wave = blockIdx.y * LM_WG_TOK + wv * (LM_TILES * LM_TOK);
    // a tile's inputs, fetched one tile ahead into two register sets used in turn (no branch around a fetch: a tile
    // past the end reads the last token's rows again and is never used)
    struct In { row_t rows[5]; lm_b8 av[LM_N]; };
    auto fetch = [&](int t0, In &in) __attribute__((always_inline)) {
        LM_LOCAL_LANE
        (void)cok;
        lm_load_x<V>(x, shift, b, Tlen, C, cl, min(t0, Tlen - 1) + 4 * g, in.rows);
        const size_t arow = (size_t)b * Tlen + min(t0 + n, Tlen - 1);
#pragma unroll
        for (int j = 0; j < LM_N; j++) in.av[j] = *reinterpret_cast<const lm_b8 *>(act + (arow * LM_N + j) * LORA + 8 * g);
    };
    auto compute = [&](int t0, const In &in) __attribute__((always_inline)) {
        LM_LOCAL_LANE
        float xf[5][V];
#pragma unroll
        for (int e = 0; e < 5; e++) lm_unpack(in.rows[e], xf[e]);
#pragma unroll
        for (int j = 0; j < LM_N; j++) {
            lm_f4 d[V];
            lm_dyn<V>(sm, j, lane, in.av[j], d);
            float cf[V];
            lm_load_f<V>(&sm.coef[j][V * n], cf);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                float o[V];
#pragma unroll
                for (int tau = 0; tau < V; tau++) o[tau] = fmaf(xf[e][tau] - xf[e + 1][tau], cf[tau] + d[tau][e], xf[e + 1][tau]);
                const int t = t0 + 4 * g + e;
                if (cok && t < Tlen) lm_store_nt((bf16 *)out.p[j] + ((size_t)b * Tlen + t) * C + cl, lm_pack(o));
            }
        }
    };
    static_assert(LM_TILES % 2 == 0, "the tiles are walked in pairs");
    if (t_wave >= Tlen) return;
    In ia, ib;
    fetch(t_wave, ia);
#pragma unroll 1
    for (int tile = 0; tile < LM_TILES; tile += 2) {
        const int t0 = t_wave + LM_TOK * tile;
        if (t0 >= Tlen) break;
        fetch(t0 + LM_TOK, ib);
        compute(t0, ia);
        if (t0 + LM_TOK >= Tlen) break;
        fetch(t0 + 2 * LM_TOK, ia);
        compute(t0 + LM_TOK, ib);
    }
}

// Backward.  With g_j the gradients of the five outputs, m_j = maa_j + dyn_j, dx = x[t-1] - x[t]:
//   gx[t]      = sum_j g_j[t] (1 - m_j[t]) + sum_j g_j[t+1] m_j[t+1]
//   gshift     = sum_j g_j[0] m_j[0]
//   gdyn_j[t]  = g_j[t] dx[t]                      (written, bf16)
//   gmaa_j     = sum_{b,t} gdyn_j[t]               (one partial row per workgroup, added in a fixed order afterwards)
// A wavefront walks its tiles from the last to the first, so that what token t+1 sends back to token t is at hand:
// inside a lane's four tokens from registers, between lanes by a shuffle, across tiles from the tile before; for a
// wavefront's last tile it is formed from token t+1 alone in an extra step that stores nothing.
template <int V>
__global__ __launch_bounds__(64 * LM_WAVES) void lora_mix_backward(int Tlen, int C, const bf16 *__restrict__ x,
        const bf16 *__restrict__ shift, const float *__restrict__ coef, const bf16 *__restrict__ act,
        const bf16 *__restrict__ w2t, ConstPtrs<LM_N> gout, bf16 *__restrict__ gx, bf16 *__restrict__ gshift,
        float *__restrict__ partial, bf16 *__restrict__ gdyn)
{
    typedef typename LmRow<V>::type row_t;
    __shared__ LmShared<V> sm;
    const int wv = threadIdx.x >> 6, lane0 = threadIdx.x & 63;
    const int c0 = blockIdx.x * (16 * V), b = blockIdx.z;
    lm_stage<V>(sm, C, c0, coef, w2t);
    const size_t plane = (size_t)gridDim.z * Tlen * C;
    const int t_wave = blockIdx.y * LM_WG_TOK + wv * (LM_TILES * LM_TOK);
    float acc[LM_N][V];
#pragma unroll
    for (int j = 0; j < LM_N; j++)
#pragma unroll
        for (int tau = 0; tau < V; tau++) acc[j][tau] = 0.f;
    float carry[V];          // what the first token of the tile after this one sends back, for the lane's channels
#pragma unroll
    for (int tau = 0; tau < V; tau++) carry[tau] = 0.f;
#pragma unroll 1
    for (int tile = LM_TILES; tile >= 0; tile--) {
        const int t0 = t_wave + LM_TOK * tile;
        if (t0 >= Tlen) continue;                // (wavefront-uniform)
        LM_LOCAL_LANE
        const bool halo = tile == LM_TILES;      // the token after the wavefront's tokens: row e = 0 of the lanes g = 0 alone
        const size_t arow = (size_t)b * Tlen + min(t0 + n, Tlen - 1);
        lm_b8 av[LM_N];
#pragma unroll
        for (int j = 0; j < LM_N; j++) av[j] = *reinterpret_cast<const lm_b8 *>(act + (arow * LM_N + j) * LORA + 8 * g);
        // the twenty gradient rows of the tile, all in flight before the first is used (no branch around the loads:
        // rows that do not count are read from a row that exists, the halo's all from its one token, and masked)
        row_t gp[LM_N][4];
#pragma unroll
        for (int j = 0; j < LM_N; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int tl = halo ? t0 : min(t0 + 4 * g + e, Tlen - 1);
                gp[j][e] = *reinterpret_cast<const row_t *>((const bf16 *)gout.p[j] + ((size_t)b * Tlen + tl) * C + cl);
            }
        float dx[4][V], own[4][V], nxt[4][V];
#pragma unroll
        for (int e = 0; e < 4; e++)
#pragma unroll
            for (int tau = 0; tau < V; tau++) { own[e][tau] = 0.f; nxt[e][tau] = 0.f; dx[e][tau] = 0.f; }
        if (!halo) {
            row_t rows[5];
            lm_load_x<V>(x, shift, b, Tlen, C, cl, t0 + 4 * g, rows);
            float prev[V];
            lm_unpack(rows[0], prev);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                float cur[V];
                lm_unpack(rows[e + 1], cur);
#pragma unroll
                for (int tau = 0; tau < V; tau++) { dx[e][tau] = prev[tau] - cur[tau]; prev[tau] = cur[tau]; }
            }
        }
#pragma unroll
        for (int j = 0; j < LM_N; j++) {
            lm_f4 d[V];
            lm_dyn<V>(sm, j, lane, av[j], d);
            float cf[V];
            lm_load_f<V>(&sm.coef[j][V * n], cf);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int t = t0 + 4 * g + e;
                const bool live = cok && t < Tlen && (!halo || (g == 0 && e == 0));
                float gj[V], gd[V];
                lm_unpack(gp[j][e], gj);
#pragma unroll
                for (int tau = 0; tau < V; tau++) {
                    if (!live) gj[tau] = 0.f;
                    const float m = cf[tau] + d[tau][e];
                    own[e][tau] = fmaf(gj[tau], 1.f - m, own[e][tau]);
                    nxt[e][tau] = fmaf(gj[tau], m, nxt[e][tau]);
                    gd[tau] = gj[tau] * dx[e][tau];
                    acc[j][tau] += gd[tau];
                    // (used here: left to itself the compiler sinks these sums below the conditional stores of all
                    // five mixes and keeps every gradient row alive until then)
                    asm volatile("" : "+v"(own[e][tau]), "+v"(nxt[e][tau]), "+v"(acc[j][tau]));
                }
                if (live && !halo) lm_store_nt(gdyn + (size_t)j * plane + ((size_t)b * Tlen + t) * C + cl, lm_pack(gd));
            }
        }
        if (!halo) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                float o[V];
#pragma unroll
                for (int tau = 0; tau < V; tau++) {
                    float right;
                    if (e < 3) right = nxt[e + 1][tau];
                    else {                       // the lanes g+1 hold token 4g+4; the last lanes take the tile after
                        const float dn = __shfl_down(nxt[0][tau], 16);
                        right = g == 3 ? carry[tau] : dn;
                    }
                    o[tau] = own[e][tau] + right;
                }
                const int t = t0 + 4 * g + e;
                if (cok && t < Tlen) lm_store_nt(gx + ((size_t)b * Tlen + t) * C + cl, lm_pack(o));
            }
            if (t0 == 0 && g == 0 && cok) *reinterpret_cast<row_t *>(gshift + (size_t)b * C + cl) = lm_pack(nxt[0]);
        }
#pragma unroll
        for (int tau = 0; tau < V; tau++) carry[tau] = __shfl(nxt[0][tau], n);       // token 0 of this tile, for the tile before
    }
    // the sums over the workgroup's tokens: over a wavefront's four lane groups, then over the wavefronts
    const int g = lane0 >> 4, n = lane0 & 15;
#pragma unroll
    for (int j = 0; j < LM_N; j++) {
        float s[V];
#pragma unroll
        for (int tau = 0; tau < V; tau++) {
            float v = acc[j][tau];
            v += __shfl_xor(v, 16);
            v += __shfl_xor(v, 32);
            s[tau] = v;
        }
        if (g == 0) lm_store_f<V>(&sm.red[wv][j][V * n], s);
    }
    __syncthreads();
    for (int s = threadIdx.x; s < LM_N * 16 * V; s += 64 * LM_WAVES) {
        const int j = s / (16 * V), c = s % (16 * V);
        if (c0 + c >= C) continue;
        float v = sm.red[0][j][c];
#pragma unroll
        for (int w = 1; w < LM_WAVES; w++) v += sm.red[w][j][c];
        partial[(((size_t)b * gridDim.y + blockIdx.y) * LM_N + j) * C + c0 + c] = v;
    }
}

inline size_t lora_mix_tiles(int Tlen) { return (size_t)(Tlen + LM_WG_TOK - 1) / LM_WG_TOK; }
inline size_t lora_mix_backward_workspace(int B, int Tlen, int C) { return (size_t)B * lora_mix_tiles(Tlen) * LM_N * C * sizeof(float); }
inline dim3 lora_mix_grid(int B, int Tlen, int C, int V) { return dim3((C + 16 * V - 1) / (16 * V), (unsigned)lora_mix_tiles(Tlen), B); }

inline hipError_t lora_mix_forward_launch(hipStream_t s, int B, int Tlen, int C, const void *x, const void *shift, const float *coef,
                                          const void *act, const void *w2t, void *const *out) {
    Ptrs<LM_N> po;
    for (int j = 0; j < LM_N; j++) po.p[j] = out[j];
    hipLaunchKernelGGL(lora_mix_forward<LM_V_FWD>, lora_mix_grid(B, Tlen, C, LM_V_FWD), dim3(64 * LM_WAVES), 0, s, Tlen, C,
                       (const bf16 *)x, (const bf16 *)shift, coef, (const bf16 *)act, (const bf16 *)w2t, po);
    return hipGetLastError();
}
inline hipError_t lora_mix_backward_launch(hipStream_t s, int B, int Tlen, int C, const void *x, const void *shift, const float *coef,
                                           const void *act, const void *w2t, const void *const *gout, void *gx, void *gshift,
                                           float *gcoef, void *gdyn, float *partial) {
    ConstPtrs<LM_N> pg;
    for (int j = 0; j < LM_N; j++) pg.p[j] = gout[j];
    hipLaunchKernelGGL(lora_mix_backward<LM_V_BWD>, lora_mix_grid(B, Tlen, C, LM_V_BWD), dim3(64 * LM_WAVES), 0, s, Tlen, C,
                       (const bf16 *)x, (const bf16 *)shift, coef, (const bf16 *)act, (const bf16 *)w2t, pg, (bf16 *)gx,
                       (bf16 *)gshift, partial, (bf16 *)gdyn);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(sum_rows, dim3((LM_N * C + 31) / 32), dim3(256), 0, s, (int)(B * lora_mix_tiles(Tlen)), LM_N * C, partial, gcoef);
    return hipGetLastError();
}

}  // namespace edges
}  // namespace wkv
