// WKV5 / WKV6 per-token recurrence in fp32: the exact path (any T, any I/O dtype).
//
// One workgroup of 256 lanes (4 wavefronts) per (batch, head).  The 64x64 fp32
// state of the head stays in VGPRs for the whole sequence: every lane keeps 16
// elements, either "column-owned" (lane = one value column j and a group of 16
// key rows) or "row-owned" (lane = one key row i and a group of 16 value
// columns), so that the contraction a step needs runs over the lane's own
// registers and finishes with two cross-lane xor shuffles (no LDS tree).
// Token data is staged through LDS 16 tokens at a time as fp32, with the next
// 16 tokens already in flight in registers while the current ones are consumed.
//
// The recurrence (i = key index, j = value index):
//     y_t[j]   = sum_i r_t[i] ( S[i][j] + u[i] k_t[i] v_t[j] )
//     S[i][j] <- w_t[i] S[i][j] + k_t[i] v_t[j]
// follows RWKV-v5/src/module/rwkv_inner.py:28-32; the backward pass evaluates
// the adjoint recurrence  G <- r_t (x) gy_t + w_t o G  and obtains the decay
// gradient from a running sum instead of stored states.
#include "common.h"

namespace wkv {

constexpr int CH = 16;            // tokens staged per step
constexpr int NT = 256;           // lanes per workgroup

__device__ __forceinline__ float group_sum(float x) {      // over the 4 lane groups of 16
    x += __shfl_xor(x, 16);
    x += __shfl_xor(x, 32);
    return x;
}

// ---------------------------------------------------------------- forward --
template <class T, bool PER_TOKEN_W>
__global__ __launch_bounds__(NT) void rec_forward(int Tlen, int C, int H,
        const T *__restrict__ r, const T *__restrict__ k, const T *__restrict__ v,
        const float *__restrict__ wraw, const float *__restrict__ u,
        const float *__restrict__ s_in, T *__restrict__ y, float *__restrict__ s_out, int floor_decay)
{
    __shared__ __align__(16) float s_r[CH][HEAD], s_k[CH][HEAD], s_v[CH][HEAD], s_w[CH][HEAD], s_y[CH][HEAD];

    const int bh = blockIdx.x, b = bh / H, h = bh % H;
    const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63;
    const int g = lane >> 4, j = 16 * wv + (lane & 15);      // column-owned: rows 16g..16g+15 of column j
    const size_t base = (size_t)b * Tlen * C + (size_t)h * HEAD;
    const int st = tid >> 4, sc = (tid & 15) * 4;            // staging: token st, channels sc..sc+3

    float S[16], uu[16], wc[16];
    const float *sp = s_in + (size_t)bh * HEAD * HEAD;
#pragma unroll
    for (int ii = 0; ii < 16; ii++) {
        S[ii] = sp[(16 * g + ii) * HEAD + j];
        uu[ii] = u[h * HEAD + 16 * g + ii];
        wc[ii] = PER_TOKEN_W ? 0.f : __expf(log_decay(wraw[h * HEAD + 16 * g + ii], floor_decay));
    }

    float pr[4], pk[4], pv[4], pw[4];
    auto fetch = [&](int t0) {
        const int t = t0 + st;
        if (t < Tlen) {
            const size_t o = base + (size_t)t * C + sc;
            load4(r + o, pr); load4(k + o, pk); load4(v + o, pv);
            if (PER_TOKEN_W) load4(wraw + o, pw);
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++) { pr[e] = pk[e] = pv[e] = 0.f; pw[e] = -1e30f; }   // decay 1, no update
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int e = 0; e < 4; e++) {
            s_r[st][sc + e] = pr[e]; s_k[st][sc + e] = pk[e]; s_v[st][sc + e] = pv[e];
            if (PER_TOKEN_W) s_w[st][sc + e] = __expf(log_decay(pw[e], floor_decay));
        }
    };

    fetch(0);
    stage();
    __syncthreads();
    for (int t0 = 0; t0 < Tlen; t0 += CH) {
        if (t0 + CH < Tlen) fetch(t0 + CH);
        const int nt = min(CH, Tlen - t0);      // the last block may be short
        for (int t = 0; t < nt; t++) {
            const float vj = s_v[t][j];
            float acc = 0.f;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float4 r4 = *reinterpret_cast<const float4 *>(&s_r[t][16 * g + 4 * q]);
                const float4 k4 = *reinterpret_cast<const float4 *>(&s_k[t][16 * g + 4 * q]);
                float4 w4;
                if (PER_TOKEN_W) w4 = *reinterpret_cast<const float4 *>(&s_w[t][16 * g + 4 * q]);
                else w4 = make_float4(wc[4 * q], wc[4 * q + 1], wc[4 * q + 2], wc[4 * q + 3]);
                const float rr[4] = {r4.x, r4.y, r4.z, r4.w}, kk[4] = {k4.x, k4.y, k4.z, k4.w},
                            ww[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int ii = 4 * q + e;
                    const float kv = kk[e] * vj;
                    acc = fmaf(rr[e], fmaf(uu[ii], kv, S[ii]), acc);
                    S[ii] = fmaf(ww[e], S[ii], kv);
                }
            }
            acc = group_sum(acc);
            if (g == 0) s_y[t][j] = acc;
        }
        __syncthreads();
        if (t0 + st < Tlen) {
            float o4[4] = {s_y[st][sc], s_y[st][sc + 1], s_y[st][sc + 2], s_y[st][sc + 3]};
            store4(y + base + (size_t)(t0 + st) * C + sc, o4);
        }
        if (t0 + CH < Tlen) stage();
        __syncthreads();
    }
    float *op = s_out + (size_t)bh * HEAD * HEAD;
#pragma unroll
    for (int ii = 0; ii < 16; ii++) op[(16 * g + ii) * HEAD + j] = S[ii];
}

// --------------------------------------------------------------- backward --
// Sweep 1 (forward in time, row-owned S):  gr_t, and q_t = r_t o gr_t kept in
// fp32 for the decay-gradient sum.  Sweep 2 (backward in time, G held twice:
// row-owned for gk, column-owned for gv):
//     gk_t[i] = sum_j v_t[j] G[i][j] + u[i] r_t[i] (v_t.gy_t)
//     gv_t[j] = sum_i k_t[i] ( G[i][j] + u[i] r_t[i] gy_t[j] )
//     D_t[i]  = A[i] - k_t[i] sum_j v_t[j] G[i][j]          (= dL/d log w_t[i])
//     A[i]   += q_t[i] - k_t[i] gk_t[i]
//     G      <- w_t o G + r_t (x) gy_t
// with A started from sum_j gS_out[i][j] S_out[i][j].
template <class T, bool PER_TOKEN_W>
__global__ __launch_bounds__(NT) void rec_backward(int Tlen, int C, int H,
        const T *__restrict__ r, const T *__restrict__ k, const T *__restrict__ v,
        const float *__restrict__ wraw, const float *__restrict__ u, const float *__restrict__ s_in,
        const T *__restrict__ gy, const float *__restrict__ gs_out,
        T *__restrict__ gr, T *__restrict__ gk, T *__restrict__ gv, float *__restrict__ gw_tok,
        float *__restrict__ gw_part, float *__restrict__ gu_part, float *__restrict__ gs_in,
        float *__restrict__ qbuf, int floor_decay)
{
    __shared__ __align__(16) float s_r[CH][HEAD], s_k[CH][HEAD], s_v[CH][HEAD], s_w[CH][HEAD], s_g[CH][HEAD],
        s_l[CH][HEAD], s_q[CH][HEAD], o_a[CH][HEAD], o_b[CH][HEAD], o_c[CH][HEAD];

    const int bh = blockIdx.x, b = bh / H, h = bh % H;
    const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63;
    const int g = lane >> 4, own = 16 * wv + (lane & 15);    // own row i (row-owned) or own column j (column-owned)
    const size_t base = (size_t)b * Tlen * C + (size_t)h * HEAD;
    const int st = tid >> 4, sc = (tid & 15) * 4;

    const float u_own = u[h * HEAD + own];
    float l_own = 0.f, w_own = 1.f;
    bool floored_own = false;
    if (!PER_TOKEN_W) {
        l_own = log_decay(wraw[h * HEAD + own], floor_decay, &floored_own);
        w_own = __expf(l_own);
    }

    float pr[4], pk[4], pv[4], pw[4], pg[4], pq[4];
    auto fetch = [&](int t0, bool second) {
        const int t = t0 + st;
        if (t >= 0 && t < Tlen) {
            const size_t o = base + (size_t)t * C + sc;
            load4(r + o, pr); load4(k + o, pk); load4(v + o, pv); load4(gy + o, pg);
            if (PER_TOKEN_W) load4(wraw + o, pw);
            if (second) load4(qbuf + o, pq);
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++) { pr[e] = pk[e] = pv[e] = pg[e] = pq[e] = 0.f; pw[e] = -1e30f; }
        }
    };
    auto stage = [&](bool second) {
#pragma unroll
        for (int e = 0; e < 4; e++) {
            s_r[st][sc + e] = pr[e]; s_k[st][sc + e] = pk[e]; s_v[st][sc + e] = pv[e]; s_g[st][sc + e] = pg[e];
            if (PER_TOKEN_W) {
                bool fl;
                const float l = log_decay(pw[e], floor_decay, &fl);
                s_w[st][sc + e] = __expf(l);
                s_l[st][sc + e] = fl ? 0.f : l;          // factor that turns dL/d log w into dL/d raw
            }
            if (second) s_q[st][sc + e] = pq[e];
        }
    };

    // ---------------- sweep 1: forward in time, S row-owned (row `own`, columns 16g..16g+15)
    float S[16];
    {
        const float *sp = s_in + (size_t)bh * HEAD * HEAD + own * HEAD + 16 * g;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const float4 x = *reinterpret_cast<const float4 *>(sp + 4 * q);
            S[4 * q] = x.x; S[4 * q + 1] = x.y; S[4 * q + 2] = x.z; S[4 * q + 3] = x.w;
        }
    }
    fetch(0, false);
    stage(false);
    __syncthreads();
    for (int t0 = 0; t0 < Tlen; t0 += CH) {
        if (t0 + CH < Tlen) fetch(t0 + CH, false);
        const int nt = min(CH, Tlen - t0);
        for (int t = 0; t < nt; t++) {
            const float ki = s_k[t][own], wi = PER_TOKEN_W ? s_w[t][own] : w_own;
            const float uk = u_own * ki;
            float acc = 0.f;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float4 v4 = *reinterpret_cast<const float4 *>(&s_v[t][16 * g + 4 * q]);
                const float4 g4 = *reinterpret_cast<const float4 *>(&s_g[t][16 * g + 4 * q]);
                const float vv[4] = {v4.x, v4.y, v4.z, v4.w}, gg[4] = {g4.x, g4.y, g4.z, g4.w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int jj = 4 * q + e;
                    acc = fmaf(gg[e], fmaf(uk, vv[e], S[jj]), acc);
                    S[jj] = fmaf(wi, S[jj], ki * vv[e]);
                }
            }
            acc = group_sum(acc);
            if (g == 0) { o_a[t][own] = acc; o_b[t][own] = acc * s_r[t][own]; }
        }
        __syncthreads();
        if (t0 + st < Tlen) {
            const size_t o = base + (size_t)(t0 + st) * C + sc;
            float a4[4] = {o_a[st][sc], o_a[st][sc + 1], o_a[st][sc + 2], o_a[st][sc + 3]};
            float b4[4] = {o_b[st][sc], o_b[st][sc + 1], o_b[st][sc + 2], o_b[st][sc + 3]};
            store4(gr + o, a4);
            store4(qbuf + o, b4);
        }
        if (t0 + CH < Tlen) stage(false);
        __syncthreads();
    }

    // ---------------- boundary: G = gS_out in both ownerships, A = sum_j gS_out o S_out
    float Gr[16], Gc[16], ucol[16], wcol[16];
    float A = 0.f;
    {
        const size_t so = (size_t)bh * HEAD * HEAD;
#pragma unroll
        for (int q = 0; q < 16; q++) {
            Gr[q] = gs_out ? gs_out[so + own * HEAD + 16 * g + q] : 0.f;
            Gc[q] = gs_out ? gs_out[so + (16 * g + q) * HEAD + own] : 0.f;
            ucol[q] = u[h * HEAD + 16 * g + q];
            wcol[q] = PER_TOKEN_W ? 0.f : __expf(log_decay(wraw[h * HEAD + 16 * g + q], floor_decay));
            A = fmaf(Gr[q], S[q], A);
        }
        A = group_sum(A);
    }
    float gu_acc = 0.f, gw_acc = 0.f;

    // the q values of sweep 1 were written by other lanes of this workgroup
    __threadfence_block();
    __syncthreads();

    // ---------------- sweep 2: backward in time
    const int last0 = ((Tlen - 1) / CH) * CH;
    fetch(last0, true);
    stage(true);
    __syncthreads();
    for (int t0 = last0; t0 >= 0; t0 -= CH) {
        if (t0 - CH >= 0) fetch(t0 - CH, true);
        for (int t = min(CH, Tlen - t0) - 1; t >= 0; t--) {
            // row-owned part (row i = own)
            const float ri = s_r[t][own], ki = s_k[t][own], wi = PER_TOKEN_W ? s_w[t][own] : w_own;
            float accG = 0.f, accP = 0.f;
            // column-owned part (column j = own)
            const float gyj = s_g[t][own];
            float accV = 0.f;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float4 v4 = *reinterpret_cast<const float4 *>(&s_v[t][16 * g + 4 * q]);
                const float4 g4 = *reinterpret_cast<const float4 *>(&s_g[t][16 * g + 4 * q]);
                const float4 r4 = *reinterpret_cast<const float4 *>(&s_r[t][16 * g + 4 * q]);
                const float4 k4 = *reinterpret_cast<const float4 *>(&s_k[t][16 * g + 4 * q]);
                float4 w4;
                if (PER_TOKEN_W) w4 = *reinterpret_cast<const float4 *>(&s_w[t][16 * g + 4 * q]);
                else w4 = make_float4(wcol[4 * q], wcol[4 * q + 1], wcol[4 * q + 2], wcol[4 * q + 3]);
                const float vv[4] = {v4.x, v4.y, v4.z, v4.w}, gg[4] = {g4.x, g4.y, g4.z, g4.w},
                            rr[4] = {r4.x, r4.y, r4.z, r4.w}, kk[4] = {k4.x, k4.y, k4.z, k4.w},
                            ww[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int x = 4 * q + e;
                    accG = fmaf(vv[e], Gr[x], accG);
                    accP = fmaf(vv[e], gg[e], accP);
                    Gr[x] = fmaf(wi, Gr[x], ri * gg[e]);
                    const float rg = rr[e] * gyj;
                    accV = fmaf(kk[e], fmaf(ucol[x], rg, Gc[x]), accV);
                    Gc[x] = fmaf(ww[e], Gc[x], rg);
                }
            }
            accG = group_sum(accG);
            accP = group_sum(accP);
            accV = group_sum(accV);
            const float gki = fmaf(u_own * ri, accP, accG);
            const float D = A - ki * accG;
            A += s_q[t][own] - ki * gki;
            gu_acc = fmaf(ri * ki, accP, gu_acc);
            if (!PER_TOKEN_W) gw_acc += D;
            if (g == 0) {
                o_a[t][own] = gki;
                o_b[t][own] = accV;
                if (PER_TOKEN_W) o_c[t][own] = D * s_l[t][own];
            }
        }
        __syncthreads();
        if (t0 + st < Tlen) {
            const size_t o = base + (size_t)(t0 + st) * C + sc;
            float a4[4] = {o_a[st][sc], o_a[st][sc + 1], o_a[st][sc + 2], o_a[st][sc + 3]};
            float b4[4] = {o_b[st][sc], o_b[st][sc + 1], o_b[st][sc + 2], o_b[st][sc + 3]};
            store4(gk + o, a4);
            store4(gv + o, b4);
            if (PER_TOKEN_W) {
                float c4[4] = {o_c[st][sc], o_c[st][sc + 1], o_c[st][sc + 2], o_c[st][sc + 3]};
                store4(gw_tok + o, c4);
            }
        }
        if (t0 - CH >= 0) stage(true);
        __syncthreads();
    }

    if (gs_in) {
        float *gp = gs_in + (size_t)bh * HEAD * HEAD + own * HEAD + 16 * g;
#pragma unroll
        for (int q = 0; q < 4; q++)
            *reinterpret_cast<float4 *>(gp + 4 * q) = make_float4(Gr[4 * q], Gr[4 * q + 1], Gr[4 * q + 2], Gr[4 * q + 3]);
    }
    if (g == 0) {
        gu_part[(size_t)bh * HEAD + own] = gu_acc;
        if (!PER_TOKEN_W) gw_part[(size_t)bh * HEAD + own] = floored_own ? 0.f : gw_acc * l_own;
    }
}

// ------------------------------------------------------------- launchers --
template <class T>
static hipError_t launch_fwd(hipStream_t s, bool per_token, int B, int Tlen, int C, int H, const void *r, const void *k,
                             const void *v, const float *w, const float *u, const float *s_in, void *y, float *s_out,
                             int floor_decay) {
    dim3 grid(B * H), block(NT);
    prof_begin(KID_REC_FORWARD, s);
    if (per_token)
        hipLaunchKernelGGL((rec_forward<T, true>), grid, block, 0, s, Tlen, C, H, (const T *)r, (const T *)k, (const T *)v,
                           w, u, s_in, (T *)y, s_out, floor_decay);
    else
        hipLaunchKernelGGL((rec_forward<T, false>), grid, block, 0, s, Tlen, C, H, (const T *)r, (const T *)k,
                           (const T *)v, w, u, s_in, (T *)y, s_out, floor_decay);
    prof_end(KID_REC_FORWARD, s);
    return hipGetLastError();
}

template <class T>
static hipError_t launch_bwd(hipStream_t s, bool per_token, int B, int Tlen, int C, int H, const void *r, const void *k,
                             const void *v, const float *w, const float *u, const float *s_in, const void *gy,
                             const float *gs_out, void *gr, void *gk, void *gv, float *gw, float *gu, float *gs_in,
                             float *ws, int floor_decay) {
    // workspace: q (B,T,C) fp32 | gu partials (B,C) | gw partials (B,C)
    float *qbuf = ws;
    float *gu_part = qbuf + (size_t)B * Tlen * C;
    float *gw_part = gu_part + (size_t)B * C;
    dim3 grid(B * H), block(NT);
    prof_begin(KID_REC_BACKWARD, s);
    if (per_token)
        hipLaunchKernelGGL((rec_backward<T, true>), grid, block, 0, s, Tlen, C, H, (const T *)r, (const T *)k,
                           (const T *)v, w, u, s_in, (const T *)gy, gs_out, (T *)gr, (T *)gk, (T *)gv, gw, gw_part,
                           gu_part, gs_in, qbuf, floor_decay);
    else
        hipLaunchKernelGGL((rec_backward<T, false>), grid, block, 0, s, Tlen, C, H, (const T *)r, (const T *)k,
                           (const T *)v, w, u, s_in, (const T *)gy, gs_out, (T *)gr, (T *)gk, (T *)gv, nullptr, gw_part,
                           gu_part, gs_in, qbuf, floor_decay);
    prof_end(KID_REC_BACKWARD, s);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(sum_over_batch, dim3((C + 255) / 256), dim3(256), 0, s, B, C, gu_part, gu);
    if (!per_token) hipLaunchKernelGGL(sum_over_batch, dim3((C + 255) / 256), dim3(256), 0, s, B, C, gw_part, gw);
    return hipGetLastError();
}

size_t recurrent_backward_workspace(int B, int Tlen, int C) {
    return ((size_t)B * Tlen * C + 2 * (size_t)B * C) * sizeof(float);
}

hipError_t recurrent_forward(hipStream_t s, int dtype, bool per_token, int B, int Tlen, int C, int H, const void *r,
                             const void *k, const void *v, const float *w, const float *u, const float *s_in, void *y,
                             float *s_out, int floor_decay) {
    switch (dtype) {
        case 0: return launch_fwd<float>(s, per_token, B, Tlen, C, H, r, k, v, w, u, s_in, y, s_out, floor_decay);
        case 1: return launch_fwd<bf16>(s, per_token, B, Tlen, C, H, r, k, v, w, u, s_in, y, s_out, floor_decay);
        default: return launch_fwd<f16>(s, per_token, B, Tlen, C, H, r, k, v, w, u, s_in, y, s_out, floor_decay);
    }
}

hipError_t recurrent_backward(hipStream_t s, int dtype, bool per_token, int B, int Tlen, int C, int H, const void *r,
                              const void *k, const void *v, const float *w, const float *u, const float *s_in,
                              const void *gy, const float *gs_out, void *gr, void *gk, void *gv, float *gw, float *gu,
                              float *gs_in, float *ws, int floor_decay) {
    switch (dtype) {
        case 0: return launch_bwd<float>(s, per_token, B, Tlen, C, H, r, k, v, w, u, s_in, gy, gs_out, gr, gk, gv, gw, gu, gs_in, ws, floor_decay);
        case 1: return launch_bwd<bf16>(s, per_token, B, Tlen, C, H, r, k, v, w, u, s_in, gy, gs_out, gr, gk, gv, gw, gu, gs_in, ws, floor_decay);
        default: return launch_bwd<f16>(s, per_token, B, Tlen, C, H, r, k, v, w, u, s_in, gy, gs_out, gr, gk, gv, gw, gu, gs_in, ws, floor_decay);
    }
}

}  // namespace wkv
