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

// The 16 x 3 multiply-adds of one token on a lane's sixteen state elements, with the per-row (or per-column) factors
// taken from the lane of this 16-lane row that holds them (a DPP operand: the broadcast costs no instruction).  The
// sixteen lanes of a row need the same sixteen per-token values (r, k, w of the rows they share, or v, gy of the columns
// they share); each lane reads ONE of them from LDS and the rest come across the row.  Read as four 16-byte pieces per
// lane and tensor, these values were 12 to 20 KB of LDS traffic per wavefront and token, and the LDS port (128 bytes
// per clock, shared by the wavefronts of a compute unit) was what bounded these kernels.
//
// Each token's instructions are ONE assembly statement: the compiler folds a DPP move into a multiply but not into a
// fused multiply-add, and the hardware does not interlock a DPP read of a register that a vector instruction wrote
// one or two slots earlier.  The statement opens with two wait states, and nothing can be placed inside it, so the
// broadcast sources (inputs of the statement) are always old enough.  Within the statement the update of an element
// is issued one element late, so that no instruction uses the result of the one before it.
#define WKV_DPP(i) " row_newbcast:" #i " row_mask:0xf bank_mask:0xf\n\t"
#define WKV_REP16(M) M(0) M(1) M(2) M(3) M(4) M(5) M(6) M(7) M(8) M(9) M(10) M(11) M(12) M(13) M(14) M(15)
#define WKV_PIPE16(A, B) A(0) A(1) B(0) A(2) B(1) A(3) B(2) A(4) B(3) A(5) B(4) A(6) B(5) A(7) B(6) A(8) B(7) \
                         A(9) B(8) A(10) B(9) A(11) B(10) A(12) B(11) A(13) B(12) A(14) B(13) A(15) B(14) B(15)
#define WKV_S_OPERAND(i) [s##i] "+v"(S[i]),

// acc += x[i] S[i];  S[i] = w[i] S[i] + k[i] v      (x, w, k broadcast from lane i of the row; v the lane's own)
#define WKV_FWD_A(i) "v_fmac_f32_dpp %[acc], %[x], %[s" #i "]" WKV_DPP(i) "v_mul_f32_dpp %[s" #i "], %[w], %[s" #i "]" WKV_DPP(i)
#define WKV_FWD_B(i) "v_fmac_f32_dpp %[s" #i "], %[k], %[v]" WKV_DPP(i)
__device__ __forceinline__ void step_bcast_w(float (&S)[16], float &acc, float x, float w, float k, float v) {
    asm("s_nop 1\n\t" WKV_PIPE16(WKV_FWD_A, WKV_FWD_B)
        : WKV_REP16(WKV_S_OPERAND) [acc] "+v"(acc)
        : [x] "v"(x), [w] "v"(w), [k] "v"(k), [v] "v"(v));
}
// acc += x[i] S[i];  S[i] = w S[i] + a[i] b         (x, a broadcast; w, b the lane's own)
#define WKV_OWN_A(i) "v_fmac_f32_dpp %[acc], %[x], %[s" #i "]" WKV_DPP(i) "v_mul_f32 %[s" #i "], %[w], %[s" #i "]\n\t"
#define WKV_OWN_B(i) "v_fmac_f32_dpp %[s" #i "], %[a], %[b]" WKV_DPP(i)
__device__ __forceinline__ void step_own_w(float (&S)[16], float &acc, float x, float w, float a, float b) {
    asm("s_nop 1\n\t" WKV_PIPE16(WKV_OWN_A, WKV_OWN_B)
        : WKV_REP16(WKV_S_OPERAND) [acc] "+v"(acc)
        : [x] "v"(x), [w] "v"(w), [a] "v"(a), [b] "v"(b));
}
__device__ __forceinline__ float token_sum(float x) {      // over the 16 lanes that stage one token
    x += __shfl_xor(x, 1);
    x += __shfl_xor(x, 2);
    x += __shfl_xor(x, 4);
    x += __shfl_xor(x, 8);
    return x;
}

// ---------------------------------------------------------------- forward --
template <class T, bool PER_TOKEN_W>
__global__ __launch_bounds__(NT) void rec_forward(int Tlen, int C, int H,
        const T *__restrict__ r, const T *__restrict__ k, const T *__restrict__ v,
        const float *__restrict__ wraw, const float *__restrict__ u,
        const float *__restrict__ s_in, T *__restrict__ y, float *__restrict__ s_out, int floor_decay)
{
    __shared__ __align__(16) float s_r[CH][HEAD], s_k[CH][HEAD], s_v[CH][HEAD], s_w[CH][HEAD];
    __shared__ __align__(16) float s_y[CH][4][HEAD];              // the four 16-row partial sums of each output
    __shared__ float s_rho[CH];                                   // sum_i r u k of each staged token

    const int bh = blockIdx.x, b = bh / H, h = bh % H;
    const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63;
    const int g = lane >> 4, j = 16 * wv + (lane & 15);      // column-owned: rows 16g..16g+15 of column j
    const size_t base = (size_t)b * Tlen * C + (size_t)h * HEAD;
    const int st = tid >> 4, sc = (tid & 15) * 4;            // staging: token st, channels sc..sc+3

    const int shared_row = 16 * g + (lane & 15);            // the row whose r, k, w this lane reads for its 16-lane row
    float S[16], us[4];
    const float *sp = s_in + (size_t)bh * HEAD * HEAD;
#pragma unroll
    for (int ii = 0; ii < 16; ii++) S[ii] = sp[(16 * g + ii) * HEAD + j];
    const float w_const = PER_TOKEN_W ? 0.f : __expf(log_decay(wraw[h * HEAD + shared_row], floor_decay));
#pragma unroll
    for (int e = 0; e < 4; e++) us[e] = u[h * HEAD + sc + e];

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
        float rho = 0.f;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            s_r[st][sc + e] = pr[e]; s_k[st][sc + e] = pk[e]; s_v[st][sc + e] = pv[e];
            if (PER_TOKEN_W) s_w[st][sc + e] = __expf(log_decay(pw[e], floor_decay));
            rho = fmaf(pr[e] * us[e], pk[e], rho);
        }
        rho = token_sum(rho);
        if (sc == 0) s_rho[st] = rho;
    };

    fetch(0);
    stage();
    __syncthreads();
    for (int t0 = 0; t0 < Tlen; t0 += CH) {
        if (t0 + CH < Tlen) fetch(t0 + CH);
        const int nt = min(CH, Tlen - t0);      // the last block may be short
        // The next token's LDS reads are issued ahead of this token's multiply-adds, and the four 16-row partial sums
        // of an output go to LDS as they are: they are added (with the bonus term v rho) when the block's outputs
        // are written out, so the token loop has no shuffle and no wait other than for its own operands.  A
        // workgroup has one wavefront per SIMD; nothing else would hide those latencies.
        float vj = s_v[0][j], r_sh = s_r[0][shared_row], k_sh = s_k[0][shared_row];
        float w_sh = PER_TOKEN_W ? s_w[0][shared_row] : w_const;
        for (int t = 0; t < nt; t++) {
            const int tn = t + 1 < CH ? t + 1 : t;
            const float vj_n = s_v[tn][j], r_n = s_r[tn][shared_row], k_n = s_k[tn][shared_row];
            const float w_n = PER_TOKEN_W ? s_w[tn][shared_row] : w_const;
            float acc = 0.f;
            step_bcast_w(S, acc, r_sh, w_sh, k_sh, vj);
            s_y[t][g][j] = acc;
            vj = vj_n; r_sh = r_n; k_sh = k_n; w_sh = w_n;
        }
        __syncthreads();
        if (t0 + st < Tlen) {
            float o4[4];
#pragma unroll
            for (int e = 0; e < 4; e++)
                o4[e] = fmaf(s_v[st][sc + e], s_rho[st],
                             (s_y[st][0][sc + e] + s_y[st][1][sc + e]) + (s_y[st][2][sc + e] + s_y[st][3][sc + e]));
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
// row-owned for gk, column-owned for gv), with P_t = v_t.gy_t and rho_t = sum_i r_t[i] u[i] k_t[i]:
//     gr_t[i] = sum_j gy_t[j] S[i][j] + u[i] k_t[i] P_t
//     gk_t[i] = sum_j v_t[j] G[i][j] + u[i] r_t[i] P_t
//     gv_t[j] = sum_i k_t[i] G[i][j] + gy_t[j] rho_t
//     D_t[i]  = A[i] - k_t[i] sum_j v_t[j] G[i][j]          (= dL/d log w_t[i])
//     A[i]   += q_t[i] - k_t[i] gk_t[i]
//     G      <- w_t o G + r_t (x) gy_t
// with A started from sum_j gS_out[i][j] S_out[i][j].
//
// The token loops only advance the states and leave the four 16-element partial sums of every contraction in LDS;
// what follows from them (the sums, the bonus terms, the running sum A over the 16 tokens of a block) is done once per
// block by all lanes: lane (g, row) takes tokens 4g..4g+3 of its row, and the A values at the starts of the four
// token quarters come from three shuffles.
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
        s_l[CH][HEAD], s_q[CH][HEAD];
    __shared__ __align__(16) float p_a[CH][4][HEAD], p_b[CH][4][HEAD];   // partial sums [token][lane group][row or column]
    __shared__ float s_p[CH], s_rho[CH];                                 // v.gy and sum r u k of each staged token

    const int bh = blockIdx.x, b = bh / H, h = bh % H;
    const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63;
    const int g = lane >> 4, own = 16 * wv + (lane & 15);    // own row i (row-owned) or own column j (column-owned)
    const int shared = 16 * g + (lane & 15);                 // the column (row-owned) or row (column-owned) whose
                                                             // per-token values this lane reads for its 16-lane row
    const size_t base = (size_t)b * Tlen * C + (size_t)h * HEAD;
    const int st = tid >> 4, sc = (tid & 15) * 4;

    const float u_own = u[h * HEAD + own];
    float l_own = 0.f, w_own = 1.f, w_shared = 1.f, us[4];
    bool floored_own = false;
    if (!PER_TOKEN_W) {
        l_own = log_decay(wraw[h * HEAD + own], floor_decay, &floored_own);
        w_own = __expf(l_own);
        w_shared = __expf(log_decay(wraw[h * HEAD + shared], floor_decay));
    }
#pragma unroll
    for (int e = 0; e < 4; e++) us[e] = u[h * HEAD + sc + e];

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
        float dot = 0.f, rho = 0.f;
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
            dot = fmaf(pv[e], pg[e], dot);
            rho = fmaf(pr[e] * us[e], pk[e], rho);
        }
        dot = token_sum(dot);
        rho = token_sum(rho);
        if (sc == 0) { s_p[st] = dot; s_rho[st] = rho; }
    };
    auto sum4 = [&](const float (&p)[CH][4][HEAD], int t, int x) {
        return (p[t][0][x] + p[t][1][x]) + (p[t][2][x] + p[t][3][x]);
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
        float ki = s_k[0][own], wi = PER_TOKEN_W ? s_w[0][own] : w_own, v_sh = s_v[0][shared], g_sh = s_g[0][shared];
        for (int t = 0; t < nt; t++) {
            const int tn = t + 1 < CH ? t + 1 : t;
            const float ki_n = s_k[tn][own], wi_n = PER_TOKEN_W ? s_w[tn][own] : w_own;
            const float v_n = s_v[tn][shared], g_n = s_g[tn][shared];
            float acc = 0.f;
            step_own_w(S, acc, g_sh, wi, v_sh, ki);      // acc += gy_j S_ij;  S_ij = w_i S_ij + v_j k_i
            p_a[t][g][own] = acc;
            ki = ki_n; wi = wi_n; v_sh = v_n; g_sh = g_n;
        }
        __syncthreads();
        if (t0 + st < Tlen) {
            const size_t o = base + (size_t)(t0 + st) * C + sc;
            float a4[4], b4[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                a4[e] = fmaf(us[e] * s_k[st][sc + e], s_p[st], sum4(p_a, st, sc + e));
                b4[e] = a4[e] * s_r[st][sc + e];
            }
            store4(gr + o, a4);
            store4(qbuf + o, b4);
        }
        // no barrier: what the lines above read of the staged block and stage() overwrites is the lane's own four
        // channels, or the token's scalar, which a lane of the same wavefront writes later in program order
        if (t0 + CH < Tlen) stage(false);
        __syncthreads();
    }

    // ---------------- boundary: G = gS_out in both ownerships, A = sum_j gS_out o S_out
    float Gr[16], Gc[16];
    float A = 0.f;
    {
        const size_t so = (size_t)bh * HEAD * HEAD;
#pragma unroll
        for (int q = 0; q < 16; q++) {
            Gr[q] = gs_out ? gs_out[so + own * HEAD + 16 * g + q] : 0.f;
            Gc[q] = gs_out ? gs_out[so + (16 * g + q) * HEAD + own] : 0.f;
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
        const int nt = min(CH, Tlen - t0);
        {
            const int tf = nt - 1;
            float ri = s_r[tf][own], wi = PER_TOKEN_W ? s_w[tf][own] : w_own, gyj = s_g[tf][own];
            float v_sh = s_v[tf][shared], g_sh = s_g[tf][shared], r_sh = s_r[tf][shared], k_sh = s_k[tf][shared];
            float w_sh = PER_TOKEN_W ? s_w[tf][shared] : w_shared;
            for (int t = tf; t >= 0; t--) {
                const int tn = t > 0 ? t - 1 : 0;
                const float ri_n = s_r[tn][own], wi_n = PER_TOKEN_W ? s_w[tn][own] : w_own, gyj_n = s_g[tn][own];
                const float v_n = s_v[tn][shared], g_n = s_g[tn][shared], r_n = s_r[tn][shared], k_n = s_k[tn][shared];
                const float w_n = PER_TOKEN_W ? s_w[tn][shared] : w_shared;
                float accG = 0.f, accV = 0.f;
                step_own_w(Gr, accG, v_sh, wi, g_sh, ri);             // row i = own:    accG += v_j G_ij;  G_ij = w_i G_ij + gy_j r_i
                step_bcast_w(Gc, accV, k_sh, w_sh, r_sh, gyj);        // column j = own: accV += k_i G_ij;  G_ij = w_i G_ij + r_i gy_j
                p_a[t][g][own] = accG;
                p_b[t][g][own] = accV;
                ri = ri_n; wi = wi_n; gyj = gyj_n; v_sh = v_n; g_sh = g_n; r_sh = r_n; k_sh = k_n; w_sh = w_n;
            }
        }
        __syncthreads();
        {   // row `own`, tokens 4g+3 .. 4g: gk, and D from the running sum A (which runs from the last token down)
            float c[4], kG[4], tot = 0.f;
#pragma unroll
            for (int e = 3; e >= 0; e--) {
                const int t = 4 * g + e;
                const float sumG = t < nt ? sum4(p_a, t, own) : 0.f;
                const float ri = s_r[t][own], ki = s_k[t][own], rkP = ri * ki * s_p[t];
                const float gki = fmaf(u_own * ri, s_p[t], sumG);
                kG[e] = ki * sumG;
                c[e] = s_q[t][own] - ki * gki;
                tot += c[e];
                gu_acc += rkP;
                p_a[t][0][own] = gki;                    // read back below; this lane is the only one to touch (t, own)
            }
            // A before token t = A + (c of all later tokens): later quarters, then later tokens of this quarter
            const int low = lane & 15;
            const float t1 = __shfl(tot, low + 16), t2 = __shfl(tot, low + 32), t3 = __shfl(tot, low + 48), t0q = __shfl(tot, low);
            float run = A + (g < 1 ? t1 : 0.f) + (g < 2 ? t2 : 0.f) + (g < 3 ? t3 : 0.f);
#pragma unroll
            for (int e = 3; e >= 0; e--) {
                const int t = 4 * g + e;
                const float D = run - kG[e];
                run += c[e];
                if (PER_TOKEN_W) p_a[t][1][own] = D * s_l[t][own];
                else if (t < nt) gw_acc += D;
            }
            A += (t0q + t1) + (t2 + t3);
        }
        __syncthreads();
        if (t0 + st < Tlen) {
            const size_t o = base + (size_t)(t0 + st) * C + sc;
            float a4[4], b4[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                a4[e] = p_a[st][0][sc + e];
                b4[e] = fmaf(s_g[st][sc + e], s_rho[st], sum4(p_b, st, sc + e));
            }
            store4(gk + o, a4);
            store4(gv + o, b4);
            if (PER_TOKEN_W) {
                float c4[4] = {p_a[st][1][sc], p_a[st][1][sc + 1], p_a[st][1][sc + 2], p_a[st][1][sc + 3]};
                store4(gw_tok + o, c4);
            }
        }
        if (t0 - CH >= 0) stage(true);           // no barrier needed, as in sweep 1
        __syncthreads();
    }

    if (gs_in) {
        float *gp = gs_in + (size_t)bh * HEAD * HEAD + own * HEAD + 16 * g;
#pragma unroll
        for (int q = 0; q < 4; q++)
            *reinterpret_cast<float4 *>(gp + 4 * q) = make_float4(Gr[4 * q], Gr[4 * q + 1], Gr[4 * q + 2], Gr[4 * q + 3]);
    }
    gu_acc = group_sum(gu_acc);
    gw_acc = group_sum(gw_acc);
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
