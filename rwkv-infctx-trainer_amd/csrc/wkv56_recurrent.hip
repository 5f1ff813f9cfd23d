// WKV5 / WKV6 per-token recurrence in fp32: the exact path (any T, any I/O dtype).
//
// Described for its first form (the second, one workgroup per head with 16 elements per lane, is the same code with
// other constants: `Shape`).  Two workgroups of 256 lanes (4 wavefronts) per (batch, head), one per half of the head.  The 64x64 fp32 state of the
// head stays in VGPRs for the whole sequence: every lane keeps 8 elements, either "column-owned" (lane = one value
// column j and a group of 8 key rows) or "row-owned" (lane = one key row i and a group of 8 value columns); a
// workgroup has the 32 columns (or rows) of its half and all eight groups.  The contraction a step needs runs over the
// lane's own registers; of the eight partial sums per output, those of lanes 32 apart are added by a shuffle that runs
// under the next token's arithmetic, and the four that remain go to LDS and are finished once per 16 tokens.
// Token data is staged through LDS 16 tokens at a time as fp32 (every workgroup stages whole tokens: the contractions
// of its half run over all 64 keys or values), with the next 16 tokens already in flight in registers.
//
// Why eight elements per lane and half a head per workgroup: a wavefront issues a vector instruction only every five
// to six clocks, a SIMD can issue one every two to three when it has several wavefronts to choose from, and the number
// of heads is seldom a multiple of the number of compute units.  Sixteen elements per lane and one workgroup per head
// left most SIMDs with one wavefront and, with 320 heads on 256 compute units, a quarter of them with twice the work.
//
// The recurrence (i = key index, j = value index):
//     y_t[j]   = sum_i r_t[i] ( S[i][j] + u[i] k_t[i] v_t[j] )  =  sum_i r_t[i] S[i][j]  +  v_t[j] rho_t,
//     S[i][j] <- w_t[i] S[i][j] + k_t[i] v_t[j]                     rho_t = sum_i r_t[i] u[i] k_t[i]
// follows RWKV-v5/src/module/rwkv_inner.py:28-32 (the bonus term leaves the 64 x 64 loop: rho_t, and v_t . gy_t for the
// backward pass, are formed once per token where the token is staged); the backward pass evaluates the adjoint
// recurrence  G <- r_t (x) gy_t + w_t o G  and obtains the decay gradient from a running sum instead of stored states.
#include "common.h"

namespace wkv {

constexpr int CH = 16;            // tokens staged per step
constexpr int NT = 256;           // lanes per workgroup
// EL = state elements per lane: 8 (two workgroups per head, each with 32 of its columns or rows: the form described
// above) or 16 (one workgroup per head, four groups of 16: half the staging work per head, for batches whose heads
// fill the compute units at least twice over anyway).  A workgroup has OWN = 4 EL columns (or rows).
template <int EL> struct Shape {
    static_assert(EL == 8 || EL == 16, "8 or 16 state elements per lane");
    static constexpr int OWN = 4 * EL, PARTS = HEAD / OWN;
};

__device__ __forceinline__ float group_sum(float x) {      // over the 4 lane groups of 16
    x += __shfl_xor(x, 16);
    x += __shfl_xor(x, 32);
    return x;
}
__device__ __forceinline__ float token_sum(float x) {      // over the 16 lanes that stage one token
    x += __shfl_xor(x, 1);
    x += __shfl_xor(x, 2);
    x += __shfl_xor(x, 4);
    x += __shfl_xor(x, 8);
    return x;
}

// The 8 x 3 multiply-adds of one token on a lane's eight state elements, with the per-row (or per-column) factors
// taken from the lane of this 16-lane row that holds them (a DPP operand: the broadcast costs no instruction).  The
// sixteen lanes of a row need the same eight per-token values (r, k, w of the rows they share, or v, gy of the columns
// they share); each lane reads ONE of them from LDS (lanes 8..15 of a row repeat lanes 0..7) and the rest come across
// the row.  Read as 16-byte pieces per lane and tensor, these values were 12 to 20 KB of LDS traffic per wavefront and
// token, and the LDS port (128 bytes per clock, shared by the wavefronts of a compute unit) was what bounded these
// kernels.
//
// Each token's instructions are ONE assembly statement: the compiler folds a DPP move into a multiply but not into a
// fused multiply-add, and the hardware does not interlock a DPP read of a register that a vector instruction wrote
// one or two slots earlier.  The statement opens with two wait states, and nothing can be placed inside it, so the
// broadcast sources (inputs of the statement) are always old enough.  Within the statement the update of an element
// is issued one element late, so that no instruction uses the result of the one before it.
#define WKV_DPP(i) " row_newbcast:" #i " row_mask:0xf bank_mask:0xf\n\t"
#define WKV_REP8(M) M(0) M(1) M(2) M(3) M(4) M(5) M(6) M(7)
#define WKV_REP16(M) WKV_REP8(M) M(8) M(9) M(10) M(11) M(12) M(13) M(14) M(15)
#define WKV_PIPE8(A, B) A(0) A(1) B(0) A(2) B(1) A(3) B(2) A(4) B(3) A(5) B(4) A(6) B(5) A(7) B(6) B(7)
#define WKV_PIPE16(A, B) A(0) A(1) B(0) A(2) B(1) A(3) B(2) A(4) B(3) A(5) B(4) A(6) B(5) A(7) B(6) A(8) B(7) \
                         A(9) B(8) A(10) B(9) A(11) B(10) A(12) B(11) A(13) B(12) A(14) B(13) A(15) B(14) B(15)
#define WKV_S_OPERAND(i) [s##i] "+v"(S[i]),

// acc += x[i] S[i];  S[i] = w[i] S[i] + k[i] v      (x, w, k broadcast from lane i of the row; v the lane's own)
#define WKV_FWD_A(i) "v_fmac_f32_dpp %[acc], %[x], %[s" #i "]" WKV_DPP(i) "v_mul_f32_dpp %[s" #i "], %[w], %[s" #i "]" WKV_DPP(i)
#define WKV_FWD_B(i) "v_fmac_f32_dpp %[s" #i "], %[k], %[v]" WKV_DPP(i)
__device__ __forceinline__ void step_bcast_w(float (&S)[8], float &acc, float x, float w, float k, float v) {
    asm("s_nop 1\n\t" WKV_PIPE8(WKV_FWD_A, WKV_FWD_B)
        : WKV_REP8(WKV_S_OPERAND) [acc] "+v"(acc)
        : [x] "v"(x), [w] "v"(w), [k] "v"(k), [v] "v"(v));
}
__device__ __forceinline__ void step_bcast_w(float (&S)[16], float &acc, float x, float w, float k, float v) {
    asm("s_nop 1\n\t" WKV_PIPE16(WKV_FWD_A, WKV_FWD_B)
        : WKV_REP16(WKV_S_OPERAND) [acc] "+v"(acc)
        : [x] "v"(x), [w] "v"(w), [k] "v"(k), [v] "v"(v));
}
// acc += x[i] S[i];  S[i] = w S[i] + a[i] b         (x, a broadcast; w, b the lane's own)
#define WKV_OWN_A(i) "v_fmac_f32_dpp %[acc], %[x], %[s" #i "]" WKV_DPP(i) "v_mul_f32 %[s" #i "], %[w], %[s" #i "]\n\t"
#define WKV_OWN_B(i) "v_fmac_f32_dpp %[s" #i "], %[a], %[b]" WKV_DPP(i)
__device__ __forceinline__ void step_own_w(float (&S)[8], float &acc, float x, float w, float a, float b) {
    asm("s_nop 1\n\t" WKV_PIPE8(WKV_OWN_A, WKV_OWN_B)
        : WKV_REP8(WKV_S_OPERAND) [acc] "+v"(acc)
        : [x] "v"(x), [w] "v"(w), [a] "v"(a), [b] "v"(b));
}
__device__ __forceinline__ void step_own_w(float (&S)[16], float &acc, float x, float w, float a, float b) {
    asm("s_nop 1\n\t" WKV_PIPE16(WKV_OWN_A, WKV_OWN_B)
        : WKV_REP16(WKV_S_OPERAND) [acc] "+v"(acc)
        : [x] "v"(x), [w] "v"(w), [a] "v"(a), [b] "v"(b));
}

// Where a lane sits.  `own`: its column (column-owned) or row (row-owned), `ol` the same counted within the workgroup;
// `grp`: its group of EL rows (or columns); `shared`: the row (or column) whose per-token values it reads for its
// 16-lane row; `slot`: where its partial sums go (EL = 8: after the lanes 32 apart have added theirs, `paired`).
template <int EL> struct Place {
    int part, bh, wv, lane, gh, slot, ol, own, grp, shared;
    __device__ Place() {
        constexpr int PARTS = Shape<EL>::PARTS;
        part = PARTS == 2 ? blockIdx.x & 1 : 0; bh = PARTS == 2 ? blockIdx.x >> 1 : blockIdx.x;
        wv = threadIdx.x >> 6; lane = threadIdx.x & 63;
        const int lg = lane >> 4;
        gh = EL == 8 ? wv >> 1 : 0; slot = EL == 8 ? 2 * gh + (lg & 1) : lg;
        ol = 16 * (EL == 8 ? wv & 1 : wv) + (lane & 15); own = Shape<EL>::OWN * part + ol;
        grp = EL == 8 ? 4 * gh + lg : lg; shared = EL * grp + (lane & (EL - 1));
    }
};
template <int EL> using Partials = float[CH][4][Shape<EL>::OWN];
// what the lane 32 lanes away holds (EL = 8: the other row group of the pair that shares a slot; EL = 16: nothing to add)
template <int EL> __device__ __forceinline__ float other_half(float x) { return EL == 8 ? __shfl_xor(x, 32) : 0.f; }
template <class P> __device__ __forceinline__ float sum4(const P &p, int t, int x) {
    return (p[t][0][x] + p[t][1][x]) + (p[t][2][x] + p[t][3][x]);
}

// ---------------------------------------------------------------- forward --
template <class T, bool PER_TOKEN_W, int EL>
__global__ __launch_bounds__(NT) void rec_forward(int Tlen, int C, int H,
        const T *__restrict__ r, const T *__restrict__ k, const T *__restrict__ v,
        const float *__restrict__ wraw, const float *__restrict__ u,
        const float *__restrict__ s_in, T *__restrict__ y, float *__restrict__ s_out, int floor_decay)
{
    __shared__ __align__(16) float s_r[CH][HEAD], s_k[CH][HEAD], s_v[CH][HEAD], s_w[CH][HEAD];
    constexpr int OWN = Shape<EL>::OWN;
    __shared__ __align__(16) Partials<EL> s_y;                    // partial sums of each output of this workgroup
    __shared__ float s_rho[CH];                                   // sum_i r u k of each staged token

    const Place<EL> at;
    const int b = at.bh / H, h = at.bh % H, tid = threadIdx.x, j = at.own;
    const size_t base = (size_t)b * Tlen * C + (size_t)h * HEAD;
    const int st = tid >> 4, sc = (tid & 15) * 4;            // staging: token st, channels sc..sc+3
    const bool writes = sc / OWN == at.part;                 // ... and the lane writes them out if they are of this workgroup

    float S[EL], us[4];
    const float *sp = s_in + (size_t)at.bh * HEAD * HEAD;
#pragma unroll
    for (int ii = 0; ii < EL; ii++) S[ii] = sp[(EL * at.grp + ii) * HEAD + j];
    const float w_const = PER_TOKEN_W ? 0.f : __expf(log_decay(wraw[h * HEAD + at.shared], floor_decay));
#pragma unroll
    for (int e = 0; e < 4; e++) us[e] = u[h * HEAD + sc + e];

    // The fetch has no branch (the token is clamped into the sequence and what came for a token outside it is
    // replaced where it is staged): loads and stores share one counter, and after a conditional load, or before a
    // register a load may still be writing is set by hand, the compiler waits for everything outstanding, which here
    // would be the stores of the block before.
    float pr[4], pk[4], pv[4], pw[4];
    bool p_in = false;
    auto fetch = [&](int t0) {
        const int t = t0 + st;
        p_in = t < Tlen;
        const size_t o = base + (size_t)min(t, Tlen - 1) * C + sc;
        load4(r + o, pr); load4(k + o, pk); load4(v + o, pv);
        if (PER_TOKEN_W) load4(wraw + o, pw);
    };
    auto stage = [&]() {
        float rho = 0.f;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            if (!p_in) { pr[e] = pk[e] = pv[e] = 0.f; pw[e] = -1e30f; }   // decay 1, no update
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
        fetch(t0 + CH);                          // (past the end: a clamped fetch that nobody stages)
        const int nt = min(CH, Tlen - t0);      // the last block may be short
        // The next token's LDS reads are issued ahead of this token's multiply-adds, and the partial sums of an
        // output go to LDS as they are: they are added up (with the bonus term v rho) when the block's outputs are
        // written out, so the token loop has no shuffle and no wait other than for its own operands.
        // Two register sets take turns (no copies, so that a token's reads are waited for only where the next token
        // uses them): `cur` is consumed while `nxt` is filled.
        struct Tok { float v, r, k, w; };
        auto read = [&](Tok &x, int t) {
            x.v = s_v[t][j]; x.r = s_r[t][at.shared]; x.k = s_k[t][at.shared];
            x.w = PER_TOKEN_W ? s_w[t][at.shared] : w_const;
        };
        float done = 0.f;                        // the partial sum of the token before, not yet paired and stored
        auto token = [&](int t, const Tok &cur, Tok &nxt) {
            read(nxt, t + 1 < CH ? t + 1 : t);
            const float there = other_half<EL>(done);
            __builtin_amdgcn_sched_barrier(0);   // the reads and the shuffle are issued before the arithmetic, not after
            float acc = 0.f;
            step_bcast_w(S, acc, cur.r, cur.w, cur.k, cur.v);
            if (t > 0) s_y[t - 1][at.slot][at.ol] = done + there;
            done = acc;
        };
        Tok ta, tb;
        read(ta, 0);
        for (int t = 0; t < nt; t += 2) {
            token(t, ta, tb);
            if (t + 1 < nt) token(t + 1, tb, ta);
        }
        s_y[nt - 1][at.slot][at.ol] = done + other_half<EL>(done);
        __syncthreads();
        float o4[4];
        if (writes) {
#pragma unroll
            for (int e = 0; e < 4; e++) o4[e] = fmaf(s_v[st][sc + e], s_rho[st], sum4(s_y, st, sc - OWN * at.part + e));
        }
        // no barrier: what the lines above read of the staged block and stage() overwrites is the lane's own four
        // channels, or the token's scalar, which a lane of the same wavefront writes later in program order
        stage();                                 // (after the last block: zeros, unused; unconditional so that no load is left
                                                 // outstanding on any path around the loop)
        // The stores come after stage(): loads and stores share one counter, stage() waits for the prefetched block
        // with a wait for everything outstanding, and a store issued before it would be waited for to the end.
        if (writes && t0 + st < Tlen) store4(y + base + (size_t)(t0 + st) * C + sc, o4);
        __syncthreads();
    }
    float *op = s_out + (size_t)at.bh * HEAD * HEAD;
#pragma unroll
    for (int ii = 0; ii < EL; ii++) op[(EL * at.grp + ii) * HEAD + j] = S[ii];
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
// The token loops only advance the states and leave the partial sums of every contraction in LDS; what follows from
// them (the sums, the bonus terms, the running sum A over the 16 tokens of a block) is done once per block: lane
// (g, row) of the first two wavefronts takes tokens 4g..4g+3 of its row, and the A values at the starts of the four
// token quarters come from three shuffles.
// (EL = 8: four workgroups per compute unit, i.e. four wavefronts per SIMD, fit by LDS; the register budget is told so)
template <class T, bool PER_TOKEN_W, int EL>
__global__ __launch_bounds__(NT, EL == 8 ? 4 : 2) void rec_backward(int Tlen, int C, int H,
        const T *__restrict__ r, const T *__restrict__ k, const T *__restrict__ v,
        const float *__restrict__ wraw, const float *__restrict__ u, const float *__restrict__ s_in,
        const T *__restrict__ gy, const float *__restrict__ gs_out,
        T *__restrict__ gr, T *__restrict__ gk, T *__restrict__ gv, float *__restrict__ gw_tok,
        float *__restrict__ gw_part, float *__restrict__ gu_part, float *__restrict__ gs_in,
        float *__restrict__ qbuf, int floor_decay)
{
    __shared__ __align__(16) float s_r[CH][HEAD], s_k[CH][HEAD], s_v[CH][HEAD], s_w[CH][HEAD], s_g[CH][HEAD],
        s_l[CH][Shape<EL>::OWN];                             // of the rows of this workgroup
    __shared__ __align__(16) Partials<EL> p_a, p_b;
    __shared__ float s_p[CH], s_rho[CH];                                 // v.gy and sum r u k of each staged token

    const Place<EL> at;
    const int b = at.bh / H, h = at.bh % H, tid = threadIdx.x, own = at.own, ol = at.ol;
    const size_t base = (size_t)b * Tlen * C + (size_t)h * HEAD;
    const int st = tid >> 4, sc = (tid & 15) * 4;
    constexpr int OWN = Shape<EL>::OWN;
    const bool writes = sc / OWN == at.part;
    const int wl = sc - OWN * at.part;                       // first of the lane's four channels within the workgroup's
    const bool scans = at.gh == 0;                           // EL = 8: wavefronts 0 and 1; lane (lane group, ol)

    const float u_own = u[h * HEAD + own];
    float l_own = 0.f, w_own = 1.f, w_shared = 1.f, us[4];
    bool floored_own = false;
    if (!PER_TOKEN_W) {
        l_own = log_decay(wraw[h * HEAD + own], floor_decay, &floored_own);
        w_own = __expf(l_own);
        w_shared = __expf(log_decay(wraw[h * HEAD + at.shared], floor_decay));
    }
#pragma unroll
    for (int e = 0; e < 4; e++) us[e] = u[h * HEAD + sc + e];

    float pr[4], pk[4], pv[4], pw[4], pg[4];
    float pq[4], q_own[4];                                   // q of the lane's row at the four tokens it scans: in flight, current
    bool p_in = false;                                       // (a fetch without branches, as in the forward)
    int p_t0 = 0;
    auto fetch = [&](int t0, bool second) {
        const int t = t0 + st;
        p_t0 = t0;
        p_in = t >= 0 && t < Tlen;
        const size_t o = base + (size_t)min(max(t, 0), Tlen - 1) * C + sc;
        load4(r + o, pr); load4(k + o, pk); load4(v + o, pv); load4(gy + o, pg);
        if (PER_TOKEN_W) load4(wraw + o, pw);
        if (second && scans) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int tq = t0 + 4 * (at.lane >> 4) + e;
                pq[e] = qbuf[base + (size_t)min(max(tq, 0), Tlen - 1) * C + own];
            }
        }
    };
    auto stage = [&](bool second) {
        float dot = 0.f, rho = 0.f;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            if (!p_in) { pr[e] = pk[e] = pv[e] = pg[e] = 0.f; pw[e] = -1e30f; }
            s_r[st][sc + e] = pr[e]; s_k[st][sc + e] = pk[e]; s_v[st][sc + e] = pv[e]; s_g[st][sc + e] = pg[e];
            if (PER_TOKEN_W) {
                bool fl;
                const float l = log_decay(pw[e], floor_decay, &fl);
                s_w[st][sc + e] = __expf(l);
                if (writes) s_l[st][wl + e] = fl ? 0.f : l;      // factor that turns dL/d log w into dL/d raw
            }
            if (second) {
                const int tq = p_t0 + 4 * (at.lane >> 4) + e;
                q_own[e] = tq >= 0 && tq < Tlen ? pq[e] : 0.f;
            }
            dot = fmaf(pv[e], pg[e], dot);
            rho = fmaf(pr[e] * us[e], pk[e], rho);
        }
        dot = token_sum(dot);
        rho = token_sum(rho);
        if (sc == 0) { s_p[st] = dot; s_rho[st] = rho; }
    };

    // ---------------- sweep 1: forward in time, S row-owned (row `own`, columns EL grp .. EL grp + EL - 1)
    float S[EL];
    {
        const float *sp = s_in + (size_t)at.bh * HEAD * HEAD + own * HEAD + EL * at.grp;
#pragma unroll
        for (int q = 0; q < EL / 4; q++) {
            const float4 x = *reinterpret_cast<const float4 *>(sp + 4 * q);
            S[4 * q] = x.x; S[4 * q + 1] = x.y; S[4 * q + 2] = x.z; S[4 * q + 3] = x.w;
        }
    }
    fetch(0, false);
    stage(false);
    __syncthreads();
    for (int t0 = 0; t0 < Tlen; t0 += CH) {
        fetch(t0 + CH, false);                   // (past the end: a clamped fetch that nobody stages)
        const int nt = min(CH, Tlen - t0);
        struct Tok { float k, w, v, g; };        // k, w of the lane's row; v, gy of the column it reads for its 16-lane row
        auto read = [&](Tok &x, int t) {
            x.k = s_k[t][own]; x.w = PER_TOKEN_W ? s_w[t][own] : w_own;
            x.v = s_v[t][at.shared]; x.g = s_g[t][at.shared];
        };
        float done = 0.f;
        auto token = [&](int t, const Tok &cur, Tok &nxt) {
            read(nxt, t + 1 < CH ? t + 1 : t);
            const float there = other_half<EL>(done);
            __builtin_amdgcn_sched_barrier(0);
            float acc = 0.f;
            step_own_w(S, acc, cur.g, cur.w, cur.v, cur.k);      // acc += gy_j S_ij;  S_ij = w_i S_ij + v_j k_i
            if (t > 0) p_a[t - 1][at.slot][ol] = done + there;
            done = acc;
        };
        Tok ta, tb;
        read(ta, 0);
        for (int t = 0; t < nt; t += 2) {
            token(t, ta, tb);
            if (t + 1 < nt) token(t + 1, tb, ta);
        }
        p_a[nt - 1][at.slot][ol] = done + other_half<EL>(done);
        __syncthreads();
        float a4[4], b4[4];
        if (writes) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                a4[e] = fmaf(us[e] * s_k[st][sc + e], s_p[st], sum4(p_a, st, wl + e));
                b4[e] = a4[e] * s_r[st][sc + e];
            }
        }
        // no barrier: what the lines above read of the staged block and stage() overwrites is the lane's own four
        // channels, or the token's scalar, which a lane of the same wavefront writes later in program order
        stage(false);                            // (unconditional, as in the forward)
        if (writes && t0 + st < Tlen) {          // (after stage(), which waits for everything outstanding: see the forward)
            const size_t o = base + (size_t)(t0 + st) * C + sc;
            store4(gr + o, a4);
            store4(qbuf + o, b4);
        }
        __syncthreads();
    }

    // ---------------- boundary: G = gS_out in both ownerships, A = sum_j gS_out o S_out
    float Gr[EL], Gc[EL];
    float A = 0.f;
    {
        const size_t so = (size_t)at.bh * HEAD * HEAD;
        float part = 0.f;
#pragma unroll
        for (int q = 0; q < EL; q++) {
            Gr[q] = gs_out ? gs_out[so + own * HEAD + EL * at.grp + q] : 0.f;
            Gc[q] = gs_out ? gs_out[so + (EL * at.grp + q) * HEAD + own] : 0.f;
            part = fmaf(Gr[q], S[q], part);
        }
        p_a[0][at.slot][ol] = part + other_half<EL>(part);
    }
    float gu_acc = 0.f, gw_acc = 0.f;

    // the q values of sweep 1 were written by other lanes of this workgroup (it reads back the rows of its half only)
    __threadfence_block();
    __syncthreads();
    if (scans) A = sum4(p_a, 0, ol);             // the same in the four lanes of a row
    __syncthreads();

    // ---------------- sweep 2: backward in time
    const int last0 = ((Tlen - 1) / CH) * CH;
    fetch(last0, true);
    stage(true);
    __syncthreads();
    for (int t0 = last0; t0 >= 0; t0 -= CH) {
        fetch(t0 - CH, true);                    // (before the start: a clamped fetch that nobody stages)
        const int nt = min(CH, Tlen - t0);
        {
            const int tf = nt - 1;
            struct Tok { float r, w, gy, vs, gs, rs, ks, ws; };      // of the lane's row / column; of the one it reads for its 16-lane row
            auto read = [&](Tok &x, int t) {
                x.r = s_r[t][own]; x.w = PER_TOKEN_W ? s_w[t][own] : w_own; x.gy = s_g[t][own];
                x.vs = s_v[t][at.shared]; x.gs = s_g[t][at.shared]; x.rs = s_r[t][at.shared]; x.ks = s_k[t][at.shared];
                x.ws = PER_TOKEN_W ? s_w[t][at.shared] : w_shared;
            };
            float doneG = 0.f, doneV = 0.f;
            auto token = [&](int t, const Tok &cur, Tok &nxt) {
                read(nxt, t > 0 ? t - 1 : 0);
                const float thereG = other_half<EL>(doneG), thereV = other_half<EL>(doneV);
                __builtin_amdgcn_sched_barrier(0);
                float accG = 0.f, accV = 0.f;
                step_own_w(Gr, accG, cur.vs, cur.w, cur.gs, cur.r);          // row i = own:    accG += v_j G_ij;  G_ij = w_i G_ij + gy_j r_i
                step_bcast_w(Gc, accV, cur.ks, cur.ws, cur.rs, cur.gy);      // column j = own: accV += k_i G_ij;  G_ij = w_i G_ij + r_i gy_j
                if (t < tf) {
                    p_a[t + 1][at.slot][ol] = doneG + thereG;
                    p_b[t + 1][at.slot][ol] = doneV + thereV;
                }
                doneG = accG; doneV = accV;
            };
            Tok ta, tb;
            read(ta, tf);
            for (int t = tf; t >= 0; t -= 2) {
                token(t, ta, tb);
                if (t > 0) token(t - 1, tb, ta);
            }
            p_a[0][at.slot][ol] = doneG + other_half<EL>(doneG);
            p_b[0][at.slot][ol] = doneV + other_half<EL>(doneV);
        }
        __syncthreads();
        if (scans) {   // row `own`, tokens 4g+3 .. 4g: gk, and D from the running sum A (which runs from the last token down)
            const int g = at.lane >> 4;
            float c[4], kG[4], tot = 0.f;
#pragma unroll
            for (int e = 3; e >= 0; e--) {
                const int t = 4 * g + e;
                const float sumG = t < nt ? sum4(p_a, t, ol) : 0.f;
                const float ri = s_r[t][own], ki = s_k[t][own];
                const float gki = fmaf(u_own * ri, s_p[t], sumG);
                kG[e] = ki * sumG;
                c[e] = q_own[e] - ki * gki;
                tot += c[e];
                gu_acc = fmaf(ri * ki, s_p[t], gu_acc);
                p_a[t][0][ol] = gki;                     // this lane alone reads and writes the slots of (t, row)
            }
            // A before token t = A + (c of all later tokens): later quarters, then later tokens of this quarter
            const int low = at.lane & 15;
            const float t0q = __shfl(tot, low), t1 = __shfl(tot, low + 16), t2 = __shfl(tot, low + 32), t3 = __shfl(tot, low + 48);
            float run = A + (g < 1 ? t1 : 0.f) + (g < 2 ? t2 : 0.f) + (g < 3 ? t3 : 0.f);
#pragma unroll
            for (int e = 3; e >= 0; e--) {
                const int t = 4 * g + e;
                const float D = run - kG[e];
                run += c[e];
                if (PER_TOKEN_W) p_a[t][1][ol] = D * s_l[t][ol];
                else if (t < nt) gw_acc += D;
            }
            A += (t0q + t1) + (t2 + t3);
        }
        __syncthreads();
        float a4[4], b4[4], c4[4];
        if (writes) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                a4[e] = p_a[st][0][wl + e];
                c4[e] = p_a[st][1][wl + e];
                b4[e] = fmaf(s_g[st][sc + e], s_rho[st], sum4(p_b, st, wl + e));
            }
        }
        stage(true);                             // no barrier needed, as in sweep 1; unconditional, as in the forward
        if (writes && t0 + st < Tlen) {          // (after stage(), as in sweep 1)
            const size_t o = base + (size_t)(t0 + st) * C + sc;
            store4(gk + o, a4);
            store4(gv + o, b4);
            if (PER_TOKEN_W) store4(gw_tok + o, c4);
        }
        __syncthreads();
    }

    if (gs_in) {
        float *gp = gs_in + (size_t)at.bh * HEAD * HEAD + own * HEAD + EL * at.grp;
#pragma unroll
        for (int q = 0; q < EL / 4; q++)
            *reinterpret_cast<float4 *>(gp + 4 * q) = make_float4(Gr[4 * q], Gr[4 * q + 1], Gr[4 * q + 2], Gr[4 * q + 3]);
    }
    gu_acc = group_sum(gu_acc);
    gw_acc = group_sum(gw_acc);
    if (scans && at.slot == 0) {      // (two lanes of a row qualify: same value, same address)
        gu_part[(size_t)at.bh * HEAD + own] = gu_acc;
        if (!PER_TOKEN_W) gw_part[(size_t)at.bh * HEAD + own] = floored_own ? 0.f : gw_acc * l_own;
    }
}

// ------------------------------------------------------------- launchers --
// Eight elements per lane (two workgroups per head) where the finer grain evens out the load of the compute units;
// sixteen where the heads fill them evenly anyway (a multiple of their number) or at least twice over: there the
// staging work that two workgroups per head do twice costs more than the grain gains.  Forward + backward per token
// on 256 compute units, ns, 8 / 16 elements: B*H = 128: 817 / 845; 256: 948 / 899; 320: 1180 / 1231; 384: 1219 / 1262;
// 512: 1572 / 1355; 768: 2361 / 2025.  RWKV_WKV_REC_EL=8|16 overrides.
static int elements_per_lane(int BH) {
    static const int forced = [] { const char *e = getenv("RWKV_WKV_REC_EL"); return e ? atoi(e) : 0; }();
    if (forced == 8 || forced == 16) return forced;
    const int ncu = cu_count();
    return (BH >= 2 * ncu || BH % ncu == 0) ? 16 : 8;
}

template <class T, int EL>
static hipError_t launch_fwd_el(hipStream_t s, bool per_token, int B, int Tlen, int C, int H, const void *r, const void *k,
                                const void *v, const float *w, const float *u, const float *s_in, void *y, float *s_out,
                                int floor_decay) {
    dim3 grid(Shape<EL>::PARTS * B * H), block(NT);
    prof_begin(KID_REC_FORWARD, s);
    if (per_token)
        hipLaunchKernelGGL((rec_forward<T, true, EL>), grid, block, 0, s, Tlen, C, H, (const T *)r, (const T *)k, (const T *)v,
                           w, u, s_in, (T *)y, s_out, floor_decay);
    else
        hipLaunchKernelGGL((rec_forward<T, false, EL>), grid, block, 0, s, Tlen, C, H, (const T *)r, (const T *)k,
                           (const T *)v, w, u, s_in, (T *)y, s_out, floor_decay);
    prof_end(KID_REC_FORWARD, s);
    return hipGetLastError();
}
template <class T>
static hipError_t launch_fwd(hipStream_t s, bool per_token, int B, int Tlen, int C, int H, const void *r, const void *k,
                             const void *v, const float *w, const float *u, const float *s_in, void *y, float *s_out,
                             int floor_decay) {
    return elements_per_lane(B * H) == 16
               ? launch_fwd_el<T, 16>(s, per_token, B, Tlen, C, H, r, k, v, w, u, s_in, y, s_out, floor_decay)
               : launch_fwd_el<T, 8>(s, per_token, B, Tlen, C, H, r, k, v, w, u, s_in, y, s_out, floor_decay);
}

template <class T, int EL>
static hipError_t launch_bwd_el(hipStream_t s, bool per_token, int B, int Tlen, int C, int H, const void *r, const void *k,
                                const void *v, const float *w, const float *u, const float *s_in, const void *gy,
                                const float *gs_out, void *gr, void *gk, void *gv, float *gw, float *gu, float *gs_in,
                                float *ws, int floor_decay) {
    // workspace: q (B,T,C) fp32 | gu partials (B,C) | gw partials (B,C)
    float *qbuf = ws;
    float *gu_part = qbuf + (size_t)B * Tlen * C;
    float *gw_part = gu_part + (size_t)B * C;
    dim3 grid(Shape<EL>::PARTS * B * H), block(NT);
    prof_begin(KID_REC_BACKWARD, s);
    if (per_token)
        hipLaunchKernelGGL((rec_backward<T, true, EL>), grid, block, 0, s, Tlen, C, H, (const T *)r, (const T *)k,
                           (const T *)v, w, u, s_in, (const T *)gy, gs_out, (T *)gr, (T *)gk, (T *)gv, gw, gw_part,
                           gu_part, gs_in, qbuf, floor_decay);
    else
        hipLaunchKernelGGL((rec_backward<T, false, EL>), grid, block, 0, s, Tlen, C, H, (const T *)r, (const T *)k,
                           (const T *)v, w, u, s_in, (const T *)gy, gs_out, (T *)gr, (T *)gk, (T *)gv, nullptr, gw_part,
                           gu_part, gs_in, qbuf, floor_decay);
    prof_end(KID_REC_BACKWARD, s);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(sum_over_batch, dim3((C + 255) / 256), dim3(256), 0, s, B, C, gu_part, gu);
    if (!per_token) hipLaunchKernelGGL(sum_over_batch, dim3((C + 255) / 256), dim3(256), 0, s, B, C, gw_part, gw);
    return hipGetLastError();
}
template <class T>
static hipError_t launch_bwd(hipStream_t s, bool per_token, int B, int Tlen, int C, int H, const void *r, const void *k,
                             const void *v, const float *w, const float *u, const float *s_in, const void *gy,
                             const float *gs_out, void *gr, void *gk, void *gv, float *gw, float *gu, float *gs_in,
                             float *ws, int floor_decay) {
    return elements_per_lane(B * H) == 16
               ? launch_bwd_el<T, 16>(s, per_token, B, Tlen, C, H, r, k, v, w, u, s_in, gy, gs_out, gr, gk, gv, gw, gu, gs_in, ws, floor_decay)
               : launch_bwd_el<T, 8>(s, per_token, B, Tlen, C, H, r, k, v, w, u, s_in, gy, gs_out, gr, gk, gv, gw, gu, gs_in, ws, floor_decay);
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
