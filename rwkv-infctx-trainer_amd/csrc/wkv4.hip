// RWKV-v4 WKV with (aa, bb, pp) state: one lane per (batch, channel) chain.
//
// The chain is serial in time, and a GPU holds few chains (B*C lanes), so two things set the speed: how many
// bytes each lane keeps in flight, and how many instructions the ONE wavefront that walks a chain has to issue per
// token.  For the first, blocks of 16 tokens of k, v (and gy) are fetched into registers several blocks ahead of the
// one being consumed; consecutive lanes are consecutive channels, so every load and store is a full coalesced row.
// For the second, only the recurrence itself stays with the walking wavefront; everything that can be formed from
// a block's starting state alone is handed to other wavefronts of the workgroup, which work on different blocks at
// the same time:
//   forward   wavefront 0 advances (p, q, o) and leaves the state at the start of every 16-token block in LDS;
//             wavefronts 1-3 take a block each (every third block) and form its 16 outputs from that state;
//   backward  wavefront 0 replays a block from the forward's checkpoint and leaves what the reverse walk needs of
//             its 16 tokens in LDS; wavefront 1 walks the block replayed just before backwards at the same time.
//             (More replaying wavefronts, the 16-byte fetches of the forward, or two pairs per workgroup were all
//             measured slower here: with the recurrence replayed the pass is bound by the instructions a compute
//             unit issues, not by one wavefront's.)
// Per token the arithmetic is kept short (one exponential per max-scaled pair, the bare reciprocal instruction) and
// free of branches, so that the tokens of a block are one straight-line stretch the scheduler can interleave.
//
// State convention (RWKV-v4neo/cuda/wkv_cuda_bf16.cu:30-52): (p, q, o) with
// p, q the decayed sums divided by e^{o}.  Backward carries the state gradient
// the same way, (gp, gq, go), and returns the decay gradient with respect to
// the raw time_decay parameter (:116-156).
//
// Backward never stores per-token intermediates for the whole sequence (the
// reference keeps three T-long arrays per lane): the forward sweep leaves a
// 5-float checkpoint (p, q, o, dp/dw, dq/dw) every 16 tokens, and the backward
// sweep replays one 16-token block at a time from its checkpoint.
#include "common.h"
#include <type_traits>

namespace wkv {

// one element of a result, stored with the non-temporal hint (results are not read again by these kernels)
__device__ __forceinline__ void stream1(float *p, float v) { __builtin_nontemporal_store(v, p); }
__device__ __forceinline__ void stream1(bf16 *p, bf16 v) { __builtin_nontemporal_store(v.bits, &p->bits); }
__device__ __forceinline__ void stream1(f16 *p, f16 v) { __builtin_nontemporal_store(v.h, &p->h); }

constexpr int CK = 16;                 // tokens per checkpoint block
constexpr float NEG_HUGE = -1e38f;

struct Chain { float p, q, o, dp, dq; };

// Two terms scaled by a common maximum exponent, e^{a-m} and e^{b-m} with m = max(a, b): one of the two is
// exactly 1, so a pair costs one exponential, e^{-|a-b|}.
struct ExpPair { float first, second; bool first_is_max; };
__device__ __forceinline__ ExpPair exp_pair(float a, float b) {
    const float d = a - b, e = __expf(-fabsf(d));
    const bool fm = d >= 0.f;
    return ExpPair{fm ? 1.f : e, fm ? e : 1.f, fm};
}

// one token: output y and the pieces backward re-uses (1 / scaled denominator, the current token's scaled weight,
// the history's scaled weight, minus the scaling exponent); advances the chain
__device__ __forceinline__ float v4_step(Chain &s, float w, float u, float kk, float vv,
                                         float &iden, float &ec, float &hist_w, float &neg_m) {
    const float uk = u + kk;
    const ExpPair a = exp_pair(s.o, uk);
    hist_w = a.first;
    ec = a.second;
    neg_m = a.first_is_max ? -s.o : -uk;
    iden = __builtin_amdgcn_rcpf(hist_w * s.q + ec);      // the bare v_rcp_f32 (1 ulp), not a full division
    const float y = (hist_w * s.p + ec * vv) * iden;
    const float wo = w + s.o;
    const ExpPair d = exp_pair(wo, kk);
    const float dh = d.first, dc = d.second;
    s.dp = dh * (s.p + s.dp);
    s.dq = dh * (s.q + s.dq);
    s.p = fmaf(dh, s.p, dc * vv);
    s.q = fmaf(dh, s.q, dc);
    s.o = d.first_is_max ? wo : kk;
    return y;
}

// the recurrence alone: the same operations on (p, q, o, dp, dq) as v4_step, in the same order
__device__ __forceinline__ void v4_advance(Chain &s, float w, float kk, float vv) {
    const float wo = w + s.o;
    const ExpPair d = exp_pair(wo, kk);
    const float dh = d.first, dc = d.second;
    s.dp = dh * (s.p + s.dp);
    s.dq = dh * (s.q + s.dq);
    s.p = fmaf(dh, s.p, dc * vv);
    s.q = fmaf(dh, s.q, dc);
    s.o = d.first_is_max ? wo : kk;
}

// A block of 16 tokens x 64 chains of one tensor on its way from memory to the lanes that own the chains.  A
// wavefront can have 64 memory instructions in flight, so what it has in flight in bytes is set by the size of one:
//   WIDE   16 bytes per lane: lane l fetches W = 16 / sizeof(T) consecutive chains of token l / (64/W) of every
//          group of 64 / (64/W) tokens (a full 256- or 128-byte row segment per 64/W lanes); a block is 4 (fp32) or
//          2 (bf16, fp16) instructions.  The pieces reach their owners through LDS: written as they came,
//          [token][chain], read back one element per lane and token.  Needs C to be a multiple of W (a piece
//          never straddles two batch rows) and 16-byte aligned tensors.
//   narrow one element per lane and token: 16 instructions per block; any C.
// Either way the block ends up in the LDS area handed in as well as in the caller's registers.
template <class T, bool WIDE> struct V4In;
template <class T> struct V4In<T, false> {
    T val[CK];
    __device__ __forceinline__ void fetch(const T *p, int /*chain0*/, int idx, int /*BC*/, int C, int Tlen, int t0, int /*lane*/) {
        const int b = idx / C, c = idx % C;
        const T *q = p + ((size_t)b * Tlen + t0) * C + c;
        if (t0 + CK <= Tlen) {          // whole block inside the sequence: no per-token checks
#pragma unroll
            for (int i = 0; i < CK; i++, q += C) val[i] = *q;
        } else {
#pragma unroll
            for (int i = 0; i < CK; i++, q += C) val[i] = t0 + i < Tlen ? *q : T{};
        }
    }
    __device__ __forceinline__ void spread(T *stage, int lane, T (&out)[CK]) const {
#pragma unroll
        for (int i = 0; i < CK; i++) { out[i] = val[i]; stage[i * 64 + lane] = val[i]; }
    }
};
template <class T> struct V4In<T, true> {
    static constexpr int W = 16 / sizeof(T), LPR = 64 / W, ROWS = 64 / LPR, NLD = CK / ROWS;
    typedef unsigned int piece_t __attribute__((ext_vector_type(4)));
    piece_t piece[NLD];
    // chain0: the wavefront's first chain (a multiple of 64); tokens past the end repeat the last one (never used)
    __device__ __forceinline__ void fetch(const T *p, int chain0, int /*idx*/, int BC, int C, int Tlen, int t0, int lane) {
        const int q = min(chain0 + (lane % LPR) * W, BC - W);
        const T *row = p + (size_t)(q / C) * Tlen * C + q % C;
#pragma unroll
        for (int i = 0; i < NLD; i++)
            piece[i] = *reinterpret_cast<const piece_t *>(row + (size_t)min(t0 + i * ROWS + lane / LPR, Tlen - 1) * C);
    }
    __device__ __forceinline__ void spread(T *stage, int lane, T (&out)[CK]) const {
#pragma unroll
        for (int i = 0; i < NLD; i++) *reinterpret_cast<piece_t *>(stage + (i * ROWS + lane / LPR) * 64 + (lane % LPR) * W) = piece[i];
#pragma unroll
        for (int i = 0; i < CK; i++) out[i] = stage[i * 64 + lane];
    }
};

// Forward.  y == nullptr: only checkpoints / final state are produced.
// ckpt layout: [block][5][B*C].
// Four wavefronts per 64 chains.  One walks the chain, V4_YW blocks (a lap) between two workgroup barriers, and
// leaves in LDS the state at the start of each block and the block's k and v; each of the other three forms the
// outputs of one block of the lap before from what it finds there (it reads nothing from memory).  The walking
// wavefront's inputs wait in registers as they came, two laps deep (converting at the fetch would make every load
// wait for its data on the spot, and nothing would be in flight); register sets and LDS slots are fixed per use, two
// laps written out.
constexpr int V4_YW = 3, V4_GROUPS = 2;
template <class T, bool WIDE>
__global__ __launch_bounds__(64 * (1 + V4_YW) * V4_GROUPS) void v4_forward(int BC, int Tlen, int C, const float *__restrict__ time_decay,
        const float *__restrict__ time_first, const T *__restrict__ k, const T *__restrict__ v,
        const float *__restrict__ s_in, T *__restrict__ y, float *__restrict__ s_out, float *__restrict__ ckpt)
{
    __shared__ float start_all[V4_GROUPS][2 * V4_YW][5][64];      // the state at a block's start: p, q, o (and dp, dq for the checkpoint)
    // k and v of the blocks of two laps, [token][chain]: left there by the walking wavefront on its way (it is also
    // how the 16-byte pieces reach their owners), read by the wavefront that forms the block's outputs a lap later
    extern __shared__ __align__(16) unsigned char kv_raw[];          // v4_forward_lds<T>() bytes
    typedef T KvBlock[CK * 64];
    KvBlock (*kv_all)[2 * V4_YW][2] = reinterpret_cast<KvBlock (*)[2 * V4_YW][2]>(kv_raw);
    // A workgroup is two groups of four wavefronts, 64 chains each.  The walking wavefront is the first of its four in
    // group 0 and the second in group 1: wavefronts go to the four SIMDs in turn, and two walkers on one SIMD would
    // share the one resource they are short of.
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), grp = wave >> 2, wl = wave & 3;
    const int role = wl == grp ? 0 : (wl < grp ? wl + 1 : wl);       // 0: walks the chain; 1 + r: outputs of every third block
    // (lanes and groups past the last chain stay, the 16-byte fetches being a wavefront's joint work and the barriers
    // the workgroup's: they read the last chains' inputs and write nothing)
    const int chain_grp = (blockIdx.x * V4_GROUPS + grp) * 64, chain0 = min(chain_grp, (BC - 1) / 64 * 64);
    const int idx = min(chain0 + lane, BC - 1);
    const bool live = chain_grp + lane < BC;
    float (*start)[5][64] = start_all[grp];
    const int b = idx / C, c = idx % C;
    const float w = -__expf(time_decay[c]), u = time_first[c];
    const size_t base = (size_t)b * Tlen * C + c;
    const int nblk = (Tlen + CK - 1) / CK, nlap = (nblk + V4_YW - 1) / V4_YW;
    typedef V4In<T, WIDE> In;

    if (role == 0) {
        Chain s{0.f, 0.f, NEG_HUGE, 0.f, 0.f};
        if (s_in) { s.p = s_in[idx * 3]; s.q = s_in[idx * 3 + 1]; s.o = s_in[idx * 3 + 2]; }
        // two laps of blocks: one being consumed, one in flight (named, not an array: every use is a fixed register set)
        static_assert(V4_YW == 3, "the laps are written out for three blocks");
        In k0, k1, k2, k3, k4, k5, v0, v1, v2, v3, v4, v5;
        // (The 16-byte fetches of the two-byte types are unconditional, also for blocks past the end, where they
        // repeat the last token and nobody uses them: after a load inside a branch the compiler waits for everything
        // outstanding instead of for the block it needs.  Measured at B8 T4096 C4096: bf16 forward 265 -> 259 us; fp32,
        // whose laps in flight are twice the bytes, 316 -> 331 us, so it keeps the conditional fetches.)
        constexpr bool AHEAD = WIDE && sizeof(T) == 2;
        auto first = [&](int d, In &ik, In &iv) __attribute__((always_inline)) {
            if (AHEAD || d < nblk) { ik.fetch(k, chain0, idx, BC, C, Tlen, d * CK, lane); iv.fetch(v, chain0, idx, BC, C, Tlen, d * CK, lane); }
        };
        first(0, k0, v0); first(1, k1, v1); first(2, k2, v2); first(3, k3, v3); first(4, k4, v4); first(5, k5, v5);
        auto block = [&](int blk, int slot, In &ik, In &iv) __attribute__((always_inline)) {
            if (!AHEAD && blk >= nblk) return;
            const bool on = blk < nblk;          // scalar
            T kk[CK], vv[CK];
            if (on) {
            // (the block's checkpoint is written by the wavefront that forms its outputs, from these five values: this
            // wavefront then has loads outstanding and nothing else, and loads alone are counted in order, so that a wait
            // for one block's inputs does not wait for the blocks fetched after it; with a store among them it would)
            start[slot][0][lane] = s.p; start[slot][1][lane] = s.q; start[slot][2][lane] = s.o;
            start[slot][3][lane] = s.dp; start[slot][4][lane] = s.dq;
            ik.spread(kv_all[grp][slot][0], lane, kk);
            iv.spread(kv_all[grp][slot][1], lane, vv);
            }
            const int nb = blk + 2 * V4_YW;
            if (AHEAD || nb < nblk) { ik.fetch(k, chain0, idx, BC, C, Tlen, nb * CK, lane); iv.fetch(v, chain0, idx, BC, C, Tlen, nb * CK, lane); }
            if (!on) return;
            const int t0 = blk * CK, cnt = min(CK, Tlen - t0);
            if (cnt == CK) {
#pragma unroll
                for (int i = 0; i < CK; i++) v4_advance(s, w, to_float(kk[i]), to_float(vv[i]));
            } else {
#pragma unroll
                for (int i = 0; i < CK; i++)
                    if (i < cnt) v4_advance(s, w, to_float(kk[i]), to_float(vv[i]));
            }
        };
        for (int rd = 0; rd <= nlap; rd += 2) {
            block(rd * V4_YW, 0, k0, v0); block(rd * V4_YW + 1, 1, k1, v1); block(rd * V4_YW + 2, 2, k2, v2);
            lds_barrier();
            block((rd + 1) * V4_YW, 3, k3, v3); block((rd + 1) * V4_YW + 1, 4, k4, v4); block((rd + 1) * V4_YW + 2, 5, k5, v5);
            lds_barrier();                       // (both halves always: blocks past the end do nothing)
        }
        if (s_out && live) { s_out[idx * 3] = s.p; s_out[idx * 3 + 1] = s.q; s_out[idx * 3 + 2] = s.o; }
    } else {
        const int r = role - 1;
        // the outputs of this wavefront's block of lap pr (whose starting state and inputs wait in slot `slot`)
        auto outputs = [&](int pr, int slot) __attribute__((always_inline)) {
            const int blk = pr * V4_YW + r;
            if (pr < 0 || blk >= nblk) return;
            if (ckpt && live) {
                float *cp = ckpt + (size_t)blk * 5 * BC + idx;
                cp[0] = start[slot][0][lane]; cp[BC] = start[slot][1][lane]; cp[2 * (size_t)BC] = start[slot][2][lane];
                cp[3 * (size_t)BC] = start[slot][3][lane]; cp[4 * (size_t)BC] = start[slot][4][lane];
            }
            if (!y) return;
            Chain s{start[slot][0][lane], start[slot][1][lane], start[slot][2][lane], 0.f, 0.f};
            const T *ks = kv_all[grp][slot][0], *vs = kv_all[grp][slot][1];
            T kk[CK], vv[CK];
#pragma unroll
            for (int i = 0; i < CK; i++) { kk[i] = ks[i * 64 + lane]; vv[i] = vs[i * 64 + lane]; }
            const int t0 = blk * CK, cnt = min(CK, Tlen - t0);
            T *yp = y + base + (size_t)t0 * C;
            if (cnt == CK) {
#pragma unroll
                for (int i = 0; i < CK; i++, yp += C) {
                    float iden, ec, hw, nm;
                    const float yy = v4_step(s, w, u, to_float(kk[i]), to_float(vv[i]), iden, ec, hw, nm);
                    if (live) stream1(yp, from_float<T>(yy));
                }
            } else {
#pragma unroll
                for (int i = 0; i < CK; i++, yp += C)
                    if (i < cnt) {
                        float iden, ec, hw, nm;
                        const float yy = v4_step(s, w, u, to_float(kk[i]), to_float(vv[i]), iden, ec, hw, nm);
                        if (live) stream1(yp, from_float<T>(yy));
                    }
            }
        };
        for (int rd = 0; rd <= nlap; rd += 2) {       // in lap rd: the block of lap rd-1
            outputs(rd - 1, V4_YW + r);
            lds_barrier();
            outputs(rd, r);
            lds_barrier();
        }
    }
}

// Backward: two wavefronts per 64 chains.  Replaying a block from its checkpoint does not depend on the reverse
// walk of the blocks after it, so the two halves of the work run side by side: wavefront 0 replays block b (and
// sums the decay / bonus gradients), leaving y, 1/denominator, the current token's weight and the scaling exponent
// of its 16 tokens in LDS; wavefront 1 meanwhile walks block b+1 backwards from what wavefront 0 left the step
// before.  One workgroup barrier per block; RB LDS buffers and RB register sets of inputs (one being consumed,
// the others in flight) used in turn.
constexpr int RB = 4;
struct V4Replay { float ys[CK][64], iden[CK][64], ec[CK][64], neg_m[CK][64]; };

template <class T>
__global__ __launch_bounds__(128) void v4_backward(int BC, int Tlen, int C, const float *__restrict__ time_decay,
        const float *__restrict__ time_first, const T *__restrict__ k, const T *__restrict__ v,
        const T *__restrict__ gy, const float *__restrict__ gs_out, const float *__restrict__ ckpt,
        float *__restrict__ gw_part, float *__restrict__ gu_part, T *__restrict__ gk, T *__restrict__ gv,
        float *__restrict__ gs_in)
{
    __shared__ V4Replay sh[RB];
    const int lane = threadIdx.x & 63, role = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int idx = blockIdx.x * 64 + lane;
    if (idx >= BC) return;          // (the same lanes leave in both wavefronts; the barriers count wavefronts)
    const int b = idx / C, c = idx % C;
    const float w = -__expf(time_decay[c]), u = time_first[c];
    const size_t base = (size_t)b * Tlen * C + c;
    const int nblk = (Tlen + CK - 1) / CK;

    // RB blocks of k, v, gy per lane: one being consumed, the others in flight
    T bk[RB][CK], bv[RB][CK], bg[RB][CK];        // (as they came; converted where they are used)
    auto fetch = [&](int blk, T (&kk)[CK], T (&vv)[CK], T (&gg)[CK]) {
        const int t0 = blk * CK;
        const size_t o0 = base + (size_t)t0 * C;
        const T *kp = k + o0, *vp = v + o0, *gp_ = gy + o0;
        if (t0 + CK <= Tlen) {          // whole block inside the sequence: no per-token checks
#pragma unroll
            for (int i = 0; i < CK; i++, kp += C, vp += C, gp_ += C) { kk[i] = *kp; vv[i] = *vp; gg[i] = *gp_; }
        } else {
#pragma unroll
            for (int i = 0; i < CK; i++, kp += C, vp += C, gp_ += C) {
                const bool in = t0 + i < Tlen;
                kk[i] = in ? *kp : T{};
                vv[i] = in ? *vp : T{};
                gg[i] = in ? *gp_ : T{};
            }
        }
    };
    auto load_ckpt = [&](int blk) {
        const float *cp = ckpt + (size_t)blk * 5 * BC + idx;
        return Chain{cp[0], cp[BC], cp[2 * (size_t)BC], cp[3 * (size_t)BC], cp[4 * (size_t)BC]};
    };

    if (role == 0) {
        // ---------------- replay: step j handles block nblk-1-j, register set and LDS buffer j % RB
        float acc_w = 0.f, acc_u = 0.f;
        Chain bs[RB];
#pragma unroll
        for (int d = 0; d < RB; d++)
            if (nblk - 1 - d >= 0) { fetch(nblk - 1 - d, bk[d], bv[d], bg[d]); bs[d] = load_ckpt(nblk - 1 - d); }
        auto replay = [&](auto full_tag, int blk, T (&kk)[CK], T (&vv)[CK], T (&gg)[CK], Chain s, V4Replay &out) {
            constexpr bool FULL = decltype(full_tag)::value;
            const int cnt = FULL ? CK : Tlen - blk * CK;
#pragma unroll
            for (int i = 0; i < CK; i++) {
                if (FULL || i < cnt) {
                    const float dp0 = s.dp, dq0 = s.dq;
                    float hw, iden, ec, nm;
                    const float ki = to_float(kk[i]), vi = to_float(vv[i]), gi = to_float(gg[i]);
                    const float yy = v4_step(s, w, u, ki, vi, iden, ec, hw, nm);
                    acc_w += gi * (dp0 - dq0 * yy) * iden * hw;
                    acc_u += gi * (vi - yy) * ec * iden;
                    out.ys[i][lane] = yy; out.iden[i][lane] = iden; out.ec[i][lane] = ec; out.neg_m[i][lane] = nm;
                }
            }
            if (blk == nblk - 1 && gs_out) {       // gradient arriving through the state handed out
                const float gp = gs_out[idx * 3], gq = gs_out[idx * 3 + 1];
                const float go = (gp == 0.f && gq == 0.f) ? NEG_HUGE : gs_out[idx * 3 + 2];
                acc_w += (gp * s.dp + gq * s.dq) * __expf(s.o + go);
            }
        };
        auto step = [&](int j, T (&kk)[CK], T (&vv)[CK], T (&gg)[CK], Chain &cs, V4Replay &out) {
            const int blk = nblk - 1 - j;
            if (blk >= 0) {
                if ((blk + 1) * CK <= Tlen) replay(std::true_type{}, blk, kk, vv, gg, cs, out);
                else replay(std::false_type{}, blk, kk, vv, gg, cs, out);
                if (blk - RB >= 0) { fetch(blk - RB, kk, vv, gg); cs = load_ckpt(blk - RB); }
            }
            lds_barrier();
        };
        for (int j = 0; j <= nblk; j += RB) {
#pragma unroll
            for (int d = 0; d < RB; d++)
                if (j + d <= nblk) step(j + d, bk[d], bv[d], bg[d], bs[d], sh[d]);
        }
        gw_part[idx] = acc_w * w;
        gu_part[idx] = acc_u;
    } else {
        // ---------------- reverse walk: step j handles block nblk-j (none at j = 0), register set and buffer (j-1) % RB
        float gp = 0.f, gq = 0.f, go = NEG_HUGE;
        if (gs_out) {
            gp = gs_out[idx * 3]; gq = gs_out[idx * 3 + 1]; go = gs_out[idx * 3 + 2];
            if (gp == 0.f && gq == 0.f) go = NEG_HUGE;
        }
#pragma unroll
        for (int d = 0; d < RB; d++)
            if (nblk - 1 - d >= 0) fetch(nblk - 1 - d, bk[d], bv[d], bg[d]);
        auto walk = [&](auto full_tag, int blk, T (&kk)[CK], T (&vv)[CK], T (&gg)[CK], const V4Replay &in) {
            constexpr bool FULL = decltype(full_tag)::value;
            const int t0 = blk * CK, cnt = FULL ? CK : Tlen - t0;
            const size_t oe = base + (size_t)(t0 + CK - 1) * C;
            T *gkp = gk + oe, *gvp = gv + oe;
#pragma unroll
            for (int i = CK - 1; i >= 0; i--, gkp -= C, gvp -= C) {
                if (FULL || i < cnt) {
                    const float ys = in.ys[i][lane], iden = in.iden[i][lane], ec = in.ec[i][lane], nm = in.neg_m[i][lane];
                    const float ki = to_float(kk[i]), vi = to_float(vv[i]), gi = to_float(gg[i]);
                    const float direct = gi * iden * ec;
                    const float later = __expf(ki + go);
                    stream1(gkp, from_float<T>(direct * (vi - ys) + later * (gp * vi + gq)));
                    stream1(gvp, from_float<T>(direct + later * gp));
                    const float wg = w + go;
                    const ExpPair e = exp_pair(wg, nm);      // gy_t / den_t carries the exponent -m_t
                    const float add = gi * iden * e.second;
                    gp = fmaf(e.first, gp, add);
                    gq = fmaf(e.first, gq, -add * ys);
                    go = e.first_is_max ? wg : nm;
                }
            }
        };
        auto step = [&](int j, T (&kk)[CK], T (&vv)[CK], T (&gg)[CK], const V4Replay &in) {
            const int blk = nblk - j;
            if (j >= 1) {
                if ((blk + 1) * CK <= Tlen) walk(std::true_type{}, blk, kk, vv, gg, in);
                else walk(std::false_type{}, blk, kk, vv, gg, in);
                if (blk - RB >= 0) fetch(blk - RB, kk, vv, gg);
            }
            lds_barrier();
        };
        for (int j = 0; j <= nblk; j += RB) {
#pragma unroll
            for (int d = 0; d < RB; d++) {
                constexpr int dummy = 0; (void)dummy;
                const int e = (d + RB - 1) % RB;
                if (j + d <= nblk) step(j + d, bk[e], bv[e], bg[e], sh[e]);
            }
        }
        if (gs_in) { gs_in[idx * 3] = gp; gs_in[idx * 3 + 1] = gq; gs_in[idx * 3 + 2] = go; }
    }
}

size_t v4_checkpoint_bytes(int B, int Tlen, int C) {
    return (size_t)((Tlen + CK - 1) / CK) * 5 * (size_t)B * C * sizeof(float);
}
size_t v4_backward_workspace(int B, int Tlen, int C) {       // gw, gu partials + room for checkpoints
    return 2 * (size_t)B * C * sizeof(float) + v4_checkpoint_bytes(B, Tlen, C);
}

// whether the 16-byte fetches apply: a piece of 16 / sizeof(T) chains must not straddle two batch rows, and the
// tensors must be 16-byte aligned
template <class T> static bool v4_wide(int C, std::initializer_list<const void *> tensors) {
    if (C % (16 / (int)sizeof(T)) != 0) return false;
    for (const void *p : tensors)
        if (p && (reinterpret_cast<uintptr_t>(p) & 15u) != 0) return false;
    return true;
}

template <class T> constexpr size_t v4_forward_lds() { return (size_t)V4_GROUPS * 2 * V4_YW * 2 * CK * 64 * sizeof(T); }

template <class T>
static hipError_t fwd(hipStream_t s, int B, int Tlen, int C, const float *td, const float *tf, const void *k,
                      const void *v, const float *s_in, void *y, float *s_out, float *ckpt) {
    const int BC = B * C;
    static PerDevice lds_limit;
    const hipError_t lds_ok = lds_limit.once([] {           // (more than the 64 KB a kernel gets by default, for fp32)
        hipError_t e = hipFuncSetAttribute((const void *)v4_forward<T, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)v4_forward_lds<T>());
        if (e == hipSuccess) e = hipFuncSetAttribute((const void *)v4_forward<T, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)v4_forward_lds<T>());
        return e;
    });
    if (lds_ok != hipSuccess) return lds_ok;
    prof_begin(KID_V4_FORWARD, s);
    const dim3 grid(((BC + 63) / 64 + V4_GROUPS - 1) / V4_GROUPS), block(64 * (1 + V4_YW) * V4_GROUPS);
    if (v4_wide<T>(C, {k, v, y}))
        hipLaunchKernelGGL((v4_forward<T, true>), grid, block, v4_forward_lds<T>(), s, BC, Tlen, C, td, tf, (const T *)k,
                           (const T *)v, s_in, (T *)y, s_out, ckpt);
    else
        hipLaunchKernelGGL((v4_forward<T, false>), grid, block, v4_forward_lds<T>(), s, BC, Tlen, C, td, tf, (const T *)k,
                           (const T *)v, s_in, (T *)y, s_out, ckpt);
    prof_end(KID_V4_FORWARD, s);
    return hipGetLastError();
}

template <class T>
static hipError_t bwd(hipStream_t s, int B, int Tlen, int C, const float *td, const float *tf, const void *k,
                      const void *v, const float *s_in, const void *gy, const float *gs_out, float *gtd, float *gtf,
                      void *gk, void *gv, float *gs_in, const float *ckpt, float *ws) {
    const int BC = B * C;
    float *gw_part = ws, *gu_part = ws + BC, *own_ckpt = ws + 2 * (size_t)BC;
    if (!ckpt) {           // no checkpoints from the forward call: make them now
        hipError_t e = fwd<T>(s, B, Tlen, C, td, tf, k, v, s_in, nullptr, nullptr, own_ckpt);
        if (e != hipSuccess) return e;
        ckpt = own_ckpt;
    }
    prof_begin(KID_V4_BACKWARD, s);
    hipLaunchKernelGGL((v4_backward<T>), dim3((BC + 63) / 64), dim3(128), 0, s, BC, Tlen, C, td, tf, (const T *)k,
                       (const T *)v, (const T *)gy, gs_out, ckpt, gw_part, gu_part, (T *)gk, (T *)gv, gs_in);
    prof_end(KID_V4_BACKWARD, s);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(sum_over_batch, dim3((C + 255) / 256), dim3(256), 0, s, B, C, gw_part, gtd);
    hipLaunchKernelGGL(sum_over_batch, dim3((C + 255) / 256), dim3(256), 0, s, B, C, gu_part, gtf);
    return hipGetLastError();
}

hipError_t v4_forward_dispatch(hipStream_t s, int dtype, int B, int Tlen, int C, const float *td, const float *tf,
                               const void *k, const void *v, const float *s_in, void *y, float *s_out, float *ckpt) {
    switch (dtype) {
        case 0: return fwd<float>(s, B, Tlen, C, td, tf, k, v, s_in, y, s_out, ckpt);
        case 1: return fwd<bf16>(s, B, Tlen, C, td, tf, k, v, s_in, y, s_out, ckpt);
        default: return fwd<f16>(s, B, Tlen, C, td, tf, k, v, s_in, y, s_out, ckpt);
    }
}

hipError_t v4_backward_dispatch(hipStream_t s, int dtype, int B, int Tlen, int C, const float *td, const float *tf,
                                const void *k, const void *v, const float *s_in, const void *gy, const float *gs_out,
                                float *gtd, float *gtf, void *gk, void *gv, float *gs_in, const float *ckpt, float *ws) {
    switch (dtype) {
        case 0: return bwd<float>(s, B, Tlen, C, td, tf, k, v, s_in, gy, gs_out, gtd, gtf, gk, gv, gs_in, ckpt, ws);
        case 1: return bwd<bf16>(s, B, Tlen, C, td, tf, k, v, s_in, gy, gs_out, gtd, gtf, gk, gv, gs_in, ckpt, ws);
        default: return bwd<f16>(s, B, Tlen, C, td, tf, k, v, s_in, gy, gs_out, gtd, gtf, gk, gv, gs_in, ckpt, ws);
    }
}

}  // namespace wkv
