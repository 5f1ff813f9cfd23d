/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the RWKV-v4 WKV recurrence with
 * its (aa, bb, pp) state.  Not linked into, loaded by or shipped with the
 * operator library.
 *
 * Restates, in plain C over explicit (batch, channel, time) loops, the
 * algorithm of the reference's only v4 implementation:
 *   forward   RWKV-v4neo/cuda/wkv_cuda_bf16.cu:7-53
 *   backward  RWKV-v4neo/cuda/wkv_cuda_bf16.cu:55-158
 * with the argument conventions of RWKV-v4neo/cuda/wkv_op_bf16.cpp:34 (the
 * kernels receive w = -exp(time_decay)), :58-60 and :85 (gw, gu are returned
 * per batch entry and summed by the caller).
 *
 * The state of a channel is (p, q, o): p and q are the decayed sums
 * sum e^{k_s} v_s and sum e^{k_s} divided by e^{o}; o is a running maximum
 * exponent that keeps them in range.  The gradient of a state travels in the
 * same form, (gp, gq, go) meaning dL/dP = gp e^{go}, dL/dQ = gq e^{go} for the
 * undivided sums P = p e^{o}, Q = q e^{o}.
 *
 * Built twice by oracle/Makefile, with REAL=float (suffix _f32) and
 * REAL=double (suffix _f64).
 *
 * Pinned by tests/test_oracle_wkv4.py: softmax closed form (torch.softmax over
 * explicit logits), empty-history and time_first -> -inf special cases,
 * autograd through an undivided fp64 statement for every gradient including
 * the state gradient, and segment chaining.
 */
#include <math.h>
#include <stdlib.h>

#ifndef REAL
#define REAL float
#define SUFFIX f32
#endif
#define CAT_(a, b) a##_##b
#define CAT(a, b) CAT_(a, b)
#define NAME(x) CAT(x, SUFFIX)

#define NEG_HUGE ((REAL)-1e38)

static inline REAL rmax(REAL a, REAL b) { return a > b ? a : b; }
static inline REAL rexp(REAL x) { return (REAL)exp((double)x); }

/* one forward step; returns y_t and advances (p,q,o); optionally reports the
 * pieces the backward pass re-uses */
static inline REAL step(REAL w, REAL u, REAL kk, REAL vv, REAL *p, REAL *q, REAL *o,
                        REAL *inv_den, REAL *cur_exp, REAL *hist_w)
{
    REAL m = rmax(*o, u + kk);
    REAL eh = rexp(*o - m);          /* weight of the history      */
    REAL ec = rexp(u + kk - m);      /* weight of the current token */
    REAL iden = (REAL)1 / (eh * *q + ec);
    REAL y = (eh * *p + ec * vv) * iden;
    if (inv_den) { *inv_den = iden; *cur_exp = u + kk - m; *hist_w = eh; }

    REAL m2 = rmax(w + *o, kk);
    REAL dh = rexp(w + *o - m2);
    REAL dc = rexp(kk - m2);
    *p = dh * *p + dc * vv;
    *q = dh * *q + dc;
    *o = m2;
    return y;
}

/* w: (C) already -exp(time_decay); u: (C); k,v,y: (B,T,C); states: (B,C,3) or NULL */
void NAME(wkv4_forward)(int B, int T, int C, const REAL *w, const REAL *u, const REAL *k, const REAL *v,
                        const REAL *last_state, REAL *y, REAL *new_state)
{
#pragma omp parallel for collapse(2)
    for (int b = 0; b < B; b++)
        for (int c = 0; c < C; c++) {
            const size_t so = ((size_t)b * C + c) * 3;
            REAL p = 0, q = 0, o = NEG_HUGE;
            if (last_state) { p = last_state[so]; q = last_state[so + 1]; o = last_state[so + 2]; }
            for (int t = 0; t < T; t++) {
                const size_t x = ((size_t)b * T + t) * C + c;
                y[x] = step(w[c], u[c], k[x], v[x], &p, &q, &o, 0, 0, 0);
            }
            if (new_state) { new_state[so] = p; new_state[so + 1] = q; new_state[so + 2] = o; }
        }
}

/* gw, gu: (B,C) per batch entry (gw already multiplied by w, i.e. w.r.t. time_decay) */
void NAME(wkv4_backward)(int B, int T, int C, const REAL *w, const REAL *u, const REAL *k, const REAL *v,
                         const REAL *last_state, const REAL *gy, const REAL *gnew_state,
                         REAL *gw, REAL *gu, REAL *gk, REAL *gv, REAL *glast_state)
{
#pragma omp parallel for collapse(2)
    for (int b = 0; b < B; b++)
        for (int c = 0; c < C; c++) {
            const size_t so = ((size_t)b * C + c) * 3;
            REAL *ys = (REAL *)malloc(sizeof(REAL) * 3 * (size_t)T);
            REAL *iden = ys + T, *cexp = ys + 2 * (size_t)T;
            const REAL wc = w[c], uc = u[c];
            REAL p = 0, q = 0, o = NEG_HUGE;
            if (last_state) { p = last_state[so]; q = last_state[so + 1]; o = last_state[so + 2]; }

            /* forward replay; dp, dq carry d(p,q)/dw in the scale of (p,q) */
            REAL acc_w = 0, acc_u = 0, dp = 0, dq = 0;
            for (int t = 0; t < T; t++) {
                const size_t x = ((size_t)b * T + t) * C + c;
                REAL p0 = p, q0 = q, o0 = o, eh = 0;
                ys[t] = step(wc, uc, k[x], v[x], &p, &q, &o, &iden[t], &cexp[t], &eh);
                acc_w += gy[x] * (dp - dq * ys[t]) * iden[t] * eh;
                acc_u += gy[x] * (v[x] - ys[t]) * rexp(cexp[t]) * iden[t];
                REAL dh = rexp(wc + o0 - o);
                dp = dh * (p0 + dp);
                dq = dh * (q0 + dq);
            }

            /* gradient arriving through the state handed out */
            REAL gp = 0, gq = 0, go = NEG_HUGE;
            if (gnew_state) {
                gp = gnew_state[so]; gq = gnew_state[so + 1]; go = gnew_state[so + 2];
                if (gp == 0 && gq == 0) go = NEG_HUGE;
                acc_w += (gp * dp + gq * dq) * rexp(o + go);
            }

            for (int t = T - 1; t >= 0; t--) {
                const size_t x = ((size_t)b * T + t) * C + c;
                REAL direct = gy[x] * iden[t] * rexp(cexp[t]);   /* through y_t's own term */
                REAL later = rexp(k[x] + go);                    /* through later tokens / state */
                gk[x] = direct * (v[x] - ys[t]) + later * (gp * v[x] + gq);
                gv[x] = direct + later * gp;

                REAL hist = cexp[t] - k[x] - uc;                 /* exponent of 1/den w.r.t. P,Q */
                REAL m = rmax(wc + go, hist);
                REAL keep = rexp(wc + go - m);
                REAL add = gy[x] * iden[t] * rexp(hist - m);
                gp = keep * gp + add;
                gq = keep * gq - add * ys[t];
                go = m;
            }
            if (glast_state) { glast_state[so] = gp; glast_state[so + 1] = gq; glast_state[so + 2] = go; }
            gw[(size_t)b * C + c] = acc_w * wc;
            gu[(size_t)b * C + c] = acc_u;
            free(ys);
        }
}
