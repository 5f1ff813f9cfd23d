// Cumulative-decay helper: from the raw decay parameter to the log-space
// tables of the chunked formulation (RWKV-v5/src/module/rwkv_inner.py:43-58,
// 72-79), in one fused pass.  log w = max(-exp(raw), ln 0.005) needs no log().
// One lane per (batch, chunk, channel); consecutive lanes are consecutive
// channels, so every row of every table is read and written coalesced.
#include "common.h"

namespace wkv {

__global__ __launch_bounds__(256) void cumsum_decay_kernel(int Bw, int Tlen, int C, int chunk, int per_token,
        const float *__restrict__ w, float *__restrict__ log_w, float *__restrict__ incl,
        float *__restrict__ inter, float *__restrict__ intra, float *__restrict__ chunk_sum)
{
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int n = blockIdx.y, b = blockIdx.z, nchunk = Tlen / chunk;
    const size_t row0 = ((size_t)b * Tlen + (size_t)n * chunk) * C + c;
    const float fixed = per_token ? 0.f : log_decay(w[c], true);

    float total = 0.f;
    if (per_token) {
        for (int t = 0; t < chunk; t++) total += log_decay(w[row0 + (size_t)t * C], true);
    } else {
        for (int t = 0; t < chunk; t++) total += fixed;
    }
    if (chunk_sum) chunk_sum[((size_t)b * nchunk + n) * C + c] = total;

    float run = 0.f;
    for (int t = 0; t < chunk; t++) {
        const size_t o = row0 + (size_t)t * C;
        const float l = per_token ? log_decay(w[o], true) : fixed;
        run += l;
        if (log_w) log_w[o] = l;
        if (incl) incl[o] = run;
        if (inter) inter[o] = total - run;
        if (intra) intra[o] = run - l;
    }
}

// The same for a chunk length known at compile time: the chunk's log decays stay in registers, so w is read once
// (CH independent loads per lane in flight) instead of once for the chunk total and once more for the tables.
template <int CH>
__global__ __launch_bounds__(256) void cumsum_decay_chunk(int Bw, int Tlen, int C, int per_token,
        const float *__restrict__ w, float *__restrict__ log_w, float *__restrict__ incl,
        float *__restrict__ inter, float *__restrict__ intra, float *__restrict__ chunk_sum)
{
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int n = blockIdx.y, b = blockIdx.z, nchunk = Tlen / CH;
    const size_t row0 = ((size_t)b * Tlen + (size_t)n * CH) * C + c;
    const float fixed = per_token ? 0.f : log_decay(w[c], true);
    float l[CH];
    if (per_token) {
#pragma unroll
        for (int t = 0; t < CH; t++) l[t] = w[row0 + (size_t)t * C];
    }
    float total = 0.f;
#pragma unroll
    for (int t = 0; t < CH; t++) {
        l[t] = per_token ? log_decay(l[t], true) : fixed;
        total += l[t];
    }
    if (chunk_sum) chunk_sum[((size_t)b * nchunk + n) * C + c] = total;
    float run = 0.f;
#pragma unroll
    for (int t = 0; t < CH; t++) {
        const size_t o = row0 + (size_t)t * C;
        run += l[t];
        if (log_w) log_w[o] = l[t];
        if (incl) incl[o] = run;
        if (inter) inter[o] = total - run;
        if (intra) intra[o] = run - l[t];
    }
}

// All outputs of the helper, including the exponentiated tables (rwkv_inner.py:80-82) and the two factors of the
// intra-chunk product re-centred on the chunk's middle token (:91-93), which the reference forms in fp64
// (precision = 64: their exponents reach +-64 * 5.3) or fp32 (precision = 32, for chunk lengths up to 32).
template <class P>
__global__ __launch_bounds__(256) void cumsum_decay_factors(int Bw, int Tlen, int C, int chunk, int per_token,
        const float *__restrict__ w, float *__restrict__ log_w, float *__restrict__ incl, float *__restrict__ inter,
        float *__restrict__ intra, float *__restrict__ chunk_sum, float *__restrict__ ws_exp, float *__restrict__ inter_exp,
        float *__restrict__ intra_exp, P *__restrict__ r_decay, P *__restrict__ k_inv_decay)
{
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int n = blockIdx.y, b = blockIdx.z, nchunk = Tlen / chunk;
    const size_t row0 = ((size_t)b * Tlen + (size_t)n * chunk) * C + c;
    const float fixed = per_token ? 0.f : log_decay(w[c], true);
    float total = 0.f, mid = 0.f;              // mid = exclusive running sum at token chunk/2
    for (int t = 0; t < chunk; t++) {
        if (t == chunk / 2) mid = total;
        total += per_token ? log_decay(w[row0 + (size_t)t * C], true) : fixed;
    }
    if (chunk_sum) chunk_sum[((size_t)b * nchunk + n) * C + c] = total;
    if (ws_exp) ws_exp[((size_t)b * nchunk + n) * C + c] = expf(total);
    float run = 0.f;
    for (int t = 0; t < chunk; t++) {
        const size_t o = row0 + (size_t)t * C;
        const float l = per_token ? log_decay(w[o], true) : fixed;
        const float excl = run;
        run += l;
        if (log_w) log_w[o] = l;
        if (incl) incl[o] = run;
        if (inter) inter[o] = total - run;
        if (intra) intra[o] = run - l;                       // as the reference forms it (:79), not the shifted sum
        if (inter_exp) inter_exp[o] = expf(total - run);
        if (intra_exp) intra_exp[o] = expf(run - l);
        if (r_decay) r_decay[o] = exp((P)(excl - mid));
        if (k_inv_decay) k_inv_decay[o] = exp((P)(mid - run));
    }
}

hipError_t cumsum_decay_factors_launch(hipStream_t s, int Bw, int Tlen, int C, int chunk, int per_token, int precision,
                                       const float *w, float *log_w, float *incl, float *inter, float *intra, float *chunk_sum,
                                       float *ws_exp, float *inter_exp, float *intra_exp, void *r_decay, void *k_inv_decay) {
    dim3 grid((C + 255) / 256, Tlen / chunk, Bw);
    if (precision == 64)
        hipLaunchKernelGGL(cumsum_decay_factors<double>, grid, dim3(256), 0, s, Bw, Tlen, C, chunk, per_token, w, log_w, incl,
                           inter, intra, chunk_sum, ws_exp, inter_exp, intra_exp, (double *)r_decay, (double *)k_inv_decay);
    else
        hipLaunchKernelGGL(cumsum_decay_factors<float>, grid, dim3(256), 0, s, Bw, Tlen, C, chunk, per_token, w, log_w, incl,
                           inter, intra, chunk_sum, ws_exp, inter_exp, intra_exp, (float *)r_decay, (float *)k_inv_decay);
    return hipGetLastError();
}

hipError_t cumsum_decay_launch(hipStream_t s, int Bw, int Tlen, int C, int chunk, int per_token, const float *w,
                               float *log_w, float *incl, float *inter, float *intra, float *chunk_sum) {
    dim3 grid((C + 255) / 256, Tlen / chunk, Bw);
    if (chunk == 128) {         // the reference's chunk_len (RWKV-v5/src/module/rwkv_inner.py:12)
        hipLaunchKernelGGL(cumsum_decay_chunk<128>, grid, dim3(256), 0, s, Bw, Tlen, C, per_token, w, log_w, incl, inter, intra,
                           chunk_sum);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(cumsum_decay_kernel, grid, dim3(256), 0, s, Bw, Tlen, C, chunk, per_token, w, log_w, incl, inter,
                       intra, chunk_sum);
    return hipGetLastError();
}

}  // namespace wkv
