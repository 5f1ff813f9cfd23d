// C ABI of the library: argument checks and dispatch.  This is the one
// translation unit hipcc builds; the kernel files are included so that every
// kernel and its launcher sit in the same code object.
#include "../../include/rwkv_wkv_hip.h"
#include "common.h"
#include "wkv56_recurrent.hip"
#include "wkv56_chunked.hip"
#include "wkv56_noalloc.hip"
#include "wkv4.hip"
#include "cumsum_decay.hip"
#include "block_edges.hip"
#include "lora_mix.hip"

using namespace wkv;

namespace {

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int check_dims56(int B, int T, int C, int H, int dtype) {
    if (B <= 0 || T <= 0 || C <= 0 || H <= 0) return WKV_ERR_DIMS;
    if (C != H * HEAD) return WKV_ERR_DIMS;
    if ((long long)B * T * C >= (1ll << 40)) return WKV_ERR_DIMS;
    if ((long long)T * C >= (1ll << 30)) return WKV_ERR_DIMS;      // the kernels address a sequence with 32-bit byte offsets
    if (dtype < WKV_F32 || dtype > WKV_F16) return WKV_ERR_DTYPE;
    return WKV_OK;
}

// the blocked matrix-core path takes bf16 streams with the decay floor switched on
// (whose range analysis relies on the decay floor); everything else goes token by token
int pick_algo56(int algo, int T, int dtype, unsigned flags) {
    (void)T;
    const bool can_chunk = dtype == WKV_BF16 && (flags & WKV_FLOOR_DECAY);
    if (algo == WKV_ALGO_AUTO) return can_chunk ? WKV_ALGO_CHUNKED : WKV_ALGO_RECURRENT;
    if (algo == WKV_ALGO_RECURRENT) return algo;
    if (algo == WKV_ALGO_CHUNKED) return can_chunk ? algo : WKV_ERR_ALGO;
    return WKV_ERR_ALGO;
}

// state_out == state_in (the state updated in place, as a serving loop does) is fine whenever every workgroup reads
// the state of its (batch, head) pair before it writes it: the per-token kernels, and the blocked ones as long as
// no sequence is cut into time segments (then the workgroups of the later segments read state_in while the one of
// the last segment writes state_out).  Buffers that overlap without being the same never are.
static int check_state_alias(const float *state_in, const float *state_out, int B, int H, bool time_split) {
    const uintptr_t a0 = reinterpret_cast<uintptr_t>(state_in), b0 = reinterpret_cast<uintptr_t>(state_out);
    const size_t bytes = (size_t)B * H * HEAD * HEAD * sizeof(float);
    if (!(a0 < b0 + bytes && b0 < a0 + bytes)) return WKV_OK;
    return (a0 == b0 && !time_split) ? WKV_OK : WKV_ERR_ALIAS;
}

int forward56(bool per_token, void *stream, int B, int T, int C, int H, int dtype, unsigned flags, int algo,
              const void *r, const void *k, const void *v, const void *w, const float *u, const float *state_in,
              void *y, float *state_out, void *workspace, size_t workspace_bytes) {
    int st = check_dims56(B, T, C, H, dtype);
    if (st) return st;
    if (!r || !k || !v || !w || !u || !state_in || !y || !state_out) return WKV_ERR_NULL;
    for (const void *p : {r, k, v, (const void *)w, (const void *)u, (const void *)state_in, (const void *)y,
                          (const void *)state_out})
        if (!aligned16(p)) return WKV_ERR_ALIGN;
    const int a = pick_algo56(algo, T, dtype, flags);
    if (a < 0) return a;
    st = check_state_alias(state_in, state_out, B, H, a == WKV_ALGO_CHUNKED && chunked::splits_time(B * H, T));
    if (st) return st;
    const bool w16 = (flags & WKV_W_BF16) != 0;
    if (w16 && (!per_token || a != WKV_ALGO_CHUNKED)) return WKV_ERR_ALGO;
    if (a == WKV_ALGO_CHUNKED) {
        // with a workspace the state at the start of every 64-token step is left there for backward
        if (workspace) {
            if (!aligned16(workspace)) return WKV_ERR_ALIGN;
            if (workspace_bytes < chunked::forward_workspace(B, T, H)) return WKV_ERR_WORKSPACE;
        }
        hipError_t e = chunked::forward_launch((hipStream_t)stream, per_token, w16, B, T, C, H, r, k, v, w, u, state_in, y,
                                               state_out, workspace, (flags & WKV_FLOOR_DECAY) ? 1 : 0);
        return e == hipSuccess ? WKV_OK : WKV_ERR_LAUNCH;
    }
    hipError_t e = recurrent_forward((hipStream_t)stream, dtype, per_token, B, T, C, H, r, k, v, (const float *)w, u, state_in, y,
                                     state_out, (flags & WKV_FLOOR_DECAY) ? 1 : 0);
    return e == hipSuccess ? WKV_OK : WKV_ERR_LAUNCH;
}

// (sizes are for the larger of the two algorithms a call with these arguments can take)
size_t forward56_workspace(int B, int T, int C, int H, int dtype, int algo) {
    if (check_dims56(B, T, C, H, dtype)) return 0;
    return pick_algo56(algo, T, dtype, WKV_FLOOR_DECAY) == WKV_ALGO_CHUNKED ? chunked::forward_workspace(B, T, H) : 0;
}

size_t backward56_workspace(int B, int T, int C, int H, int dtype, int algo) {
    if (check_dims56(B, T, C, H, dtype)) return 0;
    const size_t rec = recurrent_backward_workspace(B, T, C);
    if (pick_algo56(algo, T, dtype, WKV_FLOOR_DECAY) == WKV_ALGO_CHUNKED)
        return std::max(rec, chunked::backward_workspace(B, T, C, H));
    return rec;
}

int backward56(bool per_token, void *stream, int B, int T, int C, int H, int dtype, unsigned flags, int algo,
               const void *r, const void *k, const void *v, const void *w, const float *u, const float *state_in,
               const void *gy, const float *gstate_out, void *gr, void *gk, void *gv, void *gw, float *gu,
               float *gstate_in, void *workspace, size_t workspace_bytes) {
    int st = check_dims56(B, T, C, H, dtype);
    if (st) return st;
    if (!r || !k || !v || !w || !u || !state_in || !gy || !gr || !gk || !gv || !gw || !gu) return WKV_ERR_NULL;
    for (const void *p : {r, k, v, (const void *)w, (const void *)u, (const void *)state_in, gy,
                          (const void *)gstate_out, (const void *)gr, (const void *)gk, (const void *)gv,
                          (const void *)gw, (const void *)gu, (const void *)gstate_in, (const void *)workspace})
        if (!aligned16(p)) return WKV_ERR_ALIGN;
    const int a = pick_algo56(algo, T, dtype, flags);
    if (a < 0) return a;
    const bool w16 = (flags & WKV_W_BF16) != 0;
    if (w16 && (!per_token || a != WKV_ALGO_CHUNKED)) return WKV_ERR_ALGO;
    if (!workspace) return WKV_ERR_NULL;
    if (workspace_bytes < (a == WKV_ALGO_CHUNKED ? chunked::backward_workspace(B, T, C, H)
                                                 : recurrent_backward_workspace(B, T, C)))
        return WKV_ERR_WORKSPACE;
    if (gstate_in && gstate_out) {      // several workgroups share a head's state gradient: some read gstate_out after
                                        // others have written gstate_in, so the two are never the same memory
        const uintptr_t a0 = reinterpret_cast<uintptr_t>(gstate_in), b0 = reinterpret_cast<uintptr_t>(gstate_out);
        const size_t bytes = (size_t)B * H * HEAD * HEAD * sizeof(float);
        if (a0 < b0 + bytes && b0 < a0 + bytes) return WKV_ERR_ALIAS;
    }
    if (a == WKV_ALGO_CHUNKED) {
        hipError_t e = chunked::backward_launch((hipStream_t)stream, per_token, w16, B, T, C, H, r, k, v, w, u, state_in, gy,
                                                gstate_out, gr, gk, gv, gw, gu, gstate_in, workspace,
                                                (flags & WKV_CHECKPOINTS_VALID) != 0, (flags & WKV_FLOOR_DECAY) ? 1 : 0);
        return e == hipSuccess ? WKV_OK : WKV_ERR_LAUNCH;
    }
    hipError_t e = recurrent_backward((hipStream_t)stream, dtype, per_token, B, T, C, H, r, k, v, (const float *)w, u, state_in, gy,
                                      gstate_out, gr, gk, gv, (float *)gw, gu, gstate_in, (float *)workspace,
                                      (flags & WKV_FLOOR_DECAY) ? 1 : 0);
    return e == hipSuccess ? WKV_OK : WKV_ERR_LAUNCH;
}

int check_dims4(int B, int T, int C, int dtype) {
    if (B <= 0 || T <= 0 || C <= 0) return WKV_ERR_DIMS;
    if ((long long)B * C >= (1ll << 30)) return WKV_ERR_DIMS;
    if (dtype < WKV_F32 || dtype > WKV_F16) return WKV_ERR_DTYPE;
    return WKV_OK;
}

}  // namespace

extern "C" {

const char *wkv_strerror(int status) {
    switch (status) {
        case WKV_OK: return "ok";
        case WKV_ERR_DIMS: return "bad dimensions (sizes must be positive and C == H*64)";
        case WKV_ERR_NULL: return "a required pointer is NULL";
        case WKV_ERR_DTYPE: return "unsupported dtype";
        case WKV_ERR_ALIGN: return "pointer not 16-byte aligned";
        case WKV_ERR_WORKSPACE: return "workspace too small";
        case WKV_ERR_LAUNCH: return "HIP launch failed";
        case WKV_ERR_ALGO: return "algorithm not available for this shape/dtype";
        case WKV_ERR_ALIAS: return "state_out overlaps state_in (in place is possible only where no sequence is cut into time segments), or gstate_in overlaps gstate_out (never possible)";
        default: return "unknown status";
    }
}

int wkv_abi_version(void) { return 2; }

int wkv_init(void) {
    if (chunked::init_kernels() != hipSuccess) return WKV_ERR_LAUNCH;
    return chunked::init_static_scratch() == hipSuccess ? WKV_OK : WKV_ERR_LAUNCH;      // (for the current device)
}

int wkv_tune(int key, int value) {
    if (key == WKV_TUNE_SEGMENTS) {
        if (value < 0 || value > chunked::MAX_SEG) return WKV_ERR_DIMS;
        chunked::forced_segments() = value;
        return WKV_OK;
    }
    if (key == WKV_TUNE_PIECE_STEPS) {
        if (value < 0) return WKV_ERR_DIMS;
        chunked::forced_piece_steps() = value;
        return WKV_OK;
    }
    return WKV_ERR_DIMS;
}

int wkv_profile_begin(int kernel_id, int max_launches) {
    ProfileSlot &p = profile_slot();
    for (hipEvent_t e : p.start) (void)hipEventDestroy(e);
    for (hipEvent_t e : p.stop) (void)hipEventDestroy(e);
    p.start.clear(); p.stop.clear(); p.used = 0; p.id = KID_NONE;
    if (kernel_id == KID_NONE || max_launches <= 0) return WKV_OK;
    for (int i = 0; i < max_launches; i++) {
        hipEvent_t a, b;
        if (hipEventCreate(&a) != hipSuccess || hipEventCreate(&b) != hipSuccess) return WKV_ERR_LAUNCH;
        p.start.push_back(a); p.stop.push_back(b);
    }
    p.id = kernel_id;
    return WKV_OK;
}

int wkv_profile_end(float *ms, int capacity) {
    ProfileSlot &p = profile_slot();
    int n = 0;
    for (size_t i = 0; i < p.used && (int)i < capacity; i++) {
        if (hipEventSynchronize(p.stop[i]) != hipSuccess) break;
        float t = 0.f;
        if (hipEventElapsedTime(&t, p.start[i], p.stop[i]) != hipSuccess) break;
        if (ms) ms[n] = t;
        n++;
    }
    wkv_profile_begin(KID_NONE, 0);
    return n;
}

size_t wkv6_forward_workspace(int B, int T, int C, int H, int dtype, int algo) {
    return forward56_workspace(B, T, C, H, dtype, algo);
}
size_t wkv5_forward_workspace(int B, int T, int C, int H, int dtype, int algo) {
    return forward56_workspace(B, T, C, H, dtype, algo);
}

int wkv6_forward(void *stream, int B, int T, int C, int H, int dtype, unsigned flags, int algo, const void *r,
                 const void *k, const void *v, const void *w, const float *u, const float *state_in, void *y,
                 float *state_out, void *workspace, size_t workspace_bytes) {
    return forward56(true, stream, B, T, C, H, dtype, flags, algo, r, k, v, w, u, state_in, y, state_out, workspace,
                     workspace_bytes);
}
int wkv5_forward(void *stream, int B, int T, int C, int H, int dtype, unsigned flags, int algo, const void *r,
                 const void *k, const void *v, const float *w, const float *u, const float *state_in, void *y,
                 float *state_out, void *workspace, size_t workspace_bytes) {
    return forward56(false, stream, B, T, C, H, dtype, flags, algo, r, k, v, w, u, state_in, y, state_out, workspace,
                     workspace_bytes);
}

int wkv6_forward_noalloc(void *stream, int B, int T, int C, int H, int dtype, unsigned flags, const void *r,
                         const void *k, const void *v, const void *w, const float *u, const float *state_in, void *y,
                         float *state_out) {
    int st = check_dims56(B, T, C, H, dtype);
    if (st) return st;
    if (!r || !k || !v || !w || !u || !state_in || !y || !state_out) return WKV_ERR_NULL;
    for (const void *p : {r, k, v, (const void *)w, (const void *)u, (const void *)state_in, (const void *)y,
                          (const void *)state_out})
        if (!aligned16(p)) return WKV_ERR_ALIGN;
    if (pick_algo56(WKV_ALGO_CHUNKED, T, dtype, flags) != WKV_ALGO_CHUNKED) return WKV_ERR_ALGO;
    st = check_state_alias(state_in, state_out, B, H, chunked::splits_time(B * H, T));
    if (st) return st;
    hipError_t e = chunked::forward_static_launch((hipStream_t)stream, true, (flags & WKV_W_BF16) != 0, B, T, C, H, r, k, v, w,
                                                  u, state_in, y, state_out, (flags & WKV_FLOOR_DECAY) ? 1 : 0);
    if (e == hipErrorOutOfMemory) return WKV_ERR_WORKSPACE;
    return e == hipSuccess ? WKV_OK : WKV_ERR_LAUNCH;
}

size_t wkv6_backward_workspace(int B, int T, int C, int H, int dtype, int algo) {
    return backward56_workspace(B, T, C, H, dtype, algo);
}
size_t wkv5_backward_workspace(int B, int T, int C, int H, int dtype, int algo) {
    return backward56_workspace(B, T, C, H, dtype, algo);
}

int wkv6_backward(void *stream, int B, int T, int C, int H, int dtype, unsigned flags, int algo, const void *r,
                  const void *k, const void *v, const void *w, const float *u, const float *state_in, const void *gy,
                  const float *gstate_out, void *gr, void *gk, void *gv, void *gw, float *gu, float *gstate_in,
                  void *workspace, size_t workspace_bytes) {
    return backward56(true, stream, B, T, C, H, dtype, flags, algo, r, k, v, w, u, state_in, gy, gstate_out, gr, gk, gv,
                      gw, gu, gstate_in, workspace, workspace_bytes);
}
int wkv5_backward(void *stream, int B, int T, int C, int H, int dtype, unsigned flags, int algo, const void *r,
                  const void *k, const void *v, const float *w, const float *u, const float *state_in, const void *gy,
                  const float *gstate_out, void *gr, void *gk, void *gv, float *gw, float *gu, float *gstate_in,
                  void *workspace, size_t workspace_bytes) {
    return backward56(false, stream, B, T, C, H, dtype, flags, algo, r, k, v, w, u, state_in, gy, gstate_out, gr, gk,
                      gv, gw, gu, gstate_in, workspace, workspace_bytes);
}

size_t wkv4_checkpoint_bytes(int B, int T, int C) {
    return (B > 0 && T > 0 && C > 0) ? v4_checkpoint_bytes(B, T, C) : 0;
}
size_t wkv4_backward_workspace(int B, int T, int C, int dtype) {
    return check_dims4(B, T, C, dtype) ? 0 : v4_backward_workspace(B, T, C);
}

int wkv4_forward(void *stream, int B, int T, int C, int dtype, const float *time_decay, const float *time_first,
                 const void *k, const void *v, const float *state_in, void *y, float *state_out, void *checkpoints) {
    int st = check_dims4(B, T, C, dtype);
    if (st) return st;
    if (!time_decay || !time_first || !k || !v || !y) return WKV_ERR_NULL;
    hipError_t e = v4_forward_dispatch((hipStream_t)stream, dtype, B, T, C, time_decay, time_first, k, v, state_in, y,
                                       state_out, (float *)checkpoints);
    return e == hipSuccess ? WKV_OK : WKV_ERR_LAUNCH;
}

int wkv4_backward(void *stream, int B, int T, int C, int dtype, const float *time_decay, const float *time_first,
                  const void *k, const void *v, const float *state_in, const void *gy, const float *gstate_out,
                  float *g_time_decay, float *g_time_first, void *gk, void *gv, float *gstate_in,
                  const void *checkpoints, void *workspace, size_t workspace_bytes) {
    int st = check_dims4(B, T, C, dtype);
    if (st) return st;
    if (!time_decay || !time_first || !k || !v || !gy || !g_time_decay || !g_time_first || !gk || !gv || !workspace)
        return WKV_ERR_NULL;
    if (workspace_bytes < v4_backward_workspace(B, T, C)) return WKV_ERR_WORKSPACE;
    hipError_t e = v4_backward_dispatch((hipStream_t)stream, dtype, B, T, C, time_decay, time_first, k, v, state_in, gy,
                                        gstate_out, g_time_decay, g_time_first, gk, gv, gstate_in,
                                        (const float *)checkpoints, (float *)workspace);
    return e == hipSuccess ? WKV_OK : WKV_ERR_LAUNCH;
}

int wkv_cumsum_decay(void *stream, int Bw, int T, int C, int chunk_len, int per_token, const float *w, float *log_w,
                     float *incl, float *inter, float *intra, float *chunk_sum) {
    if (Bw <= 0 || T <= 0 || C <= 0 || chunk_len <= 0 || T % chunk_len != 0) return WKV_ERR_DIMS;
    if (T / chunk_len > 65535 || Bw > 65535) return WKV_ERR_DIMS;
    if (!w) return WKV_ERR_NULL;
    hipError_t e = cumsum_decay_launch((hipStream_t)stream, Bw, T, C, chunk_len, per_token, w, log_w, incl, inter,
                                       intra, chunk_sum);
    return e == hipSuccess ? WKV_OK : WKV_ERR_LAUNCH;
}

int wkv_cumsum_decay_factors(void *stream, int Bw, int T, int C, int chunk_len, int per_token, int precision,
                             const float *w, float *log_w, float *incl, float *inter, float *intra, float *chunk_sum,
                             float *ws_exp, float *inter_exp, float *intra_exp, void *r_decay, void *k_inv_decay) {
    if (Bw <= 0 || T <= 0 || C <= 0 || chunk_len <= 0 || T % chunk_len != 0) return WKV_ERR_DIMS;
    if (T / chunk_len > 65535 || Bw > 65535) return WKV_ERR_DIMS;
    if (precision != 32 && precision != 64) return WKV_ERR_DTYPE;
    if (!w) return WKV_ERR_NULL;
    hipError_t e = cumsum_decay_factors_launch((hipStream_t)stream, Bw, T, C, chunk_len, per_token, precision, w, log_w, incl,
                                               inter, intra, chunk_sum, ws_exp, inter_exp, intra_exp, r_decay, k_inv_decay);
    return e == hipSuccess ? WKV_OK : WKV_ERR_LAUNCH;
}

// ---- the element-wise passes around the operator (block_edges.hip)
#define WKV_BY_DTYPE(dtype, CALL)                                   \
    ((dtype) == WKV_BF16 ? CALL(bf16) : (dtype) == WKV_F16 ? CALL(f16) : CALL(float))

size_t wkv_shift_mix_backward_workspace(int B, int T, int C, int n) {
    if (B <= 0 || T <= 0 || C <= 0 || n <= 0 || n > edges::MAX_MIX) return 0;
    return edges::shift_mix_backward_workspace(B, T, C, n);
}

int wkv_shift_mix_forward(void *stream, int B, int T, int C, int dtype, int n, int lerp, const void *x, const void *shift,
                          const float *coef, const void *dyn, void *const *out) {
    if (B <= 0 || T <= 0 || C <= 0 || C % 8 != 0 || B > 65535 || n <= 0 || n > edges::MAX_MIX) return WKV_ERR_DIMS;
    if ((T + edges::TILE_R - 1) / edges::TILE_R > 65535) return WKV_ERR_DIMS;          // rows of workgroups in one launch
    if (dtype < WKV_F32 || dtype > WKV_F16) return WKV_ERR_DTYPE;
    if (!x || !shift || !coef || !out) return WKV_ERR_NULL;
    for (int j = 0; j < n; j++) {
        if (!out[j]) return WKV_ERR_NULL;
        if (!aligned16(out[j])) return WKV_ERR_ALIGN;
    }
    for (const void *p : {x, shift, (const void *)coef, dyn})
        if (!aligned16(p)) return WKV_ERR_ALIGN;
#define CALL(TY) edges::shift_mix_forward_t<TY>((hipStream_t)stream, B, T, C, n, lerp, x, shift, coef, dyn, out)
    hipError_t e = WKV_BY_DTYPE(dtype, CALL);
#undef CALL
    return e == hipSuccess ? WKV_OK : WKV_ERR_LAUNCH;
}

int wkv_shift_mix_backward(void *stream, int B, int T, int C, int dtype, int n, int lerp, const void *x, const void *shift,
                           const float *coef, const void *dyn, const void *const *gout, void *gx, void *gshift, float *gcoef,
                           void *gdyn, void *workspace, size_t workspace_bytes) {
    if (B <= 0 || T <= 0 || C <= 0 || C % 8 != 0 || B > 65535 || n <= 0 || n > edges::MAX_MIX) return WKV_ERR_DIMS;
    if ((T + edges::TILE_R - 1) / edges::TILE_R > 65535) return WKV_ERR_DIMS;          // rows of workgroups in one launch
    if (dtype < WKV_F32 || dtype > WKV_F16) return WKV_ERR_DTYPE;
    if (!x || !shift || !coef || !gout || !gx || !gshift || !gcoef || !workspace || (dyn && !gdyn)) return WKV_ERR_NULL;
    for (int j = 0; j < n; j++) {
        if (!gout[j]) return WKV_ERR_NULL;
        if (!aligned16(gout[j])) return WKV_ERR_ALIGN;
    }
    for (const void *p : {x, shift, (const void *)coef, dyn, (const void *)gx, (const void *)gshift, (const void *)gcoef,
                          (const void *)gdyn, (const void *)workspace})
        if (!aligned16(p)) return WKV_ERR_ALIGN;
    if (workspace_bytes < edges::shift_mix_backward_workspace(B, T, C, n)) return WKV_ERR_WORKSPACE;
#define CALL(TY) edges::shift_mix_backward_t<TY>((hipStream_t)stream, B, T, C, n, lerp, x, shift, coef, dyn, gout, gx, gshift, \
                                                 gcoef, gdyn, (float *)workspace)
    hipError_t e = WKV_BY_DTYPE(dtype, CALL);
#undef CALL
    return e == hipSuccess ? WKV_OK : WKV_ERR_LAUNCH;
}

static int lora_mix_dims(int B, int T, int C) {
    if (B <= 0 || T <= 0 || C <= 0 || C % 8 != 0 || B > 65535) return WKV_ERR_DIMS;
    if (edges::lora_mix_tiles(T) > 65535) return WKV_ERR_DIMS;          // rows of workgroups in one launch
    return WKV_OK;
}

size_t wkv_lora_mix_backward_workspace(int B, int T, int C) {
    if (lora_mix_dims(B, T, C) != WKV_OK) return 0;
    return edges::lora_mix_backward_workspace(B, T, C);
}

int wkv_lora_mix_forward(void *stream, int B, int T, int C, const void *x, const void *shift, const float *coef,
                         const void *act, const void *w2t, void *const *out) {
    if (int e = lora_mix_dims(B, T, C)) return e;
    if (!x || !shift || !coef || !act || !w2t || !out) return WKV_ERR_NULL;
    for (int j = 0; j < edges::LM_N; j++) {
        if (!out[j]) return WKV_ERR_NULL;
        if (!aligned16(out[j])) return WKV_ERR_ALIGN;
    }
    for (const void *p : {x, shift, (const void *)coef, act, w2t})
        if (!aligned16(p)) return WKV_ERR_ALIGN;
    hipError_t e = edges::lora_mix_forward_launch((hipStream_t)stream, B, T, C, x, shift, coef, act, w2t, out);
    return e == hipSuccess ? WKV_OK : WKV_ERR_LAUNCH;
}

int wkv_lora_mix_backward(void *stream, int B, int T, int C, const void *x, const void *shift, const float *coef,
                          const void *act, const void *w2t, const void *const *gout, void *gx, void *gshift, float *gcoef,
                          void *gdyn, void *workspace, size_t workspace_bytes) {
    if (int e = lora_mix_dims(B, T, C)) return e;
    if (!x || !shift || !coef || !act || !w2t || !gout || !gx || !gshift || !gcoef || !gdyn || !workspace) return WKV_ERR_NULL;
    for (int j = 0; j < edges::LM_N; j++) {
        if (!gout[j]) return WKV_ERR_NULL;
        if (!aligned16(gout[j])) return WKV_ERR_ALIGN;
    }
    for (const void *p : {x, shift, (const void *)coef, act, w2t, (const void *)gx, (const void *)gshift, (const void *)gcoef,
                          (const void *)gdyn, (const void *)workspace})
        if (!aligned16(p)) return WKV_ERR_ALIGN;
    if (workspace_bytes < edges::lora_mix_backward_workspace(B, T, C)) return WKV_ERR_WORKSPACE;
    hipError_t e = edges::lora_mix_backward_launch((hipStream_t)stream, B, T, C, x, shift, coef, act, w2t, gout, gx, gshift, gcoef,
                                                   gdyn, (float *)workspace);
    return e == hipSuccess ? WKV_OK : WKV_ERR_LAUNCH;
}

size_t wkv_ln_gate_backward_workspace(int rows, int C) {
    if (rows <= 0 || C <= 0) return 0;
    return edges::ln_gate_backward_workspace(rows, C);
}

int wkv_ln_gate_forward(void *stream, int rows, int C, int dtype, float scale, float eps, const void *y, const void *gate,
                        const float *weight, const float *bias, void *out) {
    if (rows <= 0 || C <= 0 || C % HEAD != 0 || (rows + edges::TILE_R - 1) / edges::TILE_R > 65535) return WKV_ERR_DIMS;
    if (dtype < WKV_F32 || dtype > WKV_F16) return WKV_ERR_DTYPE;
    if (!y || !weight || !bias || !out) return WKV_ERR_NULL;
    for (const void *p : {y, gate, (const void *)weight, (const void *)bias, (const void *)out})
        if (!aligned16(p)) return WKV_ERR_ALIGN;
#define CALL(TY) edges::ln_gate_forward_t<TY>((hipStream_t)stream, rows, C, scale, eps, y, gate, weight, bias, out)
    hipError_t e = WKV_BY_DTYPE(dtype, CALL);
#undef CALL
    return e == hipSuccess ? WKV_OK : WKV_ERR_LAUNCH;
}

int wkv_ln_gate_backward(void *stream, int rows, int C, int dtype, float scale, float eps, const void *y, const void *gate,
                         const float *weight, const float *bias, const void *gout, void *gy, void *ggate,
                         float *gweight_gbias, void *workspace, size_t workspace_bytes) {
    if (rows <= 0 || C <= 0 || C % HEAD != 0 || (rows + edges::TILE_R - 1) / edges::TILE_R > 65535) return WKV_ERR_DIMS;
    if (dtype < WKV_F32 || dtype > WKV_F16) return WKV_ERR_DTYPE;
    if (!y || !weight || !bias || !gout || !gy || !gweight_gbias || !workspace || (gate && !ggate)) return WKV_ERR_NULL;
    for (const void *p : {y, gate, (const void *)weight, (const void *)bias, gout, (const void *)gy, (const void *)ggate,
                          (const void *)gweight_gbias, (const void *)workspace})
        if (!aligned16(p)) return WKV_ERR_ALIGN;
    if (workspace_bytes < edges::ln_gate_backward_workspace(rows, C)) return WKV_ERR_WORKSPACE;
#define CALL(TY) edges::ln_gate_backward_t<TY>((hipStream_t)stream, rows, C, scale, eps, y, gate, weight, bias, gout, gy, ggate, \
                                               gweight_gbias, (float *)workspace)
    hipError_t e = WKV_BY_DTYPE(dtype, CALL);
#undef CALL
    return e == hipSuccess ? WKV_OK : WKV_ERR_LAUNCH;
}

static int check_flat(size_t n, int dtype) {
    if (n == 0 || n % 8 != 0 || n / 8 / 256 >= (1u << 31)) return WKV_ERR_DIMS;
    if (dtype < WKV_F32 || dtype > WKV_F16) return WKV_ERR_DTYPE;
    return WKV_OK;
}

int wkv_relu_square_forward(void *stream, size_t n, int dtype, const void *k, void *out) {
    if (int st = check_flat(n, dtype)) return st;
    if (!k || !out) return WKV_ERR_NULL;
    if (!aligned16(k) || !aligned16(out)) return WKV_ERR_ALIGN;
#define CALL(TY) edges::relu_square_forward_t<TY>((hipStream_t)stream, n, k, out)
    hipError_t e = WKV_BY_DTYPE(dtype, CALL);
#undef CALL
    return e == hipSuccess ? WKV_OK : WKV_ERR_LAUNCH;
}

int wkv_relu_square_backward(void *stream, size_t n, int dtype, const void *k, const void *gout, void *gk) {
    if (int st = check_flat(n, dtype)) return st;
    if (!k || !gout || !gk) return WKV_ERR_NULL;
    if (!aligned16(k) || !aligned16(gout) || !aligned16(gk)) return WKV_ERR_ALIGN;
#define CALL(TY) edges::relu_square_backward_t<TY>((hipStream_t)stream, n, k, gout, gk)
    hipError_t e = WKV_BY_DTYPE(dtype, CALL);
#undef CALL
    return e == hipSuccess ? WKV_OK : WKV_ERR_LAUNCH;
}

int wkv_sigmoid_mul_forward(void *stream, size_t n, int dtype, const void *r, const void *kv, void *out) {
    if (int st = check_flat(n, dtype)) return st;
    if (!r || !kv || !out) return WKV_ERR_NULL;
    if (!aligned16(r) || !aligned16(kv) || !aligned16(out)) return WKV_ERR_ALIGN;
#define CALL(TY) edges::sigmoid_mul_forward_t<TY>((hipStream_t)stream, n, r, kv, out)
    hipError_t e = WKV_BY_DTYPE(dtype, CALL);
#undef CALL
    return e == hipSuccess ? WKV_OK : WKV_ERR_LAUNCH;
}

int wkv_sigmoid_mul_backward(void *stream, size_t n, int dtype, const void *r, const void *kv, const void *gout, void *gr,
                             void *gkv) {
    if (int st = check_flat(n, dtype)) return st;
    if (!r || !kv || !gout || !gr || !gkv) return WKV_ERR_NULL;
    for (const void *p : {r, kv, gout, (const void *)gr, (const void *)gkv})
        if (!aligned16(p)) return WKV_ERR_ALIGN;
#define CALL(TY) edges::sigmoid_mul_backward_t<TY>((hipStream_t)stream, n, r, kv, gout, gr, gkv)
    hipError_t e = WKV_BY_DTYPE(dtype, CALL);
#undef CALL
    return e == hipSuccess ? WKV_OK : WKV_ERR_LAUNCH;
}

int wkv_l2wrap_backward(void *stream, int rows, int V, int dtype, float factor, const void *y, const float *mask, void *gy) {
    if (rows <= 0 || V <= 0) return WKV_ERR_DIMS;
    if (dtype < WKV_F32 || dtype > WKV_F16) return WKV_ERR_DTYPE;
    if (!y || !gy) return WKV_ERR_NULL;
    if (!aligned16(y) || !aligned16(gy)) return WKV_ERR_ALIGN;
#define CALL(TY) edges::l2wrap_backward_t<TY>((hipStream_t)stream, rows, V, factor, y, mask, gy)
    hipError_t e = WKV_BY_DTYPE(dtype, CALL);
#undef CALL
    return e == hipSuccess ? WKV_OK : WKV_ERR_LAUNCH;
}

}  // extern "C"
