/*
 * rwkv_wkv_hip -- C ABI of the MI355X (gfx950) WKV time-mix operators.
 *
 * One shared library, plain pointers and sizes, no framework types.  Every
 * pointer is a DEVICE pointer unless stated; every call is asynchronous on the
 * HIP stream passed in (a hipStream_t cast to void*; NULL = the default
 * stream), allocates nothing and returns 0 or a negative wkv_status.
 *
 * Layouts (all contiguous, row-major):
 *   r, k, v, y, gy, gr, gk, gv   (B, T, C) in `dtype`          C = H * 64
 *   w (WKV6), gw (WKV6)          (B, T, C) fp32 (bf16 with WKV_W_BF16), RAW decay
 *                                parameter: the decay applied is exp(-exp(w))
 *   w (WKV5), gw (WKV5), u, gu   (H, 64)   fp32 (gw, gu summed over batch and time)
 *   state                        (B, H, 64, 64) fp32, [key index][value index]
 *   WKV4: time_decay, time_first (C) fp32;  state (B, C, 3) fp32 = (aa, bb, pp)
 *
 * Reference interfaces these entry points stand in for are cited per function
 * (paths relative to the RWKV-infctx-trainer tree).
 */
#ifndef RWKV_WKV_HIP_H
#define RWKV_WKV_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    WKV_OK = 0,
    WKV_ERR_DIMS = -1,        /* non-positive size, C != H*64, T*C >= 2^30 (one sequence is addressed with 32-bit
                                 byte offsets) or B*T*C >= 2^40 */
    WKV_ERR_NULL = -2,        /* a required pointer is NULL */
    WKV_ERR_DTYPE = -3,       /* dtype not one of wkv_dtype */
    WKV_ERR_ALIGN = -4,       /* a pointer is not 16-byte aligned */
    WKV_ERR_WORKSPACE = -5,   /* workspace smaller than the matching *_workspace() query */
    WKV_ERR_LAUNCH = -6,      /* HIP reported an error at launch */
    WKV_ERR_ALGO = -7,        /* algorithm not available for this shape / dtype */
    WKV_ERR_ALIAS = -8        /* state_out overlaps state_in: with a sequence cut into time segments the last
                                 segment would write the new state while the first still reads the old one */
} wkv_status;

typedef enum { WKV_F32 = 0, WKV_BF16 = 1, WKV_F16 = 2 } wkv_dtype;

/* flags */
#define WKV_FLOOR_DECAY 1u    /* bound the decay below by 0.005 as the reference's chunked
                                 training path does (RWKV-v5/src/module/rwkv_inner.py:40,48);
                                 the gradient w.r.t. a floored w is zero */

#define WKV_CHECKPOINTS_VALID 2u   /* backward only: the workspace passed is the one the matching
                                      forward call (same arguments, same algo) was given, so the
                                      state checkpoints it left there are used instead of rebuilt */

#define WKV_W_BF16 4u         /* WKV6 with the chunked algorithm only: w and gw are bf16 (B, T, C), as a
                                 mixed-precision TimeMix produces the decay and as the reference allocates its
                                 gradient (RWKV-v6/src/module/TimeMix.py:50,90); w is widened to fp32 inside, as
                                 the reference's w.float() does.  WKV_ERR_ALGO where the call would run token by
                                 token */

/* algorithm selector */
#define WKV_ALGO_AUTO      0  /* chunked where it applies, else recurrent */
#define WKV_ALGO_RECURRENT 1  /* per-token fp32 recurrence, any T, any dtype */
#define WKV_ALGO_CHUNKED   2  /* 64-token chunks on the matrix cores, bf16 operands */

const char *wkv_strerror(int status);
int wkv_abi_version(void);

/* One-time set-up of the loaded kernels (raises the LDS limit of the blocked kernels, once per process; looks up
 * the address of wkv6_forward_noalloc's scratch array on the CURRENT device; no counterpart in the reference, whose
 * extension is configured when torch builds it, RWKV-v5/src/module/TimeMix.py:229-252).  The operators do it
 * themselves on their first call; call it beforehand, once per device with that device current, when that first
 * call would fall inside a HIP stream capture.  Needs a GPU; returns WKV_ERR_LAUNCH without one. */
int wkv_init(void);

/* Tuning knobs (no counterpart in the reference).  WKV_TUNE_SEGMENTS: number of
 * time segments one (batch, head) sequence is cut into by the chunked algorithm
 * so that short batches still fill the GPU; 0 = choose from the shape (default),
 * 1..64 = force.  Results do not depend on it beyond fp32 rounding order.  The workspace sizes the queries return
 * depend on it (more segments, more piece summaries): query again after changing it.  It may change between a
 * forward call and its backward call (only the state checkpoints pass between the two, and those do not depend
 * on it). */
#define WKV_TUNE_SEGMENTS 1
/* WKV_TUNE_PIECE_STEPS: the summary pass of the time split cuts every segment into pieces of this many 64-token
 * steps (one workgroup and one 16 KiB summary per piece); 0 = choose from the shape (default).  Same rules as above. */
#define WKV_TUNE_PIECE_STEPS 2
int wkv_tune(int key, int value);

/* Timing hook for benchmarks (no counterpart in the reference).
 * wkv_profile_begin: from now on the first `max_launches` launches of the
 * kernel `kernel_id` are bracketed by HIP events recorded on the stream the
 * kernel is launched on (the events are created here, not in the operators).
 * wkv_profile_end: waits for those events, writes the elapsed milliseconds of
 * each recorded launch to the HOST array ms[capacity], returns how many, and
 * switches the hook off.  Not thread-safe; for single-threaded benchmark loops. */
#define WKV_KERNEL_REC_FORWARD    1   /* per-token WKV5/6 forward  */
#define WKV_KERNEL_REC_BACKWARD   2   /* per-token WKV5/6 backward */
#define WKV_KERNEL_V4_FORWARD     3
#define WKV_KERNEL_V4_BACKWARD    4
#define WKV_KERNEL_CHUNK_FORWARD  10  /* chunked WKV5/6 forward    */
#define WKV_KERNEL_CHUNK_BACKWARD 11  /* chunked WKV5/6 backward   */
int wkv_profile_begin(int kernel_id, int max_launches);
int wkv_profile_end(float *ms, int capacity);

/* ---------------------------------------------------------------- WKV6 ----
 * Replaces wkv6state_cuda forward/backward as bound in
 * RWKV-v6/src/module/cuda/wkv6state_op.cpp:5-17 and called from
 * RWKV-v6/src/module/TimeMix.py:59-64,95-100; results follow the pure path
 * RWKV-v6/src/module/rwkv_inner.py:10-115 (state in, state out, fp32 state,
 * full state gradient).
 */
/* Workspaces: forward needs none; if it is given one of at least
 * wkv6_forward_workspace() bytes (the chunked algorithm only) it leaves state
 * checkpoints there.  Passing that same buffer, sized by
 * wkv6_backward_workspace() (>= the forward size), to backward together with
 * WKV_CHECKPOINTS_VALID saves backward one sweep over k, v, w. */
/* state_out == state_in (the state updated in place) is accepted by the per-token algorithm and by the chunked one
 * whenever the plan cuts no sequence of the shape into time segments (B*H at least the number of compute units, or
 * WKV_TUNE_SEGMENTS 1); where it does (short batches, e.g. the 7B shape with B = 1), and for buffers that overlap
 * without being the same, the call returns WKV_ERR_ALIAS and the caller keeps two state buffers and alternates.
 * The same holds for wkv5_forward and wkv6_forward_noalloc. */
size_t wkv6_forward_workspace(int B, int T, int C, int H, int dtype, int algo);
int wkv6_forward(void *stream, int B, int T, int C, int H, int dtype, unsigned flags, int algo,
                 const void *r, const void *k, const void *v, const void *w, const float *u,
                 const float *state_in, void *y, float *state_out,
                 void *workspace, size_t workspace_bytes);

/* wkv6_forward for callers that cannot allocate device memory and have no workspace to pass: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same
 * arguments and results as wkv6_forward with the chunked algorithm (bf16 r/k/v/y and WKV_FLOOR_DECAY required,
 * else WKV_ERR_ALGO) and no state checkpoints kept; the scratch memory of the time-parallel split (the piece
 * summaries) is a 16 MiB array inside the library, one per GPU, held until the process ends.  The call allocates
 * nothing and frees nothing.  Shapes whose summaries exceed the array (B*H*segments*pieces*16640 bytes > 16 MiB,
 * e.g. B*H above about 120 at T = 4096) are rejected with WKV_ERR_WORKSPACE.  All calls on one GPU share that
 * GPU's array: two calls that overlap in time on the same GPU (different streams) race on it. */
#define WKV_NOALLOC_SCRATCH_BYTES (16u << 20)
int wkv6_forward_noalloc(void *stream, int B, int T, int C, int H, int dtype, unsigned flags,
                         const void *r, const void *k, const void *v, const void *w, const float *u,
                         const float *state_in, void *y, float *state_out);

size_t wkv6_backward_workspace(int B, int T, int C, int H, int dtype, int algo);
/* gstate_out may be NULL (no gradient arrives through the state handed out,
 * i.e. truncated BPTT); gstate_in may be NULL when it is not wanted.  The two
 * never overlap (WKV_ERR_ALIAS, for wkv5_backward as well): the state gradient
 * of a head is shared by several workgroups, and some read gstate_out after
 * others have written gstate_in. */
int wkv6_backward(void *stream, int B, int T, int C, int H, int dtype, unsigned flags, int algo,
                  const void *r, const void *k, const void *v, const void *w, const float *u,
                  const float *state_in, const void *gy, const float *gstate_out,
                  void *gr, void *gk, void *gv, void *gw, float *gu, float *gstate_in,
                  void *workspace, size_t workspace_bytes);

/* ---------------------------------------------------------------- WKV5 ----
 * Replaces wkv5 forward_{bf16,fp16,fp32} / backward_* of
 * RWKV-v5/src/module/cuda/wkv5_op.cpp:84-129 (called from
 * RWKV-v5/src/module/TimeMix.py:79-86,119-126); results follow
 * RWKV-v5/src/module/rwkv_inner.py:10-118.  w, gw are per channel (H,64).
 */
size_t wkv5_forward_workspace(int B, int T, int C, int H, int dtype, int algo);
int wkv5_forward(void *stream, int B, int T, int C, int H, int dtype, unsigned flags, int algo,
                 const void *r, const void *k, const void *v, const float *w, const float *u,
                 const float *state_in, void *y, float *state_out,
                 void *workspace, size_t workspace_bytes);

size_t wkv5_backward_workspace(int B, int T, int C, int H, int dtype, int algo);
int wkv5_backward(void *stream, int B, int T, int C, int H, int dtype, unsigned flags, int algo,
                  const void *r, const void *k, const void *v, const float *w, const float *u,
                  const float *state_in, const void *gy, const float *gstate_out,
                  void *gr, void *gk, void *gv, float *gw, float *gu, float *gstate_in,
                  void *workspace, size_t workspace_bytes);

/* ---------------------------------------------------------------- WKV4 ----
 * Replaces cuda_forward / cuda_backward of
 * RWKV-v4neo/cuda/wkv_cuda_bf16.cu:160-172 as wrapped by
 * RWKV-v4neo/cuda/wkv_op_bf16.cpp:15-86 (torch.ops.rwkv.wkv).  time_decay is
 * the RAW parameter (w = -exp(time_decay) is formed inside, as :34 does);
 * g_time_decay, g_time_first are summed over the batch (as :85 does).
 * state_in NULL means the empty history (0, 0, -1e38).  The state gradient is
 * carried as (gp, gq, go) with go an exponent, as the reference does
 * (wkv_cuda_bf16.cu:116-152).
 * `checkpoints` (optional, wkv4_checkpoint_bytes() bytes): written by forward,
 * read by backward, saves backward one sweep over k and v.
 */
size_t wkv4_checkpoint_bytes(int B, int T, int C);
int wkv4_forward(void *stream, int B, int T, int C, int dtype,
                 const float *time_decay, const float *time_first, const void *k, const void *v,
                 const float *state_in, void *y, float *state_out, void *checkpoints);
size_t wkv4_backward_workspace(int B, int T, int C, int dtype);
int wkv4_backward(void *stream, int B, int T, int C, int dtype,
                  const float *time_decay, const float *time_first, const void *k, const void *v,
                  const float *state_in, const void *gy, const float *gstate_out,
                  float *g_time_decay, float *g_time_first, void *gk, void *gv, float *gstate_in,
                  const void *checkpoints, void *workspace, size_t workspace_bytes);

/* ------------------------------------------------------ cumsum-decay ------
 * The helper the reference's chunked path computes inline
 * (RWKV-v5/src/module/rwkv_inner.py:43-58,72-79): from the raw decay parameter
 * w (B,T,C) [or (1,1,C) broadcast when per_token == 0] to
 *   log_w      (Bw,T,C)  max(-exp(w), ln 0.005)
 *   incl       (Bw,T,C)  inclusive cumulative sum of log_w inside each chunk
 *   inter      (Bw,T,C)  chunk total - incl   (decay from a token to its chunk's end)
 *   intra      (Bw,T,C)  incl - log_w         (decay from the chunk's start to a token)
 *   chunk_sum  (Bw,T/chunk,C)
 * all fp32, in log space.  Any output pointer may be NULL.  T must be a
 * multiple of chunk_len.
 */
int wkv_cumsum_decay(void *stream, int Bw, int T, int C, int chunk_len, int per_token,
                     const float *w, float *log_w, float *incl, float *inter, float *intra,
                     float *chunk_sum);

/* The same helper with every table the reference derives from w: besides the five log-space tables above,
 *   ws_exp     (Bw,T/chunk,C) fp32  exp(chunk_sum)                        rwkv_inner.py:80
 *   inter_exp  (Bw,T,C)       fp32  exp(inter)                            :81
 *   intra_exp  (Bw,T,C)       fp32  exp(intra)                            :82
 *   r_decay    (Bw,T,C)  exp(intra - intra at the chunk's token chunk_len/2)      :91-92
 *   k_inv_decay(Bw,T,C)  exp(intra at the chunk's token chunk_len/2 - incl)       :91,93
 * the last two in fp64 (precision = 64, double*) or fp32 (precision = 32, float*), as the reference's `precision`
 * argument (:41-46): in fp32 they overflow for chunk lengths much beyond 32.  Any output pointer may be NULL. */
int wkv_cumsum_decay_factors(void *stream, int Bw, int T, int C, int chunk_len, int per_token, int precision,
                             const float *w, float *log_w, float *incl, float *inter, float *intra, float *chunk_sum,
                             float *ws_exp, float *inter_exp, float *intra_exp, void *r_decay, void *k_inv_decay);

/* ---- The element-wise passes on either side of the operator inside a block.  Tensors are contiguous (.., C)
 * in `dtype`; parameters (coef, weight, bias) and their gradients are fp32.  None of these allocates. */

/* Token shift + mixing (RWKV-v5/src/module/TimeMix.py:292-298 and ChannelMix.py:44-47 with lerp = 1;
 * RWKV-v6/src/module/TimeMix.py:262-276 and ChannelMix.py:31-35 with lerp = 0): from one read of x,
 *   out[j][b,t,:] = x[b,t,:] + (x[b,t-1,:] - x[b,t,:]) * d_j,   x[b,-1,:] = shift[b,:]
 * for j < n (n <= 5).  lerp = 1: coef[j] is the reference's time_mix_j, d_j = 1 - coef[j] (modified_lerp,
 * RWKV-v5/src/module/OptimizedOps.py:14-15).  lerp = 0: coef[j] is time_maa_j, d_j = coef[j] + dyn[j][b,t,:], with
 * dyn (n, B, T, C) the data-dependent part (the reference's mw, mk, mv, mr, mg, RWKV-v6 TimeMix.py:265-268) or NULL.
 *   x (B,T,C); shift (B,C); coef (n,C) fp32; out: HOST array of n device pointers, each (B,T,C). */
int wkv_shift_mix_forward(void *stream, int B, int T, int C, int dtype, int n, int lerp, const void *x,
                          const void *shift, const float *coef, const void *dyn, void *const *out);

/* Its backward (what autograd derives from the lines cited above): gout = HOST array of the n output gradients;
 * gx (B,T,C), gshift (B,C) in `dtype`; gcoef (n,C) fp32, summed over batch and time in a fixed order; gdyn
 * (n,B,T,C) in `dtype`, required when dyn is given.  workspace: wkv_shift_mix_backward_workspace bytes. */
size_t wkv_shift_mix_backward_workspace(int B, int T, int C, int n);
int wkv_shift_mix_backward(void *stream, int B, int T, int C, int dtype, int n, int lerp, const void *x,
                           const void *shift, const float *coef, const void *dyn, const void *const *gout, void *gx,
                           void *gshift, float *gcoef, void *gdyn, void *workspace, size_t workspace_bytes);

/* The data-dependent mix of the v6 TimeMix with its second LoRA product inside the pass
 * (RWKV-v6/src/module/TimeMix.py:264-276; replaces `torch.bmm(xxx, self.time_maa_w2)` of :265 and the five mixes of
 * :269-273, whose operands mw, mk, mv, mr, mg are then never written to memory):
 *   out[j][b,t,:] = x[b,t,:] + (x[b,t-1,:] - x[b,t,:]) * (coef[j] + act[b*T+t, j, :] @ w2[j]),   j < 5 = w, k, v, r, g
 * bf16 only.  x (B,T,C); shift (B,C); coef (5,C) fp32 = time_maa_w, _k, _v, _r, _g; act (B*T, 5, 32) =
 * tanh(xxx @ time_maa_w1) as the reference views it before its transpose (:264); w2t (5, C, 32) = time_maa_w2 with its
 * last two dimensions exchanged; out: HOST array of 5 device pointers, each (B,T,C).  C a multiple of 8. */
int wkv_lora_mix_forward(void *stream, int B, int T, int C, const void *x, const void *shift, const float *coef,
                         const void *act, const void *w2t, void *const *out);

/* Its backward: gout = HOST array of the 5 output gradients; gx (B,T,C), gshift (B,C) bf16; gcoef (5,C) fp32, summed
 * over batch and time in a fixed order; gdyn (5,B,T,C) bf16 = the gradients of the five products act @ w2[j] (what
 * autograd hands to the backward of the reference's bmm: the gradients of act and of w2 are two matrix products with
 * it, left to the caller's GEMM library).  workspace: wkv_lora_mix_backward_workspace bytes. */
size_t wkv_lora_mix_backward_workspace(int B, int T, int C);
int wkv_lora_mix_backward(void *stream, int B, int T, int C, const void *x, const void *shift, const float *coef,
                          const void *act, const void *w2t, const void *const *gout, void *gx, void *gshift,
                          float *gcoef, void *gdyn, void *workspace, size_t workspace_bytes);

/* ln_x and the gate on the operator's output (RWKV-v5/src/module/TimeMix.py:301,317-320: scale = 1/8, eps = 1e-5;
 * RWKV-v6/src/module/TimeMix.py:180,278,296-298: scale = 1, eps = 64e-5):
 *   out = (GroupNorm(y * scale; one group per 64-channel head, eps) * weight + bias) * silu(gate)
 * gate is the gate projection BEFORE its SiLU (the reference applies F.silu first and multiplies afterwards; here
 * both happen in the one pass), or NULL for the normalisation alone.  rows = B*T; y, gate, out (rows, C). */
int wkv_ln_gate_forward(void *stream, int rows, int C, int dtype, float scale, float eps, const void *y,
                        const void *gate, const float *weight, const float *bias, void *out);

/* Its backward: gy, ggate (w.r.t. the gate projection) in `dtype`; gweight_gbias (2, C) fp32 = gradient of weight,
 * then of bias, summed over rows in a fixed order.  workspace: wkv_ln_gate_backward_workspace bytes. */
size_t wkv_ln_gate_backward_workspace(int rows, int C);
int wkv_ln_gate_backward(void *stream, int rows, int C, int dtype, float scale, float eps, const void *y,
                         const void *gate, const float *weight, const float *bias, const void *gout, void *gy,
                         void *ggate, float *gweight_gbias, void *workspace, size_t workspace_bytes);

/* The activations of the channel mix (RWKV-v5/src/module/ChannelMix.py:48-49, RWKV-v6/src/module/ChannelMix.py:
 * 36-37) over n elements (n a multiple of 8): out = relu(k)^2;  out = sigmoid(r) * kv; and their backwards. */
int wkv_relu_square_forward(void *stream, size_t n, int dtype, const void *k, void *out);
int wkv_relu_square_backward(void *stream, size_t n, int dtype, const void *k, const void *gout, void *gk);
int wkv_sigmoid_mul_forward(void *stream, size_t n, int dtype, const void *r, const void *kv, void *out);
int wkv_sigmoid_mul_backward(void *stream, size_t n, int dtype, const void *r, const void *kv, const void *gout,
                             void *gr, void *gkv);

/* Backward of L2Wrap (RWKV-v5/src/model.py:140-148): gy (rows, V) is zero except, in every row, at the first
 * position of the row's maximum, where it is factor * mask[row] * max (mask (rows) fp32 or NULL = ones). */
int wkv_l2wrap_backward(void *stream, int rows, int V, int dtype, float factor, const void *y, const float *mask,
                        void *gy);

#ifdef __cplusplus
}
#endif
#endif
