"""CPU oracle for the multi-head WKV5 / WKV6 recurrence (test infrastructure).

Index convention used everywhere below (K = V = head size):

    y_t[j]   = sum_i r_t[i] * ( S_{t-1}[i,j] + u[i] * k_t[i] * v_t[j] )
    S_t[i,j] = w_t[i] * S_{t-1}[i,j] + k_t[i] * v_t[j]

with ``i`` the key index, ``j`` the value index, ``S_{-1}`` the state handed
in and ``S_{T-1}`` the state handed out.  WKV5 is the special case in which
``w_t`` is the same for every token and batch entry.

Three statements of this one function live here:

``wkv_token_loop``     the defining per-token recurrence
                       (RWKV-v5/src/module/rwkv_inner.py:28-32; the same
                       recurrence is written a second and third time in
                       RWKV-v5/src/module/TimeMix.py:369-393 and
                       RWKV-v5/src/module/cuda/wkv5_cuda.cu:167-190).
``wkv_chunked``        the chunked training path, cast for cast
                       (RWKV-v5/src/module/rwkv_inner.py:33-118,
                       RWKV-v6/src/module/rwkv_inner.py:30-115), built on
``cumsum_decay``       the cumulative-decay helper that path computes inline
                       (RWKV-v5/src/module/rwkv_inner.py:43-58,72-82,91-93).
``wkv_adjoint`` /      closed-form gradients, written from the adjoint
``decay_grad_by_scan`` equations rather than from autograd, as an independent
                       second gradient implementation.

Pinned by (tests/test_oracle_wkv56.py): an explicit double-sum closed form of
the outputs on tiny inputs, the ``w=1, u=0`` case against ``torch.cumsum``, the
single-token case, linearity in ``v`` and in the state, chunked == token loop
in fp64, helper identities, autograd == adjoint == finite differences, and
segment chaining.
"""
from __future__ import annotations

import math
from typing import NamedTuple

import torch
import torch.nn.functional as F

# smallest decay the chunked path lets through (rwkv_inner.py:40,48)
W_FLOOR = 0.005
LOG_W_FLOOR = math.log(W_FLOOR)


def decay_from_raw(x: torch.Tensor) -> torch.Tensor:
    """Raw decay parameter -> decay in (0,1): exp(-exp(x)), evaluated in fp32
    (RWKV-v5/src/module/TimeMix.py:349, RWKV-v6/src/module/TimeMix.py:331-333)."""
    return torch.exp(-torch.exp(x.float()))


# --------------------------------------------------------------------------
# 1. defining recurrence
# --------------------------------------------------------------------------
def wkv_token_loop(r, k, v, w, u, state, floor_decay: bool = False):
    """One token at a time, exactly the single-step branch of the reference
    (rwkv_inner.py:28-32) applied L times.

    r, k : (B,H,L,K)   v : (B,H,L,V)   w : (B or 1,H,L,K) decay in (0,1)
    u : (1,H,1,K)      state : (B,H,K,V)
    Runs in the dtype of its arguments.  ``floor_decay`` applies the chunked
    path's lower bound on w first (the single-step branch itself does not).
    """
    L = k.size(2)
    if floor_decay:
        w = w.clamp(W_FLOOR)
    ys = []
    for t in range(L):
        rt, kt, vt, wt = (x[:, :, t:t + 1] for x in (r, k, v, w))
        kv = kt.mT @ vt                              # (B,H,K,V)
        ys.append(rt @ (state + u.mT * kv))          # (B,H,1,V)
        state = wt.mT * state + kv
    return torch.cat(ys, dim=2), state


# --------------------------------------------------------------------------
# 2. cumulative-decay helper and the chunked path
# --------------------------------------------------------------------------
class DecayTables(NamedTuple):
    """Everything the chunked path derives from w (all but ``log_w`` chunked
    as (B or 1, H, N, T, K); T = chunk length, N = L / T)."""
    log_w: torch.Tensor          # fp32 log of the floored decay, (.,H,L,K)
    incl: torch.Tensor           # inclusive cumsum of log w inside a chunk
    excl: torch.Tensor           # exclusive cumsum (shifted by one token)
    chunk_log: torch.Tensor      # (.,H,N,1,K) sum over the chunk
    inter_log: torch.Tensor      # chunk_log - incl : decay from token to chunk end
    intra_log: torch.Tensor      # incl - log w (== excl) : decay from chunk start to token
    r_decay: torch.Tensor        # exp(excl - excl[T/2])   in fp64 / fp32
    k_inv_decay: torch.Tensor    # exp(excl[T/2] - incl)   in fp64 / fp32


def cumsum_decay(w, chunk_len: int = 128, precision: int = 64) -> DecayTables:
    """The cumsum-decay helper (rwkv_inner.py:43-58 floor + log + cumsum,
    :72-79 inter/intra, :91-93 the two re-centred intra-chunk factors)."""
    assert precision in (32, 64)
    pdt = torch.float64 if precision == 64 else torch.float32
    Bw, H, L, K = w.shape
    T = chunk_len
    assert L % T == 0
    N = L // T
    log_w = w.clamp(W_FLOOR).float().log()
    lc = log_w.view(Bw, H, N, T, K)
    incl = lc.cumsum(dim=-2)
    excl = F.pad(incl, (0, 0, 1, -1))
    chunk_log = lc.sum(dim=-2, keepdim=True)
    inter_log = chunk_log - incl
    intra_log = incl - lc
    mid = excl[..., T // 2:T // 2 + 1, :]
    r_decay = (excl - mid).to(pdt).exp()
    k_inv_decay = (mid - incl).to(pdt).exp()
    return DecayTables(log_w, incl, excl, chunk_log, inter_log, intra_log, r_decay, k_inv_decay)


def wkv_chunked(r, k, v, w, u, state, chunk_len: int = 128, precision: int = 64):
    """The training path of the reference, same operations and the same cast
    points (rwkv_inner.py:33-118): intra-chunk masked r~ k~^T in ``precision``
    bits, everything else in r.dtype, state carried chunk to chunk."""
    assert chunk_len <= 24 or precision == 64
    B, H, L, K = k.shape
    V = v.size(-1)
    T = chunk_len
    if L == 1:
        return wkv_token_loop(r, k, v, w, u, state)
    assert L % T == 0, "chunked path needs L to be a multiple of chunk_len"
    N = L // T
    tab = cumsum_decay(w, T, precision)
    dt = r.dtype

    chunk_decay = tab.chunk_log.mT.exp().to(dt).unbind(dim=-3)     # N x (.,H,K,1)
    to_end = tab.inter_log.exp().to(dt)                            # (.,H,N,T,K)
    from_start = tab.intra_log.exp().to(dt)

    rc = r.view(B, H, N, T, K)
    kc = k.view(B, H, N, T, K)
    vc = v.view(B, H, N, T, V)
    uc = u.unsqueeze(2).to(dt)                                     # (1,H,1,1,K)

    att = ((rc * tab.r_decay) @ (kc * tab.k_inv_decay).mT).to(dt).tril(-1)   # (B,H,N,T,T)
    att = att + torch.einsum('bhntk,bhntk->bhnt', rc, uc * kc).diag_embed()
    out = att @ vc

    contrib = ((kc * to_end).mT @ vc).unbind(dim=-3)               # N x (B,H,K,V)
    starts = []
    for n in range(N):
        starts.append(state)
        state = state * chunk_decay[n] + contrib[n]
    starts = torch.stack(starts, dim=2)                            # (B,H,N,K,V)

    out = out + (rc * from_start) @ starts
    return out.view(B, H, L, V), state


# --------------------------------------------------------------------------
# 3. closed-form gradients (independent of autograd)
# --------------------------------------------------------------------------
def wkv_adjoint(r, k, v, w, u, state, gy, gstate_out):
    """Gradients of  sum(gy*y) + sum(gstate_out*S_out)  from the adjoint
    recurrence  G_{t-1} = r_t (x) gy_t + w_t o G_t,  G_{T-1} = gstate_out.

    Same layouts as ``wkv_token_loop``; ``w`` is the decay actually applied.
    Returns gr, gk, gv, gw (per token, w.r.t. the decay w_t, (B,H,L,K)),
    gu (1,H,1,K) and gstate_in.
    """
    B, H, L, K = k.shape
    S_prev = []
    S = state
    for t in range(L):
        S_prev.append(S)
        S = w[:, :, t].unsqueeze(-1) * S + k[:, :, t].unsqueeze(-1) * v[:, :, t].unsqueeze(-2)
    G = gstate_out
    gr = torch.zeros_like(r)
    gk = torch.zeros_like(k)
    gv = torch.zeros_like(v)
    gw = torch.zeros(B, H, L, K, dtype=r.dtype)
    gu = torch.zeros_like(u)
    uu = u[0, :, 0]                                                  # (H,K)
    for t in reversed(range(L)):
        rt, kt, vt, gyt = r[:, :, t], k[:, :, t], v[:, :, t], gy[:, :, t]
        wt = w[:, :, t] if w.size(0) == B else w[:, :, t].expand(B, H, K)
        vg = (vt * gyt).sum(-1, keepdim=True)                        # v_t . gy_t
        gr[:, :, t] = torch.einsum('bhkv,bhv->bhk', S_prev[t], gyt) + uu * kt * vg
        gk[:, :, t] = torch.einsum('bhkv,bhv->bhk', G, vt) + uu * rt * vg
        gv[:, :, t] = torch.einsum('bhkv,bhk->bhv', G, kt) + (uu * rt * kt).sum(-1, keepdim=True) * gyt
        gw[:, :, t] = (G * S_prev[t]).sum(-1)
        gu += (rt * kt * vg).sum(0).view(1, H, 1, K)
        G = rt.unsqueeze(-1) * gyt.unsqueeze(-2) + wt.unsqueeze(-1) * G
    return gr, gk, gv, gw, gu, G


def decay_grad_by_scan(r, k, v, w, u, gy, gr, gk, state_out, gstate_out):
    """w_t * dL/dw_t  (= dL/d log w_t) without any stored state, from the scan

        A_{T-1} = sum_j gstate_out o S_out
        A_{t-1} = A_t + r_t o gr_t - k_t o gk_t
        D_t     = A_t - k_t o ( gk_t - u o r_t (v_t . gy_t) )

    which is the prefix/suffix-difference idea of
    RWKV-v6/src/module/cuda/wkv6state_cuda_v1.cu:193-293 extended by the
    boundary term the reference sets to zero (:292).  Returns D (B,H,L,K)."""
    L = k.size(2)
    uu = u[0, :, 0]
    A = (gstate_out * state_out).sum(-1)                             # (B,H,K)
    D = torch.zeros_like(gr)
    for t in reversed(range(L)):
        vg = (v[:, :, t] * gy[:, :, t]).sum(-1, keepdim=True)
        D[:, :, t] = A - k[:, :, t] * (gk[:, :, t] - uu * r[:, :, t] * vg)
        A = A + r[:, :, t] * gr[:, :, t] - k[:, :, t] * gk[:, :, t]
    return D


# --------------------------------------------------------------------------
# 4. operator-level front ends with the trainer's tensor conventions
# --------------------------------------------------------------------------
def _heads(x, B, T, H):
    return x.view(B, T, H, -1).transpose(1, 2)


def _run(r, k, v, w, u, state, T, chunk_len, precision):
    if T == 1:
        return wkv_token_loop(r, k, v, w, u, state)          # no floor on w, as the reference
    if T % chunk_len == 0:
        return wkv_chunked(r, k, v, w, u, state, chunk_len, precision)
    # Lengths the reference's pure path rejects (TimeMix.py:328): same
    # function, evaluated token by token with the floor on w kept.
    return wkv_token_loop(r, k, v, w, u, state, floor_decay=True)


def wkv5_op(B, T, C, H, state, r, k, v, w_raw, u, chunk_len=128, precision=64, dtype=torch.float32):
    """WKV5 with the trainer's tensors: r,k,v (B,T,C); w_raw, u (H,K) with
    w = exp(-exp(w_raw)) per channel; state (B,H,K,V).  Follows the pure path's
    call site RWKV-v5/src/module/TimeMix.py:345-358.  Returns y (B,T,C) and
    the new state, both in ``dtype``."""
    K = C // H
    rr, kk, vv = (_heads(x.to(dtype), B, T, H) for x in (r, k, v))
    w = decay_from_raw(w_raw).view(1, H, 1, K).expand(1, H, T, K)
    uu = u.view(1, H, 1, K).to(dtype)
    y, s = _run(rr, kk, vv, w, uu, state.to(dtype), T, chunk_len, precision)
    return y.transpose(1, 2).reshape(B, T, C), s


def wkv6_op(B, T, C, H, r, k, v, w_raw, u, state, chunk_len=128, precision=64, dtype=torch.float32):
    """WKV6 (per-token decay): w_raw (B,T,C), otherwise as ``wkv5_op``.
    Follows RWKV-v6/src/module/TimeMix.py:328-343."""
    K = C // H
    rr, kk, vv = (_heads(x.to(dtype), B, T, H) for x in (r, k, v))
    w = _heads(decay_from_raw(w_raw), B, T, H)
    uu = u.view(1, H, 1, K).to(dtype)
    y, s = _run(rr, kk, vv, w, uu, state.to(dtype), T, chunk_len, precision)
    return y.transpose(1, 2).reshape(B, T, C), s


def wkv_op_grads(version, B, T, C, H, r, k, v, w_raw, u, state, gy, gstate, **kw):
    """Forward + autograd backward through the operator-level oracle.
    Returns dict(y, state, gr, gk, gv, gw, gu, gstate) with gw w.r.t. the RAW
    decay parameter and gu in the shape of u."""
    dtype = kw.pop('dtype', torch.float32)
    leaves = [t.detach().clone().to(dtype if t is not w_raw else torch.float32).requires_grad_(True)
              for t in (r, k, v, w_raw, u, state)]
    r_, k_, v_, w_, u_, s_ = leaves
    if version == 5:
        y, s = wkv5_op(B, T, C, H, s_, r_, k_, v_, w_, u_, dtype=dtype, **kw)
    else:
        y, s = wkv6_op(B, T, C, H, r_, k_, v_, w_, u_, s_, dtype=dtype, **kw)
    loss = (y * gy.to(dtype)).sum() + (s * gstate.to(dtype)).sum()
    g = torch.autograd.grad(loss, leaves)
    return dict(y=y.detach(), state=s.detach(), gr=g[0], gk=g[1], gv=g[2], gw=g[3], gu=g[4], gstate=g[5])
