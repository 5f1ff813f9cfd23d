"""CPU oracle for the RWKV-v4 WKV recurrence (test infrastructure).

Front end to the plain-C restatement in ``wkv4_ref.c`` (which follows
RWKV-v4neo/cuda/wkv_cuda_bf16.cu:7-158) plus two torch statements of the same
function written from the mathematics instead of from the kernel:

``wkv4_undivided``   P_t = e^{w} P_{t-1} + e^{k_t} v_t,  Q_t likewise,
                     y_t = (P_{t-1} + e^{u+k_t} v_t) / (Q_{t-1} + e^{u+k_t})
                     in fp64 without the running-maximum exponent;
                     differentiable, used to pin every gradient.
``wkv4_softmax_form`` y_t as a softmax-weighted average over explicit logits.
``wkv4_torch_loop``  the kernel's stabilised recurrence vectorised over (B,C).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None
NEG_HUGE = -1e38


def lib():
    """The C oracle, building it with ``make -C oracle`` if it is not there."""
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libwkv4_oracle.so")
        if not os.path.exists(path):
            subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)
        _LIB = ctypes.CDLL(path)
    return _LIB


def _np(t, dt):
    return None if t is None else np.ascontiguousarray(t.detach().cpu().to(dt).numpy())


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def forward(time_decay, time_first, k, v, state, real="f32"):
    """(y, new_state) for raw ``time_decay``/``time_first`` (C), k,v (B,T,C),
    state (B,C,3); arithmetic in fp32 (``real='f32'``) or fp64."""
    tdt = torch.float32 if real == "f32" else torch.float64
    B, T, C = k.shape
    w = _np(-torch.exp(time_decay.to(tdt)), tdt)        # wkv_op_bf16.cpp:34 (fp32 there)
    u, kk, vv, st = _np(time_first, tdt), _np(k, tdt), _np(v, tdt), _np(state, tdt)
    y = np.empty_like(kk)
    ns = np.empty((B, C, 3), dtype=kk.dtype)
    getattr(lib(), f"wkv4_forward_{real}")(B, T, C, _ptr(w), _ptr(u), _ptr(kk), _ptr(vv), _ptr(st), _ptr(y), _ptr(ns))
    return torch.from_numpy(y), torch.from_numpy(ns)


def backward(time_decay, time_first, k, v, state, gy, gnew_state, real="f32"):
    """(g_time_decay (C), g_time_first (C), gk, gv, glast_state); the first two
    summed over the batch as the reference's wrapper does (wkv_op_bf16.cpp:85)."""
    tdt = torch.float32 if real == "f32" else torch.float64
    B, T, C = k.shape
    w = _np(-torch.exp(time_decay.to(tdt)), tdt)
    u, kk, vv, st = _np(time_first, tdt), _np(k, tdt), _np(v, tdt), _np(state, tdt)
    g, gs = _np(gy, tdt), _np(gnew_state, tdt)
    gw = np.empty((B, C), dtype=kk.dtype)
    gu = np.empty_like(gw)
    gk, gv = np.empty_like(kk), np.empty_like(kk)
    gl = np.empty((B, C, 3), dtype=kk.dtype)
    getattr(lib(), f"wkv4_backward_{real}")(B, T, C, _ptr(w), _ptr(u), _ptr(kk), _ptr(vv), _ptr(st), _ptr(g), _ptr(gs),
                                            _ptr(gw), _ptr(gu), _ptr(gk), _ptr(gv), _ptr(gl))
    f = torch.from_numpy
    return f(gw).sum(0), f(gu).sum(0), f(gk), f(gv), f(gl)


def wkv4_undivided(time_decay, time_first, k, v, P0, Q0):
    """fp64, no exponent bookkeeping; P0, Q0 (B,C) are the undivided sums
    handed in.  Returns y (B,T,C), P_T, Q_T.  Only for small |k| and T."""
    w = -torch.exp(time_decay)
    P, Q = P0, Q0
    ys = []
    for t in range(k.size(1)):
        e = torch.exp(time_first + k[:, t])
        ys.append((P + e * v[:, t]) / (Q + e))
        P = torch.exp(w) * P + torch.exp(k[:, t]) * v[:, t]
        Q = torch.exp(w) * Q + torch.exp(k[:, t])
    return torch.stack(ys, 1), P, Q


def wkv4_softmax_form(time_decay, time_first, k, v, t):
    """y at token t for an empty history before token 0: softmax over logits
    k_s + (t-1-s) w for s < t and u + k_t for s = t, applied to v."""
    w = -torch.exp(time_decay)
    s = torch.arange(t, dtype=k.dtype)
    logits = torch.cat([k[:, :t] + ((t - 1 - s).view(1, t, 1) * w), (time_first + k[:, t]).unsqueeze(1)], 1)
    return (torch.softmax(logits, dim=1) * v[:, :t + 1]).sum(1)


def wkv4_torch_loop(time_decay, time_first, k, v, state):
    """The stabilised recurrence of wkv_cuda_bf16.cu:31-46, vectorised over
    (B,C) with a Python loop over T; in the dtype of k."""
    w = -torch.exp(time_decay.to(k.dtype))
    u = time_first.to(k.dtype)
    p, q, o = state[..., 0].to(k.dtype), state[..., 1].to(k.dtype), state[..., 2].to(k.dtype)
    ys = []
    for t in range(k.size(1)):
        kk, vv = k[:, t], v[:, t]
        m = torch.maximum(o, u + kk)
        a, b = torch.exp(o - m), torch.exp(u + kk - m)
        ys.append((a * p + b * vv) / (a * q + b))
        m = torch.maximum(w + o, kk)
        a, b = torch.exp(w + o - m), torch.exp(kk - m)
        p, q, o = a * p + b * vv, a * q + b, m
    return torch.stack(ys, 1), torch.stack([p, q, o], -1)
