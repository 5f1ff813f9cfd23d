"""CPU oracle for the element-wise passes around the WKV operator inside a block (test infrastructure: only
tests, the smoke check and the benchmark's CPU baseline may use it).

Each function restates the cited lines of the reference in plain torch, cast for cast, so that autograd through it
is the reference's backward:

``token_shift``      RWKV-v5/src/module/TimeMix.py:292 (ChannelMix.py:44-45; RWKV-v6 TimeMix.py:262)
``modified_lerp``    RWKV-v5/src/module/OptimizedOps.py:14-15
``mix_v5``           RWKV-v5/src/module/TimeMix.py:295-298, ChannelMix.py:46-47
``mix_v6``           RWKV-v6/src/module/TimeMix.py:262-276, ChannelMix.py:33-35
``lora_mix_v6``      RWKV-v6/src/module/TimeMix.py:264-273 (the second LoRA product and the five mixes it feeds)
``ln_x_gate``        RWKV-v5/src/module/TimeMix.py:301,317-320 (divisor 8, eps 1e-5);
                     RWKV-v6/src/module/TimeMix.py:180,278,296-298 (divisor 1, eps 64e-5)
``relu_square``, ``sigmoid_mul``   RWKV-v5/src/module/ChannelMix.py:48-49
``L2Wrap``           RWKV-v5/src/model.py:123-148
``ChannelMix5`` / ``ChannelMix6`` forwards   RWKV-v5/src/module/ChannelMix.py:35-49, RWKV-v6/src/module/ChannelMix.py:30-37

Pinned by (tests/test_oracle_blocks.py): the mixes at coefficient 0 and 1 (identity / pure shift), token_shift against
an index loop, ln_x_gate against a written-out mean/variance normalisation and against torch's layer_norm per head,
L2Wrap against a per-row Python loop, the two activations against their textbook formulas in numpy, lora_mix_v6
against a per-token, per-mix loop of matrix-vector products (and against mix_v6 at w2 = 0).
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


def token_shift(x, shift_state):
    """xx[b,t] = x[b,t-1], xx[b,0] = shift_state[b]"""
    return torch.concat((shift_state.unsqueeze(1), x[:, :-1]), dim=1)


def modified_lerp(start_mul, start, weight):
    return start_mul * start + weight * (1 - start)


def mix_v5(x, shift_state, mixes):
    """one mixed copy of x per time_mix_* parameter"""
    xx = token_shift(x, shift_state)
    return tuple(modified_lerp(x, m, xx) for m in mixes)


def mix_v6(x, shift_state, maas, dyn=None):
    """x + dxprev * (time_maa_j [+ dyn_j]); dyn (n,B,T,C) are the reference's mw, mk, mv, mr, mg"""
    dxprev = token_shift(x, shift_state) - x
    if dyn is None:
        return tuple(x + dxprev * m for m in maas)
    return tuple(x + dxprev * (m + d) for m, d in zip(maas, dyn.unbind(0)))


def lora_mix_v6(x, shift_state, maas, act, w2):
    """the reference's five data-dependent mixes from act = tanh(xxx @ time_maa_w1) as (B*T, 5, D) and
    w2 = time_maa_w2 (5, D, C): the batched product of TimeMix.py:264-265 (transpose, bmm, view) and the mixes of
    :269-273; maas = (time_maa_w, _k, _v, _r, _g); returns (xw, xk, xv, xr, xg)"""
    B, T, C = x.shape
    dyn = torch.bmm(act.transpose(0, 1), w2).view(5, B, T, -1)
    return mix_v6(x, shift_state, maas, dyn)


def ln_x_gate(y, gate, weight, bias, n_head, eps, divisor=1.0):
    """ln_x(y / divisor) * silu(gate); gate is the gate projection before F.silu (None: no gate)"""
    shape = y.shape
    C = shape[-1]
    out = F.group_norm(y.reshape(-1, C) / divisor, n_head, weight, bias, eps).view(shape)
    return out if gate is None else out * F.silu(gate)


def relu_square(k):
    return torch.relu(k) ** 2


def sigmoid_mul(r, kv):
    return torch.sigmoid(r) * kv


class L2Wrap(torch.autograd.Function):
    @staticmethod
    def forward(ctx, loss, y, factor, currentMask):
        ctx.save_for_backward(y, torch.as_tensor(factor), currentMask)
        return loss

    @staticmethod
    def backward(ctx, grad_output):
        y, factor, currentMask = ctx.saved_tensors
        maxx, ids = torch.max(y, -1, keepdim=True)
        gy = torch.zeros_like(y)
        gy.scatter_(-1, ids, maxx * factor)
        gy = gy * currentMask.reshape(gy.shape[0], gy.shape[1], 1)
        return grad_output, gy, None, None


def channelmix5_forward(self, x, last_state):
    xx = token_shift(x, last_state)
    xk = x * self.time_mix_k + xx * (1 - self.time_mix_k)
    xr = x * self.time_mix_r + xx * (1 - self.time_mix_r)
    kv = self.value(torch.relu(self.key(xk)) ** 2)
    return torch.sigmoid(self.receptance(xr)) * kv, x[:, -1]


def channelmix6_forward(self, x, last_state):
    xx = token_shift(x, last_state)
    dxx = xx - x
    xk = x + dxx * self.time_maa_k
    xr = x + dxx * self.time_maa_r
    kv = self.value(torch.relu(self.key(xk)) ** 2)
    return torch.sigmoid(self.receptance(xr)) * kv, x[:, -1]
