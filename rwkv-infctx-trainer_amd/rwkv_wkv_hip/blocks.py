"""The element-wise passes around the WKV operator inside a block, on the HIP kernels of csrc/block_edges.hip,
and the block forwards that use them.

  token_shift_mix   token shift + mixing of the block input, any number of mixed copies from one read of x
                    (RWKV-v5/src/module/TimeMix.py:292-298, ChannelMix.py:44-47; RWKV-v6/src/module/TimeMix.py:262-276,
                    ChannelMix.py:31-35)
  lora_shift_mix    the five data-dependent mixes of the v6 TimeMix with the second LoRA product inside the pass
                    (RWKV-v6/src/module/TimeMix.py:264-276)
  ln_x_gate         GroupNorm per head times the SiLU gate (RWKV-v5 TimeMix.py:301,317-320; RWKV-v6 :278,296-298)
  relu_square, sigmoid_mul   channel-mix activations (RWKV-v5/src/module/ChannelMix.py:48-49)
  L2Wrap            RWKV-v5/src/model.py:123-148

  timemix5_forward / timemix6_forward / channelmix5_forward / channelmix6_forward take a module that holds the
  reference's parameters under the reference's names (time_mix_k ..., time_maa_x ..., receptance, key, value, gate,
  output, ln_x, time_decay, time_faaaa, n_head) and do what its _forward_cuda / forward does; the projections stay
  torch matmuls (hipBLASLt).

Every function here needs GPU tensors and the built library; there is no CPU path."""
from __future__ import annotations

import ctypes

import torch

from . import _lib
from ._lib import check
from .ops import _DT, _on_gpu, _ptr, _stream, _workspace, WKV_5, WKV_6

MAX_MIX = 5
LORA_MIXES, LORA_DIM = 5, 32      # the v6 TimeMix: five mixes, TIME_MIX_EXTRA_DIM = 32


def _ptr_array(ts):
    return (ctypes.c_void_p * len(ts))(*[t.data_ptr() for t in ts])


def _dtype_code(t):
    if t.dtype not in _DT:
        raise ValueError(f"Unsupported dtype {t.dtype}")
    return _DT[t.dtype]


class _ShiftMix(torch.autograd.Function):
    @staticmethod
    def forward(ctx, lerp, x, shift, coef, dyn):
        """coef (n, C) fp32; dyn (n, B, T, C) or None; returns n tensors (B, T, C)"""
        _on_gpu(x, shift, coef, dyn)
        B, T, C = x.shape
        n = coef.shape[0]
        assert 1 <= n <= MAX_MIX and coef.shape == (n, C) and coef.dtype == torch.float32
        x = x.contiguous()
        shift = shift.to(x.dtype).contiguous()
        assert shift.shape == (B, C)
        if dyn is not None:
            assert dyn.shape == (n, B, T, C) and dyn.dtype == x.dtype
            dyn = dyn.contiguous()
        outs = [torch.empty_like(x) for _ in range(n)]
        check(_lib.lib().wkv_shift_mix_forward(_stream(), B, T, C, _dtype_code(x), n, int(lerp), _ptr(x), _ptr(shift),
                                               _ptr(coef), _ptr(dyn), _ptr_array(outs)), "wkv_shift_mix_forward")
        ctx.lerp = int(lerp)
        ctx.save_for_backward(x, shift, coef, dyn)
        return tuple(outs)

    @staticmethod
    def backward(ctx, *gouts):
        x, shift, coef, dyn = ctx.saved_tensors
        B, T, C = x.shape
        n = coef.shape[0]
        gouts = [torch.zeros_like(x) if g is None else g.to(x.dtype).contiguous() for g in gouts]
        gx = torch.empty_like(x)
        gshift = torch.empty_like(shift)
        gcoef = torch.empty_like(coef)
        gdyn = torch.empty_like(dyn) if dyn is not None else None
        L = _lib.lib()
        ws = _workspace(L.wkv_shift_mix_backward_workspace(B, T, C, n), x.device)
        check(L.wkv_shift_mix_backward(_stream(), B, T, C, _dtype_code(x), n, ctx.lerp, _ptr(x), _ptr(shift), _ptr(coef),
                                       _ptr(dyn), _ptr_array(gouts), _ptr(gx), _ptr(gshift), _ptr(gcoef), _ptr(gdyn),
                                       _ptr(ws), ws.numel()), "wkv_shift_mix_backward")
        return None, gx, gshift, gcoef, gdyn


def token_shift_mix(x, shift_state, coefs, dyn=None, lerp=False):
    """x (B,T,C); shift_state (B,C) = the token before x[:,0]; coefs: sequence of n <= 5 parameters of C elements
    (any shape with C elements, any dtype; gradients flow back to them); dyn: optional (n,B,T,C).
    lerp=True : coefs are time_mix_*,  out_j = x * mix_j + xx * (1 - mix_j)         (v5)
    lerp=False: coefs are time_maa_*,  out_j = x + (xx - x) * (maa_j + dyn_j)       (v6)
    with xx the sequence shifted by one token.  Returns a tuple of n tensors."""
    C = x.shape[-1]
    coef = torch.stack([c.reshape(C).float() for c in coefs], 0)
    return _ShiftMix.apply(bool(lerp), x, shift_state, coef, dyn)


class _LoraMix(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, shift, coef, act, w2):
        """coef (5, C) fp32; act (B*T, 5, 32); w2 (5, 32, C); returns 5 tensors (B, T, C)"""
        _on_gpu(x, shift, coef, act, w2)
        B, T, C = x.shape
        assert x.dtype == torch.bfloat16 and act.dtype == x.dtype and w2.dtype == x.dtype
        assert coef.shape == (LORA_MIXES, C) and coef.dtype == torch.float32
        assert act.shape == (B * T, LORA_MIXES, LORA_DIM) and w2.shape == (LORA_MIXES, LORA_DIM, C)
        x, act = x.contiguous(), act.contiguous()
        shift = shift.to(x.dtype).contiguous()
        w2t = w2.transpose(1, 2).contiguous()                    # (5, C, 32): a channel's 32 factors side by side
        outs = [torch.empty_like(x) for _ in range(LORA_MIXES)]
        check(_lib.lib().wkv_lora_mix_forward(_stream(), B, T, C, _ptr(x), _ptr(shift), _ptr(coef), _ptr(act), _ptr(w2t),
                                              _ptr_array(outs)), "wkv_lora_mix_forward")
        ctx.save_for_backward(x, shift, coef, act, w2t)
        return tuple(outs)

    @staticmethod
    def backward(ctx, *gouts):
        x, shift, coef, act, w2t = ctx.saved_tensors
        B, T, C = x.shape
        gouts = [torch.zeros_like(x) if g is None else g.to(x.dtype).contiguous() for g in gouts]
        gx = torch.empty_like(x)
        gshift = torch.empty_like(shift)
        gcoef = torch.empty_like(coef)
        gdyn = torch.empty((LORA_MIXES, B * T, C), dtype=x.dtype, device=x.device)
        L = _lib.lib()
        ws = _workspace(L.wkv_lora_mix_backward_workspace(B, T, C), x.device)
        check(L.wkv_lora_mix_backward(_stream(), B, T, C, _ptr(x), _ptr(shift), _ptr(coef), _ptr(act), _ptr(w2t),
                                      _ptr_array(gouts), _ptr(gx), _ptr(gshift), _ptr(gcoef), _ptr(gdyn), _ptr(ws), ws.numel()),
              "wkv_lora_mix_backward")
        # the two reductions of the product's backward: over the channels for act, over the tokens for w2
        gact = torch.bmm(gdyn, w2t).transpose(0, 1)                               # (B*T, 5, 32)
        gw2 = torch.bmm(act.permute(1, 2, 0), gdyn)                               # (5, 32, C)
        return gx, gshift, gcoef, gact, gw2


def lora_shift_mix(x, shift_state, coefs, act, w2):
    """The five data-dependent mixes of the v6 TimeMix (RWKV-v6/src/module/TimeMix.py:264-276) from one read of x:
    out_j = x + (xx - x) * (maa_j + act[:, j] @ w2[j]),  xx the sequence shifted by one token;
    coefs = (time_maa_w, _k, _v, _r, _g); act (B*T, 5, 32) = tanh(xxx @ time_maa_w1) viewed as the reference views it;
    w2 = time_maa_w2 (5, 32, C).  The products act[:, j] @ w2[j] (the reference's mw, mk, mv, mr, mg) stay inside the
    kernel.  bf16, C a multiple of 8."""
    C = x.shape[-1]
    coef = torch.stack([c.reshape(C).float() for c in coefs], 0)
    return _LoraMix.apply(x, shift_state, coef, act, w2)


_lora_mix_on = True


def use_lora_mix(on):
    """timemix6_forward with (default) or without the fused pass, for comparisons; returns the previous setting"""
    global _lora_mix_on
    prev, _lora_mix_on = _lora_mix_on, bool(on)
    return prev


def lora_mix_available(x, act, w2):
    """whether lora_shift_mix takes these operands (else: bmm + token_shift_mix with dyn)"""
    return (_lora_mix_on and x.dtype == torch.bfloat16 and act.dtype == x.dtype and w2.dtype == x.dtype and x.shape[-1] % 8 == 0
            and act.shape[-1] == LORA_DIM and act.shape[-2] == LORA_MIXES)


class _LnGate(torch.autograd.Function):
    @staticmethod
    def forward(ctx, y, gate, weight, bias, scale, eps):
        _on_gpu(y, gate, weight, bias)
        C = y.shape[-1]
        y = y.contiguous()
        rows = y.numel() // C
        if gate is not None:
            assert gate.shape == y.shape and gate.dtype == y.dtype
            gate = gate.contiguous()
        w32, b32 = weight.float().contiguous(), bias.float().contiguous()
        out = torch.empty_like(y)
        check(_lib.lib().wkv_ln_gate_forward(_stream(), rows, C, _dtype_code(y), float(scale), float(eps), _ptr(y), _ptr(gate),
                                             _ptr(w32), _ptr(b32), _ptr(out)), "wkv_ln_gate_forward")
        ctx.scale, ctx.eps = float(scale), float(eps)
        ctx.param_dtypes = (weight.dtype, bias.dtype)
        ctx.save_for_backward(y, gate, w32, b32)
        return out

    @staticmethod
    def backward(ctx, gout):
        y, gate, w32, b32 = ctx.saved_tensors
        C = y.shape[-1]
        rows = y.numel() // C
        gout = gout.to(y.dtype).contiguous()
        gy = torch.empty_like(y)
        ggate = torch.empty_like(gate) if gate is not None else None
        gwb = torch.empty(2, C, dtype=torch.float32, device=y.device)
        L = _lib.lib()
        ws = _workspace(L.wkv_ln_gate_backward_workspace(rows, C), y.device)
        check(L.wkv_ln_gate_backward(_stream(), rows, C, _dtype_code(y), ctx.scale, ctx.eps, _ptr(y), _ptr(gate), _ptr(w32),
                                     _ptr(b32), _ptr(gout), _ptr(gy), _ptr(ggate), _ptr(gwb), _ptr(ws), ws.numel()),
              "wkv_ln_gate_backward")
        return gy, ggate, gwb[0].to(ctx.param_dtypes[0]), gwb[1].to(ctx.param_dtypes[1]), None, None


def ln_x_gate(y, gate, weight, bias, eps, scale=1.0):
    """(GroupNorm(y * scale, one group per 64 channels, eps) * weight + bias) * silu(gate); gate is the gate
    projection before its SiLU, or None.  v5: scale = 1/8, eps = 1e-5; v6: scale = 1, eps = 64e-5."""
    return _LnGate.apply(y, gate, weight, bias, scale, eps)


class _ReluSquare(torch.autograd.Function):
    @staticmethod
    def forward(ctx, k):
        _on_gpu(k)
        k = k.contiguous()
        out = torch.empty_like(k)
        check(_lib.lib().wkv_relu_square_forward(_stream(), k.numel(), _dtype_code(k), _ptr(k), _ptr(out)), "wkv_relu_square_forward")
        ctx.save_for_backward(k)
        return out

    @staticmethod
    def backward(ctx, gout):
        (k,) = ctx.saved_tensors
        gout = gout.to(k.dtype).contiguous()
        gk = torch.empty_like(k)
        check(_lib.lib().wkv_relu_square_backward(_stream(), k.numel(), _dtype_code(k), _ptr(k), _ptr(gout), _ptr(gk)),
              "wkv_relu_square_backward")
        return gk


class _SigmoidMul(torch.autograd.Function):
    @staticmethod
    def forward(ctx, r, kv):
        _on_gpu(r, kv)
        assert r.shape == kv.shape and r.dtype == kv.dtype
        r, kv = r.contiguous(), kv.contiguous()
        out = torch.empty_like(r)
        check(_lib.lib().wkv_sigmoid_mul_forward(_stream(), r.numel(), _dtype_code(r), _ptr(r), _ptr(kv), _ptr(out)),
              "wkv_sigmoid_mul_forward")
        ctx.save_for_backward(r, kv)
        return out

    @staticmethod
    def backward(ctx, gout):
        r, kv = ctx.saved_tensors
        gout = gout.to(r.dtype).contiguous()
        gr, gkv = torch.empty_like(r), torch.empty_like(kv)
        check(_lib.lib().wkv_sigmoid_mul_backward(_stream(), r.numel(), _dtype_code(r), _ptr(r), _ptr(kv), _ptr(gout), _ptr(gr),
                                                  _ptr(gkv)), "wkv_sigmoid_mul_backward")
        return gr, gkv


def relu_square(k):
    """relu(k) ** 2"""
    return _ReluSquare.apply(k)


def sigmoid_mul(r, kv):
    """sigmoid(r) * kv"""
    return _SigmoidMul.apply(r, kv)


class L2Wrap(torch.autograd.Function):
    """The reference's L2Wrap (RWKV-v5/src/model.py:123-148), same arguments: returns `loss` unchanged and sends
    factor * max(y, -1) back to the position of each row's maximum, times the token mask."""

    @staticmethod
    def forward(ctx, loss, y, factor, currentMask):
        ctx.save_for_backward(y, torch.as_tensor(factor), currentMask)
        return loss

    @staticmethod
    def backward(ctx, grad_output):
        y, factor, mask = ctx.saved_tensors
        _on_gpu(y)
        V = y.shape[-1]
        yc = y.contiguous()
        rows = yc.numel() // V
        m32 = None if mask is None else mask.reshape(rows).float().contiguous()
        gy = torch.empty_like(yc)
        check(_lib.lib().wkv_l2wrap_backward(_stream(), rows, V, _dtype_code(yc), float(factor), _ptr(yc), _ptr(m32), _ptr(gy)),
              "wkv_l2wrap_backward")
        return grad_output, gy, None, None


# ---- block forwards on these kernels -------------------------------------------------------------------------------
def timemix5_forward(self, x, last_state):
    """RWKV_TimeMix._forward_cuda of v5 (RWKV-v5/src/module/TimeMix.py:286-323): returns
    (out (B,T,C), (shift_state_out (B,C), wkv_state_out (B,H,64,64)))."""
    B, T, C = x.shape
    H = self.n_head
    xk, xv, xr, xg = token_shift_mix(x, last_state[0], (self.time_mix_k, self.time_mix_v, self.time_mix_r, self.time_mix_g),
                                     lerp=True)
    r, k, v, gate = self.receptance(xr), self.key(xk), self.value(xv), self.gate(xg)
    y, new_state = WKV_5.apply(B, T, C, H, last_state[1], r, k, v, self.time_decay.float(), self.time_faaaa)
    y = ln_x_gate(y, gate, self.ln_x.weight, self.ln_x.bias, self.ln_x.eps, scale=1.0 / 8)     # head_size_divisor = 8
    return self.output(y), (x[:, -1], new_state)


def timemix6_forward(self, x, last_state):
    """RWKV_TimeMix6_0._forward_cuda (RWKV-v6/src/module/TimeMix.py:253-302)."""
    B, T, C = x.shape
    H = self.n_head
    (xxx,) = token_shift_mix(x, last_state[0], (self.time_maa_x,))
    act = torch.tanh(xxx @ self.time_maa_w1).view(B * T, 5, -1)
    maas = (self.time_maa_w, self.time_maa_k, self.time_maa_v, self.time_maa_r, self.time_maa_g)
    if lora_mix_available(x, act, self.time_maa_w2):
        xw, xk, xv, xr, xg = lora_shift_mix(x, last_state[0], maas, act, self.time_maa_w2)
    else:       # other dtypes / LoRA sizes: the products through memory
        dyn = torch.bmm(act.transpose(0, 1), self.time_maa_w2).view(5, B, T, C)                 # mw, mk, mv, mr, mg
        xw, xk, xv, xr, xg = token_shift_mix(x, last_state[0], maas, dyn=dyn)
    r, k, v, gate = self.receptance(xr), self.key(xk), self.value(xv), self.gate(xg)
    # w = time_decay + tanh(xw @ w1) @ w2 (TimeMix.py:280-281): the broadcast addition rides on the second matmul as
    # its bias epilogue instead of being a pass of its own over (B,T,C)
    lora = torch.tanh(xw.view(B * T, C) @ self.time_decay_w1)
    w = torch.addmm(self.time_decay.reshape(C), lora, self.time_decay_w2).view(B, T, C)
    y, new_state = WKV_6.apply(B, T, C, H, r, k, v, w, self.time_faaaa, last_state[1])
    y = ln_x_gate(y, gate, self.ln_x.weight, self.ln_x.bias, self.ln_x.eps, scale=1.0)
    return self.output(y), (x[:, -1], new_state)


def channelmix5_forward(self, x, last_state):
    """RWKV_ChannelMix.forward of v5 (RWKV-v5/src/module/ChannelMix.py:35-49)."""
    xk, xr = token_shift_mix(x, last_state, (self.time_mix_k, self.time_mix_r), lerp=True)
    kv = self.value(relu_square(self.key(xk)))
    return sigmoid_mul(self.receptance(xr), kv), x[:, -1]


def channelmix6_forward(self, x, last_state):
    """RWKV_ChannelMix6_0.forward (RWKV-v6/src/module/ChannelMix.py:30-37)."""
    xk, xr = token_shift_mix(x, last_state, (self.time_maa_k, self.time_maa_r))
    kv = self.value(relu_square(self.key(xk)))
    return sigmoid_mul(self.receptance(xr), kv), x[:, -1]
