"""Test infrastructure (only tests may use it): restatement of the reference's TimeMix forward passes around the WKV
operator (RWKV-v5/src/module/TimeMix.py:286-366, RWKV-v6/src/module/TimeMix.py:253-351),
with the operator injected, so that the same module can run on the CPU oracle
(the reference's pure path) and on the HIP operators (its CUDA path)."""
import torch
import torch.nn as nn
import torch.nn.functional as F


def group_norm(mod, x, n_head):
    """nn.GroupNorm(n_head, C) on (N, C), written out (plain ops have the same
    backward on every device; the fused kernels' weight gradients differ between builds)."""
    N, C = x.shape
    xg = x.view(N, n_head, C // n_head)
    mean = xg.mean(-1, keepdim=True)
    var = xg.var(-1, unbiased=False, keepdim=True)
    xn = ((xg - mean) * torch.rsqrt(var + mod.eps)).view(N, C)
    return xn * mod.weight + mod.bias


class TimeMix5(nn.Module):
    def __init__(self, n_embd, n_head, seed=0):
        super().__init__()
        g = torch.Generator().manual_seed(seed)
        K = n_embd // n_head
        self.n_head, self.head_size = n_head, K
        u01 = lambda *s: torch.rand(*s, generator=g)
        self.time_mix_k = nn.Parameter(u01(1, 1, n_embd))
        self.time_mix_v = nn.Parameter(u01(1, 1, n_embd))
        self.time_mix_r = nn.Parameter(u01(1, 1, n_embd))
        self.time_mix_g = nn.Parameter(u01(1, 1, n_embd))
        self.time_decay = nn.Parameter(u01(n_head, K) * 5 - 6)
        self.time_faaaa = nn.Parameter(torch.randn(n_head, K, generator=g) * 0.3)
        lin = lambda: nn.Linear(n_embd, n_embd, bias=False)
        self.receptance, self.key, self.value, self.output, self.gate = lin(), lin(), lin(), lin(), lin()
        for m in (self.receptance, self.key, self.value, self.output, self.gate):
            with torch.no_grad():
                m.weight.copy_(torch.randn(n_embd, n_embd, generator=g) * (n_embd ** -0.5))
        self.ln_x = nn.GroupNorm(n_head, n_embd)

    def forward(self, x, last_state, wkv):
        """wkv(B,T,C,H,state,r,k,v,time_decay,time_faaaa) -> (y (B,T,C), new_state)"""
        B, T, C = x.shape
        H = self.n_head
        xx = torch.cat((last_state[0].unsqueeze(1), x[:, :-1]), dim=1)
        lerp = lambda mix: x * mix + xx * (1 - mix)              # modified_lerp(x, mix, xx)
        r = self.receptance(lerp(self.time_mix_r))
        k = self.key(lerp(self.time_mix_k))
        v = self.value(lerp(self.time_mix_v))
        gate = F.silu(self.gate(lerp(self.time_mix_g)))
        y, new_state = wkv(B, T, C, H, last_state[1], r, k, v, self.time_decay.float(), self.time_faaaa)
        y = group_norm(self.ln_x, y.reshape(-1, C) / 8, H).view(B, T, C)        # head_size_divisor = 8
        return self.output(y * gate), (x[:, -1], new_state)


class TimeMix6(nn.Module):
    def __init__(self, n_embd, n_head, seed=0):
        super().__init__()
        g = torch.Generator().manual_seed(seed)
        K = n_embd // n_head
        self.n_head, self.head_size = n_head, K
        u01 = lambda *s: torch.rand(*s, generator=g)
        for nm in ("x", "w", "k", "v", "r", "g"):
            setattr(self, f"time_maa_{nm}", nn.Parameter(u01(1, 1, n_embd)))
        self.time_maa_w1 = nn.Parameter((u01(n_embd, 32 * 5) - 0.5) * 0.2)
        self.time_maa_w2 = nn.Parameter((u01(5, 32, n_embd) - 0.5) * 0.2)
        self.time_decay = nn.Parameter(u01(1, 1, n_embd) * 5 - 6)
        self.time_decay_w1 = nn.Parameter((u01(n_embd, 64) - 0.5) * 0.2)
        self.time_decay_w2 = nn.Parameter((u01(64, n_embd) - 0.5) * 0.5)
        self.time_faaaa = nn.Parameter(torch.randn(n_head, K, generator=g) * 0.3)
        lin = lambda: nn.Linear(n_embd, n_embd, bias=False)
        self.receptance, self.key, self.value, self.output, self.gate = lin(), lin(), lin(), lin(), lin()
        for m in (self.receptance, self.key, self.value, self.output, self.gate):
            with torch.no_grad():
                m.weight.copy_(torch.randn(n_embd, n_embd, generator=g) * (n_embd ** -0.5))
        self.ln_x = nn.GroupNorm(n_head, n_embd, eps=1e-5 * 64)

    def forward(self, x, last_state, wkv):
        """wkv(B,T,C,H,r,k,v,w,u,state) -> (y, new_state)"""
        B, T, C = x.shape
        H = self.n_head
        dxprev = torch.cat((last_state[0].unsqueeze(1), x[:, :-1]), dim=1) - x
        xxx = x + dxprev * self.time_maa_x
        xxx = torch.tanh(xxx @ self.time_maa_w1).view(B * T, 5, -1).transpose(0, 1)
        xxx = torch.bmm(xxx, self.time_maa_w2).view(5, B, T, -1)
        mw, mk, mv, mr, mg = xxx.unbind(dim=0)
        r = self.receptance(x + dxprev * (self.time_maa_r + mr))
        k = self.key(x + dxprev * (self.time_maa_k + mk))
        v = self.value(x + dxprev * (self.time_maa_v + mv))
        gate = F.silu(self.gate(x + dxprev * (self.time_maa_g + mg)))
        xw = x + dxprev * (self.time_maa_w + mw)
        w = self.time_decay + torch.tanh(xw @ self.time_decay_w1) @ self.time_decay_w2
        y, new_state = wkv(B, T, C, H, r, k, v, w.contiguous(), self.time_faaaa, last_state[1])
        y = group_norm(self.ln_x, y.reshape(-1, C), H).view(B, T, C)
        return self.output(y * gate), (x[:, -1], new_state)


class ChannelMix5(nn.Module):
    """RWKV-v5/src/module/ChannelMix.py:7-49 with seeded parameters; forward = the oracle's restatement"""
    def __init__(self, n_embd, dim_ffn, seed=0):
        super().__init__()
        g = torch.Generator().manual_seed(seed)
        self.time_mix_k = nn.Parameter(torch.rand(1, 1, n_embd, generator=g))
        self.time_mix_r = nn.Parameter(torch.rand(1, 1, n_embd, generator=g))
        self.key = nn.Linear(n_embd, dim_ffn, bias=False)
        self.receptance = nn.Linear(n_embd, n_embd, bias=False)
        self.value = nn.Linear(dim_ffn, n_embd, bias=False)
        with torch.no_grad():
            for m in (self.key, self.receptance, self.value):
                m.weight.copy_(torch.randn(m.weight.shape, generator=g) * (m.weight.shape[1] ** -0.5))

    def forward(self, x, last_state):
        from oracle.blocks import channelmix5_forward
        return channelmix5_forward(self, x, last_state)


class ChannelMix6(nn.Module):
    """RWKV-v6/src/module/ChannelMix.py:7-37 with seeded parameters"""
    def __init__(self, n_embd, dim_ffn, seed=0):
        super().__init__()
        g = torch.Generator().manual_seed(seed)
        self.time_maa_k = nn.Parameter(torch.rand(1, 1, n_embd, generator=g))
        self.time_maa_r = nn.Parameter(torch.rand(1, 1, n_embd, generator=g))
        self.key = nn.Linear(n_embd, dim_ffn, bias=False)
        self.receptance = nn.Linear(n_embd, n_embd, bias=False)
        self.value = nn.Linear(dim_ffn, n_embd, bias=False)
        with torch.no_grad():
            for m in (self.key, self.receptance, self.value):
                m.weight.copy_(torch.randn(m.weight.shape, generator=g) * (m.weight.shape[1] ** -0.5))

    def forward(self, x, last_state):
        from oracle.blocks import channelmix6_forward
        return channelmix6_forward(self, x, last_state)
