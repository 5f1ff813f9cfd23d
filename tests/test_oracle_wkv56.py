"""Pins the WKV5/WKV6 CPU oracle by mathematics (the reference holds no
tensor-level fixture for this path): closed forms, library special cases,
invariants and three independent gradient computations."""
import math

import pytest
import torch

from oracle import wkv56 as O

torch.manual_seed(0)
D = torch.float64


def rand_case(B=2, H=2, L=12, K=5, V=4, per_token_w=True, seed=0, dtype=D, wlo=0.05):
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g, dtype=dtype)
    r, k, v = rn(B, H, L, K), rn(B, H, L, K), rn(B, H, L, V)
    w = torch.rand(B if per_token_w else 1, H, L if per_token_w else 1, K, generator=g, dtype=dtype) * (0.999 - wlo) + wlo
    if not per_token_w:
        w = w.expand(1, H, L, K)
    u = rn(1, H, 1, K)
    S = rn(B, H, K, V)
    return r, k, v, w, u, S


def closed_form(r, k, v, w, u, S):
    """y and S_out from explicit sums over token pairs; no recurrence."""
    B, H, L, K = k.shape
    V = v.size(-1)
    w = w.expand(B, H, L, K)
    y = torch.zeros(B, H, L, V, dtype=r.dtype)
    for t in range(L):
        carried = torch.ones(B, H, K, dtype=r.dtype)
        for tau in range(t):
            carried = carried * w[:, :, tau]
        y[:, :, t] += torch.einsum('bhk,bhkv->bhv', r[:, :, t] * carried, S)
        for s in range(t):
            dec = torch.ones(B, H, K, dtype=r.dtype)
            for tau in range(s + 1, t):
                dec = dec * w[:, :, tau]
            y[:, :, t] += (r[:, :, t] * dec * k[:, :, s]).sum(-1, keepdim=True) * v[:, :, s]
        y[:, :, t] += (r[:, :, t] * u[0, :, 0] * k[:, :, t]).sum(-1, keepdim=True) * v[:, :, t]
    total = w.prod(dim=2)
    S_out = total.unsqueeze(-1) * S
    for s in range(L):
        dec = w[:, :, s + 1:].prod(dim=2)
        S_out = S_out + (dec * k[:, :, s]).unsqueeze(-1) * v[:, :, s].unsqueeze(-2)
    return y, S_out


@pytest.mark.parametrize("per_token_w", [True, False])
def test_token_loop_equals_closed_form(per_token_w):
    c = rand_case(per_token_w=per_token_w, L=9)
    y, s = O.wkv_token_loop(*c)
    y2, s2 = closed_form(*c)
    assert torch.allclose(y, y2, rtol=1e-12, atol=1e-12)
    assert torch.allclose(s, s2, rtol=1e-12, atol=1e-12)


def test_no_decay_no_bonus_is_a_cumsum():
    r, k, v, w, u, S = rand_case(L=16)
    w = torch.ones_like(w)
    u = torch.zeros_like(u)
    S = torch.zeros_like(S)
    y, s = O.wkv_token_loop(r, k, v, w, u, S)
    kv = k.unsqueeze(-1) * v.unsqueeze(-2)                       # (B,H,L,K,V)
    hist = kv.cumsum(dim=2) - kv                                  # strictly earlier tokens
    assert torch.allclose(y, torch.einsum('bhlk,bhlkv->bhlv', r, hist), atol=1e-12)
    assert torch.allclose(s, kv.sum(dim=2), atol=1e-12)


def test_single_token():
    r, k, v, w, u, S = rand_case(L=1)
    y, s = O.wkv_token_loop(r, k, v, w, u, torch.zeros_like(S))
    assert torch.allclose(y, (r * u * k).sum(-1, keepdim=True) * v, atol=1e-13)
    assert torch.allclose(s, k.mT @ v, atol=1e-13)
    # zero receptance: no output, the state still moves
    y0, s0 = O.wkv_token_loop(torch.zeros_like(r), k, v, w, u, S)
    assert y0.abs().max() == 0 and not torch.equal(s0, S)


def test_linearity_in_v_and_state():
    r, k, v, w, u, S = rand_case()
    r2, k2, v2, _, _, S2 = rand_case(seed=1)
    a, b = 0.7, -1.3
    y1, s1 = O.wkv_token_loop(r, k, v, w, u, S)
    y2, s2 = O.wkv_token_loop(r, k, v2, w, u, S2)
    y3, s3 = O.wkv_token_loop(r, k, a * v + b * v2, w, u, a * S + b * S2)
    assert torch.allclose(y3, a * y1 + b * y2, atol=1e-11)
    assert torch.allclose(s3, a * s1 + b * s2, atol=1e-11)


def test_batch_and_head_permutation():
    r, k, v, w, u, S = rand_case(B=3, H=3)
    pb, ph = torch.tensor([2, 0, 1]), torch.tensor([1, 2, 0])
    y, s = O.wkv_token_loop(r, k, v, w, u, S)
    f = lambda x: x[pb][:, ph] if x.size(0) == 3 else x[:, ph]
    yp, sp = O.wkv_token_loop(f(r), f(k), f(v), f(w), f(u), f(S))
    assert torch.equal(yp, f(y)) and torch.equal(sp, f(s))


@pytest.mark.parametrize("per_token_w", [True, False])
@pytest.mark.parametrize("T,L", [(4, 16), (16, 64), (128, 256)])
def test_chunked_equals_token_loop_fp64(per_token_w, T, L):
    c = rand_case(B=2, H=2, L=L, K=8, V=8, per_token_w=per_token_w, wlo=0.006)
    y, s = O.wkv_token_loop(*c)
    y2, s2 = O.wkv_chunked(*c, chunk_len=T, precision=64)
    # the chunked path takes log(w) and its cumsum in fp32 whatever the input
    # dtype (rwkv_inner.py:51-55): with decays down to 0.006 the cumulative log
    # reaches -5*T, so agreement is to fp32 rounding of that sum
    tol = 1e-7 * 5 * T
    assert (y - y2).abs().max() <= tol * y.abs().max()
    assert (s - s2).abs().max() <= tol * s.abs().max()


def test_chunked_fp32_io_close_to_fp64():
    c = rand_case(B=1, H=2, L=256, K=64, V=64, wlo=0.3)
    y, s = O.wkv_token_loop(*c)
    c32 = tuple(x.float() for x in c)
    y2, s2 = O.wkv_chunked(*c32, chunk_len=128, precision=64)
    assert (y2.double() - y).abs().max() <= 1e-4 * y.abs().max()
    assert (s2.double() - s).abs().max() <= 1e-4 * s.abs().max()


def test_floor_on_decay():
    """w below 0.005 acts as 0.005 on the chunked path and in the floored token
    loop, and passes untouched through the single-step branch."""
    r, k, v, w, u, S = rand_case(L=8, K=4, V=4)
    w = w.clone()
    w[:, :, 3, 1] = 1e-4
    wf = w.clamp(0.005)
    y_floor, s_floor = O.wkv_token_loop(r, k, v, wf, u, S)
    y_c, s_c = O.wkv_chunked(r, k, v, w, u, S, chunk_len=4)
    y_l, s_l = O.wkv_token_loop(r, k, v, w, u, S, floor_decay=True)
    assert torch.allclose(y_c, y_floor, atol=1e-5) and torch.allclose(s_c, s_floor, atol=1e-5)
    assert torch.equal(y_l, y_floor) and torch.equal(s_l, s_floor)
    y_raw, _ = O.wkv_token_loop(r, k, v, w, u, S)
    assert not torch.allclose(y_raw, y_floor, atol=1e-6)


def test_helper_identities():
    _, _, _, w, _, _ = rand_case(L=64, K=8, wlo=0.001)
    T = 16
    tab = O.cumsum_decay(w, T, 64)
    lw = tab.log_w.view(w.size(0), w.size(1), -1, T, w.size(-1))
    assert torch.equal(tab.log_w, w.clamp(0.005).float().log())
    assert tab.log_w.min() >= math.log(0.005) - 1e-6
    assert torch.allclose(tab.inter_log + tab.incl, tab.chunk_log.expand_as(tab.incl), atol=1e-5)
    assert torch.allclose(tab.intra_log, tab.excl, atol=1e-5)
    assert torch.allclose(tab.incl - lw, tab.excl, atol=1e-5)
    assert tab.excl[..., 0, :].abs().max() == 0
    # decay over the whole chunk = decay up to the last token times the last token's decay
    assert torch.allclose(tab.intra_log[..., -1, :] + lw[..., -1, :], tab.chunk_log[..., 0, :], atol=1e-5)
    # the two re-centred factors multiply to the decay between token s (exclusive) and t (exclusive)
    t, s = 11, 3
    prod = tab.r_decay[..., t, :] * tab.k_inv_decay[..., s, :]
    direct = lw[..., s + 1:t, :].double().sum(dim=-2).exp()
    assert torch.allclose(prod, direct, rtol=1e-5)
    assert tab.r_decay.dtype == torch.float64
    assert O.cumsum_decay(w, T, 32).r_decay.dtype == torch.float32


def _autograd(c, gy, gS):
    leaves = [x.clone().requires_grad_(True) for x in c]
    y, s = O.wkv_token_loop(*leaves)
    loss = (y * gy).sum() + (s * gS).sum()
    return torch.autograd.grad(loss, leaves), y.detach(), s.detach()


@pytest.mark.parametrize("per_token_w", [True, False])
def test_adjoint_equals_autograd(per_token_w):
    c = rand_case(per_token_w=per_token_w)
    if not per_token_w:
        c = c[:3] + (c[3].contiguous(),) + c[4:]
    r, k, v, w, u, S = c
    g = torch.Generator().manual_seed(5)
    gy = torch.randn(v.shape, generator=g, dtype=D)
    gS = torch.randn(S.shape, generator=g, dtype=D)
    (ar, ak, av, aw, au, aS), y, s_out = _autograd(c, gy, gS)
    gr, gk, gv, gw, gu, gS_in = O.wkv_adjoint(r, k, v, w, u, S, gy, gS)
    for a, b in ((ar, gr), (ak, gk), (av, gv), (au, gu), (aS, gS_in)):
        assert torch.allclose(a, b, rtol=1e-11, atol=1e-11)
    if per_token_w:
        assert torch.allclose(aw, gw, rtol=1e-11, atol=1e-11)
    else:
        assert torch.allclose(aw.sum(0, keepdim=True), gw.sum(0, keepdim=True), rtol=1e-11, atol=1e-11)
    # the state-free scan gives the same decay gradient, including the boundary term
    Dscan = O.decay_grad_by_scan(r, k, v, w, u, gy, gr, gk, s_out, gS)
    assert torch.allclose(Dscan, w.expand_as(gw) * gw, rtol=1e-10, atol=1e-10)


def test_gradcheck_token_loop():
    c = tuple(x.requires_grad_(True) for x in rand_case(B=1, H=1, L=5, K=3, V=2))
    assert torch.autograd.gradcheck(lambda *a: O.wkv_token_loop(*a), c, eps=1e-6, atol=1e-6)


def test_chunked_autograd_equals_adjoint():
    c = rand_case(B=1, H=2, L=32, K=8, V=8, wlo=0.05)
    r, k, v, w, u, S = c
    g = torch.Generator().manual_seed(6)
    gy = torch.randn(v.shape, generator=g, dtype=D)
    gS = torch.randn(S.shape, generator=g, dtype=D)
    leaves = [x.clone().requires_grad_(True) for x in c]
    y, s = O.wkv_chunked(*leaves, chunk_len=8)
    got = torch.autograd.grad((y * gy).sum() + (s * gS).sum(), leaves)
    want = O.wkv_adjoint(r, k, v, w, u, S, gy, gS)
    for a, b in zip(got, want):                      # fp32 log(w) inside the chunked path
        assert (a - b).abs().max() <= 1e-5 * b.abs().max()


def test_segment_chaining_outputs_and_grads():
    """One call over 2L tokens == two chained calls over L tokens, for outputs
    and, with the state gradient passed back, for every gradient."""
    c = rand_case(L=16)
    r, k, v, w, u, S = c
    g = torch.Generator().manual_seed(7)
    gy = torch.randn(v.shape, generator=g, dtype=D)
    gS = torch.randn(S.shape, generator=g, dtype=D)
    full = O.wkv_adjoint(r, k, v, w, u, S, gy, gS)
    h = 8
    a = lambda x: x[:, :, :h]
    b = lambda x: x[:, :, h:]
    y1, s1 = O.wkv_token_loop(a(r), a(k), a(v), a(w), u, S)
    y2, s2 = O.wkv_token_loop(b(r), b(k), b(v), b(w), u, s1)
    yf, sf = O.wkv_token_loop(*c)
    assert torch.allclose(torch.cat([y1, y2], 2), yf, atol=1e-12) and torch.allclose(s2, sf, atol=1e-12)
    g2 = O.wkv_adjoint(b(r), b(k), b(v), b(w), u, s1, b(gy), gS)
    g1 = O.wkv_adjoint(a(r), a(k), a(v), a(w), u, S, a(gy), g2[5])
    for i in range(4):
        assert torch.allclose(torch.cat([g1[i], g2[i]], 2), full[i], atol=1e-11)
    assert torch.allclose(g1[4] + g2[4], full[4], atol=1e-11)
    assert torch.allclose(g1[5], full[5], atol=1e-11)


@pytest.mark.parametrize("version", [5, 6])
def test_operator_front_end(version):
    """(B,T,C) front ends: v5 == v6 with the decay broadcast; raw-decay
    gradient = chain rule through exp(-exp(x)) of the adjoint's gw."""
    B, T, H, K = 2, 8, 2, 64
    C = H * K
    g = torch.Generator().manual_seed(8)
    rn = lambda *s: torch.randn(*s, generator=g, dtype=D)
    r, k, v, gy = (rn(B, T, C) * 0.5 for _ in range(4))
    u, S, gS = rn(H, K), rn(B, H, K, K), rn(B, H, K, K)
    w5 = torch.rand(H, K, generator=g, dtype=D) * 3 - 4
    w6 = w5.view(1, 1, C).expand(B, T, C).contiguous()
    o5 = O.wkv_op_grads(5, B, T, C, H, r, k, v, w5.float(), u, S, gy, gS, dtype=D, chunk_len=4)
    o6 = O.wkv_op_grads(6, B, T, C, H, r, k, v, w6.float(), u, S, gy, gS, dtype=D, chunk_len=4)
    for n in ('y', 'state', 'gr', 'gk', 'gv', 'gu', 'gstate'):
        assert torch.allclose(o5[n], o6[n], rtol=1e-9, atol=1e-9), n
    assert torch.allclose(o5['gw'], o6['gw'].sum((0, 1)).view(H, K), rtol=1e-4, atol=1e-6)
    # chain rule against the closed-form adjoint
    hd = lambda x: x.view(B, T, H, K).transpose(1, 2)
    w = O.decay_from_raw(w6.float()).double()
    adj = O.wkv_adjoint(hd(r), hd(k), hd(v), hd(w), u.view(1, H, 1, K), S, hd(gy), gS)
    want = adj[3] * hd(w) * (-torch.exp(hd(w6)))
    assert torch.allclose(hd(o6['gw'].double()), want, rtol=1e-4, atol=1e-6)
