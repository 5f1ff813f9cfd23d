"""Pins the v4 CPU oracle (C restatement of the reference kernel's recurrence)
by mathematics: the reference has no CPU path, test or fixture for it."""
import pytest
import torch

from oracle import wkv4 as O4

D = torch.float64


def case(B=2, T=10, C=6, seed=0):
    g = torch.Generator().manual_seed(seed)
    k = torch.randn(B, T, C, generator=g, dtype=D)
    v = torch.randn(B, T, C, generator=g, dtype=D)
    td = torch.rand(C, generator=g, dtype=D) * 6 - 5
    tf = torch.randn(C, generator=g, dtype=D) * 0.5
    st = torch.zeros(B, C, 3, dtype=D)
    st[..., 2] = -1e38
    return td, tf, k, v, st


def test_forward_is_softmax_average():
    td, tf, k, v, st = case()
    y, ns = O4.forward(td, tf, k, v, st, real="f64")
    for t in range(k.size(1)):
        assert torch.allclose(y[:, t], O4.wkv4_softmax_form(td, tf, k, v, t), rtol=1e-12, atol=1e-12)
    # state handed out holds the decayed sums: P = p e^o, Q = q e^o
    T = k.size(1)
    w = -torch.exp(td)
    s = torch.arange(T, dtype=D)
    lg = k + ((T - 1 - s).view(1, T, 1) * w)
    P = (torch.exp(lg) * v).sum(1)
    Q = torch.exp(lg).sum(1)
    assert torch.allclose(ns[..., 0] * torch.exp(ns[..., 2]), P, rtol=1e-12)
    assert torch.allclose(ns[..., 1] * torch.exp(ns[..., 2]), Q, rtol=1e-12)


def test_first_token_and_minus_inf_bonus():
    td, tf, k, v, st = case(T=4)
    y, _ = O4.forward(td, tf, k, v, st, real="f64")
    assert torch.allclose(y[:, 0], v[:, 0], atol=1e-13)            # empty history: y_0 = v_0
    y2, _ = O4.forward(td, torch.full_like(tf, -200.0), k, v, st, real="f64")
    # a very negative time_first removes the current token from its own output
    w = -torch.exp(td)
    lg = torch.stack([k[:, 0] + w, k[:, 1]], 1)
    assert torch.allclose(y2[:, 2], (torch.softmax(lg, 1) * v[:, :2]).sum(1), atol=1e-12)


def test_c_matches_torch_loop_and_f32():
    td, tf, k, v, st = case(B=3, T=64, C=16, seed=1)
    y, ns = O4.forward(td, tf, k, v, st, real="f64")
    y2, ns2 = O4.wkv4_torch_loop(td, tf, k, v, st)
    assert torch.allclose(y, y2, atol=1e-12) and torch.allclose(ns, ns2, atol=1e-12)
    y3, ns3 = O4.forward(td, tf, k, v, st, real="f32")
    assert (y3.double() - y).abs().max() < 1e-5
    assert y3.dtype == torch.float32


def test_chaining_forward():
    td, tf, k, v, st = case(T=12)
    y, ns = O4.forward(td, tf, k, v, st, real="f64")
    y1, s1 = O4.forward(td, tf, k[:, :5], v[:, :5], st, real="f64")
    y2, s2 = O4.forward(td, tf, k[:, 5:], v[:, 5:], s1, real="f64")
    assert torch.allclose(torch.cat([y1, y2], 1), y, atol=1e-12)
    P = lambda s: s[..., :2] * torch.exp(s[..., 2:3])
    assert torch.allclose(P(s2), P(ns), rtol=1e-12)


@pytest.mark.parametrize("with_state", [False, True])
def test_backward_equals_autograd_of_undivided_form(with_state):
    td, tf, k, v, st = case(B=2, T=9, C=5, seed=2)
    g = torch.Generator().manual_seed(3)
    gy = torch.randn(k.shape, generator=g, dtype=D)
    B, T, C = k.shape
    if with_state:
        st = torch.stack([torch.randn(B, C, generator=g, dtype=D),
                          torch.rand(B, C, generator=g, dtype=D) + 0.5,
                          torch.randn(B, C, generator=g, dtype=D)], -1)
        gns = torch.stack([torch.randn(B, C, generator=g, dtype=D),
                           torch.randn(B, C, generator=g, dtype=D),
                           torch.randn(B, C, generator=g, dtype=D) * 0.3], -1)
    else:
        gns = torch.zeros(B, C, 3, dtype=D)
    P0 = st[..., 0] * torch.exp(st[..., 2])
    Q0 = st[..., 1] * torch.exp(st[..., 2])
    leaves = [x.clone().requires_grad_(True) for x in (td, tf, k, v, P0, Q0)]
    y, PT, QT = O4.wkv4_undivided(*leaves)
    gP, gQ = gns[..., 0] * torch.exp(gns[..., 2]), gns[..., 1] * torch.exp(gns[..., 2])
    loss = (y * gy).sum() + (PT * gP).sum() + (QT * gQ).sum()
    a_td, a_tf, a_k, a_v, a_P, a_Q = torch.autograd.grad(loss, leaves)
    gw, gu, gk, gv, gl = O4.backward(td, tf, k, v, st, gy, gns, real="f64")
    assert torch.allclose(gk, a_k, rtol=1e-9, atol=1e-10)
    assert torch.allclose(gv, a_v, rtol=1e-9, atol=1e-10)
    assert torch.allclose(gu, a_tf, rtol=1e-9, atol=1e-10)
    assert torch.allclose(gw, a_td, rtol=1e-9, atol=1e-10)
    assert torch.allclose(gl[..., 0] * torch.exp(gl[..., 2]), a_P, rtol=1e-9, atol=1e-12)
    assert torch.allclose(gl[..., 1] * torch.exp(gl[..., 2]), a_Q, rtol=1e-9, atol=1e-12)


def test_backward_chaining():
    td, tf, k, v, st = case(T=12, seed=4)
    g = torch.Generator().manual_seed(5)
    gy = torch.randn(k.shape, generator=g, dtype=D)
    zero = torch.zeros_like(st)
    full = O4.backward(td, tf, k, v, st, gy, zero, real="f64")
    _, s1 = O4.forward(td, tf, k[:, :7], v[:, :7], st, real="f64")
    b2 = O4.backward(td, tf, k[:, 7:], v[:, 7:], s1, gy[:, 7:], zero, real="f64")
    b1 = O4.backward(td, tf, k[:, :7], v[:, :7], st, gy[:, :7], b2[4], real="f64")
    assert torch.allclose(torch.cat([b1[2], b2[2]], 1), full[2], rtol=1e-10, atol=1e-12)
    assert torch.allclose(torch.cat([b1[3], b2[3]], 1), full[3], rtol=1e-10, atol=1e-12)
    assert torch.allclose(b1[0] + b2[0], full[0], rtol=1e-10, atol=1e-12)
    assert torch.allclose(b1[1] + b2[1], full[1], rtol=1e-10, atol=1e-12)
