"""Pins oracle/blocks.py (the CPU oracle of the element-wise passes around the operator) against what the
mathematics fixes: special cases, index loops and library routines that a wrong sign, index or operand would fail."""
import numpy as np
import torch
import torch.nn.functional as F

from oracle import blocks as OB


def _rand(*shape, seed=0, dtype=torch.float64):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=dtype)


def test_token_shift_is_an_index_shift():
    x, s = _rand(2, 5, 3), _rand(2, 3, seed=1)
    xx = OB.token_shift(x, s)
    for b in range(2):
        for t in range(5):
            assert torch.equal(xx[b, t], s[b] if t == 0 else x[b, t - 1])


def test_mixes_at_the_ends_of_the_coefficient_range():
    x, s = _rand(2, 6, 8), _rand(2, 8, seed=1)
    one, zero = torch.ones(1, 1, 8, dtype=x.dtype), torch.zeros(1, 1, 8, dtype=x.dtype)
    xx = OB.token_shift(x, s)
    a, b = OB.mix_v5(x, s, (one, zero))              # time_mix weighs x itself
    assert torch.equal(a, x) and torch.equal(b, xx)
    a, b = OB.mix_v6(x, s, (zero, one))              # time_maa weighs the difference to the previous token
    assert torch.equal(a, x) and torch.allclose(b, xx, atol=1e-15)
    m = torch.rand(1, 1, 8, dtype=x.dtype)
    (v5,) = OB.mix_v5(x, s, (m,))
    (v6,) = OB.mix_v6(x, s, (1 - m,))                # the two parametrisations agree at maa = 1 - mix
    assert torch.allclose(v5, v6, atol=1e-14)
    dyn = _rand(1, 2, 6, 8, seed=2)
    (d,) = OB.mix_v6(x, s, (m,), dyn)
    assert torch.allclose(d, x + (xx - x) * (m + dyn[0]), atol=1e-14)


def test_lora_mix_against_a_loop_of_matrix_vector_products():
    B, T, C, D = 2, 5, 12, 4
    x, s = _rand(B, T, C), _rand(B, C, seed=1)
    maas = [torch.rand(1, 1, C, dtype=x.dtype, generator=torch.Generator().manual_seed(10 + j)) for j in range(5)]
    act, w2 = _rand(B * T, 5, D, seed=2), _rand(5, D, C, seed=3)
    outs = OB.lora_mix_v6(x, s, maas, act, w2)
    xx = OB.token_shift(x, s)
    for j in range(5):
        for b in range(B):
            for t in range(T):
                dyn = w2[j].T @ act[b * T + t, j]                 # (C,): this token's, this mix's product
                want = x[b, t] + (xx[b, t] - x[b, t]) * (maas[j].reshape(C) + dyn)
                assert torch.allclose(outs[j][b, t], want, atol=1e-13)
    # without the second factor the mixes are the plain ones
    plain = OB.mix_v6(x, s, maas)
    zero = OB.lora_mix_v6(x, s, maas, act, torch.zeros_like(w2))
    for a, b_ in zip(plain, zero):
        assert torch.equal(a, b_)


def test_ln_x_gate_against_written_out_normalisation_and_layer_norm():
    H, C, N = 3, 192, 7
    y, gate = _rand(N, C), _rand(N, C, seed=1)
    w, b = _rand(C, seed=2), _rand(C, seed=3)
    for divisor, eps in ((8.0, 1e-5), (1.0, 64e-5)):
        got = OB.ln_x_gate(y, gate, w, b, H, eps, divisor)
        yh = (y / divisor).view(N, H, 64)
        mean = yh.mean(-1, keepdim=True)
        var = ((yh - mean) ** 2).mean(-1, keepdim=True)            # biased variance
        n = ((yh - mean) / torch.sqrt(var + eps)).view(N, C) * w + b
        want = n * gate / (1 + torch.exp(-gate))                   # silu written out
        assert torch.allclose(got, want, atol=1e-12)
        ln = F.layer_norm(yh, (64,), None, None, eps).view(N, C) * w + b
        assert torch.allclose(OB.ln_x_gate(y, None, w, b, H, eps, divisor), ln, atol=1e-12)
    # a head's output does not change when another head's input does
    y2 = y.clone(); y2[:, 64:128] += 5
    a, b2 = OB.ln_x_gate(y, None, w, b, H, 1e-5), OB.ln_x_gate(y2, None, w, b, H, 1e-5)
    assert torch.equal(a[:, :64], b2[:, :64]) and torch.equal(a[:, 128:], b2[:, 128:])


def test_activations_against_numpy():
    k, kv = _rand(4, 9), _rand(4, 9, seed=1)
    assert np.allclose(OB.relu_square(k).numpy(), np.maximum(k.numpy(), 0) ** 2)
    assert np.allclose(OB.sigmoid_mul(k, kv).numpy(), kv.numpy() / (1 + np.exp(-k.numpy())))


def test_l2wrap_backward_against_a_row_loop():
    B, T, V = 2, 3, 11
    y = _rand(B, T, V).requires_grad_(True)
    mask = torch.tensor([[1., 0., 1.], [1., 1., 0.]], dtype=y.dtype)
    loss = (y * 0).sum() + 1.0
    out = OB.L2Wrap.apply(loss, y, 1e-4 / (B * T), mask)
    assert out.item() == 1.0
    out.backward()
    want = torch.zeros(B, T, V, dtype=y.dtype)
    for b in range(B):
        for t in range(T):
            row = y[b, t].detach()
            i = int(row.argmax())
            want[b, t, i] = row[i] * (1e-4 / (B * T)) * mask[b, t]
    assert torch.allclose(y.grad, want, atol=1e-18)


def test_channelmix_forms_agree():
    import torch.nn as nn
    from oracle.timemix_restated import ChannelMix5, ChannelMix6
    C = 16
    m5, m6 = ChannelMix5(C, 4 * C, seed=1).double(), ChannelMix6(C, 4 * C, seed=1).double()
    with torch.no_grad():       # same layer expressed in both parametrisations
        m6.time_maa_k.copy_(1 - m5.time_mix_k); m6.time_maa_r.copy_(1 - m5.time_mix_r)
        for a, b in ((m5.key, m6.key), (m5.value, m6.value), (m5.receptance, m6.receptance)):
            b.weight.copy_(a.weight)
    x, s = _rand(2, 5, C), _rand(2, C, seed=1)
    a, sa = m5(x, s)
    b, sb = m6(x, s)
    assert torch.allclose(a, b, atol=1e-12) and torch.equal(sa, x[:, -1]) and torch.equal(sb, x[:, -1])
    assert isinstance(m5.key, nn.Linear)
