"""The element-wise passes around the operator (token shift + mixing, ln_x * gate, channel-mix activations, L2Wrap)
on the HIP kernels, through the C ABI, against the CPU oracle (oracle/blocks.py: the reference's lines in plain torch,
gradients by autograd).  Tolerances: rtol 1e-3 for fp32 tensors, 2e-2 for bf16 / fp16 (of |ref| + rms(ref))."""
import copy

import pytest
import torch

from oracle import blocks as OB
from oracle import wkv56 as O
from oracle.timemix_restated import ChannelMix5, ChannelMix6, TimeMix5, TimeMix6
from tests.util import assert_close

pytestmark = pytest.mark.gpu
RTOL = {torch.float32: 1e-3, torch.bfloat16: 2e-2, torch.float16: 2e-2}


def _g(seed):
    return torch.Generator().manual_seed(seed)


def _leaf(t):
    return t.clone().requires_grad_(True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,T,C", [(1, 1, 64), (2, 7, 264), (3, 130, 64), (2, 64, 2560), (1, 200, 320)])
@pytest.mark.parametrize("n,lerp,dyn", [(1, False, False), (2, True, False), (4, True, False), (2, False, False),
                                        (5, False, True), (3, False, True)])
def test_token_shift_mix(dtype, B, T, C, n, lerp, dyn):
    from rwkv_wkv_hip import blocks as K
    g = _g(B * 1000 + T + C + n)
    x = torch.randn(B, T, C, generator=g).to(dtype)
    shift = torch.randn(B, C, generator=g).to(dtype)
    coefs = [torch.rand(1, 1, C, generator=g) for _ in range(n)]
    d = (torch.randn(n, B, T, C, generator=g) * 0.3).to(dtype) if dyn else None
    gouts = [torch.randn(B, T, C, generator=g).to(dtype) for _ in range(n)]

    def run(fn, dev):
        xs, ss = _leaf(x.to(dev)), _leaf(shift.to(dev))
        cs = [_leaf(c.to(dev)) for c in coefs]
        ds = _leaf(d.to(dev)) if dyn else None
        outs = fn(xs, ss, cs, ds)
        torch.autograd.backward(list(outs), [go.to(dev) for go in gouts])
        return outs, xs.grad, ss.grad, [c.grad for c in cs], (ds.grad if dyn else None)

    # the oracle computes in fp32 from the same (already rounded) inputs
    def ref_fn(xs, ss, cs, ds):
        xf, sf = xs.float(), ss.float()
        return OB.mix_v5(xf, sf, cs) if lerp else OB.mix_v6(xf, sf, cs, None if ds is None else ds.float())
    ref = run(ref_fn, "cpu")
    got = run(lambda xs, ss, cs, ds: K.token_shift_mix(xs, ss, cs, dyn=ds, lerp=lerp), "cuda")
    torch.cuda.synchronize()
    rt = RTOL[dtype]
    for j in range(n):
        assert got[0][j].dtype == dtype
        assert_close(got[0][j], ref[0][j], rt, f"out[{j}]")
        assert_close(got[3][j], ref[3][j], max(rt, 2e-3) if dtype == torch.float32 else rt, f"gcoef[{j}]")
    assert_close(got[1], ref[1], rt, "gx")
    assert_close(got[2], ref[2], rt, "gshift")
    if dyn:
        assert_close(got[4], ref[4], rt, "gdyn")


@pytest.mark.parametrize("B,T,C", [(1, 1, 32), (2, 7, 96), (3, 130, 64), (2, 128, 2560), (1, 200, 320), (2, 129, 32),
                                   (1, 257, 128), (2, 16, 4096), (3, 300, 72), (1, 65, 8), (2, 1, 200), (1, 513, 136)])
def test_lora_shift_mix(B, T, C):
    """The five data-dependent mixes with the second LoRA product inside the kernel (bf16) against the oracle in fp32
    on the same rounded inputs: the five outputs and the gradients of x, the shift state, the five time_maa
    parameters, the activations and time_maa_w2."""
    from rwkv_wkv_hip import blocks as K
    bf = torch.bfloat16
    g = _g(B * 1000 + T + C)
    x = torch.randn(B, T, C, generator=g).to(bf)
    shift = torch.randn(B, C, generator=g).to(bf)
    coefs = [torch.rand(1, 1, C, generator=g) for _ in range(5)]
    act = torch.tanh(torch.randn(B * T, 5, 32, generator=g)).to(bf)
    w2 = (torch.randn(5, 32, C, generator=g) * 0.1).to(bf)
    gouts = [torch.randn(B, T, C, generator=g).to(bf) for _ in range(5)]

    def run(fn, dev):
        xs, ss, as_, ws = (_leaf(t.to(dev)) for t in (x, shift, act, w2))
        cs = [_leaf(c.to(dev)) for c in coefs]
        outs = fn(xs, ss, cs, as_, ws)
        torch.autograd.backward(list(outs), [go.to(dev).to(outs[0].dtype) for go in gouts])
        return outs, xs.grad, ss.grad, [c.grad for c in cs], as_.grad, ws.grad

    ref = run(lambda xs, ss, cs, as_, ws: OB.lora_mix_v6(xs.float(), ss.float(), cs, as_.float(), ws.float()), "cpu")
    assert K.lora_mix_available(x, act, w2)
    got = run(lambda xs, ss, cs, as_, ws: K.lora_shift_mix(xs, ss, cs, as_, ws), "cuda")
    torch.cuda.synchronize()
    for j in range(5):
        assert got[0][j].dtype == bf
        assert_close(got[0][j], ref[0][j], 2e-2, f"out[{j}]")
        assert_close(got[3][j], ref[3][j], 2e-2, f"gmaa[{j}]")
    assert_close(got[1], ref[1], 2e-2, "gx")
    assert_close(got[2], ref[2], 2e-2, "gshift")
    assert_close(got[4], ref[4], 2e-2, "gact")
    assert_close(got[5], ref[5], 2e-2, "gw2")


def test_lora_shift_mix_matches_the_unfused_passes():
    """the fused pass against bmm + token_shift_mix on the same device: the same mathematics with dyn rounded to bf16
    on its way through memory in the one and kept in fp32 in the other"""
    from rwkv_wkv_hip import blocks as K
    bf = torch.bfloat16
    B, T, C = 2, 200, 256
    g = _g(5)
    x, shift = torch.randn(B, T, C, generator=g).to(bf).cuda(), torch.randn(B, C, generator=g).to(bf).cuda()
    coefs = [torch.rand(1, 1, C, generator=g).cuda() for _ in range(5)]
    act = torch.tanh(torch.randn(B * T, 5, 32, generator=g)).to(bf).cuda()
    w2 = (torch.randn(5, 32, C, generator=g) * 0.1).to(bf).cuda()
    with torch.no_grad():
        fused = K.lora_shift_mix(x, shift, coefs, act, w2)
        dyn = torch.bmm(act.transpose(0, 1), w2).view(5, B, T, C)
        plain = K.token_shift_mix(x, shift, coefs, dyn=dyn)
    for j in range(5):
        assert_close(fused[j], plain[j].float().cpu(), 2e-2, f"out[{j}]")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,C", [(1, 64), (9, 320), (130, 128), (64, 2560), (257, 4096)])
@pytest.mark.parametrize("divisor,eps,gated", [(8.0, 1e-5, True), (1.0, 64e-5, True), (1.0, 1e-5, False)])
def test_ln_x_gate(dtype, rows, C, divisor, eps, gated):
    from rwkv_wkv_hip import blocks as K
    g = _g(rows + C)
    y = (torch.randn(rows, C, generator=g) * 3 + 0.5).to(dtype)
    gate = torch.randn(rows, C, generator=g).to(dtype) if gated else None
    w, b = torch.randn(C, generator=g), torch.randn(C, generator=g)
    go = torch.randn(rows, C, generator=g).to(dtype)

    def run(fn, dev):
        ys, ws, bs = _leaf(y.to(dev)), _leaf(w.to(dev)), _leaf(b.to(dev))
        gs = _leaf(gate.to(dev)) if gated else None
        out = fn(ys, gs, ws, bs)
        out.backward(go.to(dev).to(out.dtype))
        return out, ys.grad, (gs.grad if gated else None), ws.grad, bs.grad
    ref = run(lambda ys, gs, ws, bs: OB.ln_x_gate(ys.float(), None if gs is None else gs.float(), ws, bs, C // 64, eps, divisor), "cpu")
    got = run(lambda ys, gs, ws, bs: K.ln_x_gate(ys, gs, ws, bs, eps, scale=1.0 / divisor), "cuda")
    torch.cuda.synchronize()
    rt = RTOL[dtype]
    assert got[0].dtype == dtype
    assert_close(got[0], ref[0], rt, "out")
    assert_close(got[1], ref[1], rt, "gy")
    if gated:
        assert_close(got[2], ref[2], rt, "ggate")
    assert_close(got[3], ref[3], max(rt, 2e-3), "gweight")
    assert_close(got[4], ref[4], max(rt, 2e-3), "gbias")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(1, 1, 8), (2, 7, 264), (2, 128, 8960)])
def test_channel_mix_activations(dtype, shape):
    from rwkv_wkv_hip import blocks as K
    g = _g(sum(shape))
    k, kv, go = (torch.randn(*shape, generator=g).to(dtype) for _ in range(3))

    def run(mod, dev, f32):
        cast = (lambda t: t.float()) if f32 else (lambda t: t)
        ks, rs, kvs = _leaf(k.to(dev)), _leaf(k.to(dev)), _leaf(kv.to(dev))
        a = mod.relu_square(cast(ks))
        b = mod.sigmoid_mul(cast(rs), cast(kvs))
        torch.autograd.backward([a, b], [go.to(dev).to(a.dtype), go.to(dev).to(b.dtype)])
        return a, b, ks.grad, rs.grad, kvs.grad
    ref, got = run(OB, "cpu", True), run(K, "cuda", False)
    torch.cuda.synchronize()
    for name, a, b in zip(("relu^2", "sigmoid*kv", "gk", "gr", "gkv"), got, ref):
        assert a.dtype == dtype
        assert_close(a, b, RTOL[dtype], name)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,T,V", [(1, 1, 8), (2, 5, 50277), (2, 3, 65536)])
def test_l2wrap(dtype, B, T, V):
    """bf16 logits tie often: the kernel, like torch on the CPU, takes the first position of the maximum."""
    from rwkv_wkv_hip import blocks as K
    g = _g(V)
    y = torch.randn(B, T, V, generator=g).to(dtype)
    y[0, 0, V // 2] = y[0, 0, V - 1] = 9.0                        # a forced tie
    mask = (torch.rand(B, T, generator=g) > 0.3).float()
    factor = 1e-4 / (B * T)

    def run(mod, dev):
        ys = _leaf(y.to(dev))
        loss = ys.float().sum() * 0 + 2.0
        mod.L2Wrap.apply(loss, ys, factor, mask.to(dev)).backward()
        return ys.grad
    ref, got = run(OB, "cpu"), run(K, "cuda")
    torch.cuda.synchronize()
    assert got.dtype == dtype
    assert torch.equal((got != 0).cpu(), ref != 0), "position of the maximum"
    assert_close(got, ref, RTOL[dtype], "gy")


def _run_module(fwd, mod, x, state, gy, extra_grads=()):
    mod.zero_grad()
    x = x.clone().requires_grad_(True)
    state = tuple(s.clone().requires_grad_(True) for s in state) if isinstance(state, tuple) else state.clone().requires_grad_(True)
    y, new = fwd(mod, x, state)
    outs, gs = [y], [gy]
    if isinstance(new, tuple):
        outs.append(new[1]); gs.append(torch.ones_like(new[1]) * 0.1)
    torch.autograd.backward(outs, gs)
    grads = {n: p.grad.detach().float().cpu() for n, p in mod.named_parameters() if p.grad is not None}
    sg = state[0].grad if isinstance(state, tuple) else state.grad
    return y.detach(), x.grad.detach(), sg.detach(), grads


@pytest.mark.parametrize("version", [5, 6])
@pytest.mark.parametrize("T", [128, 72])
def test_timemix_forward_on_the_kernels(version, T):
    """timemix5_forward / timemix6_forward (every element-wise pass and the operator on HIP kernels) against the
    restated reference module on the CPU oracle: output, input / shift-state gradients and every parameter gradient."""
    from rwkv_wkv_hip import blocks as K
    B, C, H = 2, 128, 2
    g = _g(11)
    x, shift, gy = torch.randn(B, T, C, generator=g), torch.randn(B, C, generator=g), torch.randn(B, T, C, generator=g)
    state = torch.randn(B, H, 64, 64, generator=g) * 0.1
    cpu = (TimeMix5 if version == 5 else TimeMix6)(C, H, seed=5)
    with torch.no_grad():
        cpu.ln_x.weight.copy_(torch.randn(C, generator=g)); cpu.ln_x.bias.copy_(torch.randn(C, generator=g))
    gpu = copy.deepcopy(cpu).cuda()
    if version == 5:
        ref_fwd = lambda m, xs, st: m(xs, st, lambda B, T, C, H, s, r, k, v, w, u: O.wkv5_op(B, T, C, H, s, r, k, v, w, u))
        our_fwd = K.timemix5_forward
    else:
        ref_fwd = lambda m, xs, st: m(xs, st, lambda B, T, C, H, r, k, v, w, u, s: O.wkv6_op(B, T, C, H, r, k, v, w, u, s))
        our_fwd = K.timemix6_forward
    ref = _run_module(ref_fwd, cpu, x, (shift, state), gy)
    got = _run_module(our_fwd, gpu, x.cuda(), (shift.cuda(), state.cuda()), gy.cuda())
    torch.cuda.synchronize()
    for name, a, b in zip(("y", "gx", "gshift"), got[:3], ref[:3]):
        assert_close(a, b, 2e-3, f"timemix v{version} {name}")
    assert set(got[3]) == set(ref[3])
    for n in ref[3]:
        assert_close(got[3][n], ref[3][n], 3e-3, f"timemix v{version} grad {n}")


@pytest.mark.parametrize("version", [5, 6])
def test_timemix_forward_on_the_kernels_bf16_module(version):
    """The whole module in bf16 (weights, matmuls, every element-wise pass), as mixed-precision training runs it, against
    the fp32 CPU module: compared in norm (the matmuls round too); the carried state, which only the operator touches and
    which stays fp32, element-wise."""
    from rwkv_wkv_hip import blocks as K
    B, T, C, H = 2, 128, 128, 2
    g = _g(13)
    x, shift = torch.randn(B, T, C, generator=g), torch.randn(B, C, generator=g)
    state = torch.randn(B, H, 64, 64, generator=g) * 0.1
    gy = torch.randn(B, T, C, generator=g)
    cpu = (TimeMix5 if version == 5 else TimeMix6)(C, H, seed=8)
    gpu = copy.deepcopy(cpu).cuda().bfloat16()
    if version == 5:
        ref_fwd = lambda m, xs, st: m(xs, st, lambda B, T, C, H, s, r, k, v, w, u: O.wkv5_op(B, T, C, H, s, r, k, v, w, u))
        our_fwd = K.timemix5_forward
    else:
        ref_fwd = lambda m, xs, st: m(xs, st, lambda B, T, C, H, r, k, v, w, u, s: O.wkv6_op(B, T, C, H, r, k, v, w, u, s))
        our_fwd = K.timemix6_forward
    ref = _run_module(ref_fwd, cpu, x, (shift, state), gy)
    got = _run_module(our_fwd, gpu, x.cuda().bfloat16(), (shift.cuda().bfloat16(), state.cuda()), gy.cuda().bfloat16())
    torch.cuda.synchronize()
    assert got[0].dtype == torch.bfloat16
    for name, a, b in zip(("y", "gx", "gshift"), got[:3], ref[:3]):
        rel = ((a.float().cpu() - b).norm() / b.norm()).item()
        assert rel < 4e-2, f"timemix bf16 v{version} {name}: relative error {rel}"
    for n in ref[3]:
        a, b = got[3][n], ref[3][n]
        rel = ((a - b).norm() / (b.norm() + 1e-6)).item()
        assert rel < 8e-2, f"timemix bf16 v{version} grad {n}: relative error {rel}"
    with torch.no_grad():
        _, (_, s_ref) = ref_fwd(cpu, x, (shift, state))
        _, (_, s_got) = our_fwd(gpu, x.cuda().bfloat16(), (shift.cuda().bfloat16(), state.cuda()))
    assert s_got.dtype == torch.float32
    assert_close(s_got, s_ref, 6e-2, f"timemix bf16 v{version} state")


@pytest.mark.parametrize("version", [5, 6])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_channelmix_forward_on_the_kernels(version, dtype):
    from rwkv_wkv_hip import blocks as K
    B, T, C = 2, 70, 128
    g = _g(12)
    x, shift, gy = torch.randn(B, T, C, generator=g), torch.randn(B, C, generator=g), torch.randn(B, T, C, generator=g)
    cpu = (ChannelMix5 if version == 5 else ChannelMix6)(C, 4 * C, seed=6)
    gpu = copy.deepcopy(cpu).cuda().to(dtype)
    ref = _run_module(lambda m, xs, st: m(xs, st), cpu, x, shift, gy)
    fwd = K.channelmix5_forward if version == 5 else K.channelmix6_forward
    got = _run_module(fwd, gpu, x.cuda().to(dtype), shift.cuda().to(dtype), gy.cuda().to(dtype))
    torch.cuda.synchronize()
    if dtype == torch.float32:
        for name, a, b in zip(("y", "gx", "gshift"), got[:3], ref[:3]):
            assert_close(a, b, 2e-3, f"channelmix v{version} {name}")
        for n in ref[3]:
            assert_close(got[3][n], ref[3][n], 3e-3, f"channelmix v{version} grad {n}")
    else:       # the whole module (weights, matmuls) is bf16 here, the reference fp32: compare in norm
        for name, a, b in zip(("y", "gx"), got[:2], ref[:2]):
            rel = ((a.float().cpu() - b).norm() / b.norm()).item()
            assert rel < 3e-2, f"channelmix bf16 v{version} {name}: relative error {rel}"


def test_full_shape_7b_edges():
    """The 7B shape of one segment (B1 T4096 C4096, bf16): every pass against the CPU oracle on the whole tensor."""
    from rwkv_wkv_hip import blocks as K
    B, T, C = 1, 4096, 4096
    g = _g(77)
    bf = torch.bfloat16
    x, shift = torch.randn(B, T, C, generator=g).to(bf), torch.randn(B, C, generator=g).to(bf)
    coefs = [torch.rand(C, generator=g) for _ in range(5)]
    dyn = (torch.randn(5, B, T, C, generator=g) * 0.3).to(bf)
    with torch.no_grad():
        ref = OB.mix_v6(x.float(), shift.float(), coefs, dyn.float())
        got = K.token_shift_mix(x.cuda(), shift.cuda(), [c.cuda() for c in coefs], dyn=dyn.cuda())
        for j in range(5):
            assert_close(got[j], ref[j], 2e-2, f"7B mix out[{j}]")
        y, gate = (torch.randn(B, T, C, generator=g) * 2).to(bf), torch.randn(B, T, C, generator=g).to(bf)
        w, b = torch.randn(C, generator=g), torch.randn(C, generator=g)
        ref = OB.ln_x_gate(y.float(), gate.float(), w, b, C // 64, 64e-5)
        got = K.ln_x_gate(y.cuda(), gate.cuda(), w.cuda(), b.cuda(), 64e-5)
        assert_close(got, ref, 2e-2, "7B ln_x*gate")
