"""The operators inside the reference's TimeMix call sites: a restated TimeMix
module run once on the CPU oracle (the reference's pure path) and once on the
HIP operators (its CUDA path) gives the same output, state and parameter gradients."""
import copy

import pytest
import torch

from oracle import wkv56 as O
from oracle.timemix_restated import TimeMix5, TimeMix6
from tests.util import assert_close

pytestmark = pytest.mark.gpu


def _run(mod, x, shift, state, wkv, gy):
    mod.zero_grad()
    x = x.clone().requires_grad_(True)
    state = state.clone().requires_grad_(True)
    y, (s_shift, s_wkv) = mod(x, (shift, state), wkv)
    torch.autograd.backward([y, s_wkv], [gy, torch.ones_like(s_wkv) * 0.1])
    grads = {n: p.grad.detach().float().cpu() for n, p in mod.named_parameters() if p.grad is not None}
    return y.detach(), s_wkv.detach(), x.grad.detach(), state.grad.detach(), grads


@pytest.mark.parametrize("version", [5, 6])
@pytest.mark.parametrize("T", [128, 96])
def test_timemix_fp32(version, T):
    import rwkv_wkv_hip as W
    B, C, H = 2, 128, 2
    g = torch.Generator().manual_seed(3)
    x = torch.randn(B, T, C, generator=g)
    shift = torch.randn(B, C, generator=g)
    state = torch.randn(B, H, 64, 64, generator=g) * 0.1
    gy = torch.randn(B, T, C, generator=g)
    cls = TimeMix5 if version == 5 else TimeMix6
    cpu = cls(C, H, seed=7)
    gpu = copy.deepcopy(cpu).cuda()
    if version == 5:
        ref_wkv = lambda B, T, C, H, st, r, k, v, w, u: O.wkv5_op(B, T, C, H, st, r, k, v, w, u)
        our_wkv = lambda B, T, C, H, st, r, k, v, w, u: W.WKV_5.apply(B, T, C, H, st.contiguous(), r, k, v, w.contiguous(), u)
    else:
        ref_wkv = lambda B, T, C, H, r, k, v, w, u, st: O.wkv6_op(B, T, C, H, r, k, v, w, u, st)
        our_wkv = lambda B, T, C, H, r, k, v, w, u, st: W.WKV_6.apply(B, T, C, H, r, k, v, w, u, st.contiguous())
    ref = _run(cpu, x, shift, state, ref_wkv, gy)
    got = _run(gpu, x.cuda(), shift.cuda(), state.cuda(), our_wkv, gy.cuda())
    torch.cuda.synchronize()
    for name, a, b in zip(("y", "state", "gx", "gstate"), got[:4], ref[:4]):
        assert_close(a, b, 2e-3, f"timemix v{version} {name}")
    for n in ref[4]:
        assert_close(got[4][n], ref[4][n], 3e-3, f"timemix v{version} grad {n}")


@pytest.mark.parametrize("version", [5, 6])
def test_timemix_bf16_in_place_wrappers(version):
    """bf16 module through the reference's in-place calling convention (RUN_*),
    against the fp32 CPU module: loose tolerance, the Linear layers round too."""
    import rwkv_wkv_hip as W
    B, T, C, H = 2, 128, 128, 2
    g = torch.Generator().manual_seed(4)
    x = torch.randn(B, T, C, generator=g)
    shift = torch.randn(B, C, generator=g)
    state = torch.randn(B, H, 64, 64, generator=g) * 0.1
    cls = TimeMix5 if version == 5 else TimeMix6
    cpu = cls(C, H, seed=9)
    gpu = copy.deepcopy(cpu).cuda().bfloat16()
    with torch.no_grad():
        if version == 5:
            y_ref, (_, s_ref) = cpu(x, (shift, state), lambda B, T, C, H, st, r, k, v, w, u: O.wkv5_op(B, T, C, H, st, r, k, v, w, u))

            def wkv(B, T, C, H, st, r, k, v, w, u):
                st = st.clone().to(torch.float32).contiguous()          # TimeMix.py:306
                y = W.RUN_WKV5_CUDA(B, T, C, H, st, r, k, v, w.float().contiguous(), u.to(r.dtype))
                return y, st
        else:
            y_ref, (_, s_ref) = cpu(x, (shift, state), lambda B, T, C, H, r, k, v, w, u, st: O.wkv6_op(B, T, C, H, r, k, v, w, u, st))

            def wkv(B, T, C, H, r, k, v, w, u, st):
                st = st.to(torch.float32).clone().contiguous()
                y = W.RUN_WKV6STATE_CUDA(B, T, C, H, r, k, v, w, u, st)
                return y, st
        y, (_, s) = gpu(x.cuda().bfloat16(), (shift.cuda().bfloat16(), state.cuda()), wkv)
    torch.cuda.synchronize()
    assert y.dtype == torch.bfloat16 and s.dtype == torch.float32
    # the whole module runs in bf16 here (weights, Linear outputs, GroupNorm), the reference in fp32
    # (so y is compared in norm; the carried state, which only the operator touches, element-wise)
    rel = ((y.float().cpu() - y_ref).norm() / y_ref.norm()).item()
    assert rel < 3e-2, f"timemix bf16 v{version} y: relative error {rel}"
    assert_close(s, s_ref, 6e-2, f"timemix bf16 v{version} state")


@pytest.mark.parametrize("version", [5, 6])
def test_in_place_wrappers_train(version):
    """Training through the reference's in-place convention: forward with RUN_*, which overwrites the state
    buffer, then backward.  Gradients equal those of the functional operators on the same inputs."""
    import rwkv_wkv_hip as W
    from rwkv_wkv_hip import configs
    wl = configs.make(1 if version == 5 else 3, B=2, T=128, C=128, H=2, dtype=torch.bfloat16)
    B, T, C, H = wl.B, wl.T, wl.C, wl.H
    g = {n: x.cuda() for n, x in wl.tensors.items()}
    names = ("r", "k", "v", "w", "u")

    def leaves():
        return {n: g[n].clone().requires_grad_(True) for n in names}
    La, Lb = leaves(), leaves()
    st = g["state"].clone()
    if version == 5:
        y = W.RUN_WKV5_CUDA(B, T, C, H, st, La["r"], La["k"], La["v"], La["w"], La["u"])
        y2, s2 = W.WKV_5.apply(B, T, C, H, g["state"], Lb["r"], Lb["k"], Lb["v"], Lb["w"], Lb["u"])
    else:
        y = W.RUN_WKV6STATE_CUDA(B, T, C, H, La["r"], La["k"], La["v"], La["w"], La["u"], st)
        y2, s2 = W.WKV_6.apply(B, T, C, H, Lb["r"], Lb["k"], Lb["v"], Lb["w"], Lb["u"], g["state"])
    y.backward(g["dy"])
    y2.backward(g["dy"])
    torch.cuda.synchronize()
    assert torch.equal(y, y2) and torch.equal(st, s2), "in-place wrapper and functional operator disagree"
    for n in names:
        assert torch.equal(La[n].grad, Lb[n].grad), f"gradient of {n} differs"


@pytest.mark.parametrize("version", [5, 6])
def test_in_place_wrappers_write_into_a_layer_slice(version):
    """The state buffer handed to RUN_* is one layer's slice of an (N_layer, B, H, 64, 64) tensor, as the trainer keeps
    it: the kernel writes the new state there directly and leaves the other layers alone."""
    import rwkv_wkv_hip as W
    from rwkv_wkv_hip import configs
    wl = configs.make(1 if version == 5 else 3, B=2, T=128, C=128, H=2, dtype=torch.bfloat16)
    B, T, C, H = wl.B, wl.T, wl.C, wl.H
    g = {n: x.cuda() for n, x in wl.tensors.items()}
    layers = torch.full((3, B, H, 64, 64), 5.0, device="cuda")
    layers[1].copy_(g["state"])
    with torch.no_grad():
        if version == 5:
            y = W.RUN_WKV5_CUDA(B, T, C, H, layers[1], g["r"], g["k"], g["v"], g["w"], g["u"])
            y2, s2 = W.WKV_5.apply(B, T, C, H, g["state"], g["r"], g["k"], g["v"], g["w"], g["u"])
        else:
            y = W.RUN_WKV6STATE_CUDA(B, T, C, H, g["r"], g["k"], g["v"], g["w"], g["u"], layers[1])
            y2, s2 = W.WKV_6.apply(B, T, C, H, g["r"], g["k"], g["v"], g["w"], g["u"], g["state"])
    torch.cuda.synchronize()
    assert torch.equal(y, y2) and torch.equal(layers[1], s2)
    assert bool((layers[0] == 5.0).all()) and bool((layers[2] == 5.0).all())
