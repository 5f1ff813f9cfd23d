"""Activation checkpointing (the reference wraps every block in deepspeed.checkpointing.checkpoint,
RWKV-v5/src/model.py:674-683): the operator's forward runs once without autograd and once more when backward
recomputes the block.  With the recompute cache the second run takes over the first one's outputs and state
checkpoints.  Same gradients as without the cache, bit for bit and against the oracle, and half the kernel launches."""
import pytest
import torch
from torch.utils.checkpoint import checkpoint

from oracle import wkv56 as O
from tests.util import assert_close

pytestmark = pytest.mark.gpu


def _model(version, g, B, T, C, H, in_place):
    """two 'layers', each one operator call, the second fed by the first"""
    import rwkv_wkv_hip as W

    def layer(r, k, v, w, u, s):
        if in_place:
            st = s.detach().clone()
            y = (W.RUN_WKV5_CUDA(B, T, C, H, st, r, k, v, w, u) if version == 5
                 else W.RUN_WKV6STATE_CUDA(B, T, C, H, r, k, v, w, u, st))
            return y, st
        return (W.WKV_5.apply(B, T, C, H, s, r, k, v, w, u) if version == 5 else W.WKV_6.apply(B, T, C, H, r, k, v, w, u, s))

    def run(leaves, use_ckpt):
        call = (lambda *a: checkpoint(layer, *a, use_reentrant=True)) if use_ckpt else layer
        y1, s1 = call(leaves["r"], leaves["k"], leaves["v"], leaves["w"], leaves["u"], leaves["state"])
        y2, s2 = call(y1, leaves["k"], leaves["v"], leaves["w"], leaves["u"], s1)
        loss = (y2.float() * g["dy"].float()).sum() + (0 if in_place else (s2 * g["dstate"]).sum())
        loss.backward()
        return {n: t.grad.clone() for n, t in leaves.items() if t.grad is not None}, y2.detach()
    return run


@pytest.mark.parametrize("version", [5, 6])
@pytest.mark.parametrize("in_place", [False, True])
def test_recompute_reuses_first_forward(version, in_place):
    import rwkv_wkv_hip as W
    from rwkv_wkv_hip import configs
    wl = configs.make(1 if version == 5 else 3, B=2, T=256, C=128, H=2, dtype=torch.bfloat16)
    B, T, C, H = wl.B, wl.T, wl.C, wl.H
    g = {n: x.cuda() for n, x in wl.tensors.items()}
    run = _model(version, g, B, T, C, H, in_place)
    fresh = lambda: {n: g[n].clone().requires_grad_(True) for n in ("r", "k", "v", "w", "u", "state")}
    plain, y_plain = run(fresh(), use_ckpt=False)
    n0 = W.stats["forward_launches"]
    ck, y_ck = run(fresh(), use_ckpt=True)
    launches_ckpt = W.stats["forward_launches"] - n0
    n0, r0 = W.stats["forward_launches"], W.stats["forward_reused"]
    with W.recompute_cache():
        cached, y_cached = run(fresh(), use_ckpt=True)
    launches_cached, reused = W.stats["forward_launches"] - n0, W.stats["forward_reused"] - r0
    torch.cuda.synchronize()
    assert launches_ckpt == 4 and launches_cached == 2 and reused == 2
    assert torch.equal(y_plain, y_ck) and torch.equal(y_plain, y_cached)
    for n in plain:
        assert torch.equal(plain[n], ck[n]), f"checkpointed gradient of {n} differs"
        assert torch.equal(plain[n], cached[n]), f"gradient of {n} differs with the recompute cache"
