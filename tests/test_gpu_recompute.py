"""Activation checkpointing (the reference wraps every block in deepspeed.checkpointing.checkpoint,
RWKV-v5/src/model.py:674-683): the operator's forward runs once without autograd and once more when backward
recomputes the block.  With the recompute cache the second run takes over the first one's outputs and state
checkpoints: half the kernel launches, and gradients that match the CPU oracle's (two chained operator calls,
autograd through both; bf16 I/O: rtol 2e-2 with a floor of 2e-2 rms) and the uncached run's bit for bit."""
import pytest
import torch
from torch.utils.checkpoint import checkpoint

from oracle import wkv56 as O
from tests.util import assert_close

pytestmark = pytest.mark.gpu


def _model(version, g, B, T, C, H, in_place, keyed=False):
    """two 'layers', each one operator call, the second fed by the first"""
    import rwkv_wkv_hip as W

    def op(r, k, v, w, u, s):
        if in_place:
            st = s.detach().clone()
            y = (W.RUN_WKV5_CUDA(B, T, C, H, st, r, k, v, w, u) if version == 5
                 else W.RUN_WKV6STATE_CUDA(B, T, C, H, r, k, v, w, u, st))
            return y, st
        return (W.WKV_5.apply(B, T, C, H, s, r, k, v, w, u) if version == 5 else W.WKV_6.apply(B, T, C, H, r, k, v, w, u, s))

    def layer(i):
        def f(*a):
            if keyed:
                with W.call_key(("layer", i)):
                    return op(*a)
            return op(*a)
        return f

    def run(leaves, use_ckpt):
        call = (lambda f, *a: checkpoint(f, *a, use_reentrant=True)) if use_ckpt else (lambda f, *a: f(*a))
        y1, s1 = call(layer(0), leaves["r"], leaves["k"], leaves["v"], leaves["w"], leaves["u"], leaves["state"])
        y2, s2 = call(layer(1), y1, leaves["k"], leaves["v"], leaves["w"], leaves["u"], s1)
        loss = (y2.float() * g["dy"].float()).sum() + (0 if in_place else (s2 * g["dstate"]).sum())
        loss.backward()
        return {n: t.grad.clone() for n, t in leaves.items() if t.grad is not None}, y2.detach()
    return run


def _oracle_two_layers(version, wl, in_place):
    """The same two chained calls on the CPU oracle, autograd through both; y of the first call is rounded to the I/O
    dtype where the GPU path stores it.  In-place convention: no gradient through the state (TimeMix.py:139-140)."""
    t = wl.tensors
    B, T, C, H = wl.B, wl.T, wl.C, wl.H
    L = {n: t[n].detach().clone().float().requires_grad_(True) for n in ("r", "k", "v", "w", "u", "state")}

    def op(r, s):
        s_ = s.detach() if in_place else s
        if version == 5:
            return O.wkv5_op(B, T, C, H, s_, r, L["k"], L["v"], L["w"], L["u"])
        return O.wkv6_op(B, T, C, H, r, L["k"], L["v"], L["w"], L["u"], s_)
    y1, s1 = op(L["r"], L["state"])
    y2, s2 = op(y1.to(wl.dtype).float(), s1)
    loss = (y2 * t["dy"].float()).sum() + (0 if in_place else (s2 * t["dstate"]).sum())
    loss.backward()
    return {n: x.grad for n, x in L.items() if x.grad is not None}, y2.detach()


@pytest.mark.parametrize("version", [5, 6])
@pytest.mark.parametrize("in_place", [False, True])
@pytest.mark.parametrize("keyed", [False, True])
def test_recompute_reuses_first_forward(version, in_place, keyed):
    import rwkv_wkv_hip as W
    from rwkv_wkv_hip import configs
    wl = configs.make(1 if version == 5 else 3, B=2, T=256, C=128, H=2, dtype=torch.bfloat16)
    B, T, C, H = wl.B, wl.T, wl.C, wl.H
    g = {n: x.cuda() for n, x in wl.tensors.items()}
    run = _model(version, g, B, T, C, H, in_place, keyed)
    fresh = lambda: {n: g[n].clone().requires_grad_(True) for n in ("r", "k", "v", "w", "u", "state")}
    plain, y_plain = run(fresh(), use_ckpt=False)
    n0 = W.stats["forward_launches"]
    ck, y_ck = run(fresh(), use_ckpt=True)
    launches_ckpt = W.stats["forward_launches"] - n0
    n0, r0 = W.stats["forward_launches"], W.stats["forward_reused"]
    with W.recompute_cache():
        cached, y_cached = run(fresh(), use_ckpt=True)       # (leaving the block verifies the take-overs)
    launches_cached, reused = W.stats["forward_launches"] - n0, W.stats["forward_reused"] - r0
    torch.cuda.synchronize()
    assert launches_ckpt == 4 and launches_cached == 2 and reused == 2
    # parity: the cached run against the oracle's two chained calls
    ref, y_ref = _oracle_two_layers(version, wl, in_place)
    assert_close(y_cached, y_ref, 2e-2, "y of the second layer")
    for n in ref:
        if in_place and n == "state":
            continue
        assert_close(cached[n], ref[n], 2e-2, f"gradient of {n} with the recompute cache")
    # and bit for bit what the uncached runs give
    assert torch.equal(y_plain, y_ck) and torch.equal(y_plain, y_cached)
    for n in plain:
        assert torch.equal(plain[n], ck[n]), f"checkpointed gradient of {n} differs"
        assert torch.equal(plain[n], cached[n]), f"gradient of {n} differs with the recompute cache"


def _segment_inputs(seed):
    from rwkv_wkv_hip import configs
    wl = configs.make(3, B=1, T=128, C=128, H=2, dtype=torch.bfloat16, seed=seed)
    return wl, {n: x.cuda() for n, x in wl.tensors.items()}


def test_grad_call_that_is_no_recomputation():
    """The reference's outer per-segment checkpoint (RWKV-v5/src/model.py:1248) runs the early segments without
    autograd and the last one with: that last call is no recomputation.  Unkeyed, it meets the kept run of the
    segment before (same signature) and the cache says so loudly on leaving; keyed, it runs the kernels itself and
    its results are the ones of a run without any cache."""
    import rwkv_wkv_hip as W
    wl_a, a = _segment_inputs(1)
    wl_b, b = _segment_inputs(2)
    B, T, C, H = wl_a.B, wl_a.T, wl_a.C, wl_a.H
    call = lambda t, s, lv=None: W.WKV_6.apply(B, T, C, H, (lv or t)["r"], t["k"], t["v"], t["w"], t["u"], s)

    def two_segments(keyed):
        leaves = {"r": b["r"].clone().requires_grad_(True)}
        with torch.no_grad():
            if keyed:
                with W.call_key(("seg", 0)):
                    _, s1 = call(a, a["state"])
            else:
                _, s1 = call(a, a["state"])
        if keyed:
            with W.call_key(("seg", 1)):
                y2, _ = call(b, s1, leaves)
        else:
            y2, _ = call(b, s1, leaves)
        y2.backward(b["dy"])
        return y2.detach(), leaves["r"].grad

    y_ref, g_ref = two_segments(False)                      # no cache installed
    with pytest.raises(W.WKVError, match="different inputs"):
        with W.recompute_cache():
            two_segments(False)
    r0 = W.stats["forward_reused"]
    with W.recompute_cache() as cache:
        y_k, g_k = two_segments(True)
        assert len(cache.entries) == 1                      # segment 0's run is still kept (it was never recomputed)
    assert W.stats["forward_reused"] == r0
    assert torch.equal(y_k, y_ref) and torch.equal(g_k, g_ref)


def test_kept_runs_are_bounded():
    import rwkv_wkv_hip as W
    wl, a = _segment_inputs(3)
    B, T, C, H = wl.B, wl.T, wl.C, wl.H
    with W.recompute_cache(W.RecomputeCache(max_bytes=1)) as cache:
        with torch.no_grad():
            for _ in range(3):
                W.WKV_6.apply(B, T, C, H, a["r"], a["k"], a["v"], a["w"], a["u"], a["state"])
        assert len(cache.entries) == 1 and cache.bytes > 1          # (one run is always kept: the bound drops older ones)
    with W.recompute_cache(W.RecomputeCache(max_entries=2)) as cache:
        with torch.no_grad():
            for _ in range(5):
                W.WKV_6.apply(B, T, C, H, a["r"], a["k"], a["v"], a["w"], a["u"], a["state"])
        assert len(cache.entries) == 2
