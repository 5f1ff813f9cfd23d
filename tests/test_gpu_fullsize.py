"""Parity at the full benchmark shapes: (a) the CPU oracle over the WHOLE tensors
(one batch row at a time for v5/v6, to bound host memory; heads and batch rows
are independent recurrences), (b) the per-token fp32 kernel as a second,
independent device implementation, and (c) size-independent properties (segment
chaining)."""
import pytest
import torch

from oracle import wkv4 as O4
from oracle import wkv56 as O
from tests.util import assert_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def gpu_fwd_bwd(version, t, B, T, C, H, algo, with_state_grad=True):
    import rwkv_wkv_hip as W
    W.set_algo(algo)
    L = {n: t[n].detach().clone().requires_grad_(True) for n in ("r", "k", "v", "w", "u", "state")}
    if version == 5:
        y, s = W.WKV_5.apply(B, T, C, H, L["state"], L["r"], L["k"], L["v"], L["w"], L["u"])
    else:
        y, s = W.WKV_6.apply(B, T, C, H, L["r"], L["k"], L["v"], L["w"], L["u"], L["state"])
    torch.autograd.backward([y, s], [t["dy"], t["dstate"]])
    torch.cuda.synchronize()
    W.set_algo("auto")
    return dict(y=y.detach(), state=s.detach(), gr=L["r"].grad, gk=L["k"].grad, gv=L["v"].grad, gw=L["w"].grad,
                gu=L["u"].grad, gstate=L["state"].grad)


def head_slice(x, B, T, H, heads):
    return x.view(B, T, H, 64)[:, :, heads].reshape(B, T, len(heads) * 64).contiguous()


def oracle_by_batch_row(version, cpu, B, T, C, H):
    """wkv_op_grads over all heads, one batch row per call; per-row gu / WKV5 gw summed."""
    rows = []
    for b in range(B):
        sl = slice(b, b + 1)
        w = cpu["w"] if version == 5 else cpu["w"][sl]
        rows.append(O.wkv_op_grads(version, 1, T, C, H, cpu["r"][sl].float(), cpu["k"][sl].float(), cpu["v"][sl].float(),
                                   w, cpu["u"], cpu["state"][sl], cpu["dy"][sl].float(), cpu["dstate"][sl]))
    out = {}
    for n in rows[0]:
        if n == "gu" or (n == "gw" and version == 5):
            out[n] = torch.stack([r[n] for r in rows]).sum(0)
        else:
            out[n] = torch.cat([r[n] for r in rows], 0)
    return out


def test_cfg0_wkv5_forward_fp32():
    """The reference's own CPU-runnable case: WKV5 forward, B1 T512 C768 H12, fp32, zero state
    (plus the backward of the same call), against the oracle at rtol 1e-3."""
    from rwkv_wkv_hip import configs
    wl = configs.make(0)
    B, T, C, H = wl.B, wl.T, wl.C, wl.H
    print(f"case cfg0: v5 B{B} T{T} C{C} H{H} fp32", flush=True)
    cpu = wl.tensors
    t = {n: x.to(DEV) for n, x in cpu.items()}
    got = gpu_fwd_bwd(5, t, B, T, C, H, "auto")
    ref = O.wkv_op_grads(5, B, T, C, H, cpu["r"], cpu["k"], cpu["v"], cpu["w"], cpu["u"], cpu["state"], cpu["dy"],
                         cpu["dstate"])
    for n in ref:
        assert_close(got[n].cpu(), ref[n], 1e-3, f"cfg0 {n}")


@pytest.mark.parametrize("cfg", [1, 3])
def test_full_shape_v5_v6(cfg):
    from rwkv_wkv_hip import configs
    wl = configs.make(cfg)
    version, B, T, C, H = wl.version, wl.B, wl.T, wl.C, wl.H
    print(f"case full cfg{cfg}: v{version} B{B} T{T} C{C} H{H}", flush=True)
    cpu = wl.tensors
    t = {n: x.to(DEV) for n, x in cpu.items()}
    fast = gpu_fwd_bwd(version, t, B, T, C, H, "chunked")
    slow = gpu_fwd_bwd(version, t, B, T, C, H, "recurrent")
    for n in fast:
        assert_close(fast[n], slow[n], 2e-2, f"cfg{cfg} blocked vs per-token {n}")
    # (a) the oracle over every head of every batch row; gu (and the WKV5 gw) are sums over the batch
    ref = oracle_by_batch_row(version, cpu, B, T, C, H)
    for n in ref:
        assert_close(fast[n].cpu(), ref[n], 2e-2, f"cfg{cfg} oracle {n}")
    # (c) one call over T == two chained calls over T/2, state gradient handed back
    import rwkv_wkv_hip as W
    h = T // 2
    a = lambda x: x[:, :h].contiguous()
    b = lambda x: x[:, h:].contiguous()
    L = {n: t[n].detach().clone().requires_grad_(True) for n in ("r", "k", "v", "w", "u", "state")}
    if version == 5:
        y1, s1 = W.WKV_5.apply(B, h, C, H, L["state"], a(L["r"]), a(L["k"]), a(L["v"]), L["w"], L["u"])
        y2, s2 = W.WKV_5.apply(B, h, C, H, s1, b(L["r"]), b(L["k"]), b(L["v"]), L["w"], L["u"])
    else:
        y1, s1 = W.WKV_6.apply(B, h, C, H, a(L["r"]), a(L["k"]), a(L["v"]), a(L["w"]), L["u"], L["state"])
        y2, s2 = W.WKV_6.apply(B, h, C, H, b(L["r"]), b(L["k"]), b(L["v"]), b(L["w"]), L["u"], s1)
    torch.autograd.backward([y1, y2, s2], [a(t["dy"]), b(t["dy"]), t["dstate"]])
    torch.cuda.synchronize()
    assert_close(torch.cat([y1, y2], 1), fast["y"], 2e-2, "chain y")
    assert_close(s2, fast["state"], 1e-3, "chain state")
    for n, gn in (("r", "gr"), ("k", "gk"), ("v", "gv"), ("w", "gw"), ("u", "gu"), ("state", "gstate")):
        assert_close(L[n].grad, fast[gn], 2e-2, f"chain {gn}")


@pytest.mark.parametrize("version", [5, 6])
def test_more_pairs_than_one_round_of_compute_units(version):
    """B*H = 260: the blocked path runs the first 256 (batch, head) pairs in one piece and cuts the other four in
    time (two launches per kernel, two regions of partial sums).  All outputs against the per-token kernel, and
    the oracle on one head of each group for every batch row (so the batch-summed gu / v5 gw are covered)."""
    from rwkv_wkv_hip import configs
    B, H, T = 5, 52, 1024
    C = H * 64
    wl = configs.make(1 if version == 5 else 3, B=B, T=T, C=C, H=H, dtype=torch.bfloat16)
    print(f"case two groups v{version} B{B} H{H} T{T}", flush=True)
    cpu = wl.tensors
    t = {n: x.to(DEV) for n, x in cpu.items()}
    fast = gpu_fwd_bwd(version, t, B, T, C, H, "chunked")
    slow = gpu_fwd_bwd(version, t, B, T, C, H, "recurrent")
    for n in fast:
        assert_close(fast[n], slow[n], 2e-2, f"two groups v{version} blocked vs per-token {n}")
    heads = [1, H - 1]             # (b, 1) is below pair 256 for every b; (4, 51) is pair 259
    hs = lambda x: head_slice(x, B, T, H, heads)
    sub_w = cpu["w"][heads] if version == 5 else hs(cpu["w"])
    ref = O.wkv_op_grads(version, B, T, 128, 2, hs(cpu["r"]).float(), hs(cpu["k"]).float(), hs(cpu["v"]).float(), sub_w,
                         cpu["u"][heads], cpu["state"][:, heads], hs(cpu["dy"]).float(), cpu["dstate"][:, heads])
    pick = {"y": hs, "gr": hs, "gk": hs, "gv": hs,
            "gw": (lambda x: x[heads]) if version == 5 else hs,
            "gu": lambda x: x[heads], "state": lambda x: x[:, heads], "gstate": lambda x: x[:, heads]}
    for n in ref:
        assert_close(pick[n](fast[n].cpu()), ref[n], 2e-2, f"two groups v{version} oracle heads {heads} {n}")


def test_full_shape_v4():
    import rwkv_wkv_hip as W
    from rwkv_wkv_hip import configs
    wl = configs.make(2)
    B, T, C = wl.B, wl.T, wl.C
    print(f"case full cfg2: v4 B{B} T{T} C{C} fp32", flush=True)
    cpu = wl.tensors
    t = {n: x.to(DEV) for n, x in cpu.items()}
    L = {n: t[n].clone().requires_grad_(True) for n in ("time_decay", "time_first", "k", "v", "state")}
    y, s = W.wkv_op(L["time_decay"], L["time_first"], L["k"], L["v"], L["state"])
    torch.autograd.backward([y, s], [t["dy"], t["dstate"]])
    torch.cuda.synchronize()
    # the C oracle over all channels (channels are independent chains)
    yr, sr = O4.forward(cpu["time_decay"], cpu["time_first"], cpu["k"], cpu["v"], cpu["state"])
    ref = O4.backward(cpu["time_decay"], cpu["time_first"], cpu["k"], cpu["v"], cpu["state"], cpu["dy"], cpu["dstate"])
    assert_close(y, yr, 1e-3, "v4 y")
    und = lambda st: st[..., :2].float().cpu() * torch.exp(st[..., 2:3].float().cpu())
    assert_close(und(s), und(sr), 1e-3, "v4 state")
    assert_close(L["time_decay"].grad, ref[0], 2e-3, "v4 g_time_decay")
    assert_close(L["time_first"].grad, ref[1], 2e-3, "v4 g_time_first")
    assert_close(L["k"].grad, ref[2], 1e-3, "v4 gk")
    assert_close(L["v"].grad, ref[3], 1e-3, "v4 gv")
    # chaining: T == T/2 + T/2 through the carried state
    h = T // 2
    y1, s1 = W.wkv_op(t["time_decay"], t["time_first"], t["k"][:, :h].contiguous(), t["v"][:, :h].contiguous(), t["state"])
    y2, s2 = W.wkv_op(t["time_decay"], t["time_first"], t["k"][:, h:].contiguous(), t["v"][:, h:].contiguous(), s1)
    assert_close(torch.cat([y1, y2], 1), y, 1e-4, "v4 chain y")


def test_full_shape_v4_bf16():
    """cfg2 at its full width in the reference kernel's own dtype (bf16 k, v, y and gradients,
    RWKV-v4neo/cuda/wkv_op_bf16.cpp:45-51): B8 T4096 C4096 against the C oracle on the rounded inputs,
    rtol 2e-2 (floor 2e-2 rms); the parameter gradients are sums over 32768 rounded terms per channel."""
    import rwkv_wkv_hip as W
    from rwkv_wkv_hip import configs
    wl = configs.make(2, dtype=torch.bfloat16)
    B, T, C = wl.B, wl.T, wl.C
    print(f"case full cfg2: v4 B{B} T{T} C{C} bf16", flush=True)
    cpu = wl.tensors
    t = {n: x.to(DEV) for n, x in cpu.items()}
    L = {n: t[n].clone().requires_grad_(True) for n in ("time_decay", "time_first", "k", "v", "state")}
    y, s = W.wkv_op(L["time_decay"], L["time_first"], L["k"], L["v"], L["state"])
    assert y.dtype == torch.bfloat16
    torch.autograd.backward([y, s], [t["dy"], t["dstate"]])
    torch.cuda.synchronize()
    f32 = lambda x: x.float()
    yr, sr = O4.forward(cpu["time_decay"], f32(cpu["time_first"]), f32(cpu["k"]), f32(cpu["v"]), cpu["state"])
    ref = O4.backward(cpu["time_decay"], f32(cpu["time_first"]), f32(cpu["k"]), f32(cpu["v"]), cpu["state"], f32(cpu["dy"]),
                      cpu["dstate"])
    assert_close(y, yr, 2e-2, "v4 bf16 y")
    und = lambda st: st[..., :2].float().cpu() * torch.exp(st[..., 2:3].float().cpu())
    assert_close(und(s), und(sr), 1e-3, "v4 bf16 state")
    assert_close(L["time_decay"].grad, ref[0], 2e-2, "v4 bf16 g_time_decay")
    assert_close(L["time_first"].grad, ref[1], 2e-2, "v4 bf16 g_time_first")
    assert_close(L["k"].grad, ref[2], 2e-2, "v4 bf16 gk")
    assert_close(L["v"].grad, ref[3], 2e-2, "v4 bf16 gv")


def test_long_context_chain_7b_shape():
    """cfg4: 64 consecutive 4096-token segments at B1 C4096 H64, fp32 state carried
    segment to segment on the GPU, forward + backward per segment.  All 64 heads are
    followed on the CPU oracle with their own carried state: per-segment outputs and
    gradients within tolerance and no drift of the carried state."""
    import rwkv_wkv_hip as W
    from rwkv_wkv_hip import configs
    B, T, C, H, NSEG = 1, 4096, 4096, 64, 64
    heads = list(range(H))
    hs = lambda x: x
    state = None
    ref_state = None
    worst = {}
    for seg in range(NSEG):
        wl = configs.make(4, segment=seg)
        cpu = wl.tensors
        if seg == 0:
            state = cpu["state"].to(DEV)
            ref_state = cpu["state"][:, heads].clone()
        t = {n: x.to(DEV) for n, x in cpu.items()}
        t["state"] = state
        got = gpu_fwd_bwd(6, t, B, T, C, H, "auto")
        ref = O.wkv_op_grads(6, B, T, 64 * len(heads), len(heads), hs(cpu["r"]).float(), hs(cpu["k"]).float(),
                             hs(cpu["v"]).float(), hs(cpu["w"]), cpu["u"][heads], ref_state, hs(cpu["dy"]).float(),
                             cpu["dstate"][:, heads])
        pick = {"y": hs, "gr": hs, "gk": hs, "gv": hs, "gw": hs, "gu": lambda x: x[heads],
                "state": lambda x: x[:, heads], "gstate": lambda x: x[:, heads]}
        for n in ref:
            a, b = pick[n](got[n].cpu()).float(), ref[n].float()
            assert_close(a, b, 2e-2, f"segment {seg} {n}")
            worst[n] = max(worst.get(n, 0.0), ((a - b).abs().max() / b.pow(2).mean().sqrt()).item())
        drift = ((got["state"][:, heads].cpu() - ref["state"]).norm() / ref["state"].norm()).item()
        worst["drift"] = max(worst.get("drift", 0.0), drift)
        assert drift < 1e-3, f"state drift {drift} at segment {seg}"
        state = got["state"]
        ref_state = ref["state"]
        if seg % 16 == 0:
            print(f"segment {seg}: drift {drift:.2e}", flush=True)
    print("worst max-error / rms per tensor over the chain:", {k: f"{v:.2e}" for k, v in worst.items()}, flush=True)


def test_full_shape_cumsum_decay_helper():
    """The helper at the shape `bench.py --helper` times (raw decay of cfg3: B8 T4096 C2560, chunk length 128, where
    the chunk's log decays stay in registers): every log-space table of every element against the oracle, one batch
    row at a time, and the exponentiated tables and fp64 re-centred factors of the first and last row."""
    import rwkv_wkv_hip as W
    from rwkv_wkv_hip import configs
    wl = configs.make(3)
    B, T, C, H, chunk = wl.B, wl.T, wl.C, wl.H, 128
    print(f"case helper B{B} T{T} C{C} chunk {chunk}", flush=True)
    raw = wl.tensors["w"].clone()
    raw[0, 9, 5] = 3.0                      # below the floor
    raw[B - 1, T - 1, C - 1] = 2.0
    out = W.cumsum_decay(raw.to(DEV), chunk, factors=True, precision=64)
    torch.cuda.synchronize()
    back = lambda x: x.reshape(1, H, T, 64).transpose(1, 2).reshape(T, C)
    lg = lambda x: x.double().log().float()
    for b in range(B):
        w = O.decay_from_raw(raw[b:b + 1]).view(1, T, H, 64).transpose(1, 2)
        tab = O.cumsum_decay(w, chunk, 64)
        assert_close(out["log_w"][b], back(tab.log_w), 1e-5, f"log_w row {b}")
        assert_close(out["incl"][b], back(tab.incl), 1e-5, f"incl row {b}")
        assert_close(out["inter"][b], back(tab.inter_log), 1e-5, f"inter row {b}")
        assert_close(out["intra"][b], back(tab.intra_log), 1e-5, f"intra row {b}")
        cs = tab.chunk_log[..., 0, :].transpose(1, 2).reshape(T // chunk, C)
        assert_close(out["chunk_sum"][b], cs, 1e-5, f"chunk_sum row {b}")
        if b in (0, B - 1):
            # (exponentials below the smallest normal fp32 come back as 0 from the GPU: absolute floor 1e-37; the
            # exponents are fp32 sums of up to 128 terms summed in another order by torch: 2e-4 relative)
            near = lambda a, r, n: torch.testing.assert_close(a.cpu(), r, rtol=2e-4, atol=1e-37, msg=lambda m: f"{n}: {m}")
            near(out["ws_exp"][b], cs.exp(), "ws_exp")
            near(out["inter_exp"][b], back(tab.inter_log).exp(), "inter_exp")
            near(out["intra_exp"][b], back(tab.intra_log).exp(), "intra_exp")
            assert_close(lg(out["r_decay"][b].cpu()), lg(back(tab.r_decay)), 1e-5, f"log r_decay row {b}")
            assert_close(lg(out["k_inv_decay"][b].cpu()), lg(back(tab.k_inv_decay)), 1e-5, f"log k_inv_decay row {b}")
    assert out["log_w"][0, 9, 5].item() == pytest.approx(-5.298317, abs=1e-5)
