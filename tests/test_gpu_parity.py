"""GPU parity: the HIP operators (through the C ABI and the autograd front
ends) against the CPU oracle on identical seeded inputs.

Tolerances (written where used): rtol 1e-3 for fp32 I/O, 2e-2 for bf16/fp16
I/O, each with an absolute floor of rtol * rms(reference tensor).  The oracle
runs in fp32 on the already-rounded inputs."""
import pytest
import torch

from oracle import wkv4 as O4
from oracle import wkv56 as O
from tests.util import assert_close

pytestmark = pytest.mark.gpu

RTOL = {torch.float32: 1e-3, torch.bfloat16: 2e-2, torch.float16: 2e-2}
NAMES = ("y", "state", "gr", "gk", "gv", "gw", "gu", "gstate")


def dev():
    return torch.device("cuda:0")


def run_gpu56(version, wl, with_gstate=True, algo="auto"):
    import rwkv_wkv_hip as W
    W.set_algo(algo)
    B, T, C, H = wl.B, wl.T, wl.C, wl.H
    g = {n: x.to(dev()) for n, x in wl.tensors.items()}
    leaves = {n: g[n].clone().requires_grad_(True) for n in ("r", "k", "v", "w", "u", "state")}
    if version == 5:
        y, s = W.WKV_5.apply(B, T, C, H, leaves["state"], leaves["r"], leaves["k"], leaves["v"], leaves["w"], leaves["u"])
    else:
        y, s = W.WKV_6.apply(B, T, C, H, leaves["r"], leaves["k"], leaves["v"], leaves["w"], leaves["u"], leaves["state"])
    if with_gstate:
        torch.autograd.backward([y, s], [g["dy"], g["dstate"]])
    else:
        y.backward(g["dy"])
    torch.cuda.synchronize()
    W.set_algo("auto")
    return dict(y=y, state=s, gr=leaves["r"].grad, gk=leaves["k"].grad, gv=leaves["v"].grad, gw=leaves["w"].grad,
                gu=leaves["u"].grad, gstate=leaves["state"].grad)


def run_oracle56(version, wl, with_gstate=True):
    t = wl.tensors
    gs = t["dstate"] if with_gstate else torch.zeros_like(t["dstate"])
    return O.wkv_op_grads(version, wl.B, wl.T, wl.C, wl.H, t["r"].float(), t["k"].float(), t["v"].float(), t["w"],
                          t["u"], t["state"], t["dy"].float(), gs)


def compare(got, ref, rtol, tag):
    for n in NAMES:
        assert_close(got[n], ref[n], rtol, f"{tag}:{n}")


@pytest.mark.parametrize("version", [5, 6])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T", [1, 7, 16, 17, 128, 200, 256])
def test_recurrent_matches_oracle(version, dtype, T):
    from rwkv_wkv_hip import configs
    cfg = 1 if version == 5 else 3
    wl = configs.make(cfg, B=2, T=T, C=128, H=2, dtype=dtype)
    print(f"case v{version} {dtype} T={T}", flush=True)
    got = run_gpu56(version, wl, algo="recurrent")
    ref = run_oracle56(version, wl)
    compare(got, ref, RTOL[dtype], f"v{version}/{dtype}/T{T}")


@pytest.mark.parametrize("version", [5, 6])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("B,T", [(8, 40), (4, 33), (4, 1), (4, 16)])
def test_recurrent_with_many_heads(version, dtype, B, T):
    """The per-token kernels pick their form by how the heads fill the compute units: B*H = 512 (twice the 256 compute
    units of an MI355X) and 256 (once) take one workgroup per head with sixteen state elements per lane, where the
    small shapes of the other tests take two workgroups per head with eight.  T = 40 and 33: whole and ragged blocks
    of sixteen staged tokens, and a last block of one; T = 1 and 16: a single token, a single whole block."""
    from rwkv_wkv_hip import configs
    wl = configs.make(1 if version == 5 else 3, seed=5, B=B, T=T, C=4096, H=64, dtype=dtype)
    print(f"case v{version} {dtype} B={B} T={T}", flush=True)
    got = run_gpu56(version, wl, algo="recurrent")
    ref = run_oracle56(version, wl)
    compare(got, ref, RTOL[dtype], f"v{version}/{dtype}/B{B}T{T}")


@pytest.mark.parametrize("version", [5, 6])
def test_floor_on_decay_and_its_zero_gradient(version):
    """Raw decays large enough that exp(-exp(w)) < 0.005: the operator uses
    0.005 and returns a zero gradient there, as the chunked reference path."""
    from rwkv_wkv_hip import configs
    wl = configs.make(1 if version == 5 else 3, B=1, T=128, C=64, H=1, dtype=torch.float32)
    w = wl.tensors["w"]
    if version == 5:
        w[0, 3] = 2.5
        w[0, 17] = 1.8
    else:
        w[0, 5, 3] = 2.5
        w[0, 77, 40] = 4.0
    got = run_gpu56(version, wl, algo="recurrent")
    ref = run_oracle56(version, wl)
    compare(got, ref, 1e-3, f"floor v{version}")
    gw = got["gw"].cpu()
    if version == 5:
        assert gw[0, 3] == 0 and gw[0, 17] == 0 and gw[0, 4] != 0
    else:
        assert gw[0, 5, 3] == 0 and gw[0, 77, 40] == 0 and gw[0, 5, 4] != 0


@pytest.mark.parametrize("version", [5, 6])
@pytest.mark.parametrize("B,T,H", [(2, 128, 2), (4, 40, 64)])      # (few heads, many heads: the two forms of the kernels)
def test_no_state_gradient_truncated_bptt(version, B, T, H):
    from rwkv_wkv_hip import configs
    wl = configs.make(1 if version == 5 else 3, B=B, T=T, C=64 * H, H=H, dtype=torch.bfloat16)
    got = run_gpu56(version, wl, with_gstate=False, algo="recurrent")
    ref = run_oracle56(version, wl, with_gstate=False)
    for n in NAMES:
        assert_close(got[n], ref[n], 2e-2, f"trunc v{version}:{n}")


def test_segment_chain_equals_one_call_v6():
    """Two chained calls over T tokens each, with the state gradient handed
    back, equal one call over 2T tokens (outputs and every gradient)."""
    import rwkv_wkv_hip as W
    from rwkv_wkv_hip import configs
    W.set_algo("recurrent")
    wl = configs.make(3, B=2, T=256, C=128, H=2, dtype=torch.float32)
    B, T, C, H = wl.B, wl.T, wl.C, wl.H
    g = {n: x.to(dev()) for n, x in wl.tensors.items()}
    L1 = {n: g[n].clone().requires_grad_(True) for n in ("r", "k", "v", "w", "u", "state")}
    y, s = W.WKV_6.apply(B, T, C, H, L1["r"], L1["k"], L1["v"], L1["w"], L1["u"], L1["state"])
    torch.autograd.backward([y, s], [g["dy"], g["dstate"]])
    L2 = {n: g[n].clone().requires_grad_(True) for n in ("r", "k", "v", "w", "u", "state")}
    h = T // 2
    a = lambda x: x[:, :h].contiguous()
    b = lambda x: x[:, h:].contiguous()
    y1, s1 = W.WKV_6.apply(B, h, C, H, a(L2["r"]), a(L2["k"]), a(L2["v"]), a(L2["w"]), L2["u"], L2["state"])
    y2, s2 = W.WKV_6.apply(B, h, C, H, b(L2["r"]), b(L2["k"]), b(L2["v"]), b(L2["w"]), L2["u"], s1)
    torch.autograd.backward([y1, y2, s2], [a(g["dy"]), b(g["dy"]), g["dstate"]])
    torch.cuda.synchronize()
    W.set_algo("auto")
    assert_close(torch.cat([y1, y2], 1), y, 1e-5, "chain y")
    assert_close(s2, s, 1e-5, "chain state")
    for n in ("r", "k", "v", "w", "u", "state"):
        assert_close(L2[n].grad, L1[n].grad, 1e-4, f"chain g{n}")


def test_in_place_wrappers_keep_reference_convention():
    import rwkv_wkv_hip as W
    from rwkv_wkv_hip import configs
    wl = configs.make(1, B=1, T=32, C=128, H=2, dtype=torch.bfloat16)
    g = {n: x.to(dev()) for n, x in wl.tensors.items()}
    B, T, C, H = wl.B, wl.T, wl.C, wl.H
    st = g["state"].clone()
    y = W.RUN_WKV5_CUDA(B, T, C, H, st, g["r"], g["k"], g["v"], g["w"], g["u"].to(torch.bfloat16))
    y2, ns = W.WKV_5.apply(B, T, C, H, g["state"], g["r"], g["k"], g["v"], g["w"], g["u"])
    assert y.shape == (B, T, C) and y.dtype == torch.bfloat16
    assert torch.equal(st, ns) and not torch.equal(st, g["state"])
    wl6 = configs.make(3, B=1, T=32, C=128, H=2, dtype=torch.bfloat16)
    g6 = {n: x.to(dev()) for n, x in wl6.tensors.items()}
    s6 = g6["state"].clone()
    y6 = W.WKV6STATE_CUDA.apply(B, T, C, H, g6["r"], g6["k"], g6["v"], g6["w"], g6["u"], s6)
    _, ns6 = W.WKV_6.apply(B, T, C, H, g6["r"], g6["k"], g6["v"], g6["w"], g6["u"], g6["state"])
    assert torch.equal(s6, ns6) and y6.dtype == torch.bfloat16


# ------------------------------------------------------------------ v4 -----
def v4_case(B, T, C, dtype, seed=0, with_state=False):
    from rwkv_wkv_hip import configs
    wl = configs.make(2, B=B, T=T, C=C, dtype=dtype, seed=seed)
    t = wl.tensors
    if with_state:
        g = torch.Generator().manual_seed(seed + 50)
        t["state"] = torch.stack([torch.randn(B, C, generator=g), torch.rand(B, C, generator=g) + 0.5,
                                  torch.randn(B, C, generator=g)], -1)
        t["dstate"] = torch.stack([torch.randn(B, C, generator=g), torch.randn(B, C, generator=g),
                                   torch.randn(B, C, generator=g) * 0.3], -1)
    return wl


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,with_state", [(1, False), (16, False), (37, True), (128, True), (300, False)])
def test_v4_matches_oracle(dtype, T, with_state):
    import rwkv_wkv_hip as W
    B, C = 3, 96
    wl = v4_case(B, T, C, dtype, with_state=with_state)
    t = wl.tensors
    print(f"case v4 {dtype} T={T} state={with_state}", flush=True)
    f32 = lambda x: x.float()
    y_ref, s_ref = O4.forward(t["time_decay"], f32(t["time_first"]), f32(t["k"]), f32(t["v"]), t["state"])
    ref = O4.backward(t["time_decay"], f32(t["time_first"]), f32(t["k"]), f32(t["v"]), t["state"], f32(t["dy"]),
                      t["dstate"])
    g = {n: x.to(dev()) for n, x in t.items()}
    L = {n: g[n].clone().requires_grad_(True) for n in ("time_decay", "time_first", "k", "v", "state")}
    y, s = W.wkv_op(L["time_decay"], L["time_first"], L["k"], L["v"], L["state"])
    torch.autograd.backward([y, s], [g["dy"], g["dstate"]])
    torch.cuda.synchronize()
    rt = RTOL[dtype]
    assert_close(y, y_ref, rt, "v4 y")
    und = lambda st: st[..., :2].float().cpu() * torch.exp(st[..., 2:3].float().cpu())
    assert_close(und(s), und(s_ref), 1e-3, "v4 state (undivided sums)")
    assert_close(L["time_decay"].grad, ref[0], rt, "v4 g_time_decay")
    assert_close(L["time_first"].grad, ref[1], rt, "v4 g_time_first")
    assert_close(L["k"].grad, ref[2], rt, "v4 gk")
    assert_close(L["v"].grad, ref[3], rt, "v4 gv")
    assert_close(und(L["state"].grad), und(ref[4]), rt, "v4 gstate (undivided)")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,T,C", [(1, 50, 8), (2, 33, 100), (3, 17, 130), (1, 200, 64), (5, 97, 52), (2, 49, 256), (1, 96, 328)])
def test_v4_shapes(dtype, B, T, C):
    """Widths that take the 16-byte fetches of the forward (C a multiple of 4 for fp32, of 8 for the 16-bit types) and
    widths that do not, chains that do not fill the last wavefront or the second group of the last workgroup, lengths
    that end inside a block, inside a lap of three blocks and on their boundaries: y, the state and every gradient."""
    import rwkv_wkv_hip as W
    wl = v4_case(B, T, C, dtype, seed=B + T + C, with_state=True)
    t = wl.tensors
    print(f"case v4 shapes {dtype} B={B} T={T} C={C}", flush=True)
    f32 = lambda x: x.float()
    y_ref, s_ref = O4.forward(t["time_decay"], f32(t["time_first"]), f32(t["k"]), f32(t["v"]), t["state"])
    ref = O4.backward(t["time_decay"], f32(t["time_first"]), f32(t["k"]), f32(t["v"]), t["state"], f32(t["dy"]),
                      t["dstate"])
    g = {n: x.to(dev()) for n, x in t.items()}
    L = {n: g[n].clone().requires_grad_(True) for n in ("time_decay", "time_first", "k", "v", "state")}
    y, s = W.wkv_op(L["time_decay"], L["time_first"], L["k"], L["v"], L["state"])
    torch.autograd.backward([y, s], [g["dy"], g["dstate"]])
    torch.cuda.synchronize()
    rt = RTOL[dtype]
    assert y.dtype == dtype
    assert_close(y, y_ref, rt, "v4 y")
    und = lambda st: st[..., :2].float().cpu() * torch.exp(st[..., 2:3].float().cpu())
    assert_close(und(s), und(s_ref), 1e-3, "v4 state (undivided sums)")
    assert_close(L["time_decay"].grad, ref[0], rt, "v4 g_time_decay")
    assert_close(L["time_first"].grad, ref[1], rt, "v4 g_time_first")
    assert_close(L["k"].grad, ref[2], rt, "v4 gk")
    assert_close(L["v"].grad, ref[3], rt, "v4 gv")
    assert_close(und(L["state"].grad), und(ref[4]), rt, "v4 gstate (undivided)")


def test_v4_backward_without_forward_checkpoints():
    """The C entry point rebuilds its checkpoints when none are passed."""
    import ctypes
    from rwkv_wkv_hip import _lib
    L = _lib.lib()
    B, T, C = 2, 50, 64
    wl = v4_case(B, T, C, torch.float32, seed=3, with_state=True)
    t = wl.tensors
    ref = O4.backward(t["time_decay"], t["time_first"], t["k"], t["v"], t["state"], t["dy"], t["dstate"])
    g = {n: x.to(dev()).contiguous() for n, x in t.items()}
    gtd, gtf = torch.empty(C, device=dev()), torch.empty(C, device=dev())
    gk, gv, gst = torch.empty_like(g["k"]), torch.empty_like(g["v"]), torch.empty_like(g["state"])
    ws = torch.empty(L.wkv4_backward_workspace(B, T, C, 0), dtype=torch.uint8, device=dev())
    p = lambda x: x.data_ptr()
    st = L.wkv4_backward(None, B, T, C, 0, p(g["time_decay"]), p(g["time_first"]), p(g["k"]), p(g["v"]), p(g["state"]),
                         p(g["dy"]), p(g["dstate"]), p(gtd), p(gtf), p(gk), p(gv), p(gst), None, p(ws), ws.numel())
    torch.cuda.synchronize()
    assert st == 0
    assert_close(gk, ref[2], 1e-3, "gk")
    assert_close(gv, ref[3], 1e-3, "gv")
    assert_close(gtd, ref[0], 1e-3, "gtd")


# -------------------------------------------------------------- helper -----
@pytest.mark.parametrize("chunk", [16, 128])
def test_cumsum_decay_helper(chunk):
    import rwkv_wkv_hip as W
    B, T, H, K = 2, 256, 3, 64
    C = H * K
    g = torch.Generator().manual_seed(11)
    raw = torch.randn(B, T, C, generator=g) * 0.8 - 0.5
    raw[0, 9, 5] = 3.0                                   # below the floor
    out = W.cumsum_decay(raw.to(dev()), chunk)
    w = O.decay_from_raw(raw).view(B, T, H, K).transpose(1, 2)           # (B,H,T,K)
    tab = O.cumsum_decay(w, chunk, 64)
    back = lambda x: x.reshape(B, H, T, K).transpose(1, 2).reshape(B, T, C)
    assert_close(out["log_w"], back(tab.log_w), 1e-5, "log_w")
    assert_close(out["incl"], back(tab.incl), 1e-5, "incl")
    assert_close(out["inter"], back(tab.inter_log), 1e-5, "inter")
    assert_close(out["intra"], back(tab.intra_log), 1e-5, "intra")
    cs = tab.chunk_log[..., 0, :].transpose(1, 2).reshape(B, T // chunk, C)
    assert_close(out["chunk_sum"], cs, 1e-5, "chunk_sum")
    assert out["log_w"][0, 9, 5].item() == pytest.approx(-5.298317, abs=1e-5)
    # every table of the reference's helper, including the exponentiated ones and the re-centred fp64 factors
    full = W.cumsum_decay(raw.to(dev()), chunk, factors=True, precision=64)
    for n in ("log_w", "incl", "inter", "intra", "chunk_sum"):
        assert torch.equal(full[n], out[n]), n
    # (exponentials below the smallest normal fp32, 1.2e-38, come back as 0 from the GPU: absolute floor 1e-37; the
    # exponents are fp32 sums of up to 128 terms of size ~5, summed in another order by torch: 2e-4 relative)
    near = lambda a, b, n: torch.testing.assert_close(a.cpu(), b, rtol=2e-4, atol=1e-37, msg=lambda m: f"{n}: {m}")
    near(full["ws_exp"], cs.exp(), "ws_exp")
    near(full["inter_exp"], back(tab.inter_log).exp(), "inter_exp")
    near(full["intra_exp"], back(tab.intra_log).exp(), "intra_exp")
    assert full["r_decay"].dtype == torch.float64
    lg = lambda x: x.double().log().float()          # compared in log space: the factors span hundreds of orders of magnitude
    assert_close(lg(full["r_decay"].cpu()), lg(back(tab.r_decay)), 1e-5, "log r_decay")
    assert_close(lg(full["k_inv_decay"].cpu()), lg(back(tab.k_inv_decay)), 1e-5, "log k_inv_decay")
    if chunk == 16:
        f32 = W.cumsum_decay(raw.to(dev()), chunk, factors=True, precision=32)
        assert f32["r_decay"].dtype == torch.float32
        assert_close(f32["r_decay"], back(O.cumsum_decay(w, chunk, 32).r_decay), 1e-4, "r_decay fp32")
    # per-channel (WKV5) form
    out5 = W.cumsum_decay(raw[0, 0].to(dev()), chunk, per_token=T)
    w5 = O.decay_from_raw(raw[0, 0]).view(1, H, 1, K).expand(1, H, T, K)
    tab5 = O.cumsum_decay(w5, chunk, 64)
    assert_close(out5["incl"], tab5.incl.reshape(1, H, T, K).transpose(1, 2).reshape(1, T, C), 1e-5, "incl v5")


# ------------------------------------------------- blocked matrix-core path --
def run_gpu56_forward(version, wl, algo):
    import rwkv_wkv_hip as W
    W.set_algo(algo)
    B, T, C, H = wl.B, wl.T, wl.C, wl.H
    g = {n: x.to(dev()) for n, x in wl.tensors.items()}
    with torch.no_grad():
        if version == 5:
            y, s = W.WKV_5.apply(B, T, C, H, g["state"], g["r"], g["k"], g["v"], g["w"], g["u"])
        else:
            y, s = W.WKV_6.apply(B, T, C, H, g["r"], g["k"], g["v"], g["w"], g["u"], g["state"])
    torch.cuda.synchronize()
    W.set_algo("auto")
    return y, s


@pytest.mark.parametrize("version", [5, 6])
@pytest.mark.parametrize("T", [16, 50, 64, 128, 200, 512])
def test_chunked_forward_matches_oracle(version, T):
    from rwkv_wkv_hip import configs
    wl = configs.make(1 if version == 5 else 3, B=2, T=T, C=192, H=3, dtype=torch.bfloat16)
    print(f"case chunked fwd v{version} T={T}", flush=True)
    y, s = run_gpu56_forward(version, wl, "chunked")
    t = wl.tensors
    with torch.no_grad():
        if version == 5:
            y_ref, s_ref = O.wkv5_op(wl.B, T, wl.C, wl.H, t["state"], t["r"], t["k"], t["v"], t["w"], t["u"])
        else:
            y_ref, s_ref = O.wkv6_op(wl.B, T, wl.C, wl.H, t["r"], t["k"], t["v"], t["w"], t["u"], t["state"])
    assert_close(y, y_ref, 2e-2, "y")
    assert_close(s, s_ref, 2e-2, "state")
    # and against the per-token fp32 kernel on the same device
    y2, s2 = run_gpu56_forward(version, wl, "recurrent")
    assert_close(y, y2, 2e-2, "y vs recurrent")
    assert_close(s, s2, 2e-2, "state vs recurrent")


def test_chunked_forward_strong_decay_and_floor():
    """Decays at and below the floor for whole blocks: the re-centred factors
    reach e^{+-42} and must neither overflow nor lose the result."""
    from rwkv_wkv_hip import configs
    wl = configs.make(3, B=1, T=128, C=128, H=2, dtype=torch.bfloat16)
    w = wl.tensors["w"]
    w[:, :, :32] = 1.9            # exp(-exp(1.9)) = 1.2e-3 < 0.005 -> floored
    w[:, :, 32:64] = 1.6          # exp(-exp(1.6)) = 7.1e-3, just above the floor
    w[:, 40:60, 64:96] = 5.0
    y, s = run_gpu56_forward(6, wl, "chunked")
    t = wl.tensors
    with torch.no_grad():
        y_ref, s_ref = O.wkv6_op(wl.B, wl.T, wl.C, wl.H, t["r"], t["k"], t["v"], t["w"], t["u"], t["state"])
    assert_close(y, y_ref, 2e-2, "y")
    assert_close(s, s_ref, 2e-2, "state")


@pytest.mark.parametrize("version", [5, 6])
@pytest.mark.parametrize("T", [16, 40, 64, 128, 200, 512])
def test_chunked_forward_backward_matches_oracle(version, T):
    from rwkv_wkv_hip import configs
    wl = configs.make(1 if version == 5 else 3, B=2, T=T, C=192, H=3, dtype=torch.bfloat16)
    print(f"case chunked fwd+bwd v{version} T={T}", flush=True)
    got = run_gpu56(version, wl, algo="chunked")
    ref = run_oracle56(version, wl)
    compare(got, ref, 2e-2, f"chunked v{version}/T{T}")


@pytest.mark.parametrize("version", [5, 6])
def test_chunked_truncated_bptt_and_floor(version):
    from rwkv_wkv_hip import configs
    wl = configs.make(1 if version == 5 else 3, B=1, T=192, C=128, H=2, dtype=torch.bfloat16)
    w = wl.tensors["w"]
    if version == 5:
        w[0, 3] = 2.5
        w[1, 17] = 1.8
    else:
        w[0, 5, 3] = 2.5
        w[0, 100:140, 64:96] = 1.9
    got = run_gpu56(version, wl, with_gstate=False, algo="chunked")
    ref = run_oracle56(version, wl, with_gstate=False)
    compare(got, ref, 2e-2, f"chunked trunc/floor v{version}")
    gw = got["gw"].cpu()
    if version == 5:
        assert gw[0, 3] == 0 and gw[1, 17] == 0 and gw[0, 4] != 0
    else:
        assert gw[0, 5, 3] == 0 and (gw[0, 100:140, 64:96] == 0).all() and gw[0, 5, 4] != 0


def test_chunked_backward_rebuilds_checkpoints_when_not_given():
    """Backward through the C ABI without WKV_CHECKPOINTS_VALID equals backward with it."""
    from rwkv_wkv_hip import _lib, configs
    L = _lib.lib()
    wl = configs.make(3, B=1, T=256, C=128, H=2, dtype=torch.bfloat16)
    B, T, C, H = wl.B, wl.T, wl.C, wl.H
    g = {n: x.to(dev()).contiguous() for n, x in wl.tensors.items()}
    p = lambda x: x.data_ptr()
    outs = []
    for valid in (True, False):
        ws = torch.zeros(L.wkv6_backward_workspace(B, T, C, H, 1, 2), dtype=torch.uint8, device=dev())
        y, so = torch.empty_like(g["r"]), torch.empty_like(g["state"])
        flags = _lib.FLOOR_DECAY
        if valid:
            assert L.wkv6_forward(None, B, T, C, H, 1, flags, 2, p(g["r"]), p(g["k"]), p(g["v"]), p(g["w"]), p(g["u"]),
                                  p(g["state"]), p(y), p(so), p(ws), ws.numel()) == 0
            flags |= _lib.CHECKPOINTS_VALID
        gr, gk, gv = (torch.empty_like(g["r"]) for _ in range(3))
        gw, gu, gs = torch.empty_like(g["w"]), torch.empty_like(g["u"]), torch.empty_like(g["state"])
        assert L.wkv6_backward(None, B, T, C, H, 1, flags, 2, p(g["r"]), p(g["k"]), p(g["v"]), p(g["w"]), p(g["u"]),
                               p(g["state"]), p(g["dy"]), p(g["dstate"]), p(gr), p(gk), p(gv), p(gw), p(gu), p(gs),
                               p(ws), ws.numel()) == 0
        torch.cuda.synchronize()
        outs.append((gr, gk, gv, gw, gu, gs))
    for a, b_ in zip(*outs):
        assert torch.equal(a, b_)


@pytest.mark.parametrize("version", [5, 6])
@pytest.mark.parametrize("nseg,T", [(1, 1024), (2, 1024), (4, 1024), (3, 1000), (5, 1344), (8, 832)])
def test_chunked_time_segments(version, nseg, T):
    """The time-parallel split (segment summaries folded in order) gives the same
    outputs and gradients as the oracle for any number of segments, ragged ones included."""
    from rwkv_wkv_hip import _lib, configs
    L = _lib.lib()
    wl = configs.make(1 if version == 5 else 3, B=1, T=T, C=128, H=2, dtype=torch.bfloat16)
    print(f"case segments v{version} nseg={nseg} T={T}", flush=True)
    assert L.wkv_tune(_lib.TUNE_SEGMENTS, nseg) == 0
    try:
        got = run_gpu56(version, wl, algo="chunked")
    finally:
        assert L.wkv_tune(_lib.TUNE_SEGMENTS, 0) == 0
    ref = run_oracle56(version, wl)
    compare(got, ref, 2e-2, f"segments v{version}/n{nseg}/T{T}")


def _slow_decay_case(kind, T):
    """cfg3 data with the raw decay moved so that the summary passes of the time split cannot stop early.
    RWKV-v6 initialises time_decay in [-6, -1] (decay 0.9975 .. 0.69 per token), the training case; the benchmark
    distribution N(-1, 0.5) forgets within about a hundred tokens."""
    from rwkv_wkv_hip import configs
    wl = configs.make(3, B=1, T=T, C=256, H=4, dtype=torch.bfloat16)
    w = wl.tensors["w"]
    if kind == "all":                   # every head keeps its state across whole segments: no piece stops
        w -= 5.0
    elif kind == "half":                # heads 0, 1 slow, heads 2, 3 fast: neighbouring pieces report 0 and non-zero decays
        w[:, :, :128] -= 5.0
    elif kind == "turns":               # head 1 turns slow in the middle of a segment, head 2 turns fast there;
        w[:, T // 4 + 96:, 64:128] -= 5.0       # single channels of head 3 stay slow while the others forget
        w[:, :T // 4 + 96, 128:192] -= 5.0
        w[:, :, 192:200] -= 6.0
    return wl


@pytest.mark.parametrize("kind", ["all", "half", "turns"])
@pytest.mark.parametrize("nseg,pps", [(2, 0), (4, 0), (2, 8), (4, 3)])
def test_chunked_time_segments_slow_decay(kind, nseg, pps):
    """The time split with decays that do not forget inside a piece: the summary passes walk their pieces to the end
    (no early exit), heads that stop and heads that do not sit side by side, and the chaining of the summaries in the
    main kernels' prologues runs over every piece.  pps = steps per piece (0: the planner's choice, 2-step pieces
    at this size; 8 and 3: pieces of several steps, ragged ones included).  All eight outputs against the oracle."""
    from rwkv_wkv_hip import _lib
    L = _lib.lib()
    T = 2048
    wl = _slow_decay_case(kind, T)
    print(f"case slow decay {kind} nseg={nseg} pps={pps}", flush=True)
    assert L.wkv_tune(_lib.TUNE_SEGMENTS, nseg) == 0 and L.wkv_tune(_lib.TUNE_PIECE_STEPS, pps) == 0
    try:
        got = run_gpu56(6, wl, algo="chunked")
    finally:
        assert L.wkv_tune(_lib.TUNE_SEGMENTS, 0) == 0 and L.wkv_tune(_lib.TUNE_PIECE_STEPS, 0) == 0
    ref = run_oracle56(6, wl)
    compare(got, ref, 2e-2, f"slow decay {kind}/n{nseg}/p{pps}")       # bf16 I/O: rtol 2e-2, floor 2e-2 rms


@pytest.mark.parametrize("nseg,T", [(1, 200), (3, 1000)])
@pytest.mark.parametrize("shift", [0.0, -5.0])
def test_chunked_v6_takes_bf16_decay(nseg, T, shift):
    """The raw decay handed over in bf16 (what a mixed-precision TimeMix produces and the reference widens with
    w.float(), RWKV-v6/src/module/TimeMix.py:50) is read as it is by the blocked kernels, and its gradient comes
    back in bf16 (as the reference allocates it, :90): same results as the oracle on the widened tensor."""
    import ctypes
    from rwkv_wkv_hip import _lib, configs
    L = _lib.lib()
    wl = configs.make(3, B=2, T=T, C=128, H=2, dtype=torch.bfloat16)
    wl.tensors["w"] = (wl.tensors["w"] + shift).to(torch.bfloat16)          # (shift -5: no piece of the split's passes stops early)
    print(f"case bf16 decay nseg={nseg} T={T} shift={shift}", flush=True)
    assert L.wkv_tune(_lib.TUNE_SEGMENTS, nseg) == 0
    try:
        got = run_gpu56(6, wl, algo="chunked")
    finally:
        assert L.wkv_tune(_lib.TUNE_SEGMENTS, 0) == 0
    assert got["gw"].dtype == torch.bfloat16
    wide = configs.make(3, B=2, T=T, C=128, H=2, dtype=torch.bfloat16)
    wide.tensors["w"] = wl.tensors["w"].float()
    ref = run_oracle56(6, wide)
    compare(got, ref, 2e-2, f"bf16 decay n{nseg}/T{T}")
    # token by token there is no bf16 decay at the C boundary: the entry point says so
    B, C, H = wl.B, wl.C, wl.H
    g = {n: x.to(dev()).contiguous() for n, x in wl.tensors.items()}
    y, s = torch.empty_like(g["r"]), torch.empty_like(g["state"])
    p = lambda x: ctypes.c_void_p(x.data_ptr())
    st = L.wkv6_forward(None, B, T, C, H, 1, _lib.FLOOR_DECAY | _lib.W_BF16, 1, p(g["r"]), p(g["k"]), p(g["v"]), p(g["w"]),
                        p(g["u"]), p(g["state"]), p(y), p(s), None, 0)
    assert st == -7


def test_chunked_needs_the_decay_floor():
    """T = 1 follows the reference's single-step branch (no floor on the decay); the blocked
    path's range analysis relies on the floor, so it refuses and 'auto' takes the per-token path."""
    import rwkv_wkv_hip as W
    from rwkv_wkv_hip import configs
    wl = configs.make(3, B=1, T=1, C=64, H=1, dtype=torch.bfloat16)
    g = {n: x.to(dev()) for n, x in wl.tensors.items()}
    W.set_algo("chunked")
    try:
        with pytest.raises(W.WKVError):
            W.WKV_6.apply(1, 1, 64, 1, g["r"], g["k"], g["v"], g["w"], g["u"], g["state"])
    finally:
        W.set_algo("auto")
    y, s = W.WKV_6.apply(1, 1, 64, 1, g["r"], g["k"], g["v"], g["w"], g["u"], g["state"])
    t = wl.tensors
    y_ref, s_ref = O.wkv6_op(1, 1, 64, 1, t["r"], t["k"], t["v"], t["w"], t["u"], t["state"])
    assert_close(y, y_ref, 2e-2, "y")
    assert_close(s, s_ref, 1e-3, "state")


@pytest.mark.parametrize("nseg_fwd,nseg_bwd", [(4, 2), (2, 8), (0, 3)])
def test_plan_may_change_between_forward_and_backward(nseg_fwd, nseg_bwd):
    """The number of time segments (wkv_tune) differs between the forward call and its backward call: only the
    state checkpoints pass between the two, so every gradient still matches the oracle."""
    import rwkv_wkv_hip as W
    from rwkv_wkv_hip import _lib, configs
    L = _lib.lib()
    wl = configs.make(3, B=1, T=1024, C=128, H=2, dtype=torch.bfloat16)
    B, T, C, H = wl.B, wl.T, wl.C, wl.H
    g = {n: x.to(dev()) for n, x in wl.tensors.items()}
    leaves = {n: g[n].clone().requires_grad_(True) for n in ("r", "k", "v", "w", "u", "state")}
    try:
        assert L.wkv_tune(_lib.TUNE_SEGMENTS, nseg_fwd) == 0
        y, s = W.WKV_6.apply(B, T, C, H, leaves["r"], leaves["k"], leaves["v"], leaves["w"], leaves["u"], leaves["state"])
        assert L.wkv_tune(_lib.TUNE_SEGMENTS, nseg_bwd) == 0
        torch.autograd.backward([y, s], [g["dy"], g["dstate"]])
        torch.cuda.synchronize()
    finally:
        L.wkv_tune(_lib.TUNE_SEGMENTS, 0)
    got = dict(y=y, state=s, gr=leaves["r"].grad, gk=leaves["k"].grad, gv=leaves["v"].grad, gw=leaves["w"].grad,
               gu=leaves["u"].grad, gstate=leaves["state"].grad)
    compare(got, run_oracle56(6, wl), 2e-2, f"plan {nseg_fwd}->{nseg_bwd}")


def _sweep_cases():
    """Seeded random shapes and decay regimes for the blocked path: ragged lengths, one to seven heads, forced and
    automatic time splits with forced piece lengths, fast / slow / mixed / floored decays, with and without a state
    gradient arriving."""
    import random
    rnd = random.Random(20240611)
    cases = []
    for i in range(24):
        version = 5 if i % 3 == 0 else 6
        B, H = rnd.choice([1, 2, 3]), rnd.choice([1, 2, 3, 5, 7])
        T = rnd.choice([rnd.randint(2, 63), rnd.randint(64, 400), rnd.randint(401, 1500), 64 * rnd.randint(1, 20)])
        nseg = rnd.choice([0, 1, 2, 3, 5])
        pps = rnd.choice([0, 0, 1, 3])
        regime = rnd.choice(["fast", "slow", "mixed", "floor"])
        cases.append((i, version, B, H, T, nseg, pps, regime, rnd.random() < 0.75))
    return cases


@pytest.mark.parametrize("case", _sweep_cases(), ids=lambda c: f"{c[0]}-v{c[1]}-B{c[2]}H{c[3]}T{c[4]}-n{c[5]}p{c[6]}-{c[7]}")
def test_chunked_random_sweep(case):
    from rwkv_wkv_hip import _lib, configs
    L = _lib.lib()
    i, version, B, H, T, nseg, pps, regime, with_gstate = case
    wl = configs.make(1 if version == 5 else 3, B=B, T=T, C=64 * H, H=H, dtype=torch.bfloat16, seed=5000 + i)
    w = wl.tensors["w"]
    g = torch.Generator().manual_seed(7000 + i)
    if regime == "slow":
        w -= 4.0 if version == 6 else 0.0            # (WKV5 draws its decay from U(-6, 0): slow channels are in it already)
    elif regime == "mixed":
        mask = torch.rand(w.shape[-1] if version == 6 else w.shape, generator=g) < 0.5
        w[..., mask] -= 4.5 if version == 6 else 0.0
        if version == 5:
            w[mask] -= 2.0
    elif regime == "floor":
        hit = torch.rand(w.shape, generator=g) < 0.05
        w[hit] = 2.5                                  # exp(-exp(2.5)) = 5e-6: held at the floor of 0.005
    print(f"case sweep {case}", flush=True)
    assert L.wkv_tune(_lib.TUNE_SEGMENTS, nseg) == 0 and L.wkv_tune(_lib.TUNE_PIECE_STEPS, pps) == 0
    try:
        got = run_gpu56(version, wl, with_gstate=with_gstate, algo="chunked")
    finally:
        assert L.wkv_tune(_lib.TUNE_SEGMENTS, 0) == 0 and L.wkv_tune(_lib.TUNE_PIECE_STEPS, 0) == 0
    ref = run_oracle56(version, wl, with_gstate=with_gstate)
    compare(got, ref, 2e-2, f"sweep {case}")              # bf16 I/O: rtol 2e-2, floor 2e-2 rms
    if regime == "floor":
        hit_gw = got["gw"].float().cpu()[hit]
        assert (hit_gw == 0).all(), "no gradient where the floor holds"
