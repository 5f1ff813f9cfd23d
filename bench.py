#!/usr/bin/env python3
"""Benchmark of the WKV hot path on one MI355X.

Default workload (``--cfg 4``): WKV6 forward+backward on one 4096-token BPTT
segment at the RWKV-v6 7B layer shape (B=1, C=4096, H=64, head 64; bf16 r/k/v/dy,
fp32 raw decay, fp32 state), the state carried from step to step and the state
gradient fed back, i.e. one link of the long-context chain per step.  A "step"
is one forward + one backward call through the C ABI with all inputs resident
in HBM.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--cfg 1|2|3|4] [--algo auto|recurrent|chunked]
                    [--launch graph|eager] [--no-extras]

Besides the line's own figures (``value``, ``ms_per_step``: the workload as BASELINE.json states it) the default run
times the same K steps two more ways and reports them under their own keys: ``slow_decay`` (WKV6: the raw decay
shifted by -5, i.e. no channel forgets inside a segment, which is what a freshly initialised RWKV-v6 layer looks
like and the worst case of the time split's summary passes) and ``cold`` (the backward call of a segment runs two
steps after its forward call, with other segments' calls in between, so that nothing it reads is still in the
last-level cache: what a training step with a whole layer stack between forward and backward sees).

The K timed steps are launched from HIP graphs (one graph of K steps up to
K = 128; beyond that a 120-step body replayed K // 120 times plus one graph with
the rest), or as plain launches with ``--launch eager`` (and whenever the capture
fails).  They are timed twice: between two HIP events on the launch stream with
the queue primed (``ms_per_step``, ``value``) and between two device
synchronisations by the host clock (``ms_per_step_host``).
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "rwkv-infctx-trainer_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=600)      # 0.2 s of GPU time at cfg4: short runs measure the launch
    ap.add_argument("--warmup", type=int, default=30)      # and synchronisation latencies of the host more than the kernels
    ap.add_argument("--cfg", type=int, default=4, choices=[1, 2, 3, 4])
    ap.add_argument("--algo", default="auto", choices=["auto", "recurrent", "chunked"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-heads", type=int, default=16, help="heads of the workload the CPU baseline times")
    ap.add_argument("--rotate", type=int, default=3, help="distinct input sets cycled through")
    ap.add_argument("--launch", default="graph", choices=["graph", "eager"],
                    help="timed steps replayed from a HIP graph of one rotation period, or launched one by one")
    ap.add_argument("--w-dtype", default="fp32", choices=["fp32", "bf16"],
                    help="WKV6 only: dtype of the raw decay tensor and its gradient (fp32 is what the workload is "
                         "defined with; bf16 is what a mixed-precision TimeMix hands over)")
    ap.add_argument("--io-dtype", default=None, choices=["bf16", "fp16", "fp32"],
                    help="dtype of r, k, v, dy and of y, gr, gk, gv.  Default: what the workload states (bf16 for WKV5/WKV6, "
                         "fp32 for WKV4).  The reference binds all three for WKV5 (RWKV-v5/src/module/cuda/wkv5_op.cpp:84-129) "
                         "and bf16 alone for WKV4 (RWKV-v4neo/cuda/wkv_op_bf16.cpp:45-51)")
    ap.add_argument("--helper", action="store_true",
                    help="time the cumulative-decay helper alone (all tables, chunk length 128) on the raw decay tensor of "
                         "--cfg 3 instead of the operators")
    ap.add_argument("--edges", action="store_true",
                    help="time the element-wise passes around the operator (token shift + mixing, ln_x * gate, channel-mix "
                         "activations, L2Wrap backward) at the cfg3 and cfg4 shapes instead of the operator")
    ap.add_argument("--block", action="store_true",
                    help="time one whole RWKV-v6 TimeMix + ChannelMix layer (cfg4 width, fwd+bwd): element-wise passes on the "
                         "HIP kernels against the same layer with torch element-wise ops around the same WKV operator")
    ap.add_argument("--block-way", default="both", choices=["both", "kernels", "torch"],
                    help="--block: time only the layer on the HIP element-wise kernels, only the one with torch element-wise "
                         "ops, or both (for a profile of one of them alone)")
    ap.add_argument("--w-shift", type=float, default=0.0,
                    help="WKV6 only: added to the raw decay parameter (negative = slower decay; -5 makes every channel "
                         "remember for thousands of tokens, the worst case of the time-parallel split's summary passes)")
    ap.add_argument("--settle-ms", type=float, default=100.0,
                    help="untimed replays of the captured steps for this long before the timed region (the first replays "
                         "of a fresh graph run ~8 %% slower than the steady state a long run measures)")
    ap.add_argument("--segments", type=int, default=0, help="force the number of parallel time segments (0 = auto)")
    ap.add_argument("--no-extras", action="store_true", help="skip the slow-decay and cold-cache measurements of the default run")
    ap.add_argument("--cold", action="store_true",
                    help="make the cold-cache order (backward of the segment two steps back, then forward of this step's) the "
                         "one that value / ms_per_step report")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="also run three plain 256 MiB device copies first (reference point for the FETCH_SIZE / "
                         "WRITE_SIZE counters of a profiler run)")
    return ap.parse_args()


class Runner56:
    """WKV5 / WKV6 forward+backward through the C ABI on preallocated buffers."""

    def __init__(self, cfg, algo, rotate, w_dtype="fp32", w_shift=0.0, io_dtype="bf16"):
        import torch
        from rwkv_wkv_hip import _lib, configs
        self.torch, self._lib, self.L = torch, _lib, _lib.lib()
        dev = torch.device("cuda:0")
        self.sets = []
        for i in range(rotate):
            wl = configs.make(cfg, seed=1000 + cfg + i)
            self.sets.append({n: t.to(dev).contiguous() for n, t in wl.tensors.items()})
        self.wl = wl
        self.version = wl.version
        self.w16 = w_dtype == "bf16" and wl.version == 6
        io = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[io_dtype]
        if io != wl.dtype:
            for st in self.sets:
                for n in ("r", "k", "v", "dy"):
                    st[n] = st[n].to(io)
            wl.dtype = io
        if w_shift and wl.version == 6:
            for st in self.sets:
                st["w"] = st["w"] + w_shift
        if self.w16:
            for st in self.sets:
                st["w"] = st["w"].to(torch.bfloat16)
        B, T, C, H = wl.B, wl.T, wl.C, wl.H
        self.dims = (B, T, C, H)
        self.dt = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}[wl.dtype]
        self.algo = {"auto": 0, "recurrent": 1, "chunked": 2}[algo]
        s0 = self.sets[0]
        self.y, self.gr, self.gk, self.gv = (torch.empty_like(s0["r"]) for _ in range(4))
        self.gw = torch.empty_like(s0["w"])
        self.gu = torch.empty_like(s0["u"])
        self.state = [s0["state"].clone(), torch.empty_like(s0["state"])]
        # the state gradient a backward call hands back is the one the next step's backward call is given
        self.gstate = [s0["dstate"].clone(), torch.empty_like(s0["state"])]
        L = self.L
        q = (L.wkv5_forward_workspace, L.wkv5_backward_workspace) if self.version == 5 else \
            (L.wkv6_forward_workspace, L.wkv6_backward_workspace)
        nws = max(q[0](B, T, C, H, self.dt, self.algo), q[1](B, T, C, H, self.dt, self.algo), 16)
        self.ws = torch.empty(nws, dtype=torch.uint8, device=dev)
        self.ws_cold = None                             # second workspace, cold-cache order only
        self.have_ckpt = q[0](B, T, C, H, self.dt, self.algo) > 0      # the forward call leaves its checkpoints in the workspace
        self.fwd = L.wkv5_forward if self.version == 5 else L.wkv6_forward
        self.bwd = L.wkv5_backward if self.version == 5 else L.wkv6_backward
        self.stream = torch.cuda.current_stream().cuda_stream
        self.i = 0
        self.tokens_per_step = B * T
        elems = B * T * C
        st = B * H * 64 * 64 * 4
        wb = 2 if self.w16 else 4                       # bytes of a decay / decay-gradient element
        eb = 4 if io == torch.float32 else 2            # bytes of an r, k, v, y, gradient element
        fwd_b = (4 * eb + wb) if self.version == 6 else 4 * eb
        bwd_b = (7 * eb + 2 * wb) if self.version == 6 else 7 * eb
        self.bytes_step = (fwd_b + bwd_b) * elems + 5 * st
        self.bytes_fwd = fwd_b * elems + 2 * st
        self.bytes_bwd = bwd_b * elems + 3 * st
        self.dtype_name = {"bf16": "bf16", "fp16": "f16", "fp32": "f32"}[io_dtype]
        self.desc = (f"cfg{cfg}: WKV{self.version} fwd+bwd B{B} T{T} C{C} H{H} head 64, {io_dtype} r/k/v/dy, "
                     f"{'bf16' if self.w16 else 'fp32'} raw decay, fp32 state, state carried step to step, state "
                     f"gradient fed back" + (f", raw decay shifted by {w_shift}" if w_shift else ""))

    def _forward(self, s, s_in, s_out, ws):
        B, T, C, H = self.dims
        p = lambda t: t.data_ptr()
        flags = self._lib.FLOOR_DECAY | (self._lib.W_BF16 if self.w16 else 0)
        st = self.fwd(self.stream, B, T, C, H, self.dt, flags, self.algo, p(s["r"]), p(s["k"]), p(s["v"]), p(s["w"]),
                      p(s["u"]), p(s_in), p(self.y), p(s_out), p(ws), ws.numel())
        assert st == 0, self.L.wkv_strerror(st)

    def _backward(self, s, s_in, g_out, g_in, ws):
        B, T, C, H = self.dims
        p = lambda t: t.data_ptr()
        flags = self._lib.FLOOR_DECAY | (self._lib.W_BF16 if self.w16 else 0)
        if self.have_ckpt:
            flags |= self._lib.CHECKPOINTS_VALID
        st = self.bwd(self.stream, B, T, C, H, self.dt, flags, self.algo, p(s["r"]), p(s["k"]), p(s["v"]), p(s["w"]),
                      p(s["u"]), p(s_in), p(s["dy"]), p(g_out), p(self.gr), p(self.gk), p(self.gv), p(self.gw),
                      p(self.gu), p(g_in), p(ws), ws.numel())
        assert st == 0, self.L.wkv_strerror(st)

    def step(self):
        """forward, then backward, of one segment"""
        i = self.i
        self.i += 1
        s = self.sets[i % len(self.sets)]
        self._forward(s, self.state[i % 2], self.state[(i + 1) % 2], self.ws)
        self._backward(s, self.state[i % 2], self.gstate[i % 2], self.gstate[(i + 1) % 2], self.ws)

    def step_cold(self):
        """Cold-cache order: the backward call of the segment whose forward call ran two steps ago (its checkpoints
        wait in the workspace this step's forward call then takes over), then this step's forward call.  Same calls,
        same bytes per step; between a segment's forward and its backward lie two other calls' worth of traffic."""
        torch = self.torch
        if self.ws_cold is None:
            self.ws_cold = torch.empty_like(self.ws)
        i = self.i
        self.i += 1
        n = len(self.sets)
        ws = (self.ws, self.ws_cold)[i % 2]
        if i >= 2:
            self._backward(self.sets[(i - 2) % n], self.state[i % 2], self.gstate[i % 2], self.gstate[(i + 1) % 2], ws)
        self._forward(self.sets[i % n], self.state[i % 2], self.state[(i + 1) % 2], ws)

    def kernel_ids(self):
        return {"forward": (1, 10), "backward": (2, 11)}


class Runner4:
    """WKV4 forward+backward through the C ABI (cfg2; fp32 as the workload states it, or bf16 k/v/y/gradients, the only
    dtype the reference's own kernel has, RWKV-v4neo/cuda/wkv_op_bf16.cpp:45-51)."""

    def __init__(self, cfg, algo, rotate, io_dtype="fp32"):
        import torch
        from rwkv_wkv_hip import _lib, configs
        self.torch, self._lib, self.L = torch, _lib, _lib.lib()
        dev = torch.device("cuda:0")
        io = {"bf16": torch.bfloat16, "fp32": torch.float32}[io_dtype]
        self.dt = {torch.float32: 0, torch.bfloat16: 1}[io]
        self.sets = []
        for i in range(rotate):
            wl = configs.make(cfg, seed=1000 + cfg + i)
            st = {n: t.to(dev).contiguous() for n, t in wl.tensors.items()}
            for n in ("k", "v", "dy"):
                st[n] = st[n].to(io)
            self.sets.append(st)
        B, T, C = wl.B, wl.T, wl.C
        self.dims = (B, T, C)
        s0 = self.sets[0]
        self.y, self.gk, self.gv = (torch.empty_like(s0["k"]) for _ in range(3))
        self.gtd, self.gtf = torch.empty(C, device=dev), torch.empty(C, device=dev)
        self.state = [s0["state"].clone(), torch.empty_like(s0["state"])]
        self.gstate = torch.empty_like(s0["state"])
        self.ckpt = torch.empty(self.L.wkv4_checkpoint_bytes(B, T, C), dtype=torch.uint8, device=dev)
        self.ws = torch.empty(self.L.wkv4_backward_workspace(B, T, C, self.dt), dtype=torch.uint8, device=dev)
        self.stream = torch.cuda.current_stream().cuda_stream
        self.i = 0
        self.tokens_per_step = B * T
        elems = B * T * C
        eb = 4 if io == torch.float32 else 2
        self.bytes_step, self.bytes_fwd, self.bytes_bwd = 8 * eb * elems, 3 * eb * elems, 5 * eb * elems
        self.dtype_name = "f32" if io == torch.float32 else "bf16"
        self.desc = f"cfg{cfg}: WKV4 fwd+bwd B{B} T{T} C{C} {io_dtype} k/v/dy, (aa,bb,pp) state fp32 carried step to step"

    def step(self):
        B, T, C = self.dims
        s = self.sets[self.i % len(self.sets)]
        s_in, s_out = self.state[self.i % 2], self.state[(self.i + 1) % 2]
        self.i += 1
        p = lambda t: t.data_ptr()
        st = self.L.wkv4_forward(self.stream, B, T, C, self.dt, p(s["time_decay"]), p(s["time_first"]), p(s["k"]), p(s["v"]),
                                 p(s_in), p(self.y), p(s_out), p(self.ckpt))
        assert st == 0
        st = self.L.wkv4_backward(self.stream, B, T, C, self.dt, p(s["time_decay"]), p(s["time_first"]), p(s["k"]), p(s["v"]),
                                  p(s_in), p(s["dy"]), None, p(self.gtd), p(self.gtf), p(self.gk), p(self.gv),
                                  p(self.gstate), p(self.ckpt), p(self.ws), self.ws.numel())
        assert st == 0

    def kernel_ids(self):
        return {"forward": (3,), "backward": (4,)}


def capture_steps(runner, nsteps, step=None):
    """`nsteps` consecutive steps (input rotation x state ping-pong) recorded into a HIP graph.
    The library allocates nothing and synchronises nothing in a call, so its launches
    record as they are.  Returns None when the capture fails."""
    torch = runner.torch
    eager_stream, i0 = runner.stream, runner.i
    try:
        g = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            with torch.cuda.graph(g, stream=side):
                runner.stream = torch.cuda.current_stream().cuda_stream
                for _ in range(nsteps):
                    (step or runner.step)()
        torch.cuda.current_stream().wait_stream(side)
        return g
    except Exception as e:            # noqa: BLE001 - any capture problem means plain launches
        print(f"bench.py: HIP graph capture failed ({e}); timing plain launches", file=sys.stderr)
        runner.i = i0
        return None
    finally:
        runner.stream = eager_stream


def capture_period(runner, period):
    assert runner.i % period == 0
    return capture_steps(runner, period)


def time_kernel(runner, kid, steps):
    """Average launch duration (ms) of kernel `kid` over `steps` steps, by HIP
    events recorded inside the library on the launch stream."""
    L = runner.L
    assert L.wkv_profile_begin(kid, steps) == 0
    for _ in range(steps):
        runner.step()
    runner.torch.cuda.synchronize()
    buf = (ctypes.c_float * steps)()
    n = L.wkv_profile_end(buf, steps)
    if n == 0:
        return None
    return sum(buf[:n]) / n


def cpu_baseline(cfg, heads):
    """The CPU restatement of the reference's pure-PyTorch path (chunk 128,
    fp64 intra-chunk), fwd + autograd bwd, timed on the host cores on a head
    subset of the same workload (heads are independent, cost is linear)."""
    import torch
    from oracle import wkv56 as O
    from rwkv_wkv_hip import configs
    spec = configs.SHAPES[cfg]
    if spec["version"] == 4:
        return None
    ncores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else os.cpu_count()
    ncores = min(ncores, 16)
    torch.set_num_threads(ncores)
    B, T, H = spec["B"], spec["T"], spec["H"]
    hs = min(heads, H)
    bs = 1
    wl = configs.make(cfg, B=bs, H=hs, C=hs * 64)
    t = wl.tensors
    v = spec["version"]
    run = lambda: O.wkv_op_grads(v, bs, T, hs * 64, hs, t["r"].float(), t["k"].float(), t["v"].float(), t["w"], t["u"],
                                 t["state"], t["dy"].float(), t["dstate"])
    run()
    times = []
    t_all = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_all < 10 and len(times) < 8):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    tok_s = (bs * T) / (med * (H / hs))            # scaled to all heads of the layer; per batch row
    out = {"value": tok_s, "unit": "tokens/s", "cores": ncores, "kind": "port",
           "sample": (f"CPU restatement of rwkv_inner (chunk_len 128, fp64 intra-chunk, eager torch "
                      f"{torch.__version__}) fwd + autograd bwd on {hs} of {H} heads of one batch row, T={T}; "
                      f"median of {len(times)} runs = {med:.3f} s, scaled by {H}/{hs} heads"),
           "threads": torch.get_num_threads()}
    # the reference's own CPU-runnable case: WKV5 forward only, B1 T512 C768 H12 fp32
    w0 = configs.make(0)
    t0s = w0.tensors
    f0 = lambda: O.wkv5_op(1, 512, 768, 12, t0s["state"], t0s["r"], t0s["k"], t0s["v"], t0s["w"], t0s["u"])
    with torch.no_grad():
        f0()
        ts = []
        for _ in range(5):
            a = time.perf_counter()
            f0()
            ts.append(time.perf_counter() - a)
    ts.sort()
    out["cfg0_forward_tokens_per_s"] = 512 / ts[2]
    return out


def kernel_source_hash():
    """Fingerprint of the kernel sources the library is built from (the counters of a
    profiler run describe exactly one version of the kernels): the code without its
    comments and white space, so that a reworded comment does not disown a measurement."""
    import glob
    import hashlib
    import re
    h = hashlib.sha256()
    for path in sorted(glob.glob(os.path.join(ROOT, "rwkv-infctx-trainer_amd", "csrc", "*.h*"))):
        code = open(path, encoding="utf-8").read()
        code = re.sub(r"/\*.*?\*/", "", code, flags=re.S)
        code = re.sub(r"//[^\n]*", "", code)
        h.update(os.path.basename(path).encode())
        h.update("".join(code.split()).encode())
    return h.hexdigest()[:16]


def measured_traffic(cfg, algo, segments, kernel):
    """HBM bytes per launch of the dominant kernel from the committed rocprofv3 counter
    summary of this same workload and this same version of the kernel sources
    (profiles/), or None when there is none that matches."""
    path = os.path.join(ROOT, "profiles", f"wkv6_cfg{cfg}_traffic.json")
    if not os.path.exists(path):
        return None
    rec = json.load(open(path))
    same = (rec.get("algo") == algo and rec.get("segments") == (segments or "auto") and rec.get("kernel") == kernel
            and rec.get("source_hash") == kernel_source_hash())
    return rec["traffic_bytes_per_launch"] if same else None


def bench_helper(a):
    """The cumulative-decay helper alone: every table of rwkv_inner.py:43-93 from the raw decay tensor of cfg3
    (B8 T4096 C2560, chunk length 128).  Algorithmic bytes: 4 read + 4 per fp32 table + 8 per fp64 factor."""
    import torch
    from rwkv_wkv_hip import _lib, configs
    L = _lib.lib()
    wl = configs.make(3)
    B, T, C = wl.B, wl.T, wl.C
    w = wl.tensors["w"].cuda().contiguous()
    f32 = lambda *sh: torch.empty(*sh, dtype=torch.float32, device="cuda")
    out = [f32(B, T, C) for _ in range(4)] + [f32(B, T // 128, C)]
    exps = [f32(B, T // 128, C), f32(B, T, C), f32(B, T, C)]
    facs = [torch.empty(B, T, C, dtype=torch.float64, device="cuda") for _ in range(2)]
    p = lambda t: t.data_ptr()
    stream = torch.cuda.current_stream().cuda_stream
    res = {}
    for name, fn, nbytes in (
            ("log_tables", lambda: L.wkv_cumsum_decay(stream, B, T, C, 128, 1, p(w), *[p(t) for t in out]), 20 * B * T * C),
            ("all_tables", lambda: L.wkv_cumsum_decay_factors(stream, B, T, C, 128, 1, 64, p(w), *[p(t) for t in out + exps + facs]),
             44 * B * T * C)):
        for _ in range(max(a.warmup, 3)):
            assert fn() == 0
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        n = max(a.steps // 10, 10)
        ev0.record()
        for _ in range(n):
            fn()
        ev1.record()
        torch.cuda.synchronize()
        ms = ev0.elapsed_time(ev1) / n
        res[name] = {"ms": ms, "algorithmic_bytes": nbytes, "GBs": nbytes / ms / 1e6, "frac_of_hbm_peak": nbytes / ms / 1e6 / HBM_PEAK_GBS}
    print(json.dumps({"metric": "cumulative-decay helper, B8 T4096 C2560, chunk 128", "unit": "ms", "n_gpus": 1, "data": "synthetic",
                      "dtype": "f32", "value": res["log_tables"]["ms"], "higher_is_better": False, "kernels": res}))


def bench_edges(a):
    """The element-wise passes around the operator (csrc/block_edges.hip), each kernel alone, bf16, at the token
    counts and widths of cfg3 (B8 T4096 C2560) and cfg4 (B1 T4096 C4096).  Algorithmic bytes: every tensor the
    reference's lines read or write, once (2 B per bf16 element; parameters are negligible).  Inputs and outputs
    rotate over several sets so that nothing is served from the 256 MB last-level cache."""
    import ctypes
    import torch
    from rwkv_wkv_hip import _lib
    L = _lib.lib()
    stream = torch.cuda.current_stream().cuda_stream
    bf = torch.bfloat16
    p = lambda t: None if t is None else t.data_ptr()
    arr = lambda ts: (ctypes.c_void_p * len(ts))(*[t.data_ptr() for t in ts])
    res = {}

    def timed(name, calls, nbytes):
        for _ in range(max(a.warmup // 10, 2)):
            for c in calls:
                assert c() == 0
        n = max(a.steps // 20, 5)
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
        for _ in range(n):
            for c in calls:
                c()
        ev1.record()
        torch.cuda.synchronize()
        ms = ev0.elapsed_time(ev1) / (n * len(calls))
        res[name] = {"ms": round(ms, 5), "algorithmic_bytes": nbytes, "GBs": round(nbytes / ms / 1e6, 1),
                     "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)}

    for tag, B, T, C in (("cfg3", 8, 4096, 2560), ("cfg4", 1, 4096, 4096)):
        E = B * T * C
        rot = 3 if tag == "cfg3" else 6
        rnd = lambda *sh: torch.randn(*sh, device="cuda", dtype=bf)
        sets = []
        for _ in range(rot):
            sets.append(dict(x=rnd(B, T, C), shift=rnd(B, C), dyn=rnd(5, B, T, C) * 0.3, o=[rnd(B, T, C) for _ in range(5)],
                             gx=rnd(B, T, C), gshift=rnd(B, C), gdyn=torch.empty(5, B, T, C, device="cuda", dtype=bf)))
        coef = torch.rand(5, C, device="cuda")
        gcoef = torch.empty(5, C, device="cuda")
        ws = torch.empty(max(L.wkv_shift_mix_backward_workspace(B, T, C, 5), L.wkv_ln_gate_backward_workspace(B * T, C)),
                         dtype=torch.uint8, device="cuda")
        wb, gwb = torch.randn(2, C, device="cuda"), torch.empty(2, C, device="cuda")
        mk = lambda f: [(lambda s=s: f(s)) for s in sets]
        timed(f"{tag} shift_mix v5 forward (4 mixes)", mk(lambda s: L.wkv_shift_mix_forward(
            stream, B, T, C, 1, 4, 1, p(s["x"]), p(s["shift"]), p(coef), None, arr(s["o"][:4]))), 10 * E)
        timed(f"{tag} shift_mix v5 backward (4 mixes)", mk(lambda s: L.wkv_shift_mix_backward(
            stream, B, T, C, 1, 4, 1, p(s["x"]), p(s["shift"]), p(coef), None, arr(s["o"][:4]), p(s["gx"]), p(s["gshift"]), p(gcoef),
            None, p(ws), ws.numel())), 12 * E)
        timed(f"{tag} shift_mix v6 forward (5 mixes + data-dependent part)", mk(lambda s: L.wkv_shift_mix_forward(
            stream, B, T, C, 1, 5, 0, p(s["x"]), p(s["shift"]), p(coef), p(s["dyn"]), arr(s["o"]))), 22 * E)
        timed(f"{tag} shift_mix v6 backward (5 mixes + data-dependent part)", mk(lambda s: L.wkv_shift_mix_backward(
            stream, B, T, C, 1, 5, 0, p(s["x"]), p(s["shift"]), p(coef), p(s["dyn"]), arr(s["o"]), p(s["gx"]), p(s["gshift"]), p(gcoef),
            p(s["gdyn"]), p(ws), ws.numel())), 34 * E)
        # the same five mixes with the second LoRA product inside the pass: x and the activations in, five mixes out
        # (backward: x, five gradients in; gx and the five product gradients out); the 32-wide activations and
        # factors are 160 / 4096 of a tensor each and are counted
        act = [torch.tanh(torch.randn(B * T, 5, 32, device="cuda")).to(bf) for _ in range(rot)]
        w2t = (torch.randn(5, C, 32, device="cuda") * 0.1).to(bf)
        ws2 = torch.empty(L.wkv_lora_mix_backward_workspace(B, T, C), dtype=torch.uint8, device="cuda")
        small = 2 * (B * T * 160 + 160 * C)
        timed(f"{tag} lora_mix v6 forward (5 mixes, LoRA product inside)", [
            (lambda s=s, a_=a_: L.wkv_lora_mix_forward(stream, B, T, C, p(s["x"]), p(s["shift"]), p(coef), p(a_), p(w2t), arr(s["o"])))
            for s, a_ in zip(sets, act)], 12 * E + small)
        timed(f"{tag} lora_mix v6 backward (5 mixes, LoRA product inside)", [
            (lambda s=s, a_=a_: L.wkv_lora_mix_backward(stream, B, T, C, p(s["x"]), p(s["shift"]), p(coef), p(a_), p(w2t), arr(s["o"]),
                                                        p(s["gx"]), p(s["gshift"]), p(gcoef), p(s["gdyn"]), p(ws2), ws2.numel()))
            for s, a_ in zip(sets, act)], 24 * E + small)
        del act
        timed(f"{tag} ln_x * gate forward", mk(lambda s: L.wkv_ln_gate_forward(
            stream, B * T, C, 1, 1.0, 64e-5, p(s["x"]), p(s["o"][0]), p(wb[0]), p(wb[1]), p(s["gx"]))), 6 * E)
        timed(f"{tag} ln_x * gate backward", mk(lambda s: L.wkv_ln_gate_backward(
            stream, B * T, C, 1, 1.0, 64e-5, p(s["x"]), p(s["o"][0]), p(wb[0]), p(wb[1]), p(s["o"][1]), p(s["gx"]), p(s["o"][2]),
            p(gwb), p(ws), ws.numel())), 10 * E)
        timed(f"{tag} relu^2 forward", mk(lambda s: L.wkv_relu_square_forward(stream, E, 1, p(s["x"]), p(s["gx"]))), 4 * E)
        timed(f"{tag} relu^2 backward", mk(lambda s: L.wkv_relu_square_backward(stream, E, 1, p(s["x"]), p(s["o"][0]), p(s["gx"]))), 6 * E)
        timed(f"{tag} sigmoid * kv forward", mk(lambda s: L.wkv_sigmoid_mul_forward(stream, E, 1, p(s["x"]), p(s["o"][0]), p(s["gx"]))), 6 * E)
        timed(f"{tag} sigmoid * kv backward", mk(lambda s: L.wkv_sigmoid_mul_backward(
            stream, E, 1, p(s["x"]), p(s["o"][0]), p(s["o"][1]), p(s["gx"]), p(s["o"][2]))), 10 * E)
        del sets
    rows, V = 4096, 65536
    ys = [torch.randn(rows, V, device="cuda", dtype=bf) for _ in range(2)]
    gys = [torch.empty_like(y) for y in ys]
    timed("L2Wrap backward (4096 rows, vocabulary 65536)",
          [(lambda i=i: L.wkv_l2wrap_backward(stream, rows, V, 1, 1e-4 / rows, p(ys[i]), None, p(gys[i]))) for i in range(2)], 4 * rows * V)
    key = "cfg4 shift_mix v6 backward (5 mixes + data-dependent part)"
    print(json.dumps({"metric": "element-wise passes around the WKV operator, bf16", "unit": "GB/s", "n_gpus": 1, "data": "synthetic",
                      "dtype": "bf16", "value": res[key]["GBs"], "higher_is_better": True, "kernels": res}))


def bench_block(a):
    """One RWKV-v6 layer's TimeMix and ChannelMix (RWKV-v6/src/module/TimeMix.py:253-302, ChannelMix.py:30-37) at the
    cfg4 width (B1 T4096 C4096 H64, dim_ffn 14336, bf16), forward + backward, two ways: every element-wise pass on the
    HIP kernels (rwkv_wkv_hip.blocks), and the same layer written with torch element-wise ops as the reference writes
    it.  Both use the same WKV6 operator and the same torch matmuls, so the difference is the element-wise passes."""
    import torch
    import torch.nn as nn
    import torch.nn.functional as F
    import rwkv_wkv_hip as W
    from rwkv_wkv_hip import blocks as K
    B, T, C, H, FFN = 1, 4096, 4096, 64, 14336
    dev, bf = "cuda", torch.bfloat16
    g = torch.Generator(device="cpu").manual_seed(5)

    class TimeMix(nn.Module):
        def __init__(self):
            super().__init__()
            self.n_head = H
            u01 = lambda *sh: torch.rand(*sh, generator=g)
            for nm in ("x", "w", "k", "v", "r", "g"):
                setattr(self, f"time_maa_{nm}", nn.Parameter(u01(1, 1, C)))
            self.time_maa_w1 = nn.Parameter((u01(C, 160) - 0.5) * 0.02)
            self.time_maa_w2 = nn.Parameter((u01(5, 32, C) - 0.5) * 0.02)
            self.time_decay = nn.Parameter(u01(1, 1, C) * 5 - 6)
            self.time_decay_w1 = nn.Parameter((u01(C, 64) - 0.5) * 0.02)
            self.time_decay_w2 = nn.Parameter((u01(64, C) - 0.5) * 0.02)
            self.time_faaaa = nn.Parameter(torch.randn(H, 64, generator=g) * 0.3)
            self.receptance, self.key, self.value, self.gate, self.output = (nn.Linear(C, C, bias=False) for _ in range(5))
            self.ln_x = nn.GroupNorm(H, C, eps=64e-5)

    class ChannelMix(nn.Module):
        def __init__(self):
            super().__init__()
            self.time_maa_k = nn.Parameter(torch.rand(1, 1, C, generator=g))
            self.time_maa_r = nn.Parameter(torch.rand(1, 1, C, generator=g))
            self.key, self.receptance, self.value = nn.Linear(C, FFN, bias=False), nn.Linear(C, C, bias=False), nn.Linear(FFN, C, bias=False)

    def timemix_torch(m, x, st):            # the reference's lines, element-wise work in torch
        dxprev = torch.concat((st[0].unsqueeze(1), x[:, :-1]), dim=1) - x
        xxx = x + dxprev * m.time_maa_x
        xxx = torch.tanh(xxx @ m.time_maa_w1).view(B * T, 5, -1).transpose(0, 1)
        mw, mk, mv, mr, mg = torch.bmm(xxx, m.time_maa_w2).view(5, B, T, -1).unbind(dim=0)
        xk, xv, xr = x + dxprev * (m.time_maa_k + mk), x + dxprev * (m.time_maa_v + mv), x + dxprev * (m.time_maa_r + mr)
        xg, xw = x + dxprev * (m.time_maa_g + mg), x + dxprev * (m.time_maa_w + mw)
        r, k, v, gate = m.receptance(xr), m.key(xk), m.value(xv), F.silu(m.gate(xg))
        w = m.time_decay + torch.tanh(xw @ m.time_decay_w1) @ m.time_decay_w2
        y, ns = W.WKV_6.apply(B, T, C, H, r, k, v, w.contiguous(), m.time_faaaa, st[1])
        y = m.ln_x(y.view(-1, C)).view(B, T, C)
        return m.output(y * gate), (x[:, -1], ns)

    def channelmix_torch(m, x, st):
        dxx = torch.concat((st.unsqueeze(1), x[:, :-1]), dim=1) - x
        xk, xr = x + dxx * m.time_maa_k, x + dxx * m.time_maa_r
        kv = m.value(torch.relu(m.key(xk)) ** 2)
        return torch.sigmoid(m.receptance(xr)) * kv, x[:, -1]

    tm, cm = TimeMix().to(dev).to(bf), ChannelMix().to(dev).to(bf)
    x = (torch.randn(B, T, C, generator=g) * 0.5).to(dev).to(bf).requires_grad_(True)
    shift = torch.randn(B, C, generator=g).to(dev).to(bf)
    state = (torch.randn(B, H, 64, 64, generator=g) * 0.1).to(dev)
    gy = torch.randn(B, T, C, generator=g).to(dev).to(bf)
    res = {}

    def timed(name, fn):
        def once():
            x.grad = None
            for p in list(tm.parameters()) + list(cm.parameters()):
                p.grad = None
            y = fn()
            y.backward(gy)
        for _ in range(3):
            once()
        n = max(a.steps // 30, 10)
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        ev0.record()
        for _ in range(n):
            once()
        ev1.record()
        torch.cuda.synchronize()
        res[name] = round(ev0.elapsed_time(ev1) / n, 4)
    if a.block_way in ("both", "kernels"):
        timed("timemix_kernels_ms", lambda: K.timemix6_forward(tm, x, (shift, state))[0])
        timed("channelmix_kernels_ms", lambda: K.channelmix6_forward(cm, x, shift)[0])
        K.use_lora_mix(False)       # the same with the second LoRA product and its five results through memory
        timed("timemix_kernels_lora_through_memory_ms", lambda: K.timemix6_forward(tm, x, (shift, state))[0])
        K.use_lora_mix(True)
    if a.block_way in ("both", "torch"):
        timed("timemix_torch_elementwise_ms", lambda: timemix_torch(tm, x, (shift, state))[0])
        timed("channelmix_torch_elementwise_ms", lambda: channelmix_torch(cm, x, shift)[0])
    if a.block_way != "both":
        way = "kernels" if a.block_way == "kernels" else "torch_elementwise"
        print(json.dumps({"metric": f"RWKV-v6 layer (TimeMix + ChannelMix) fwd+bwd, B1 T4096 C4096 H64 bf16, {a.block_way} way only", "unit": "ms",
                          "n_gpus": 1, "data": "synthetic", "dtype": "bf16", "higher_is_better": False,
                          "value": round(res[f"timemix_{way}_ms"] + res[f"channelmix_{way}_ms"], 4), "parts": res}))
        return
    with torch.no_grad():       # the two ways agree
        ya, yb = K.timemix6_forward(tm, x, (shift, state))[0].float(), timemix_torch(tm, x, (shift, state))[0].float()
        res["timemix_rel_diff"] = round(((ya - yb).norm() / yb.norm()).item(), 5)
        ya, yb = K.channelmix6_forward(cm, x, shift)[0].float(), channelmix_torch(cm, x, shift)[0].float()
        res["channelmix_rel_diff"] = round(((ya - yb).norm() / yb.norm()).item(), 5)
    layer_k = res["timemix_kernels_ms"] + res["channelmix_kernels_ms"]
    layer_t = res["timemix_torch_elementwise_ms"] + res["channelmix_torch_elementwise_ms"]
    print(json.dumps({"metric": "RWKV-v6 layer (TimeMix + ChannelMix) fwd+bwd, B1 T4096 C4096 H64 bf16, host-launched (autograd)", "unit": "ms",
                      "n_gpus": 1, "data": "synthetic", "dtype": "bf16", "value": round(layer_k, 4), "higher_is_better": False,
                      "torch_elementwise_ms": round(layer_t, 4), "speedup": round(layer_t / layer_k, 3), "parts": res}))


def measure(runner, step, a):
    """Warm up, then time exactly a.steps calls of `step` twice (host clock between two device synchronisations; HIP
    events on the launch stream with the queue primed).  Returns ms per step both ways and how the steps were launched."""
    torch = runner.torch
    period = 2 * a.rotate if a.rotate % 2 else a.rotate        # input rotation x state ping-pong
    runner.i = 0
    for _ in range(-(-max(a.warmup, 2) // period) * period if a.launch == "graph" else max(a.warmup, 2)):
        step()
    torch.cuda.synchronize()
    # The K timed steps as few graph launches as possible: up to 128 steps are ONE graph; a longer run replays a
    # body of 120 steps (whole rotation periods) K // 120 times, plus one more graph with what is left.  A graph
    # launch costs the host (and the idle GPU) about 0.2 ms, so a short run (the 20-step default of an automated
    # harness) would otherwise measure launch latencies rather than the kernels.
    body = tail = None
    body_steps = a.steps if a.steps <= 128 else 120
    if a.launch == "graph" and body_steps > 0:
        body = capture_steps(runner, body_steps, step)
        if body is not None and a.steps % body_steps:
            tail = capture_steps(runner, a.steps % body_steps, step)
            if tail is None:
                body = None
    graph = body
    if graph is not None:
        graph.replay()                 # untimed: the first replay uploads the graph
        if tail is not None:
            tail.replay()
        torch.cuda.synchronize()

    def run_k_steps():
        if graph is not None:
            for _ in range(a.steps // body_steps):
                graph.replay()
            if tail is not None:
                tail.replay()
        else:
            for _ in range(a.steps):
                step()

    if a.settle_ms > 0 and graph is not None:      # untimed: the first replays of a fresh graph are slower than the steady state
        t_end = time.perf_counter() + a.settle_ms * 1e-3
        while time.perf_counter() < t_end:
            run_k_steps()
            torch.cuda.synchronize()
    # (1) the K steps between two device synchronisations, by the host's clock.  This includes the latency of the
    # first launch (about 0.2 - 0.6 ms for a graph: the GPU idles until the launch arrives), which is a property
    # of the host, not of the kernels, and weighs 10 % and more on a 20-step run.
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    run_k_steps()
    torch.cuda.synchronize()
    ms_step_host = (time.perf_counter() - t0) / a.steps * 1e3
    # (2) the same K steps once more, between two HIP events on the launch stream, with untimed plain steps
    # queued in front so that the GPU is still busy when the timed launches arrive: the events then bracket
    # exactly the K steps' execution.  This is the figure reported as ms_per_step / value.
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(period):            # (a whole period, so that the replayed graphs meet the state they were captured in)
        step()
    ev0.record()
    run_k_steps()
    ev1.record()
    torch.cuda.synchronize()
    launch = ((f"hip graph of {body_steps} steps per replay" + (f" + one of {a.steps % body_steps}" if tail is not None else ""))
              if graph is not None else "eager")
    return {"ms_per_step": ev0.elapsed_time(ev1) / a.steps, "ms_per_step_host": ms_step_host, "launch": launch,
            "settle_ms": a.settle_ms if graph is not None else 0.0}


def main():
    a = parse()
    if a.gpus != 1:
        print("bench.py: this build measures one GPU only (every (batch, head) recurrence is independent; "
              "no multi-GPU path is part of it); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    if a.helper:
        return bench_helper(a)
    if a.edges:
        return bench_edges(a)
    if a.block:
        return bench_block(a)
    if a.cfg == 2 and a.io_dtype == "fp16":
        sys.exit("bench.py: --cfg 2 takes --io-dtype fp32 (the workload as stated, the default there) or bf16")
    runner = Runner4(a.cfg, a.algo, a.rotate, a.io_dtype or "fp32") if a.cfg == 2 else Runner56(a.cfg, a.algo, a.rotate, a.w_dtype, a.w_shift, a.io_dtype or "bf16")
    assert runner.L.wkv_tune(runner._lib.TUNE_SEGMENTS, a.segments) == 0

    if a.traffic_probe:
        src = torch.ones(256 << 20, dtype=torch.uint8, device="cuda:0")
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
    step = runner.step_cold if (a.cold and a.cfg != 2) else runner.step
    m = measure(runner, step, a)
    ms_step, ms_step_host, tok_s = m["ms_per_step"], m["ms_per_step_host"], runner.tokens_per_step / (m["ms_per_step"] * 1e-3)

    # per-kernel launch durations (HIP events around the kernel, on its stream)
    ksteps = min(a.steps, 20)
    kern = {}
    runner.i = 0
    for phase, ids in runner.kernel_ids().items():
        for kid in ids:
            ms = time_kernel(runner, kid, ksteps)
            if ms is not None:
                kern[phase] = {"kernel_id": kid, "ms": ms}
    dom = max(kern, key=lambda k: kern[k]["ms"])
    dom_bytes = runner.bytes_bwd if dom == "backward" else runner.bytes_fwd
    achieved = dom_bytes / (kern[dom]["ms"] * 1e-3) / 1e9
    kname = f"{dom} (kernel id {kern[dom]['kernel_id']})"
    roofline = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": achieved / HBM_PEAK_GBS, "traffic": measured_traffic(a.cfg, a.algo, a.segments, kname) if a.w_dtype == "fp32" else None,
                "kernel": kname,
                "algorithmic_bytes_per_launch": dom_bytes, "avg_launch_ms": kern[dom]["ms"],
                "kernels_ms": {k: v["ms"] for k, v in kern.items()},
                "whole_step_GBs": runner.bytes_step / (ms_step * 1e-3) / 1e9,
                "whole_step_frac": runner.bytes_step / (ms_step * 1e-3) / 1e9 / HBM_PEAK_GBS}

    out = {"metric": "WKV fwd+bwd tokens/sec at v6-7B shape (1 GPU); % of peak HBM GB/s" if a.cfg == 4
           else f"WKV fwd+bwd tokens/sec (cfg{a.cfg})",
           "value": tok_s, "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
           "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": runner.dtype_name, "data": "synthetic",
           "config": {"workload": runner.desc + (", cold-cache order (backward of the segment two steps back, then this step's forward)" if a.cold and a.cfg != 2 else ""),
                      "algo": a.algo, "segments": a.segments or "auto", "launch": m["launch"]},
           "ms_per_step_host": ms_step_host, "untimed_settle_ms": m["settle_ms"],
           "timing": "ms_per_step and value: HIP events on the launch stream around exactly the K steps, the queue "
                     "primed with untimed plain steps; ms_per_step_host: the same K steps between two device "
                     "synchronisations by the host clock (includes the latency of the first launch)",
           "roofline": roofline}
    if not a.no_extras and a.cfg != 2 and not a.cold:
        frac = lambda ms, r: r.bytes_step / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS
        c = measure(runner, runner.step_cold, a)
        out["cold"] = {"ms_per_step": c["ms_per_step"], "whole_step_frac": frac(c["ms_per_step"], runner),
                       "order": "backward of the segment whose forward ran two steps ago, then this step's forward; two workspaces"}
        if runner.version == 6 and not a.w_shift:
            del runner
            torch.cuda.empty_cache()
            slow = Runner56(a.cfg, a.algo, a.rotate, a.w_dtype, -5.0, a.io_dtype or "bf16")
            sd = measure(slow, slow.step, a)
            out["slow_decay"] = {"ms_per_step": sd["ms_per_step"], "whole_step_frac": frac(sd["ms_per_step"], slow),
                                 "raw_decay_shift": -5.0}
    if not a.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(a.cfg, a.cpu_heads)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
