"""wkv6_forward_noalloc: the forward entry point that allocates nothing (its scratch memory is an array inside the
library) gives bit for bit what wkv6_forward gives with a caller's workspace - same kernels, same plan - on two
calls in a row, the second on a smaller input, and rejects shapes beyond the array with a clear error."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(B, T, H, seed):
    from rwkv_wkv_hip import _lib, configs
    L = _lib.lib()
    C = H * 64
    wl = configs.make(3, seed=seed, B=B, T=T, C=C, H=H, dtype=torch.bfloat16)
    g = {n: x.cuda().contiguous() for n, x in wl.tensors.items()}
    p = lambda t: t.data_ptr()
    stream = torch.cuda.current_stream().cuda_stream
    flags = _lib.FLOOR_DECAY
    y0, s0 = torch.empty_like(g["r"]), torch.empty_like(g["state"])
    y1, s1 = torch.full_like(g["r"], 7.0), torch.full_like(g["state"], 7.0)
    ws = torch.empty(L.wkv6_forward_workspace(B, T, C, H, _lib.WKV_BF16, _lib.ALGO_CHUNKED), dtype=torch.uint8, device="cuda")
    st = L.wkv6_forward(stream, B, T, C, H, _lib.WKV_BF16, flags, _lib.ALGO_CHUNKED, p(g["r"]), p(g["k"]), p(g["v"]),
                        p(g["w"]), p(g["u"]), p(g["state"]), p(y0), p(s0), p(ws), ws.numel())
    assert st == 0, L.wkv_strerror(st)
    torch.cuda.synchronize()
    # device memory as the driver counts it (hipMemGetInfo): an allocation inside the library would show here,
    # whichever allocator made it; torch's own counter beside it
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    st = L.wkv6_forward_noalloc(stream, B, T, C, H, _lib.WKV_BF16, flags, p(g["r"]), p(g["k"]), p(g["v"]), p(g["w"]),
                                p(g["u"]), p(g["state"]), p(y1), p(s1))
    assert st == 0, L.wkv_strerror(st)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before and torch.cuda.mem_get_info()[0] == free_before
    return (y0, s0), (y1, s1)


def test_noalloc_forward_matches_workspace_forward_twice():
    from rwkv_wkv_hip import _lib
    assert _lib.lib().wkv_init() == 0          # (also looks up the scratch array's address: nothing left for the first call)
    for B, T, H, seed in ((1, 2048, 4, 11), (1, 1024, 2, 12)):        # both are cut into several time segments
        print(f"case noalloc B{B} T{T} H{H}", flush=True)
        (y0, s0), (y1, s1) = _both(B, T, H, seed)
        assert torch.equal(y0, y1), "y differs"
        assert torch.equal(s0, s1), "state differs"
        assert torch.isfinite(y1.float()).all()


def test_noalloc_forward_rejects_what_does_not_fit():
    """A plan whose piece summaries exceed the 16 MiB array is refused before anything is launched.  The plan is
    forced (8 segments for 128 (batch, head) pairs: 128 x 8 summaries of 16.6 KB at least), and every pointer is a
    real buffer of the right size, so that the call would be harmless even if the check were missing."""
    from rwkv_wkv_hip import _lib, configs
    L = _lib.lib()
    B, T, H = 2, 1024, 64
    C = H * 64
    wl = configs.make(3, seed=13, B=B, T=T, C=C, H=H, dtype=torch.bfloat16)
    g = {n: x.cuda().contiguous() for n, x in wl.tensors.items()}
    y, s = torch.empty_like(g["r"]), torch.empty_like(g["state"])
    p = lambda t: t.data_ptr()
    stream = torch.cuda.current_stream().cuda_stream
    assert L.wkv_tune(_lib.TUNE_SEGMENTS, 8) == 0
    try:
        st = L.wkv6_forward_noalloc(stream, B, T, C, H, _lib.WKV_BF16, _lib.FLOOR_DECAY, p(g["r"]), p(g["k"]), p(g["v"]),
                                    p(g["w"]), p(g["u"]), p(g["state"]), p(y), p(s))
    finally:
        assert L.wkv_tune(_lib.TUNE_SEGMENTS, 0) == 0
    torch.cuda.synchronize()
    assert st == -5 and b"workspace" in L.wkv_strerror(st)
    # fp32 streams do not take the blocked algorithm
    f = {n: (x.float() if x.dtype == torch.bfloat16 else x) for n, x in g.items()}
    yf = torch.empty_like(f["r"])
    st = L.wkv6_forward_noalloc(stream, B, T, C, H, _lib.WKV_F32, _lib.FLOOR_DECAY, p(f["r"]), p(f["k"]), p(f["v"]), p(f["w"]),
                                p(f["u"]), p(f["state"]), p(yf), p(s))
    assert st == -7


def test_state_in_place_where_no_sequence_is_cut():
    """state_out == state_in: accepted by the per-token kernels and by the blocked ones when the plan cuts nothing in
    time (same results as with two buffers), refused (WKV_ERR_ALIAS) when it does, and always for partial overlap."""
    from rwkv_wkv_hip import _lib, configs
    L = _lib.lib()
    B, T, H = 1, 512, 2
    C = H * 64
    wl = configs.make(3, seed=14, B=B, T=T, C=C, H=H, dtype=torch.bfloat16)
    g = {n: x.cuda().contiguous() for n, x in wl.tensors.items()}
    p = lambda t: t.data_ptr()
    stream = torch.cuda.current_stream().cuda_stream

    def fwd(algo, s_in, s_out, nseg):
        y = torch.empty_like(g["r"])
        assert L.wkv_tune(_lib.TUNE_SEGMENTS, nseg) == 0
        try:
            st = L.wkv6_forward(stream, B, T, C, H, _lib.WKV_BF16, _lib.FLOOR_DECAY, algo, p(g["r"]), p(g["k"]), p(g["v"]),
                                p(g["w"]), p(g["u"]), p(s_in), p(y), p(s_out), None, 0)
        finally:
            assert L.wkv_tune(_lib.TUNE_SEGMENTS, 0) == 0
        torch.cuda.synchronize()
        return st, y
    for algo in (_lib.ALGO_RECURRENT, _lib.ALGO_CHUNKED):
        two = torch.empty_like(g["state"])
        st, y2 = fwd(algo, g["state"], two, 1)
        assert st == 0
        one = g["state"].clone()
        st, y1 = fwd(algo, one, one, 1)
        assert st == 0, L.wkv_strerror(st)
        assert torch.equal(y1, y2) and torch.equal(one, two)
    one = g["state"].clone()
    assert fwd(_lib.ALGO_CHUNKED, one, one, 4)[0] == -8                 # cut in time: two buffers needed
    big = torch.zeros(2 * g["state"].numel(), device="cuda")
    assert fwd(_lib.ALGO_RECURRENT, big[:g["state"].numel()], big[64:64 + g["state"].numel()], 1)[0] == -8      # partial overlap


def test_noalloc_forward_under_graph_capture():
    """What the entry point is for: recorded into a HIP graph (after wkv_init, nothing is left to set up inside the
    capture) and replayed, with plain launches in between; every replay gives the bits of the plain call."""
    from rwkv_wkv_hip import _lib, configs
    L = _lib.lib()
    assert L.wkv_init() == 0
    B, T, H = 1, 1024, 3
    C = H * 64
    wl = configs.make(3, seed=15, B=B, T=T, C=C, H=H, dtype=torch.bfloat16)
    g = {n: x.cuda().contiguous() for n, x in wl.tensors.items()}
    p = lambda t: t.data_ptr()
    y, s = torch.empty_like(g["r"]), torch.empty_like(g["state"])

    def call(stream):
        st = L.wkv6_forward_noalloc(stream, B, T, C, H, _lib.WKV_BF16, _lib.FLOOR_DECAY, p(g["r"]), p(g["k"]), p(g["v"]),
                                    p(g["w"]), p(g["u"]), p(g["state"]), p(y), p(s))
        assert st == 0, L.wkv_strerror(st)
    call(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    want = (y.clone(), s.clone())
    graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            call(torch.cuda.current_stream().cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(3):
        y.fill_(3.0); s.fill_(3.0)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want[0]) and torch.equal(s, want[1]), f"replay {rep} differs"
        call(torch.cuda.current_stream().cuda_stream)          # the program's own work between the replays
        torch.cuda.synchronize()
