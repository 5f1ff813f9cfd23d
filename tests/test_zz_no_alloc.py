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
    before = torch.cuda.memory_allocated()
    st = L.wkv6_forward_noalloc(stream, B, T, C, H, _lib.WKV_BF16, flags, p(g["r"]), p(g["k"]), p(g["v"]), p(g["w"]),
                                p(g["u"]), p(g["state"]), p(y1), p(s1))
    assert st == 0, L.wkv_strerror(st)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    return (y0, s0), (y1, s1)


def test_noalloc_forward_matches_workspace_forward_twice():
    for B, T, H, seed in ((1, 2048, 4, 11), (1, 1024, 2, 12)):        # both are cut into several time segments
        print(f"case noalloc B{B} T{T} H{H}", flush=True)
        (y0, s0), (y1, s1) = _both(B, T, H, seed)
        assert torch.equal(y0, y1), "y differs"
        assert torch.equal(s0, s1), "state differs"
        assert torch.isfinite(y1.float()).all()


def test_noalloc_forward_rejects_what_does_not_fit():
    from rwkv_wkv_hip import _lib
    L = _lib.lib()
    one = ctypes.c_void_p(4096)         # never dereferenced: the size check comes before any launch
    two = ctypes.c_void_p(1 << 30)
    st = L.wkv6_forward_noalloc(None, 8, 4096, 2560, 40, _lib.WKV_BF16, _lib.FLOOR_DECAY, one, one, one, one, one, one,
                                one, two)
    assert st == -5 and b"workspace" in L.wkv_strerror(st)
    # fp32 streams do not take the blocked algorithm
    st = L.wkv6_forward_noalloc(None, 1, 128, 64, 1, _lib.WKV_F32, _lib.FLOOR_DECAY, one, one, one, one, one, one, one, two)
    assert st == -7
