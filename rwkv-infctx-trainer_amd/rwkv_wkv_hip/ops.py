"""torch.autograd front ends with the reference trainer's call signatures.

WKV_5.apply(B, T, C, H, state, r, k, v, w, u)  -> (y, new_state)
WKV_6.apply(B, T, C, H, r, k, v, w, u, s)      -> (y, new_state)
wkv_op(time_decay, time_first, k, v, wkv_state) -> (y, new_state)

Argument order and meaning are those of WKV5_CUDA / WKV6STATE_CUDA
(RWKV-v5/src/module/TimeMix.py:20-31, RWKV-v6/src/module/TimeMix.py:19-26) and
of torch.ops.rwkv.wkv (RWKV-v4neo/src/model.py:130-132): ``w`` is the RAW decay
parameter and the gradient returned for it is with respect to that raw
parameter.  Unlike the reference's kernels the functions are functional (the
new state is returned, and is differentiable); RUN_WKV5_CUDA /
RUN_WKV6STATE_CUDA keep the reference's in-place convention on top of them.

All tensors must live on the GPU; the work is done by librwkv_wkv_hip.so on the
current HIP stream.
"""
from __future__ import annotations

import os

import torch

from . import _lib
from ._lib import WKVError, check

HEAD = 64
_DT = {torch.float32: _lib.WKV_F32, torch.bfloat16: _lib.WKV_BF16, torch.float16: _lib.WKV_F16}
_ALGO = {"auto": _lib.ALGO_AUTO, "recurrent": _lib.ALGO_RECURRENT, "chunked": _lib.ALGO_CHUNKED}
_algo = _ALGO[os.environ.get("RWKV_WKV_ALGO", "auto")]


def set_algo(name: str):
    """'auto' | 'recurrent' | 'chunked' for the WKV5/WKV6 operators."""
    global _algo
    _algo = _ALGO[name]


def _ptr(t):
    return None if t is None else t.data_ptr()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _on_gpu(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise WKVError("rwkv_wkv_hip operators need GPU tensors (there is no CPU path)")


def _check_rkv(B, T, C, H, r, k, v):
    dtype = r.dtype
    if dtype not in _DT:
        raise ValueError(f"Unsupported dtype {dtype} for WKV")
    assert dtype == k.dtype and dtype == v.dtype
    assert r.is_contiguous() and k.is_contiguous() and v.is_contiguous()
    assert r.shape == (B, T, C) and k.shape == (B, T, C) and v.shape == (B, T, C)
    return _DT[dtype]


def _workspace(nbytes, device):
    return torch.empty(max(int(nbytes), 16), dtype=torch.uint8, device=device)


def _blocked(version, B, T, C, H, dtype):
    """True when a call with these arguments takes the blocked (matrix-core) algorithm."""
    L = _lib.lib()
    fq = L.wkv5_forward_workspace if version == 5 else L.wkv6_forward_workspace
    return T > 1 and dtype in _DT and fq(B, T, C, H, _DT[dtype], _algo) > 0


stats = {"forward_launches": 0, "forward_reused": 0}      # counters for tests and diagnostics


class RecomputeCache:
    """Opt-in reuse of a forward pass by the recomputation that activation checkpointing runs later.

    Under activation checkpointing (the reference wraps every block in ``deepspeed.checkpointing.checkpoint``,
    RWKV-v5/src/model.py:674-683) the operator's forward runs twice per layer and segment: once without autograd
    while the model runs forward, once more when backward recomputes the block.  With a cache installed
    (``with recompute_cache(): ...`` around the training step) the first run keeps its outputs and its state
    checkpoints, and the recomputation takes them over instead of running the kernels again: one forward pass of the
    operator less per layer and segment, paid for with y, the new state and the checkpoints (about 6 bytes per token
    and channel) held from forward to backward.

    Which kept run a call with autograd on may take over:

    * keyed (recommended): the caller names each call, ``with call_key((layer, segment)): ...`` around the block's
      forward.  A kept run is taken over only by a call with the same key and signature (operator, shape, dtypes);
      any other call runs the kernels.  This is safe for every pattern, including the reference's outer per-segment
      checkpoint (RWKV-v5/src/model.py:1248: segments 0..S-2 run without autograd, the last one with) and nested
      checkpoints.
    * unkeyed: last kept, first taken over, by signature.  This is what plain activation checkpointing of a stack of
      equal layers does (the recomputation replays the blocks in reverse order) and nothing else: a call with
      autograd on that is not a recomputation would take over another call's results.  That is why every take-over
      is verified: 1024 elements spread over r, kept on the device from the first run, are compared with the
      recomputation's r by a few asynchronous device operations, and ``check()`` (called on leaving the ``with`` block;
      one synchronisation per step) raises if any take-over met different inputs.  The step's gradients are then
      wrong and must be discarded; switch to keys.

    Kept runs that are never taken over (forward-only work inside the block, segments outside the BPTT range) stay
    until the ``with`` block is left; ``max_bytes`` bounds what they hold (oldest dropped first).  Under nested
    checkpoints an inner recomputation runs without autograd again and keeps its run a second time: harmless, the
    copy is dropped on leaving."""

    SAMPLE = 1024

    def __init__(self, max_entries: int = 4096, max_bytes: int = 16 << 30, verify: bool = True):
        self.entries, self.max_entries, self.max_bytes, self.verify = [], max_entries, max_bytes, verify
        self.bytes, self.bad = 0, None

    @classmethod
    def _sample(cls, r):
        flat = r.reshape(-1)
        step = max(flat.numel() // cls.SAMPLE, 1)
        return flat[::step][:cls.SAMPLE].clone()

    @staticmethod
    def _nbytes(payload):
        return sum(t.numel() * t.element_size() for t in payload if torch.is_tensor(t))

    def push(self, key, sig, r, payload):
        n = self._nbytes(payload)
        while self.entries and (len(self.entries) >= self.max_entries or self.bytes + n > self.max_bytes):
            self.bytes -= self.entries.pop(0)[4]
        self.entries.append((key, sig, self._sample(r) if self.verify else None, payload, n))
        self.bytes += n

    def pop(self, key, sig, r):
        hit = None
        if key is None:         # unkeyed: the most recent kept run, if it is unkeyed too and has this signature
            if self.entries and self.entries[-1][0] is None and self.entries[-1][1] == sig:
                hit = self.entries.pop()
        else:
            for i in range(len(self.entries) - 1, -1, -1):
                if self.entries[i][0] == key and self.entries[i][1] == sig:
                    hit = self.entries.pop(i)
                    break
        if hit is None:
            return None
        self.bytes -= hit[4]
        if hit[2] is not None:      # asynchronous: no host synchronisation here
            differs = (hit[2] != self._sample(r)).any()
            self.bad = differs if self.bad is None else (self.bad | differs)
        return hit[3]

    def check(self):
        """Raises if a take-over since the last check met inputs that differ from the kept run's (synchronises)."""
        bad, self.bad = self.bad, None
        if bad is not None and bool(bad.item()):
            raise WKVError("recompute cache: a kept forward run was taken over by a call with different inputs (a call "
                           "with autograd on that was not the recomputation of that run); the gradients of this step "
                           "are wrong.  Name the calls with call_key() or keep such calls outside recompute_cache()")

    def clear(self):
        self.entries.clear()
        self.bytes = 0


_cache = None
_key = None


class recompute_cache:
    """Context manager that installs a ``RecomputeCache`` for the operators called inside it; on leaving, the
    take-overs are verified (``RecomputeCache.check``) and what is still kept is dropped."""

    def __init__(self, cache: RecomputeCache = None):
        self.cache = cache or RecomputeCache()

    def __enter__(self):
        global _cache
        self.prev, _cache = _cache, self.cache
        return self.cache

    def __exit__(self, exc_type, *exc):
        global _cache
        _cache = self.prev
        self.cache.clear()
        if exc_type is None:
            self.cache.check()
        else:
            self.cache.bad = None
        return False


class call_key:
    """Names the operator calls made inside it for the recompute cache (any hashable: e.g. (layer, segment)).  The
    same key must be in force when the block's forward is recomputed, which it is when the ``with`` sits inside the
    checkpointed function."""

    def __init__(self, key):
        self.key = key

    def __enter__(self):
        global _key
        self.prev, _key = _key, self.key
        return self

    def __exit__(self, *exc):
        global _key
        _key = self.prev
        return False


def _forward56_cached(version, B, T, C, H, r, k, v, w32, u32, s32, need_grad, out_state=None):
    """_forward56 behind the recompute cache (when one is installed)."""
    cache = _cache
    if cache is None:
        return _forward56(version, B, T, C, H, r, k, v, w32, u32, s32, need_grad, out_state)
    sig = (version, B, T, C, H, r.dtype, w32.dtype, tuple(w32.shape), out_state is not None)
    if need_grad:
        hit = cache.pop(_key, sig, r)
        if hit is not None:          # the recomputation of a forward run that kept its results
            y, new_state, ws, algo = hit
            if out_state is not None:
                out_state.copy_(new_state)
                new_state = out_state
            stats["forward_reused"] += 1
            return y, new_state, ws, algo
        return _forward56(version, B, T, C, H, r, k, v, w32, u32, s32, True, out_state)
    y, new_state, ws, algo = _forward56(version, B, T, C, H, r, k, v, w32, u32, s32, True, out_state)    # keep checkpoints
    cache.push(_key, sig, r, (y, new_state.clone() if out_state is not None else new_state, ws, algo))
    return y, new_state, ws, algo


def _forward56(version, B, T, C, H, r, k, v, w32, u32, s32, need_grad, out_state=None):
    """Returns y, new_state and, when a backward call will follow, the
    workspace in which the forward kernel left its state checkpoints (sized
    for that backward call) together with the algorithm that was in force.
    `w32` is fp32, or (WKV6, blocked algorithm) bf16 as it came."""
    L = _lib.lib()
    dt = _check_rkv(B, T, C, H, r, k, v)
    _on_gpu(r, k, v, w32, u32, s32)
    y = torch.empty_like(r)
    new_state = torch.empty_like(s32) if out_state is None else out_state       # (must not overlap s32)
    flags = _lib.FLOOR_DECAY if T > 1 else 0
    if w32.dtype == torch.bfloat16:
        flags |= _lib.W_BF16
    algo = _algo
    fn, fq, bq = (L.wkv5_forward, L.wkv5_forward_workspace, L.wkv5_backward_workspace) if version == 5 else \
                 (L.wkv6_forward, L.wkv6_forward_workspace, L.wkv6_backward_workspace)
    ws = None
    if need_grad and fq(B, T, C, H, dt, algo) > 0:
        ws = _workspace(max(fq(B, T, C, H, dt, algo), bq(B, T, C, H, dt, algo)), r.device)
    check(fn(_stream(), B, T, C, H, dt, flags, algo, _ptr(r), _ptr(k), _ptr(v), _ptr(w32), _ptr(u32), _ptr(s32),
             _ptr(y), _ptr(new_state), _ptr(ws), 0 if ws is None else ws.numel()), f"wkv{version}_forward")
    stats["forward_launches"] += 1
    return y, new_state, ws, algo


def _backward56(version, B, T, C, H, r, k, v, w32, u32, s32, gy, gstate, ws, algo):
    L = _lib.lib()
    dt = _DT[r.dtype]
    gr, gk, gv = torch.empty_like(r), torch.empty_like(k), torch.empty_like(v)
    gw = torch.empty_like(w32)
    gu = torch.empty_like(u32)
    gs = torch.empty_like(s32)
    flags = _lib.FLOOR_DECAY if T > 1 else 0
    if w32.dtype == torch.bfloat16:
        flags |= _lib.W_BF16           # gw comes back in bf16 too (torch.empty_like above)
    fn, wsq = (L.wkv5_backward, L.wkv5_backward_workspace) if version == 5 else (L.wkv6_backward, L.wkv6_backward_workspace)
    need = wsq(B, T, C, H, dt, algo)
    if ws is not None and ws.numel() >= need:
        flags |= _lib.CHECKPOINTS_VALID
    else:           # no forward workspace, or one sized for another plan (wkv_tune changed in between): rebuild inside
        ws = _workspace(need, r.device)
    check(fn(_stream(), B, T, C, H, dt, flags, algo, _ptr(r), _ptr(k), _ptr(v), _ptr(w32), _ptr(u32), _ptr(s32),
             _ptr(gy), _ptr(gstate), _ptr(gr), _ptr(gk), _ptr(gv), _ptr(gw), _ptr(gu), _ptr(gs), _ptr(ws), ws.numel()),
          f"wkv{version}_backward")
    return gr, gk, gv, gw, gu, gs


class _WKV5Fn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, grad_mode, B, T, C, H, state, r, k, v, w, u):
        assert state.dtype == torch.float32 and w.dtype == torch.float32
        assert state.is_contiguous() and w.is_contiguous() and u.is_contiguous()
        assert state.shape == (B, H, HEAD, HEAD) and H * HEAD == C
        u32 = u.float().contiguous().view(H, HEAD)
        w32 = w.view(H, HEAD)
        need_grad = grad_mode and any(ctx.needs_input_grad)      # no checkpoints kept under torch.no_grad()
        with torch.no_grad():
            y, new_state, ws, algo = _forward56_cached(5, B, T, C, H, r, k, v, w32, u32, state, need_grad)
        ctx.dims = (B, T, C, H)
        ctx.meta = (w.shape, u.shape, u.dtype)
        ctx.ws, ctx.algo = ws, algo
        ctx.save_for_backward(r, k, v, w32, u32, state)
        return y, new_state

    @staticmethod
    def backward(ctx, gy, gstate):
        B, T, C, H = ctx.dims
        r, k, v, w32, u32, state = ctx.saved_tensors
        wshape, ushape, udtype = ctx.meta
        gy = gy.contiguous()
        assert gy.dtype == r.dtype
        gstate = None if gstate is None else gstate.float().contiguous()
        with torch.no_grad():
            gr, gk, gv, gw, gu, gs = _backward56(5, B, T, C, H, r, k, v, w32, u32, state, gy, gstate, ctx.ws, ctx.algo)
        return (None, None, None, None, None, gs, gr, gk, gv, gw.view(wshape), gu.view(ushape).to(udtype))


class WKV_5:
    """WKV5: per-channel decay.  ``WKV_5.apply(B, T, C, H, state, r, k, v, w, u) -> (y, new_state)`` with state
    (B,H,64,64) fp32 [key][value]; r,k,v (B,T,C) in one dtype; w (H,64) fp32 raw; u (H,64).  Differentiable in
    everything, the state included.  (A thin front of the autograd Function: it notes whether autograd is recording,
    which the Function itself cannot see, so that a call under torch.no_grad() keeps no checkpoints.)"""

    @staticmethod
    def apply(B, T, C, H, state, r, k, v, w, u):
        return _WKV5Fn.apply(torch.is_grad_enabled(), B, T, C, H, state, r, k, v, w, u)


class _WKV6Fn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, grad_mode, B, T, C, H, r, k, v, w, u, s):
        assert s.is_contiguous() and w.is_contiguous() and u.is_contiguous()
        assert s.shape == (B, H, HEAD, HEAD) and H * HEAD == C and w.shape == (B, T, C)
        u32 = u.float().contiguous().view(H, HEAD)
        native_w = w.dtype == torch.bfloat16 and r.dtype == torch.bfloat16 and _blocked(6, B, T, C, H, r.dtype)
        w32 = w if native_w else w.float()
        s32 = s.float()
        need_grad = grad_mode and any(ctx.needs_input_grad)
        with torch.no_grad():
            y, new_state, ws, algo = _forward56_cached(6, B, T, C, H, r, k, v, w32, u32, s32, need_grad)
        ctx.dims = (B, T, C, H)
        ctx.meta = (w.dtype, u.shape, u.dtype, s.dtype)
        ctx.ws, ctx.algo = ws, algo
        ctx.save_for_backward(r, k, v, w32, u32, s32)
        return y, new_state.to(s.dtype)

    @staticmethod
    def backward(ctx, gy, gstate):
        B, T, C, H = ctx.dims
        r, k, v, w32, u32, s32 = ctx.saved_tensors
        wdtype, ushape, udtype, sdtype = ctx.meta
        gy = gy.contiguous()
        assert gy.dtype == r.dtype
        gstate = None if gstate is None else gstate.float().contiguous()
        with torch.no_grad():
            gr, gk, gv, gw, gu, gs = _backward56(6, B, T, C, H, r, k, v, w32, u32, s32, gy, gstate, ctx.ws, ctx.algo)
        return (None, None, None, None, None, gr, gk, gv, gw.to(wdtype), gu.view(ushape).to(udtype), gs.to(sdtype))


class WKV_6:
    """WKV6: per-token decay.  ``WKV_6.apply(B, T, C, H, r, k, v, w, u, s) -> (y, new_state)`` with r,k,v (B,T,C);
    w (B,T,C) raw (any float dtype, used in fp32; a bf16 w is read as it is by the blocked algorithm and its
    gradient comes back in bf16, as in the reference, RWKV-v6/src/module/TimeMix.py:50,90); u (H,64);
    s (B,H,64,64) [key][value]."""

    @staticmethod
    def apply(B, T, C, H, r, k, v, w, u, s):
        return _WKV6Fn.apply(torch.is_grad_enabled(), B, T, C, H, r, k, v, w, u, s)


class _RunInPlace5(torch.autograd.Function):
    """WKV5 with the reference's in-place state convention: y is returned, the new state is written by the kernel
    straight into the caller's buffer (e.g. one layer's slice of the trainer's (N_layer,B,H,64,64) tensor,
    RWKV-v5/src/model.py:53-61), the incoming state survives in a private copy for backward (the reference's
    ``state.clone()``, TimeMix.py:60).  No gradient flows through the state, as in the reference (:139-140)."""

    @staticmethod
    def forward(ctx, grad_mode, B, T, C, H, state, r, k, v, w, u):
        u32, w32 = u.float().contiguous().view(H, HEAD), w.view(H, HEAD)
        s_in = state.clone()
        with torch.no_grad():
            y, _, ws, algo = _forward56_cached(5, B, T, C, H, r, k, v, w32, u32, s_in, grad_mode and any(ctx.needs_input_grad),
                                               out_state=state)
        ctx.dims, ctx.meta, ctx.ws, ctx.algo = (B, T, C, H), (w.shape, u.shape, u.dtype), ws, algo
        ctx.save_for_backward(r, k, v, w32, u32, s_in)
        return y

    @staticmethod
    def backward(ctx, gy):
        B, T, C, H = ctx.dims
        r, k, v, w32, u32, s_in = ctx.saved_tensors
        wshape, ushape, udtype = ctx.meta
        with torch.no_grad():
            gr, gk, gv, gw, gu, _ = _backward56(5, B, T, C, H, r, k, v, w32, u32, s_in, gy.contiguous(), None, ctx.ws, ctx.algo)
        return (None, None, None, None, None, None, gr, gk, gv, gw.view(wshape), gu.view(ushape).to(udtype))


class _RunInPlace6(torch.autograd.Function):
    """WKV6 counterpart of ``_RunInPlace5`` (RWKV-v6/src/module/TimeMix.py:51,111-118)."""

    @staticmethod
    def forward(ctx, grad_mode, B, T, C, H, r, k, v, w, u, s):
        u32 = u.float().contiguous().view(H, HEAD)
        native_w = w.dtype == torch.bfloat16 and r.dtype == torch.bfloat16 and _blocked(6, B, T, C, H, r.dtype)
        w32 = w if native_w else w.float()
        s_in = s.clone()
        with torch.no_grad():
            y, _, ws, algo = _forward56_cached(6, B, T, C, H, r, k, v, w32, u32, s_in, grad_mode and any(ctx.needs_input_grad),
                                               out_state=s)
        ctx.dims, ctx.meta, ctx.ws, ctx.algo = (B, T, C, H), (w.dtype, u.shape, u.dtype), ws, algo
        ctx.save_for_backward(r, k, v, w32, u32, s_in)
        return y

    @staticmethod
    def backward(ctx, gy):
        B, T, C, H = ctx.dims
        r, k, v, w32, u32, s_in = ctx.saved_tensors
        wdtype, ushape, udtype = ctx.meta
        with torch.no_grad():
            gr, gk, gv, gw, gu, _ = _backward56(6, B, T, C, H, r, k, v, w32, u32, s_in, gy.contiguous(), None, ctx.ws, ctx.algo)
        return (None, None, None, None, None, gr, gk, gv, gw.to(wdtype), gu.view(ushape).to(udtype), None)


def _direct_state(state, B, H):
    return state.dtype == torch.float32 and state.is_contiguous() and state.shape == (B, H, HEAD, HEAD) and not state.requires_grad


def RUN_WKV5_CUDA(B, T, C, H, state, r, k, v, w, u):
    """The reference's calling convention (RWKV-v5/src/module/TimeMix.py:145-154): returns y and leaves the new
    state in ``state``.  An fp32 contiguous state buffer is written by the kernel directly (no copy afterwards);
    anything else goes through the functional operator and a copy."""
    if _direct_state(state, B, H) and w.dtype == torch.float32 and w.is_contiguous() and u.is_contiguous():
        return _RunInPlace5.apply(torch.is_grad_enabled(), B, T, C, H, state, r, k, v, w, u)
    y, new_state = WKV_5.apply(B, T, C, H, state.clone(), r, k, v, w, u)
    with torch.no_grad():
        state.copy_(new_state)
    return y


def RUN_WKV6STATE_CUDA(B, T, C, H, r, k, v, w, u, s):
    """The reference's calling convention (RWKV-v6/src/module/TimeMix.py:111-118): returns y and leaves the new
    state in ``s`` (written by the kernel directly when ``s`` is an fp32 contiguous buffer)."""
    if _direct_state(s, B, H) and w.is_contiguous() and u.is_contiguous() and w.shape == (B, T, C):
        return _RunInPlace6.apply(torch.is_grad_enabled(), B, T, C, H, r, k, v, w, u, s)
    y, new_state = WKV_6.apply(B, T, C, H, r, k, v, w, u, s.clone())
    with torch.no_grad():
        s.copy_(new_state)
    return y


class _WKV4(torch.autograd.Function):
    @staticmethod
    def forward(ctx, grad_mode, time_decay, time_first, k, v, wkv_state):
        L = _lib.lib()
        assert k.dim() == 3 and v.shape == k.shape and k.dtype == v.dtype
        B, T, C = k.shape
        assert time_decay.shape == (C,) and time_first.shape == (C,) and wkv_state.shape == (B, C, 3)
        if k.dtype not in _DT:
            raise ValueError(f"Unsupported dtype {k.dtype} for WKV")
        _on_gpu(time_decay, time_first, k, v, wkv_state)
        td, tf = time_decay.float().contiguous(), time_first.float().contiguous()
        k, v, st = k.contiguous(), v.contiguous(), wkv_state.float().contiguous()
        y = torch.empty_like(k)
        new_state = torch.empty_like(st)
        need_grad = grad_mode and any(ctx.needs_input_grad)
        ckpt = _workspace(L.wkv4_checkpoint_bytes(B, T, C), k.device) if need_grad else None
        check(L.wkv4_forward(_stream(), B, T, C, _DT[k.dtype], _ptr(td), _ptr(tf), _ptr(k), _ptr(v), _ptr(st),
                             _ptr(y), _ptr(new_state), _ptr(ckpt)), "wkv4_forward")
        ctx.save_for_backward(td, tf, k, v, st, ckpt)
        ctx.meta = (time_decay.dtype, time_first.dtype)
        return y, new_state

    @staticmethod
    def backward(ctx, gy, gnew_state):
        L = _lib.lib()
        td, tf, k, v, st, ckpt = ctx.saved_tensors
        B, T, C = k.shape
        gy = gy.contiguous()
        gns = None if gnew_state is None else gnew_state.float().contiguous()
        gtd, gtf = torch.empty_like(td), torch.empty_like(tf)
        gk, gv = torch.empty_like(k), torch.empty_like(v)
        gst = torch.empty_like(st)
        ws = _workspace(L.wkv4_backward_workspace(B, T, C, _DT[k.dtype]), k.device)
        check(L.wkv4_backward(_stream(), B, T, C, _DT[k.dtype], _ptr(td), _ptr(tf), _ptr(k), _ptr(v), _ptr(st),
                              _ptr(gy), _ptr(gns), _ptr(gtd), _ptr(gtf), _ptr(gk), _ptr(gv), _ptr(gst), _ptr(ckpt),
                              _ptr(ws), ws.numel()), "wkv4_backward")
        return None, gtd.to(ctx.meta[0]), gtf.to(ctx.meta[1]), gk, gv, gst


def wkv_op(time_decay, time_first, k, v, wkv_state):
    """RWKV-v4 WKV with the signature of torch.ops.rwkv.wkv
    (RWKV-v4neo/src/model.py:130-132): time_decay, time_first (C); k, v (B,T,C);
    wkv_state (B,C,3) = (aa, bb, pp).  Returns (y, new_state)."""
    return _WKV4.apply(torch.is_grad_enabled(), time_decay, time_first, k, v, wkv_state)


def cumsum_decay(w, chunk_len=128, per_token=True, factors=False, precision=64):
    """Decay tables of the chunked formulation from the raw decay parameter w (B,T,C) fp32, or (C,) expanded over
    T tokens when ``per_token`` is an int T.  Returns dict(log_w, incl, inter, intra, chunk_sum), all in log space;
    with ``factors=True`` also the exponentiated tables ws_exp, inter_exp, intra_exp (fp32) and the two re-centred
    factors r_decay, k_inv_decay of the intra-chunk product (fp64 for ``precision=64``, fp32 for 32), i.e.
    everything RWKV-v5/src/module/rwkv_inner.py:43-93 derives from w."""
    L = _lib.lib()
    _on_gpu(w)
    w = w.float().contiguous()
    if w.dim() == 3:
        Bw, T, C = w.shape
        pt = 1
    else:
        (C,), Bw, T, pt = w.shape, 1, int(per_token), 0
    new = lambda dt=torch.float32: torch.empty(Bw, T, C, dtype=dt, device=w.device)
    out = {n: new() for n in ("log_w", "incl", "inter", "intra")}
    out["chunk_sum"] = torch.empty(Bw, T // chunk_len, C, dtype=torch.float32, device=w.device)
    if not factors:
        check(L.wkv_cumsum_decay(_stream(), Bw, T, C, chunk_len, pt, _ptr(w), _ptr(out["log_w"]), _ptr(out["incl"]),
                                 _ptr(out["inter"]), _ptr(out["intra"]), _ptr(out["chunk_sum"])), "wkv_cumsum_decay")
        return out
    pdt = torch.float64 if precision == 64 else torch.float32
    out["ws_exp"] = torch.empty_like(out["chunk_sum"])
    out["inter_exp"], out["intra_exp"] = new(), new()
    out["r_decay"], out["k_inv_decay"] = new(pdt), new(pdt)
    check(L.wkv_cumsum_decay_factors(_stream(), Bw, T, C, chunk_len, pt, precision, _ptr(w), _ptr(out["log_w"]),
                                     _ptr(out["incl"]), _ptr(out["inter"]), _ptr(out["intra"]), _ptr(out["chunk_sum"]),
                                     _ptr(out["ws_exp"]), _ptr(out["inter_exp"]), _ptr(out["intra_exp"]),
                                     _ptr(out["r_decay"]), _ptr(out["k_inv_decay"])), "wkv_cumsum_decay_factors")
    return out
