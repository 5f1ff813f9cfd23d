"""Seeded synthetic inputs for the five benchmark / parity workloads.

Every tensor is drawn on the CPU in fp32 from one ``torch.Generator`` in a fixed
order (r, k, v, raw decay, u, state, dy, dstate), then rounded to its storage
dtype, so a CPU checker and the GPU operator see bit-identical inputs.  The
second parameter of N(.,.) is a standard deviation.

cfg0  WKV5 forward only  B1 T512  C768  H12 fp32, zero state
cfg1  WKV5 fwd+bwd       B8 T4096 C2048 H32 bf16 r/k/v, fp32 w/u/state
cfg2  WKV4 fwd+bwd       B8 T4096 C4096 fp32, state aa=bb=0 pp=-1e38
cfg3  WKV6 fwd+bwd       B8 T4096 C2560 H40 bf16 r/k/v, per-token raw decay N(-1,0.5)
cfg4  WKV6 chain         B1 C4096 H64, 64 segments of T4096, state carried (7B layer shape)

The shapes can be overridden (``B=, T=, C=, H=``) to get a small case with the
same distributions.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Optional

import torch

HEAD = 64

SHAPES = {
    0: dict(version=5, B=1, T=512, C=768, H=12, dtype=torch.float32),
    1: dict(version=5, B=8, T=4096, C=2048, H=32, dtype=torch.bfloat16),
    2: dict(version=4, B=8, T=4096, C=4096, H=None, dtype=torch.float32),
    3: dict(version=6, B=8, T=4096, C=2560, H=40, dtype=torch.bfloat16),
    4: dict(version=6, B=1, T=4096, C=4096, H=64, dtype=torch.bfloat16, segments=64),
}


@dataclass
class Workload:
    cfg: int
    version: int
    B: int
    T: int
    C: int
    H: Optional[int]
    dtype: torch.dtype
    tensors: Dict[str, torch.Tensor] = field(default_factory=dict)

    def to(self, device):
        self.tensors = {n: t.to(device) for n, t in self.tensors.items()}
        return self

    def __getitem__(self, name):
        return self.tensors[name]


def _normal(g, shape, std=1.0, mean=0.0):
    return torch.randn(shape, generator=g, dtype=torch.float32) * std + mean


def _uniform(g, shape, lo, hi):
    return torch.rand(shape, generator=g, dtype=torch.float32) * (hi - lo) + lo


def make(cfg: int, seed: Optional[int] = None, segment: int = 0, **override) -> Workload:
    """Draw the inputs of workload ``cfg``.  ``segment`` selects the segment of
    the cfg4 chain (seed 1004 + segment); its ``state`` entry is the chain's
    initial state and only meaningful for segment 0."""
    spec = dict(SHAPES[cfg])
    spec.pop('segments', None)
    spec.update(override)
    version, B, T, C, H, dtype = (spec[n] for n in ('version', 'B', 'T', 'C', 'H', 'dtype'))
    if seed is None:
        seed = 1000 + cfg + (segment if cfg == 4 else 0)
    g = torch.Generator().manual_seed(seed)
    wl = Workload(cfg, version, B, T, C, H, dtype)
    t = wl.tensors
    if version == 4:
        t['k'] = _normal(g, (B, T, C)).to(dtype)
        t['v'] = _normal(g, (B, T, C)).to(dtype)
        t['time_decay'] = _uniform(g, (C,), -5.0, 1.0)
        t['time_first'] = _normal(g, (C,), 0.5).to(dtype)
        st = torch.zeros(B, C, 3)
        st[:, :, 2] = -1e38
        t['state'] = st
        t['dy'] = _normal(g, (B, T, C)).to(dtype)
        t['dstate'] = torch.zeros(B, C, 3)
        t['dstate'][:, :, 2] = -1e38
        return wl
    K = C // H
    assert K == HEAD and K * H == C
    for n in ('r', 'k', 'v'):
        t[n] = _normal(g, (B, T, C), 0.5).to(dtype)
    if version == 5:
        t['w'] = _uniform(g, (H, K), -6.0, 0.0)                  # raw; decay = exp(-exp(w))
    else:
        t['w'] = _normal(g, (B, T, C), 0.5, -1.0)                # raw, per token
    t['u'] = _normal(g, (H, K), 0.5)
    if cfg == 0:
        t['state'] = torch.zeros(B, H, K, K)
    else:
        t['state'] = _normal(g, (B, H, K, K), 0.1)
    t['dy'] = _normal(g, (B, T, C)).to(dtype)
    t['dstate'] = _normal(g, (B, H, K, K))
    return wl
