"""The forward + backward calls of a step recorded into a HIP graph: every replay
must reproduce what the same steps give when launched one by one (the library
allocates nothing and synchronises nothing inside a call, and its reductions run
in a fixed order, so the comparison is exact).  Plain launches run between the
replays, and each replay is checked, not only the first."""
import os
import sys

import pytest
import torch

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def test_graph_replays_match_plain_launches():
    import bench
    r = bench.Runner56(4, "auto", 3)
    period = 6
    init = r.state[0].clone()
    outs = lambda: [t.clone() for t in (r.y, r.gr, r.gk, r.gv, r.gw, r.gu, r.gstate_in, r.state[0], r.state[1])]
    for _ in range(period):
        r.step()
    torch.cuda.synchronize()
    want = outs()
    g = bench.capture_period(r, period)
    assert g is not None, "capture failed"
    for rep in range(3):
        r.state[0].copy_(init)
        g.replay()
        torch.cuda.synchronize()
        got = outs()
        for a, b in zip(got, want):
            assert torch.equal(a, b), f"replay {rep} differs from the plain launches"
        for _ in range(period):          # the program's own work between the replays
            r.step()
        torch.cuda.synchronize()
