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


def _replays_match(r, step, period, state_bufs):
    """`period` steps launched one by one from a saved memory image, then the same steps recorded into a graph and
    replayed three times from that image, with plain launches in between: every replay gives the same bits."""
    import bench
    outs = lambda: [t.clone() for t in (r.y, r.gr, r.gk, r.gv, r.gw, r.gu, r.gstate[0], r.gstate[1], r.state[0], r.state[1])]
    image = [t.clone() for t in state_bufs]

    def restore():
        for t, saved in zip(state_bufs, image):
            t.copy_(saved)
    assert r.i % period == 0
    for _ in range(period):
        step()
    torch.cuda.synchronize()
    want = outs()
    g = bench.capture_steps(r, period, step)
    assert g is not None, "capture failed"
    for rep in range(3):
        restore()
        g.replay()
        torch.cuda.synchronize()
        got = outs()
        for a, b in zip(got, want):
            assert torch.equal(a, b), f"replay {rep} differs from the plain launches"
        for _ in range(period):          # the program's own work between the replays
            step()
        torch.cuda.synchronize()


def test_graph_replays_match_plain_launches():
    import bench
    r = bench.Runner56(4, "auto", 3)
    _replays_match(r, r.step, 6, [r.state[0], r.gstate[0]])


def test_graph_replays_match_plain_launches_cold_order():
    """The cold-cache order of the benchmark (backward of the segment two steps back, then this step's forward; two
    workspaces): the checkpoints waiting in the workspaces are part of the memory image a replay starts from."""
    import bench
    r = bench.Runner56(4, "auto", 3)
    for _ in range(6):                   # (the first two steps of this order have no backward call yet)
        r.step_cold()
    torch.cuda.synchronize()
    _replays_match(r, r.step_cold, 6, [r.state[0], r.gstate[0], r.ws, r.ws_cold])
