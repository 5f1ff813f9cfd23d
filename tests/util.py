import os

import torch


def assert_close(got, ref, rtol, name=""):
    """|got - ref| <= rtol * |ref| + rtol * rms(ref), element by element."""
    got = got.detach().float().cpu()
    ref = ref.detach().float().cpu()
    assert got.shape == ref.shape, f"{name}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(got).all(), f"{name}: non-finite values"
    err = (got - ref).abs()
    bound = rtol * ref.abs() + rtol * ref.pow(2).mean().sqrt()
    if os.environ.get("WKV_SHOW_MARGIN"):       # worst error as a fraction of what the tolerance allows
        print(f"margin {name}: {(err / bound).max().item():.3f}", flush=True)
    bad = err > bound
    if bad.any():
        i = torch.argmax(err - bound)
        raise AssertionError(f"{name}: {int(bad.sum())} of {bad.numel()} elements off; worst err "
                             f"{err.flatten()[i].item():.4e} (ref {ref.flatten()[i].item():.4e}, "
                             f"rms {ref.pow(2).mean().sqrt().item():.4e}, rtol {rtol})")
