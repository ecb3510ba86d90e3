import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o
    o.lib()
    return o


@pytest.fixture(scope="session")
def dev():
    """The HIP device front end; skips (never falls back) when no GPU is visible."""
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from tensorlib_amd import HipDevice
    return HipDevice(0)


def assert_close_f16(got, want, rtol=1e-2, atol=1e-3, what=""):
    """north_star parity gate: |got - want| <= atol + rtol*|want| elementwise on fp16 values."""
    import numpy as np
    g = np.asarray(got, dtype=np.float32)
    w = np.asarray(want, dtype=np.float32)
    assert g.shape == w.shape, f"{what}: shape {g.shape} vs {w.shape}"
    both_nan = np.isnan(g) & np.isnan(w)
    same_inf = np.isinf(w) & (g == w)
    with np.errstate(invalid="ignore"):
        err = np.abs(g - w)
        tol = atol + rtol * np.abs(w)
        bad = ~((err <= tol) | both_nan | same_inf)
    if bad.any():
        idx = np.argwhere(bad)[0]
        raise AssertionError(
            f"{what}: {int(bad.sum())}/{bad.size} elements outside atol={atol} rtol={rtol}; first at {tuple(idx)}: "
            f"got {g[tuple(idx)]} want {w[tuple(idx)]}; max abs err {np.nanmax(np.where(bad, err, 0))}")


def assert_close_scaled(got, want, rtol=1e-2, scale_tol=1e-2, what=""):
    """Gate for op CHAINS (a transformer block, the whole model): every one of the ~25 ops of a block
    rounds to fp16, and two correct fp32-accumulating implementations differ by a rounding step
    after each of them, so the absolute slack is tied to the tensor's own scale:
    |got - want| <= rtol*|want| + scale_tol*rms(want)."""
    import numpy as np
    w = np.asarray(want, dtype=np.float32)
    rms = float(np.sqrt(np.mean(np.square(w[np.isfinite(w)])))) if w.size else 0.0
    assert_close_f16(got, want, rtol, scale_tol * rms, what + f" (rms {rms:.3g})")
