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


def rope_cos_sin_differences(dev, oracle, n_pos, head_dim):
    """Boolean [n_pos, head_dim/2]: where the GPU's half(cos), half(sin) of the rotary angle differ from the CPU
    loop's.  The kernels evaluate cos and sin as correctly rounded fp32 values; the host libm the CPU loop calls
    (cosf, sinf: tensorLib/src/device/cpu/CPU.cpp:446-447) is off by one fp32 ulp for about 1 % of the angles, and
    in a handful of the 262144 entries of a 2048 x 64 table that moves the value across a half rounding boundary.
    Everything else in the rotation is reproduced rounding by rounding, so RoPE outputs must be bit-equal wherever
    this mask is False.  Asserts that the mask is nearly empty and that each difference is one half ulp."""
    import numpy as np
    ones = np.zeros((1, n_pos, 1, head_dim), np.float16)
    ones[..., 0::2] = 1.0                       # rotating (1, 0) returns (cos, sin) as the CPU loop rounds them
    cpu = oracle.rope(ones, 0).reshape(n_pos, head_dim // 2, 2).view(np.uint16).astype(np.int32)
    gpu = dev.rope_table(n_pos, head_dim).cpu().numpy().reshape(n_pos, head_dim // 2, 2).view(np.uint16).astype(np.int32)
    diff = cpu != gpu
    assert int(diff.sum()) <= max(4, n_pos * head_dim // 32768), f"{int(diff.sum())} table entries differ from libm's"
    assert np.all(np.abs(cpu - gpu)[diff] == 1), "a cos/sin entry differs by more than one half ulp"
    return diff.any(axis=2)


def assert_rope_equal(got, want, differs, start, what=""):
    """got, want: [..., T, H, D] with T on axis -3; bit equality except in the pairs flagged by
    rope_cos_sin_differences (positions start .. start+T), where one half ulp of cos or sin may show."""
    import numpy as np
    g = np.asarray(got)
    w = np.asarray(want)
    assert g.shape == w.shape, f"{what}: shape {g.shape} vs {w.shape}"
    T, D = g.shape[-3], g.shape[-1]
    m = np.repeat(differs[start:start + T], 2, axis=1)[:, None, :]          # [T, 1, D]
    m = np.broadcast_to(m, g.shape)
    same = g.view(np.uint16) == w.view(np.uint16)
    assert np.all(same | m), f"{what}: {int((~same & ~m).sum())} elements differ from the CPU loop"
    assert_close_f16(g[m], w[m], 1e-2, 2e-3, what + " (pairs whose cos/sin differ by a half ulp)")
