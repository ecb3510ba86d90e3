"""Host-side logic that needs no GPU: the shape/broadcast rules of Tensor::matmul
(tensorLib/src/ops/matmul.cpp:209-286, checked against numpy as the reference's own
test_batched_matmul does, tensorLib/test/python/test_tensor.py:38-121), the synthetic-input
generator, and the loud failure when no GPU is present."""
import numpy as np
import pytest

from tensorlib_amd import synth
from tensorlib_amd.device import half_bits, plan_matmul


def test_plan_matmul_matches_numpy_broadcasting():
    rng = np.random.default_rng(0)
    for _ in range(200):
        nb_a, nb_b = rng.integers(0, 4, 2)
        batch = [int(rng.integers(1, 4)) for _ in range(max(nb_a, nb_b))]
        ab = [b if rng.random() < 0.7 else 1 for b in batch[len(batch) - nb_a:]]
        bb = [b if rng.random() < 0.7 else 1 for b in batch[len(batch) - nb_b:]]
        M, K, N = (int(v) for v in rng.integers(1, 9, 3))
        a = np.zeros(ab + [M, K], np.float32)
        b = np.zeros(bb + [K, N], np.float32)
        want = np.matmul(a, b).shape
        pa, pb, ob, m, n, k = plan_matmul(a.shape, b.shape)
        assert tuple(ob + [m, n]) == want and (m, n, k) == (M, N, K)
        assert len(pa) == len(pb) == len(ob)


@pytest.mark.parametrize("sa,sb", [((5,), (5, 2)), ((4, 5), (6, 3)), ((2, 4, 5), (3, 5, 2)), ((4, 5), (5,))])
def test_plan_matmul_rejects_like_the_reference(sa, sb):
    with pytest.raises(ValueError):
        plan_matmul(sa, sb)


def test_plan_matmul_checks_result_shape():
    plan_matmul((4, 5), (5, 3), (4, 3))
    with pytest.raises(ValueError, match="result shape"):
        plan_matmul((4, 5), (5, 3), (4, 4))


def test_synth_is_deterministic_and_has_the_stated_moments():
    a = synth.normal_f16(123, (512, 512), 0.02)
    b = synth.normal_f16(123, (512, 512), 0.02)
    assert a.dtype == np.float16 and np.array_equal(a.view(np.uint16), b.view(np.uint16))
    assert not np.array_equal(a, synth.normal_f16(124, (512, 512), 0.02))
    assert abs(a.astype(np.float64).std() - 0.02) < 5e-4 and abs(a.astype(np.float64).mean()) < 2e-4
    ids = synth.token_ids(5, 128, 32000)
    assert ids.min() >= 3 and ids.max() < 32000 and ids.dtype == np.int32


def test_algorithmic_bytes_match_the_baseline_table():
    assert synth.gemv_bytes(4096, 4096) == 33_570_816
    assert synth.gemv_bytes(11008, 4096) == 90_207_744 == synth.gemv_bytes(4096, 11008)
    assert synth.gemv_bytes(32000, 4096) == 262_216_192
    assert synth.gemm_flops(2048, 4096, 4096) == 68_719_476_736


def test_half_bits():
    assert half_bits(1.0) == 0x3C00 and half_bits(-2.0) == 0xC000
    assert half_bits(np.sqrt(128.0)) == int(np.float16(11.3125).view(np.uint16))


def test_no_gpu_means_loud_failure():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from tensorlib_amd import HipDevice, TensorLibError
    with pytest.raises(TensorLibError):
        HipDevice(0)


# ------------------------------------------------ arithmetic identities the kernels rely on ----

def _round_to_f32(fr):
    """Exact round-to-nearest-even of a Fraction to a float32 value (returned as Fraction)."""
    from fractions import Fraction
    if fr == 0:
        return Fraction(0)
    sign = -1 if fr < 0 else 1
    a = abs(fr)
    e = a.numerator.bit_length() - a.denominator.bit_length() - 24
    while a / Fraction(2) ** e >= 2 ** 24:
        e += 1
    while a / Fraction(2) ** e < 2 ** 23:
        e -= 1
    e = max(e, -149)
    scaled = a / Fraction(2) ** e
    n = scaled.numerator // scaled.denominator
    rem = scaled - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and n % 2 == 1):
        n += 1
    return sign * n * Fraction(2) ** e


def test_score_quotient_by_newton_step_equals_the_division_for_every_half():
    """The attention kernels form half(x / d) as q = x*r, q += fma(-q, d, x) * r with r = float32(1/d).  For every
    finite fp16 x and both divisors in use (half(sqrt(64)) = 8, half(sqrt(128)) = 11.3125) this must round to the
    same fp16 value as the fp32 division the reference performs (Transformer.cpp:94, half operator/)."""
    from fractions import Fraction
    for d_half in (np.float16(np.sqrt(64.0)), np.float16(np.sqrt(128.0))):
        d = Fraction(float(d_half))
        r = _round_to_f32(1 / d)
        bits = np.arange(0, 0x7C00, dtype=np.uint16)            # non-negative finite halves; the scheme is odd in x
        xs = bits.view(np.float16)
        bad = []
        for xv in xs:                                            # exact rational arithmetic, one rounding per operation
            x = Fraction(float(xv))
            q0 = _round_to_f32(x * r)
            rem = _round_to_f32(x - q0 * d)
            q1 = _round_to_f32(q0 + rem * r)
            want32 = _round_to_f32(x / d)
            got16, want16 = np.float16(np.float32(float(q1))), np.float16(np.float32(float(want32)))
            if got16 != want16:
                bad.append(float(xv))
        assert not bad, (float(d_half), bad[:5])
