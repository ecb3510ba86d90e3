"""Pins of the CPU oracle (oracle/tl_oracle.c) that do not go through the oracle's own formula.

The reference holds no golden vectors for this path (every reference test draws unseeded random
inputs) and its CPU backend cannot be compiled here (it needs cuda_fp16.h), so each oracle
function is pinned by what the mathematics fixes: exact integer cases, identities, closed forms
evaluated in float64 by numpy/scipy, brute-force Python loops on tiny inputs, and inputs built so
that a plausible mistake (wrong summation order, transposed operand, wrong RoPE pairing or
frequency, softmax without the max shift, argmax tie order ...) fails.
"""
import numpy as np
import pytest
from scipy.special import softmax as scipy_softmax

from tensorlib_amd import synth


def f16_round(x64):
    """Round float64 -> fp16 (nearest even) the way IEEE does, via numpy."""
    with np.errstate(over="ignore"):
        return np.asarray(x64, dtype=np.float64).astype(np.float16)


def ulp16(x):
    x = np.abs(np.asarray(x, dtype=np.float64))
    e = np.floor(np.log2(np.maximum(x, 2.0 ** -14)))
    return 2.0 ** (e - 10)


# ------------------------------------------------------------------------ conversions ----

def test_half_to_float_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = oracle.h2f(bits)
    nan = np.isnan(want)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
    assert np.isnan(got[nan]).all()


def test_float_to_half_rounding(oracle):
    rng = np.random.default_rng(0)
    x = rng.integers(0, 2 ** 32, size=2_000_000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    with np.errstate(all="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = oracle.f2h(x)
    ok = ~np.isnan(x)
    assert np.array_equal(got[ok], want[ok])
    # every midpoint between adjacent halves (ties-to-even) and its float neighbours
    h = np.arange(0x7c00, dtype=np.uint16).view(np.float16).astype(np.float64)
    mid = ((h[:-1] + h[1:]) / 2).astype(np.float32)
    c = np.concatenate([mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf)),
                        np.array([65504, 65519.996, 65520, 65536, 1e9, np.inf, 2.0 ** -25, 2.0 ** -24, 0.0], np.float32)])
    c = np.concatenate([c, -c])
    with np.errstate(all="ignore"):
        assert np.array_equal(oracle.f2h(c), c.astype(np.float16).view(np.uint16))


# ----------------------------------------------------------------------------- matmul ----

def test_matmul2d_integer_exact(oracle):
    for (M, N, K) in [(1, 7, 5), (3, 4, 64), (17, 9, 300), (1, 50, 4096)]:
        A = synth.small_ints_f16(1, (M, K), -3, 3)
        B = synth.small_ints_f16(2, (N, K), -3, 3)
        want = A.astype(np.int64) @ B.astype(np.int64).T
        assert np.abs(want).max() < 2048
        assert np.array_equal(oracle.matmul2d(A, B).astype(np.int64), want)


def test_matmul2d_operand_layout(oracle):
    """A is [M,K], B is [N,K] (not [K,N]): non-square shapes and unit vectors pin the layout."""
    B = synth.normal_f16(3, (6, 11), 1.0)
    for k in range(11):
        e = np.zeros((1, 11), np.float16)
        e[0, k] = 1.0
        assert np.array_equal(oracle.matmul2d(e, B)[0].view(np.uint16), B[:, k].view(np.uint16))
    A = synth.normal_f16(4, (5, 8), 1.0)
    assert np.array_equal(oracle.matmul2d(A, np.eye(8, dtype=np.float16)).view(np.uint16), A.view(np.uint16))


def test_matmul2d_brute_force_python(oracle):
    """Tiny shapes against a pure-Python restatement with numpy float32 scalars: bit-exact."""
    rng = np.random.default_rng(5)
    for (M, N, K) in [(1, 1, 1), (2, 3, 5), (3, 2, 17)]:
        A = rng.standard_normal((M, K)).astype(np.float16)
        B = rng.standard_normal((N, K)).astype(np.float16)
        want = np.empty((M, N), np.float16)
        for i in range(M):
            for j in range(N):
                s = np.float32(0)
                for k in range(K):
                    s = np.float32(s + np.float32(A[i, k]) * np.float32(B[j, k]))
                want[i, j] = np.float16(s)
        assert np.array_equal(oracle.matmul2d(A, B).view(np.uint16), want.view(np.uint16))


def test_matmul2d_against_float64(oracle):
    """fp32 accumulation of exact products: at most ~1 fp16 ulp from the correctly rounded result."""
    A = synth.normal_f16(6, (8, 4096), 1.0)
    B = synth.normal_f16(7, (64, 4096), 0.02)
    got = oracle.matmul2d(A, B).astype(np.float64)
    ref = A.astype(np.float64) @ B.astype(np.float64).T
    assert np.all(np.abs(got - ref) <= 1.01 * ulp16(ref))
    # torch/numpy fp32 matmul of the same operands, the reference's own tolerance (test_tensor.py:121)
    ref32 = A.astype(np.float32) @ B.astype(np.float32).T
    np.testing.assert_allclose(got, ref32, rtol=1e-3, atol=2e-3)


def test_matmul2d_sums_k_ascending_in_fp32(oracle):
    """big + many tiny - big: with a sequential ascending fp32 sum every tiny term is absorbed and
    the result is exactly 0; any other order (or a wider accumulator) returns about 3.9."""
    K = 4002
    a = np.full((1, K), 0.03125, np.float16)
    b = np.full((1, K), 0.03125, np.float16)
    a[0, 0], b[0, 0] = 128.0, 256.0
    a[0, -1], b[0, -1] = -128.0, 256.0
    assert float(oracle.matmul2d(a, b)[0, 0]) == 0.0
    assert abs((a.astype(np.float64) @ b.astype(np.float64).T).item() - 4000 * 2.0 ** -10) < 1e-9


def test_matmul2d_entries_and_batched_agree_with_full(oracle):
    A = synth.normal_f16(8, (9, 40), 1.0)
    B = synth.normal_f16(9, (13, 40), 1.0)
    C = oracle.matmul2d(A, B)
    ii, jj = np.meshgrid(np.arange(9), np.arange(13), indexing="ij")
    assert np.array_equal(oracle.matmul2d_entries(A, B, ii.ravel(), jj.ravel()).view(np.uint16), C.ravel().view(np.uint16))
    Ab = synth.normal_f16(10, (4, 3, 16), 1.0)
    Bb = synth.normal_f16(11, (4, 5, 16), 1.0)
    got = oracle.matmul2d_batched(Ab, Bb, 4, 3, 5, 16, 48, 80)
    for b in range(4):
        assert np.array_equal(got[b].view(np.uint16), oracle.matmul2d(Ab[b], Bb[b]).view(np.uint16))
    got = oracle.matmul2d_batched(Ab[0], Bb, 4, 3, 5, 16, 0, 80)  # stride 0 broadcasts A
    for b in range(4):
        assert np.array_equal(got[b].view(np.uint16), oracle.matmul2d(Ab[0], Bb[b]).view(np.uint16))


def test_matmul2d_f32(oracle):
    rng = np.random.default_rng(12)
    A = rng.standard_normal((7, 33)).astype(np.float32)
    B = rng.standard_normal((5, 33)).astype(np.float32)
    np.testing.assert_allclose(oracle.matmul2d_f32(A, B), A.astype(np.float64) @ B.astype(np.float64).T, rtol=1e-5, atol=1e-5)


# ------------------------------------------------------------------------------- RoPE ----

def test_rope_closed_form(oracle):
    """Complex-multiply form of the reference's own test (tensorLib/test/python/test_ops.py:65-86)."""
    B, T, H, D, start = 2, 9, 4, 128, 5
    x = synth.normal_f16(20, (B, T, H, D), 1.0)
    got = oracle.rope(x, start).astype(np.float64)
    xc = x.astype(np.float64).reshape(B, T, H, D // 2, 2)
    z = xc[..., 0] + 1j * xc[..., 1]
    freqs = 1.0 / (10000.0 ** (np.arange(0, D, 2) / D))
    ang = np.outer(np.arange(start, start + T), freqs)
    rot = z * np.exp(1j * ang)[None, :, None, :]
    want = np.stack([rot.real, rot.imag], axis=-1).reshape(B, T, H, D)
    # cos/sin rounded to half and four half roundings: a few fp16 ulps of slack
    assert np.all(np.abs(got - want) <= 3 * ulp16(want) + 2e-3)


def test_rope_pairing_and_frequency_index(oracle):
    """(1, 0) in pair p at position t must become (cos, sin) of t * 10000^(-2p/D): fails for the
    half-split pairing convention or an off-by-one in the frequency exponent."""
    D, t = 64, 7
    for p in (0, 1, 5, 31):
        x = np.zeros((1, 1, 1, D), np.float16)
        x[0, 0, 0, 2 * p] = 1.0
        out = oracle.rope(x, t).astype(np.float64)[0, 0, 0]
        th = t * 10000.0 ** (-2.0 * p / D)
        assert abs(out[2 * p] - np.cos(th)) < 1e-3 and abs(out[2 * p + 1] - np.sin(th)) < 1e-3
        out[2 * p] = out[2 * p + 1] = 0
        assert np.all(out == 0)


def test_rope_position_zero_is_identity(oracle):
    x = synth.normal_f16(21, (1, 1, 3, 16), 1.0)
    assert np.array_equal(oracle.rope(x, 0).view(np.uint16), x.view(np.uint16))


def test_rope_uses_start_pos_plus_t(oracle):
    x = synth.normal_f16(22, (1, 4, 2, 32), 1.0)
    full = oracle.rope(x, 10)
    for t in range(4):
        one = oracle.rope(x[:, t:t + 1], 10 + t)
        assert np.array_equal(full[:, t:t + 1].view(np.uint16), one.view(np.uint16))


# ---------------------------------------------------------------------------- softmax ----

def test_softmax_against_scipy(oracle):
    x = synth.normal_f16(30, (37, 300), 3.0)
    got = oracle.softmax(x).astype(np.float64)
    want = scipy_softmax(x.astype(np.float64), axis=1)
    assert np.all(np.abs(got - want) <= 0.51 * ulp16(want) + 1e-6 * want + 6e-8)
    assert np.all(np.abs(got.sum(1) - 1) < 2e-3)


def test_softmax_large_inputs_need_max_shift(oracle):
    x = np.array([[60000.0, 59999.0, -60000.0]], np.float16)  # exp overflows without the shift
    got = oracle.softmax(x).astype(np.float64)
    want = scipy_softmax(x.astype(np.float64), axis=1)
    assert np.all(np.isfinite(got)) and np.all(np.abs(got - want) < 1e-3)


def test_softmax_literal_half_chain_is_close_but_not_the_gate(oracle):
    """The literal half-carried sum drifts with row length; it is reported, not gated on."""
    x = synth.normal_f16(31, (8, 1024), 1.0)
    lit = oracle.softmax(x, literal=True).astype(np.float64)
    ref = scipy_softmax(x.astype(np.float64), axis=1)
    rel = np.abs(lit - ref) / ref
    assert rel.max() < 0.05          # same function ...
    assert rel.max() > 1e-3          # ... but visibly less accurate than the fp32-sum form


def test_softmax_literal_carries_its_sum_in_half(oracle):
    """What the half arithmetic of softmax.cpp:20-24 fixes, worked by hand.  A row of n equal values: every
    exponential is 1 and the running half sum counts 1, 2, ... exactly up to 2048; from there 2048 + 1 is a tie
    that rounds to even, i.e. back to 2048, so for n > 2048 every output is 1/2048 = 2^-11 whatever n is, where a
    float sum gives 1/n.  For n <= 2048 the outputs are half(1/n)."""
    for n in (1, 3, 7, 100, 2048):
        row = np.full((1, n), 0.75, np.float16)
        assert np.all(oracle.softmax(row, literal=True) == np.float16(1.0 / n)), n
    for n in (2049, 3000, 4096):
        row = np.full((1, n), -3.0, np.float16)
        assert np.all(oracle.softmax(row, literal=True) == np.float16(2.0 ** -11)), n
        assert np.all(oracle.softmax(row) == np.float16(1.0 / n)), n        # the fp32-sum form, for contrast


def test_softmax_literal_rounds_the_shifted_input_to_half(oracle):
    """x - max is a half operation (softmax.cpp:20): 0.001 and 0.003 are different halves, but 10 away from the
    row maximum both differences round to the same half, -10 (spacing 2^-7 there), so the literal chain gives
    them the same probability, which a float subtraction does not."""
    a, b = np.float16(0.001), np.float16(0.003)
    assert a != b and np.float16(np.float32(a) - 10) == np.float16(np.float32(b) - 10)
    row = np.array([[10.0, a, b]], np.float16)
    lit = oracle.softmax(row, literal=True)[0]
    assert lit[1] == lit[2] and lit[1] > 0
    f32 = oracle.softmax(row)[0]
    assert f32[1] != f32[2]


# ---------------------------------------------------------------------------- RMSNorm ----

def _rms_ref(x, w, eps):
    x64, w64 = x.astype(np.float64), w.astype(np.float64)
    return x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + eps) * w64


def test_rms_norm_exact_and_fused(oracle):
    x = synth.normal_f16(40, (5, 4096), 1.5)
    w = synth.normal_f16(41, (4096,), 1.0)
    ref = _rms_ref(x, w, 1e-5)
    exact = oracle.rms_norm(x, w, 1e-5, "exact").astype(np.float64)
    assert np.all(np.abs(exact - ref) <= 0.51 * ulp16(ref) + 1e-7)
    fused = oracle.rms_norm(x, w, 1e-5, "fused").astype(np.float64)
    assert np.all(np.abs(fused - ref) <= 3 * ulp16(ref) + 1e-6)


def test_rms_norm_eps_and_mean_not_sum(oracle):
    """All-zero rows give 0 (eps keeps it finite); scaling hidden size must not change the result
    (mean, not sum, under the root)."""
    z = np.zeros((1, 64), np.float16)
    w = np.ones(64, np.float16)
    assert np.all(oracle.rms_norm(z, w, 1e-5, "fused") == 0)
    x = np.full((1, 64), 3.0, np.float16)
    x2 = np.full((1, 256), 3.0, np.float16)
    assert np.allclose(oracle.rms_norm(x, w, 1e-5, "exact").astype(np.float32), 1.0, atol=1e-3)
    assert np.allclose(oracle.rms_norm(x2, np.ones(256, np.float16), 1e-5, "exact").astype(np.float32), 1.0, atol=1e-3)


def test_rms_norm_plain_literal_drifts(oracle):
    """The literal CPU chain sums 4096 squares in half precision and is several per cent off the
    definition, which is why it cannot be the parity gate for an fp32-accumulating kernel."""
    x = synth.normal_f16(42, (4, 4096), 1.0)
    w = np.ones(4096, np.float16)
    lit = oracle.rms_norm(x, w, 1e-5, "plain_literal").astype(np.float64)
    ref = _rms_ref(x, w, 1e-5)
    big = np.abs(ref) > 0.5
    rel = np.abs(lit - ref)[big] / np.abs(ref)[big]
    assert rel.max() < 1.0 and rel.mean() > 1e-2


def test_rms_norm_plain_literal_saturating_mean(oracle):
    """Hand-worked consequences of summing the squares sequentially in half (CPU.cpp:340-354): 4096 ones sum to
    2048 (2048 + 1 ties back to 2048), so mean = 2048/4096 = 0.5, + half(1e-5) is still 0.5, rsqrt gives
    half(1.41421) = 1.4140625 and every output is 1.4140625 where the definition gives 1.  With 2.0 the squares
    are 4 and the sum stops at 8192 (8192 + 4 ties to even): mean 2, rsqrt half(0.70711) = 0.70703125, output
    half(2 * 0.70703125) = 1.4140625 again.  Up to 2048 ones nothing saturates and the output is 1."""
    w = np.ones(4096, np.float16)
    out = oracle.rms_norm(np.ones((2, 4096), np.float16), w, 1e-5, "plain_literal")
    assert np.all(out == np.float16(1.4140625))
    out2 = oracle.rms_norm(np.full((1, 4096), 2.0, np.float16), w, 1e-5, "plain_literal")
    assert np.all(out2 == np.float16(1.4140625))
    out3 = oracle.rms_norm(np.ones((1, 2048), np.float16), np.ones(2048, np.float16), 1e-5, "plain_literal")
    assert np.all(out3 == np.float16(1.0))
    # the weight is applied after the normalisation, as a half multiply (rmsNorm.cpp:52-55)
    w3 = np.full(4096, 3.0, np.float16)
    out4 = oracle.rms_norm(np.ones((1, 4096), np.float16), w3, 1e-5, "plain_literal")
    assert np.all(out4 == np.float16(np.float32(1.4140625) * 3))
    # and for contrast the fp32-sum variant returns 1 on the same input
    assert np.all(oracle.rms_norm(np.ones((1, 4096), np.float16), w, 1e-5, "fused") == np.float16(1.0))


# ------------------------------------------------------------------------ elementwise ----

def test_silu_closed_form(oracle):
    x = np.arange(-2048, 2048, dtype=np.float32).astype(np.float16) / np.float16(128)
    ref = x.astype(np.float64) / (1 + np.exp(-x.astype(np.float64)))
    got = oracle.silu(x).astype(np.float64)
    assert np.all(np.abs(got - ref) <= 0.51 * ulp16(ref) + 1e-6)
    assert oracle.silu(np.array([0.0], np.float16))[0] == 0


def test_silu_cpu_literal_has_flipped_sign(oracle):
    """tensorLib/src/device/cpu/CPU.cpp:216-219 computes x/(1+exp(+x)) = -silu(-x)."""
    x = synth.normal_f16(50, (1000,), 2.0)
    lit = oracle.silu(x, cpu_literal=True).astype(np.float64)
    want = -oracle.silu((-x).astype(np.float16)).astype(np.float64)
    assert np.all(np.abs(lit - want) <= 2 * ulp16(want) + 1e-6)
    # hand values: far right the half sigmoid 1/(1+e^x) underflows to 0 and the result is 0 where silu(x) = x;
    # far left it is exactly 1 and the result is x where silu(x) = 0; at 0 it is 0 * 0.5
    pts = np.array([20.0, 30.0, -20.0, -30.0, 0.0], np.float16)
    assert np.array_equal(oracle.silu(pts, cpu_literal=True), np.array([0.0, 0.0, -20.0, -30.0, 0.0], np.float16))


@pytest.mark.parametrize("op,fn", [("add", np.add), ("sub", np.subtract), ("mul", np.multiply), ("div", np.divide)])
def test_binary_ops_match_ieee_half(oracle, op, fn):
    a = synth.normal_f16(60, (5000,), 3.0)
    b = synth.normal_f16(61, (5000,), 3.0)
    with np.errstate(all="ignore"):
        want = fn(a.astype(np.float32), b.astype(np.float32)).astype(np.float16)
    assert np.array_equal(oracle.binary(a, b, op).view(np.uint16), want.view(np.uint16))
    s = np.float16(11.3125)
    with np.errstate(all="ignore"):
        want = fn(a.astype(np.float32), np.float32(s)).astype(np.float16)
    assert np.array_equal(oracle.binary_scalar(a, s, op).view(np.uint16), want.view(np.uint16))


def test_sqrt_head_dim_rounds_to_11_3125():
    assert float(np.float16(np.sqrt(128.0))) == 11.3125


def test_silu_mul_is_two_rounded_ops(oracle):
    a = synth.normal_f16(62, (3000,), 2.0)
    b = synth.normal_f16(63, (3000,), 1.0)
    want = oracle.binary(oracle.silu(a), b, "mul")
    assert np.array_equal(oracle.silu_mul(a, b).view(np.uint16), want.view(np.uint16))


# ----------------------------------------------------------------------------- layout ----

def test_contiguous_and_set_item_against_numpy_strides(oracle):
    base = synth.normal_f16(70, (6, 5, 8), 1.0)
    # transpose(0,1) then slice [:, 1:4]
    view = base.transpose(1, 0, 2)[:, 1:4]
    stride = [s // 2 for s in view.strides]
    off = (view.__array_interface__["data"][0] - base.__array_interface__["data"][0]) // 2
    got = oracle.contiguous(base, view.shape, stride, off)
    assert np.array_equal(got.view(np.uint16), np.ascontiguousarray(view).view(np.uint16))
    src = synth.normal_f16(71, view.shape, 1.0)
    want = base.copy()
    want.transpose(1, 0, 2)[:, 1:4] = src
    assert np.array_equal(oracle.set_item_ewise(base, src, view.shape, stride, off).view(np.uint16), want.view(np.uint16))
    # stride 0 = broadcast
    row = synth.normal_f16(72, (8,), 1.0)
    got = oracle.contiguous(row, (3, 8), (0, 1), 0)
    assert np.array_equal(got.view(np.uint16), np.broadcast_to(row, (3, 8)).copy().view(np.uint16))


def test_argmax_first_maximum(oracle):
    x = np.array([[1, 5, 5, 2], [7, 7, 7, 7], [-3, -2, -1, -1], [0, -1, -2, 9]], np.float16)
    assert oracle.argmax(x).tolist() == [1, 0, 2, 3]
    r = synth.normal_f16(80, (50, 999), 1.0)
    assert np.array_equal(oracle.argmax(r), np.argmax(r.astype(np.float32), axis=1))


def test_embedding_is_a_row_gather(oracle):
    t = synth.normal_f16(90, (20, 12), 1.0)
    ids = np.array([3, 3, 19, 0], np.int32)
    assert np.array_equal(oracle.embedding(t, ids).view(np.uint16), t[ids].view(np.uint16))


# ------------------------------------------------------------------ composed chains ----

def test_attention_chain_against_float64(oracle):
    """The composed attention chain (per-head matmul2d, ScalarDiv, mask, softmax, matmul2d) against the
    textbook causal attention in float64: catches a transposed operand, a wrong mask edge or scale."""
    H, S, D, start = 3, 7, 32, 4
    T = start + S
    q = synth.normal_f16(300, (H, S, D), 1.0)
    ck = synth.normal_f16(301, (T + 2, H, D), 1.0)
    cv = synth.normal_f16(302, (T + 2, H, D), 1.0)
    got = oracle.attention_chain(q, ck, cv, start).astype(np.float64)
    k = ck[:T].astype(np.float64).transpose(1, 0, 2)          # [H, T, D]
    v = cv[:T].astype(np.float64).transpose(1, 0, 2)
    sc = np.einsum("hsd,htd->hst", q.astype(np.float64), k) / np.sqrt(D)
    sc = np.where(np.arange(T)[None, None, :] > start + np.arange(S)[None, :, None], -np.inf, sc)
    want = np.einsum("hst,htd->shd", scipy_softmax(sc, axis=-1), v)
    assert np.abs(got - want).max() < 6e-3
    # a single new token sees every cached position: no mask is applied (Transformer.cpp:234)
    got1 = oracle.attention_chain(q[:, :1], ck, cv, T - 1).astype(np.float64)
    sc1 = np.einsum("hsd,htd->hst", q[:, :1].astype(np.float64), k) / np.sqrt(D)
    want1 = np.einsum("hst,htd->shd", scipy_softmax(sc1, axis=-1), v)
    assert np.abs(got1 - want1).max() < 6e-3
