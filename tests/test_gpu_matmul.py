"""GPU parity of the matmul hot path (GEMV + HGEMM) against the CPU oracle, through the C ABI.

Gate (north_star): |gpu - cpu| <= 1e-3 + 1e-2 * |cpu| elementwise on the fp16 outputs; the
integer-valued and unit-vector cases must match bit for bit.
"""
import numpy as np
import pytest
import torch

from tensorlib_amd import synth
from tests.conftest import assert_close_f16

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-2, 1e-3

# Llama2-7B decode GEMV sweep (N <- K)
SWEEP = [(4096, 4096), (11008, 4096), (4096, 11008), (32000, 4096)]


def _gemv_case(dev, oracle, N, K, seed, variant=0, w_std=0.02):
    W = synth.normal_f16(seed, (N, K), w_std)
    x = synth.normal_f16(seed + 1, (K,), 1.0)
    from tensorlib_amd import TensorLibError
    dev.set_gemv_variant(variant)
    try:
        y = dev.gemv(dev.from_numpy(x), dev.from_numpy(W)).cpu().numpy()
    except TensorLibError as e:
        # a forced single-tile variant refuses rows longer than its register tile
        assert variant != 0 and "cannot hold" in str(e), e
        return
    finally:
        dev.set_gemv_variant(0)
    want = oracle.matmul2d(x[None, :], W)[0]
    assert_close_f16(y, want, RTOL, ATOL, f"gemv {N}<-{K} variant {variant}")


def test_gemv_config_single(dev, oracle):
    """W[4096,4096] ~ N(0,0.02), x ~ N(0,1)."""
    _gemv_case(dev, oracle, 4096, 4096, seed=100)


@pytest.mark.parametrize("N,K", SWEEP)
def test_gemv_decode_sweep(dev, oracle, N, K):
    """The four Llama2-7B decode shapes, through matmul2d with M == 1."""
    W = synth.normal_f16(200 + N % 97, (N, K), 0.02)
    x = synth.normal_f16(300 + K % 89, (1, K), 1.0)
    y = dev.matmul2d(dev.from_numpy(x), dev.from_numpy(W)).cpu().numpy()
    want = oracle.matmul2d(x, W)
    assert_close_f16(y, want, RTOL, ATOL, f"matmul2d M=1 {N}<-{K}")


def test_gemv_every_variant(dev, oracle):
    names = dev.gemv_variants()
    assert len(names) > 4
    for v in range(1, len(names)):
        for (N, K) in [(4096, 4096), (1024, 11008), (37, 520), (5, 8), (130, 4104)]:
            _gemv_case(dev, oracle, N, K, seed=400 + v, variant=v)


@pytest.mark.parametrize("N,K", [(1, 1), (3, 7), (64, 127), (257, 1001), (100, 128), (33, 64), (1000, 256),
                                 (128, 1024), (7, 24), (19, 8192), (2, 40000)])
def test_gemv_ragged_shapes(dev, oracle, N, K):
    """Shapes off the fast path: K % 8 != 0, short rows (attention's K = 128), x larger than LDS."""
    _gemv_case(dev, oracle, N, K, seed=500 + N, w_std=0.05)


def test_gemv_integer_inputs_bit_exact(dev, oracle):
    """Integer-valued operands with |sum| < 2048: every fp32 partial sum is exact, so any summation
    order must give the oracle's bits."""
    for (N, K) in [(4096, 4096), (4096, 11008), (300, 136)]:
        W = synth.small_ints_f16(600, (N, K), -2, 2)
        x = synth.small_ints_f16(601, (K,), -1, 1)
        y = dev.gemv(dev.from_numpy(x), dev.from_numpy(W)).cpu().numpy()
        want = oracle.matmul2d(x[None, :], W)[0]
        assert np.abs(want.astype(np.float32)).max() < 2048
        assert np.array_equal(y.view(np.uint16), want.view(np.uint16))


def test_gemv_unit_vector_selects_column(dev):
    """x = e_k must return column k of W exactly (catches index/lane mapping mistakes)."""
    N, K = 512, 4096
    W = synth.normal_f16(700, (N, K), 1.0)
    Wd = dev.from_numpy(W)
    for k in [0, 1, 7, 8, 63, 64, 511, 512, 2047, 4095]:
        x = np.zeros(K, np.float16)
        x[k] = 1.0
        y = dev.gemv(dev.from_numpy(x), Wd).cpu().numpy()
        assert np.array_equal(y.view(np.uint16), W[:, k].view(np.uint16)), k


def test_gemv_unaligned_pointers(dev, oracle):
    """Operands not 16-byte aligned must take the generic kernel and still be right."""
    N, K = 50, 264
    W = synth.normal_f16(710, (N * K + 8,), 0.1)
    x = synth.normal_f16(711, (K + 8,), 1.0)
    Wd, xd = dev.from_numpy(W), dev.from_numpy(x)
    y = dev.gemv(xd[1:K + 1].view(-1), Wd[3:3 + N * K].view(N, K))
    want = oracle.matmul2d(x[None, 1:K + 1], W[3:3 + N * K].reshape(N, K))[0]
    assert_close_f16(y.cpu().numpy(), want, RTOL, ATOL, "unaligned gemv")


# ------------------------------------------------------------------------------ HGEMM ----

def _hgemm_case(dev, oracle, M, N, K, seed, variant=0, full=True, a_std=1.0, b_std=0.02):
    A = synth.normal_f16(seed, (M, K), a_std)
    B = synth.normal_f16(seed + 1, (N, K), b_std)
    dev.set_hgemm_variant(variant)
    try:
        C = dev.hgemm(dev.from_numpy(A), dev.from_numpy(B)).cpu().numpy()
    finally:
        dev.set_hgemm_variant(0)
    what = f"hgemm {M}x{N}x{K} variant {variant}"
    if full:
        assert_close_f16(C, oracle.matmul2d(A, B), RTOL, ATOL, what)
    else:
        # sampled parity: 8 full rows + 8192 uniformly drawn entries
        rng = np.random.default_rng(seed)
        rows = np.unique(np.concatenate([[0, M - 1], rng.integers(0, M, 6)]))
        assert_close_f16(C[rows], oracle.matmul2d(A[rows], B), RTOL, ATOL, what + " rows")
        ii, jj = rng.integers(0, M, 8192), rng.integers(0, N, 8192)
        assert_close_f16(C[ii, jj], oracle.matmul2d_entries(A, B, ii, jj), RTOL, ATOL, what + " entries")
    return C


@pytest.mark.parametrize("M,N,K", [(128, 4096, 4096), (128, 4096, 11008)])
def test_hgemm_prefill_full_oracle(dev, oracle, M, N, K):
    _hgemm_case(dev, oracle, M, N, K, seed=800 + K % 13)


@pytest.mark.parametrize("M", [128, 512, 2048])
@pytest.mark.parametrize("N,K", [(4096, 4096), (11008, 4096), (32000, 4096), (4096, 11008)])
def test_hgemm_prefill_shapes_sampled(dev, oracle, M, N, K):
    """The twelve prefill shapes at full size: oracle on sampled rows and entries."""
    _hgemm_case(dev, oracle, M, N, K, seed=900 + M + N % 31, full=False)


@pytest.mark.parametrize("M", [512, 2048])
@pytest.mark.parametrize("N,K", [(4096, 4096), (11008, 4096), (32000, 4096), (4096, 11008)])
def test_hgemm_prefill_whole_matrix_against_second_gpu_path(dev, oracle, M, N, K):
    """Every entry of the large prefill products, not a sample.  The checker is the library's plain fp32 kernel
    (tl_matmul2d_f32 on the operands widened to fp32: one thread per entry, one fp32 accumulator, k ascending),
    which shares nothing with the MFMA kernels.  Products of two halves are exact in fp32, so that kernel's sum is
    the CPU loop's sum (CPU.cpp:76-89) and its fp16 rounding must equal the oracle bit for bit, which is asserted
    on eight rows.  The MFMA result may differ from it by the fp32 summation order only: the two fp32 sums differ
    by rounding noise of the partial sums (magnitude ~1, K terms: a few 1e-6, bounded here by 2e-5), which after
    the fp16 rounding is at most one fp16 ulp on top of that noise, and inside the parity gate everywhere."""
    A = synth.normal_f16(2000 + M, (M, K), 1.0)
    B = synth.normal_f16(2001 + N % 97, (N, K), 0.02)
    Ad, Bd = dev.from_numpy(A), dev.from_numpy(B)
    ref = dev.matmul2d_f32(Ad.float(), Bd.float()).half()
    rng = np.random.default_rng(M + N)
    rows = np.unique(np.concatenate([[0, M - 1], rng.integers(0, M, 6)]))
    want = oracle.matmul2d(A[rows], B)
    assert np.array_equal(ref[torch.as_tensor(rows, device=ref.device)].cpu().numpy().view(np.uint16), want.view(np.uint16)), \
        "the fp32 checker kernel does not reproduce the CPU loop"
    C = dev.hgemm(Ad, Bd)
    cf, rf = C.float(), ref.float()
    err = (cf - rf).abs()
    # spacing of fp16 at the larger of the two magnitudes (2^-24 below the smallest normal): x = m * 2^e with
    # m in [0.5, 1) has spacing 2^(e - 11)
    _, e = torch.frexp(torch.maximum(cf.abs(), rf.abs()).clamp_min(2.0 ** -14))
    ulp = torch.pow(2.0, (e - 11).float())
    assert bool((err <= ulp + 2e-5).all()), f"{int((err > ulp + 2e-5).sum())} entries differ by more than one fp16 ulp"
    assert bool((err <= ATOL + RTOL * rf.abs()).all()), "whole-matrix parity gate"
    assert float((err > 0).float().mean()) < 0.2, "an unexpected share of entries rounds differently"


@pytest.mark.parametrize("M,N,K", [(2048, 8328, 128), (1100, 16520, 64), (2048, 8192 + 8, 192)])
def test_hgemm_column_range_split_launches(dev, oracle, M, N, K):
    """Shapes whose 256x256 tiles fill whole rounds of the chip plus a nearly empty one are issued as two launches
    over two column ranges of C (row stride N in both): every entry is written, matches the plain fp32 kernel inside
    the parity gate, and whole rows (which cross the seam) match the oracle."""
    A = synth.normal_f16(2100 + M, (M, K), 1.0)
    B = synth.normal_f16(2101 + N % 89, (N, K), 0.05)
    Ad, Bd = dev.from_numpy(A), dev.from_numpy(B)
    ref = dev.matmul2d_f32(Ad.float(), Bd.float()).half()
    C = dev.empty(M, N)
    C.fill_(float("nan"))
    dev.hgemm(Ad, Bd, C)
    assert not bool(torch.isnan(C).any()), "entries left unwritten"
    rows = np.array([0, 255, 256, M - 1])
    assert_close_f16(C.cpu().numpy()[rows], oracle.matmul2d(A[rows], B), RTOL, ATOL, "rows against the oracle")
    err = (C.float() - ref.float()).abs()
    assert bool((err <= ATOL + RTOL * ref.float().abs()).all())
    assert float((err > 0).float().mean()) < 0.2


def test_hgemm_every_variant_ragged(dev, oracle):
    names = dev.hgemm_variants()
    for v in range(1, len(names)):
        for (M, N, K) in [(300, 500, 264), (2, 3, 8), (129, 257, 72), (64, 64, 64), (257, 130, 1000), (300, 517, 256),
                          (1, 9, 64), (513, 255, 128), (260, 1030, 192)]:
            _hgemm_case(dev, oracle, M, N, K, seed=1000 + v, variant=v, b_std=0.1)


@pytest.mark.parametrize("M,N,K", [(2, 2, 1), (5, 7, 3), (33, 65, 127), (17, 100, 1001), (300, 2, 9)])
def test_hgemm_unaligned_k(dev, oracle, M, N, K):
    _hgemm_case(dev, oracle, M, N, K, seed=1100 + K, b_std=0.1)


def test_hgemm_rows_longer_than_the_ring_kernels_address(dev, oracle):
    """The direct-to-LDS kernels address a tile's rows with 32-bit byte offsets, good for K up to 2^22; a longer
    K (still a multiple of 64) must be routed to the register-staged kernel and come out right."""
    M, N, K = 4, 16, (1 << 22) + 64
    A = synth.normal_f16(1190, (M, K), 0.05)
    B = synth.normal_f16(1191, (N, K), 0.05)
    C = dev.hgemm(dev.from_numpy(A), dev.from_numpy(B)).cpu().numpy()
    assert_close_f16(C, oracle.matmul2d(A, B), RTOL, ATOL, "hgemm K = 2^22 + 64")


def test_hgemm_integer_inputs_bit_exact(dev, oracle):
    M, N, K = 256, 384, 512
    A = synth.small_ints_f16(1200, (M, K), -2, 2)
    B = synth.small_ints_f16(1201, (N, K), -2, 2)
    C = dev.hgemm(dev.from_numpy(A), dev.from_numpy(B)).cpu().numpy()
    want = oracle.matmul2d(A, B)
    assert np.array_equal(C.view(np.uint16), want.view(np.uint16))
    ref = (A.astype(np.float64) @ B.astype(np.float64).T)
    assert np.array_equal(C.astype(np.float64), ref)


def test_matmul2d_drawn_shapes_integer_exact(dev):
    """Sixty shapes drawn with a fixed seed from the edges of every dispatch rule (M = 1 and few rows, N and K around
    the tile sizes, multiples of 8 and 64 and odd values) through the boundary entry; small-integer inputs make every
    sum exact in fp32 and in fp16, so a wrong index, a skipped tail or a stale tile shows as a wrong value.  The
    expected values come from float64 on the host."""
    import random
    rnd = random.Random(20240611)
    Ms = [1, 2, 3, 15, 16, 17, 31, 33, 64, 100, 128, 129, 255, 256, 300, 512, lambda: rnd.randint(1, 700)]
    Ns = [1, 7, 8, 16, 48, 63, 64, 65, 128, 200, 256, 320, 1000, 1024, lambda: rnd.randint(1, 3000), lambda: 8 * rnd.randint(1, 400)]
    Ks = [1, 7, 8, 24, 64, 72, 128, 192, 256, 320, 512, 1000, 1024, lambda: rnd.randint(1, 3000), lambda: 8 * rnd.randint(1, 300),
          lambda: 64 * rnd.randint(1, 60)]
    pick = lambda xs: (lambda c: c() if callable(c) else c)(rnd.choice(xs))
    for i in range(60):
        M, N, K = pick(Ms), pick(Ns), pick(Ks)
        A = synth.small_ints_f16(7000 + 2 * i, (M, K), -2, 2)
        B = synth.small_ints_f16(7001 + 2 * i, (N, K), -2, 2)
        C = torch.full((M, N), 5.0, device="cuda", dtype=torch.float16)
        dev.matmul2d(dev.from_numpy(A), dev.from_numpy(B), C)
        want = A.astype(np.float64) @ B.astype(np.float64).T
        assert np.abs(want).max() <= 2048, (M, N, K)           # every sum is an fp16 integer
        assert np.array_equal(C.cpu().numpy().astype(np.float64), want), (i, M, N, K)


FEW_ROWS_SHAPES = [(2, 16, 2048), (3, 48, 2304), (15, 4096, 4096), (16, 4112, 4096), (17, 1008, 3072), (31, 4096, 4096),
                   (32, 11008, 4096), (8, 12288, 4096), (5, 32000, 4096), (32, 16384, 2560), (9, 272, 3840)]


@pytest.mark.parametrize("shape", FEW_ROWS_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_hgemm_few_rows_kernel(dev, oracle, shape):
    """2 <= M <= 32 with K in 2048..4096 goes to the kernel that keeps X in registers and streams W once: every block
    count per workgroup (fewer blocks than CUs, uneven shares), every row count around its 16-row groups, wavefronts
    with 1 to 4 pieces of K.  Small integers are exact whatever the order of summation; random data is checked
    against the oracle (all rows; sampled columns when W is large) and against the tile kernels."""
    M, N, K = shape
    A = synth.small_ints_f16(7300 + M, (M, K), -2, 2)
    B = synth.small_ints_f16(7301 + N, (N, K), -2, 2)
    C = torch.full((M, N), 5.0, device="cuda", dtype=torch.float16)
    dev.hgemm(dev.from_numpy(A), dev.from_numpy(B), C)
    want = A.astype(np.float64) @ B.astype(np.float64).T
    assert np.abs(want).max() <= 2048
    assert np.array_equal(C.cpu().numpy().astype(np.float64), want)

    A = synth.normal_f16(7310 + M, (M, K), 1.0)
    B = synth.normal_f16(7311 + N, (N, K), 0.02)
    Ad, Bd = dev.from_numpy(A), dev.from_numpy(B)
    got = dev.hgemm(Ad, Bd).cpu().numpy()
    cols = np.arange(N) if N * K <= (1 << 24) else np.unique(np.random.default_rng(N).integers(0, N, 512))
    ref = oracle.matmul2d(A, np.ascontiguousarray(B[cols]))
    assert_close_f16(got[:, cols], ref, RTOL, ATOL, f"few-rows hgemm {shape}")
    try:
        dev.lib.tl_set_hgemm_fewrows(-1)
        tiles = dev.hgemm(Ad, Bd).cpu().numpy()
    finally:
        dev.lib.tl_set_hgemm_fewrows(0)
    assert_close_f16(got, tiles, RTOL, ATOL, f"few-rows hgemm vs tile kernels {shape}")


def test_hgemm_few_rows_kernel_leaves_the_rest_of_c_alone(dev):
    """The kernel stores 8-byte pieces of rows below M only: a C with more rows than M keeps them."""
    M, N, K = 13, 4096, 4096
    A = synth.small_ints_f16(7400, (M, K), -2, 2)
    B = synth.small_ints_f16(7401, (N, K), -2, 2)
    C = torch.full((M + 3, N), 5.0, device="cuda", dtype=torch.float16)
    dev.hgemm(dev.from_numpy(A), dev.from_numpy(B), C[:M])
    want = A.astype(np.float64) @ B.astype(np.float64).T
    out = C.cpu().numpy().astype(np.float64)
    assert np.array_equal(out[:M], want)
    assert np.all(out[M:] == 5.0)


@pytest.mark.parametrize("shape", [(640, 512, 8192), (576, 1280, 11008), (384, 1024, 8192), (256, 768, 11008),
                                   (192, 5120, 5120), (64, 8192, 4096)],
                         ids=lambda s: "x".join(map(str, s)))
def test_hgemm_long_k_is_split_over_wide_tiles(dev, shape):
    """Few tiles and a long K: the dispatch keeps wide tiles and splits K over workgroups (fp32 slabs, ordered second
    pass), also above 512 rows.  Small integers are exact whatever the split; the fused projection + add + RMSNorm entry
    consumes the same slabs and must give the bits of the two-step path."""
    M, N, K = shape
    A = synth.small_ints_f16(7500 + M, (M, K), -2, 2)
    B = synth.small_ints_f16(7501 + N, (N, K), -1, 1)
    Ad, Bd = dev.from_numpy(A), dev.from_numpy(B)
    C = dev.hgemm(Ad, Bd).cpu().numpy()
    want = A.astype(np.float64) @ B.astype(np.float64).T
    assert np.abs(want).max() <= 2048
    assert np.array_equal(C.astype(np.float64), want)

    A = synth.normal_f16(7510 + M, (M, K), 1.0)
    B = synth.normal_f16(7511 + N, (N, K), 0.02)
    R = synth.normal_f16(7512 + M, (M, N), 1.0)
    g = synth.normal_f16(7513 + N, (N,), 1.0)
    Ad, Bd, Rd, gd = (dev.from_numpy(x) for x in (A, B, R, g))
    s1, n1 = dev.hgemm_add_rms_norm(Ad, Bd, Rd, gd, 1e-5)
    P = dev.hgemm(Ad, Bd)
    s2, n2 = dev.add_rms_norm(P, Rd, gd, 1e-5)
    # the fused entry sums the slabs in fp32 and adds the residual before the one rounding of the sum, the two-step
    # path rounds the product first: they agree to an ulp of the sum, and the plain product must match float64
    ref = A.astype(np.float64) @ B.astype(np.float64).T
    assert_close_f16(P.cpu().numpy(), ref.astype(np.float16), RTOL, ATOL, f"split long-K hgemm {shape}")
    assert_close_f16(s1.cpu().numpy(), (ref + R.astype(np.float64)).astype(np.float16), RTOL, ATOL, f"fused sum {shape}")
    assert_close_f16(s1.cpu().numpy(), s2.cpu().numpy(), RTOL, 2e-3, f"fused vs two-step sum {shape}")


SQUARE_TILE_PLANS = [
    # (M, N, K), expected (variant, splits)
    ((256, 8192, 8192), ("p128x128x64w2x2s4", 2)),
    ((192, 5120, 5120), ("p128x128x64w2x2s4", 3)),
    ((48, 12288, 4096), ("p128x128x64w2x2s4", 2)),
    ((512, 8192, 2048), ("p128x128x64w2x2s4", 1)),
    ((384, 6144, 4096), ("p128x128x64w2x2s4", 1)),   # two rounds of 128x64 tiles avoided
    ((512, 8192, 16384), ("p128x256x64w2x4s3", 2)),  # very long K: wide tiles on two splits, not 128x192 unsplit
    ((48, 4096, 4096), ("p128x64x64w4x1s4", 4)),     # fewer than 5120 columns: the narrow-tile rule stays
    ((16, 4096, 4096), ("fewrows", 1)),
]


@pytest.mark.parametrize("shape,plan", SQUARE_TILE_PLANS, ids=lambda v: "x".join(map(str, v)) if isinstance(v[0], int) else None)
def test_hgemm_square_tiles_fill_one_round(dev, shape, plan):
    """Up to 512 rows and from 5120 columns on, 128x128 tiles are split over K until one round of them fills the chip.
    The plan the dispatch took is read back through tl_hgemm_last_plan; small integers are exact whatever the plan."""
    M, N, K = shape
    A = synth.small_ints_f16(7600 + M, (M, K), -2, 2)
    B = synth.small_ints_f16(7601 + N, (N, K), -1, 1)
    Ad, Bd = dev.from_numpy(A), dev.from_numpy(B)
    C = dev.hgemm(Ad, Bd)
    assert dev.hgemm_last_plan() == plan
    want = torch.from_numpy(A).cuda().double() @ torch.from_numpy(B).cuda().double().T
    assert float(want.abs().max()) <= 2048
    assert torch.equal(C.double(), want)


@pytest.mark.parametrize("shape", [(130, 5130, 4096), (257, 7000, 4160), (64, 8200, 8192), (500, 8100, 4096)],
                         ids=lambda s: "x".join(map(str, s)))
def test_hgemm_square_tiles_ragged_edges_and_batches(dev, shape):
    """The same rule on shapes whose last tiles are partly filled, and as a batch of two (no split of K there: the
    second pass of a split writes a dense single C)."""
    M, N, K = shape
    A = synth.small_ints_f16(7700 + M, (2, M, K), -2, 2)
    B = synth.small_ints_f16(7701 + N, (N, K), -1, 1)
    Ad, Bd = dev.from_numpy(A), dev.from_numpy(B)
    want = torch.from_numpy(A).cuda().double() @ torch.from_numpy(B).cuda().double().T
    assert float(want.abs().max()) <= 2048
    C = dev.hgemm(Ad[0].contiguous(), Bd)
    assert dev.hgemm_last_plan()[0] == "p128x128x64w2x2s4"
    assert torch.equal(C.double(), want[0])
    Cb = dev.matmul(Ad, Bd.t())
    assert dev.hgemm_last_plan()[1] == 1
    assert torch.equal(Cb.double(), want)


GATED_SHAPES = [(128, 11008, 4096), (512, 11008, 4096), (2048, 11008, 4096), (48, 11008, 4096), (16, 11008, 4096),
                (200, 1000, 4160), (130, 5128, 4096), (700, 6000, 2048), (1, 11008, 4096), (64, 1376, 4100),
                (300, 72, 128), (3000, 2752, 1024)]


@pytest.mark.parametrize("shape", GATED_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_hgemm_silu_mul_equals_two_steps(dev, shape):
    """The two FFN projections with the SwiGLU gate in the GEMM's epilogue against GEMM into a [M, 2*hidden] buffer
    followed by the gate kernel: the gate sees the same fp16-rounded projections, so every bit agrees.  Shapes: the
    Llama2-7B w1|w3 at several prompt lengths, hidden not a multiple of any tile, rows past the last tile, K with a tail
    (two-step path inside the entry), one row (GEMV), a handful of rows (two-step by choice)."""
    M, hidden, K = shape
    X = dev.from_numpy(synth.normal_f16(7800 + M, (M, K), 1.0))
    W13 = dev.from_numpy(synth.normal_f16(7801 + hidden, (2 * hidden, K), 0.02))
    try:
        # every workgroup walks all of K from its first tile: both paths then add the same products in the same order
        dev.lib.tl_set_hgemm_k_rotation(0, 0)
        dev.lib.tl_set_hgemm_splits(1)
        want = dev.silu_mul_rows(dev.matmul2d(X, W13))
        got = dev.hgemm_silu_mul(X, W13)
        assert got.shape == (M, hidden)
        assert torch.equal(got, want)
    finally:
        dev.lib.tl_set_hgemm_k_rotation(-1, -1)
        dev.lib.tl_set_hgemm_splits(0)
    # with the rotated walks of the default dispatch (the order of the fp32 sums then differs from tile to tile):
    # against float64 of the defining formula, to the tolerance of the GEMM
    got = dev.hgemm_silu_mul(X, W13)
    a = X.double() @ W13[:hidden].double().T
    b = X.double() @ W13[hidden:].double().T
    ref = (a.half().double() / (1.0 + torch.exp(-a.half().double())) * b.half().double())
    assert_close_f16(got.cpu().numpy(), ref.cpu().numpy().astype(np.float16), RTOL, ATOL, f"gated {shape}")


@pytest.mark.parametrize("M", [128, 512, 2048])
def test_hgemm_silu_mul_against_the_oracle(dev, oracle, M):
    """The gated w1|w3 projection against the CPU restatement directly, on eight sampled rows at the Llama2-7B size:
    oracle.silu_mul(oracle.matmul2d(X, W1), oracle.matmul2d(X, W3)) at the gate of the single kernels."""
    hidden, K = 11008, 4096
    X = synth.normal_f16(7850 + M, (M, K), 1.0)
    W13 = synth.normal_f16(7851, (2 * hidden, K), 0.02)
    got = dev.hgemm_silu_mul(dev.from_numpy(X), dev.from_numpy(W13)).cpu().numpy()
    if M >= 512:   # whole 256-row tiles: the gated build of the AGPR kernel serves (at least the last columns of) these
        assert dev.hgemm_last_plan()[0] == "a256x256x64w2x2"
    rng = np.random.default_rng(M)
    rows = np.unique(np.concatenate([[0, M - 1], rng.integers(0, M, 6)]))
    want = oracle.silu_mul(oracle.matmul2d(X[rows], W13[:hidden]), oracle.matmul2d(X[rows], W13[hidden:]))
    assert_close_f16(got[rows], want, RTOL, ATOL, f"gated {M}x{hidden}x{K} against the oracle")


def test_hgemm_silu_mul_drawn_shapes(dev):
    """Forty drawn shapes (rows 2..700, hidden a multiple of 8 up to 3000, K a multiple of 64 up to 2048) through the
    automatic dispatch: tiles partly filled in both directions, column ranges, every tile shape the dispatch reaches."""
    rng = np.random.default_rng(20240611)
    seen = set()
    try:
        dev.lib.tl_set_hgemm_k_rotation(0, 0)
        dev.lib.tl_set_hgemm_splits(1)
        for i in range(40):
            M = int(rng.integers(2, 701))
            hidden = 8 * int(rng.integers(1, 376))
            K = 64 * int(rng.integers(1, 33))
            X = dev.from_numpy(synth.normal_f16(7900 + i, (M, K), 1.0))
            W13 = dev.from_numpy(synth.normal_f16(8000 + i, (2 * hidden, K), 0.05))
            want = dev.silu_mul_rows(dev.matmul2d(X, W13))
            got = dev.hgemm_silu_mul(X, W13)
            seen.add(dev.hgemm_last_plan()[0])
            assert torch.equal(got, want), (M, hidden, K, dev.hgemm_last_plan())
    finally:
        dev.lib.tl_set_hgemm_k_rotation(-1, -1)
        dev.lib.tl_set_hgemm_splits(0)
    assert len(seen) >= 2, seen


def test_hgemm_silu_mul_every_pipelined_variant(dev):
    """Each pipelined tile shape has a gated build of its own (the pairing of rows follows the wavefront tile): all of
    them against the two-step path, on a shape with partly filled last tiles in both directions."""
    M, hidden, K = 300, 1096, 512
    X = dev.from_numpy(synth.normal_f16(7810, (M, K), 1.0))
    W13 = dev.from_numpy(synth.normal_f16(7811, (2 * hidden, K), 0.05))
    names = dev.hgemm_variants()
    tried = 0
    try:
        dev.lib.tl_set_hgemm_k_rotation(0, 0)   # same order of the fp32 sums on both paths
        dev.lib.tl_set_hgemm_splits(1)
        want = dev.silu_mul_rows(dev.matmul2d(X, W13))
        for i, name in enumerate(names):
            if not name.startswith("p"):
                continue
            dev.set_hgemm_variant(i)
            got = dev.hgemm_silu_mul(X, W13)
            assert dev.hgemm_last_plan() == (name, 1), name
            assert torch.equal(got, want), name
            tried += 1
    finally:
        dev.set_hgemm_variant(0)
        dev.lib.tl_set_hgemm_k_rotation(-1, -1)
        dev.lib.tl_set_hgemm_splits(0)
    assert tried >= 10


def test_hgemm_k_rotation_and_splits_visit_every_k_tile_once(dev, oracle):
    """Workgroups start their walk over K at a rotated tile and wrap, per split: with small-integer data the
    result is exact whatever the order, so a skipped or repeated K tile shows as a wrong bit."""
    names = dev.hgemm_variants()
    try:
        for (M, N, K) in [(128, 640, 448), (300, 1100, 704), (512, 2112, 1024)]:
            A = synth.small_ints_f16(1250 + K, (M, K), -2, 2)
            B = synth.small_ints_f16(1251 + K, (N, K), -2, 2)
            want = oracle.matmul2d(A, B).view(np.uint16)
            Ad, Bd = dev.from_numpy(A), dev.from_numpy(B)
            for name in ("auto", "p256x256x64w2x4s2", "p128x128x64w2x4s4", "p128x64x64w4x1s4"):
                dev.set_hgemm_variant(names.index(name))
                for splits in (0, 1, 3):
                    dev.lib.tl_set_hgemm_splits(splits)
                    for rot in ((-1, -1), (0, 0), (1, 0), (5, 3), (0, 2), (1000003, 17)):
                        dev.lib.tl_set_hgemm_k_rotation(*rot)
                        C = dev.hgemm(Ad, Bd).cpu().numpy()
                        assert np.array_equal(C.view(np.uint16), want), (M, N, K, name, splits, rot)
    finally:
        dev.set_hgemm_variant(0)
        dev.lib.tl_set_hgemm_splits(0)
        dev.lib.tl_set_hgemm_k_rotation(-1, -1)


def test_hgemm_tile_bands_cover_every_tile_once(dev):
    """Tiles are numbered band by band (a band = a few rows of tiles over all columns); whatever the band height,
    and with a last band that is lower than the others, the numbering must reach every tile.  A carries a row
    block pattern, B a column block pattern, K = 64: C[i, j] then names its tile, so a tile computed from the
    wrong panels shows, and a C poisoned beforehand shows a tile that nobody wrote."""
    names = dev.hgemm_variants()
    try:
        for (M, N, name) in [(9 * 256 + 40, 5 * 256 + 8, "p256x256x64w2x4s2"), (19 * 128, 3 * 256, "p128x256x64w2x4s3"),
                             (11 * 128 + 1, 7 * 128, "t128x128x64w2x2"), (4096 + 256, 2048, "auto")]:
            A = np.zeros((M, 64), np.float16)
            B = np.zeros((N, 64), np.float16)
            A[:, 0] = (np.arange(M) // 128) % 64
            A[:, 1] = 1
            B[:, 0] = 1
            B[:, 1] = (np.arange(N) // 128) % 64
            want = (A[:, :1].astype(np.float32) + B[:, 1].astype(np.float32)[None, :]).astype(np.float16)
            Ad, Bd = dev.from_numpy(A), dev.from_numpy(B)
            dev.set_hgemm_variant(names.index(name))
            for band in (0, 1, 3, 4, 8, 1000):
                dev.lib.tl_set_hgemm_tile_band(band)
                C = torch.full((M, N), -7.0, dtype=torch.float16, device=Ad.device)
                dev.hgemm(Ad, Bd, C)
                assert np.array_equal(C.cpu().numpy().view(np.uint16), want.view(np.uint16)), (M, N, name, band)
    finally:
        dev.set_hgemm_variant(0)
        dev.lib.tl_set_hgemm_tile_band(0)


def test_hgemm_identity(dev):
    """B = I returns A; A = I returns B^T (catches a transposed operand or tile mapping)."""
    n = 320
    A = synth.normal_f16(1300, (200, n), 1.0)
    eye = np.eye(n, dtype=np.float16)
    C = dev.hgemm(dev.from_numpy(A), dev.from_numpy(eye)).cpu().numpy()
    assert np.array_equal(C.view(np.uint16), A.view(np.uint16))
    B = synth.normal_f16(1301, (136, n), 1.0)
    C2 = dev.hgemm(dev.from_numpy(eye), dev.from_numpy(B)).cpu().numpy()
    assert np.array_equal(C2.view(np.uint16), np.ascontiguousarray(B.T).view(np.uint16))


# ------------------------------------------------------- batched / Tensor::matmul plumbing ----

def test_batched_attention_shapes(dev, oracle):
    """The per-head loops of Attention::forward as one batched call: decode (M=1) and prefill."""
    H, T, D = 32, 200, 128
    for S in (1, 40):
        q = synth.normal_f16(1400, (H, S, D), 1.0)
        keys = synth.normal_f16(1401, (H, T, D), 1.0)
        sc = dev.matmul(dev.from_numpy(q), dev.from_numpy(keys).transpose(1, 2)).cpu().numpy()
        want = oracle.matmul2d_batched(q, keys, H, S, T, D, S * D, T * D)
        assert_close_f16(sc, want, RTOL, ATOL, f"scores S={S}")
        p = synth.normal_f16(1402, (H, S, T), 0.1)
        vals_c = synth.normal_f16(1403, (H, D, T), 1.0)  # values_c layout: [H, D, T]
        o = dev.matmul(dev.from_numpy(p), dev.from_numpy(vals_c).transpose(1, 2)).cpu().numpy()
        want = oracle.matmul2d_batched(p, vals_c, H, S, D, T, S * T, D * T)
        assert_close_f16(o, want, RTOL, ATOL, f"p.v S={S}")


def test_matmul_broadcast_semantics(dev):
    """Tensor::matmul batch broadcasting must agree with np.matmul (the reference's own
    test_batched_matmul, tensorLib/test/python/test_tensor.py:103-121, on fp16 data)."""
    rng = np.random.default_rng(7)
    cases = [((3, 4, 5), (5, 6)), ((2, 1, 4, 8), (3, 8, 5)), ((4, 8), (2, 3, 8, 2)), ((2, 3, 7, 16), (2, 3, 16, 9)),
             ((5, 1, 3, 4), (1, 6, 4, 2))]
    for sa, sb in cases:
        a = rng.integers(-3, 4, sa).astype(np.float16)
        b = rng.integers(-3, 4, sb).astype(np.float16)
        got = dev.matmul(dev.from_numpy(a), dev.from_numpy(b)).cpu().numpy()
        want = np.matmul(a.astype(np.float32), b.astype(np.float32))
        assert got.shape == want.shape
        assert np.array_equal(got.astype(np.float32), want), (sa, sb)


def test_matmul_error_behaviour(dev):
    a = dev.empty(4, 5)
    with pytest.raises(ValueError):
        dev.matmul(a, dev.empty(6, 3))
    with pytest.raises(ValueError):
        dev.matmul(dev.empty(5), dev.empty(5, 2))
    with pytest.raises(ValueError):
        dev.matmul(dev.empty(2, 4, 5), dev.empty(3, 5, 2))
    with pytest.raises(ValueError):
        dev.matmul(a, dev.empty(5, 3), out=dev.empty(4, 4))


def test_matmul2d_degenerate_sizes(dev):
    """M == 0 or N == 0: nothing to write; K == 0: the empty sum, i.e. zeros (CPU<half>::matmul2d's loop over k does
    not run, tensorLib/src/device/cpu/CPU.cpp:76-89) -- for the GEMV (M == 1) and the GEMM path alike."""
    import ctypes
    A = torch.ones(8, 16, dtype=torch.float16, device="cuda")
    B = torch.ones(24, 16, dtype=torch.float16, device="cuda")
    vp = lambda t: ctypes.c_void_p(t.data_ptr())
    for (M, N) in [(0, 24), (8, 0), (0, 0), (1, 0)]:
        C = torch.full((8, 24), -7.0, dtype=torch.float16, device="cuda")
        assert dev.lib.tl_matmul2d_f16(vp(A), vp(B), vp(C), M, N, 16) == 0
        torch.cuda.synchronize()
        assert bool((C == -7.0).all()), (M, N)
    for M in (1, 8):
        C = torch.full((M, 24), -7.0, dtype=torch.float16, device="cuda")
        assert dev.lib.tl_matmul2d_f16(vp(A), vp(B), vp(C), M, 24, 0) == 0
        torch.cuda.synchronize()
        assert bool((C == 0).all()), M


def test_matmul2d_f32(dev, oracle):
    rng = np.random.default_rng(11)
    for (M, N, K) in [(1, 1, 1), (17, 33, 65), (128, 100, 300)]:
        A = rng.standard_normal((M, K)).astype(np.float32)
        B = rng.standard_normal((N, K)).astype(np.float32)
        C = dev.matmul2d_f32(dev.from_numpy(A), dev.from_numpy(B)).cpu().numpy()
        np.testing.assert_allclose(C, oracle.matmul2d_f32(A, B), rtol=1e-4, atol=1e-4)


def test_linearity_at_full_size(dev):
    """Size-independent property at the largest decode shape: W.(x1 + x2) == W.x1 + W.x2 for
    integer-valued operands (exact in fp32)."""
    N, K = 32000, 4096
    W = synth.small_ints_f16(1500, (N, K), -2, 2)
    x1 = synth.small_ints_f16(1501, (K,), -1, 1)
    x2 = synth.small_ints_f16(1502, (K,), -1, 1)
    Wd = dev.from_numpy(W)
    y1 = dev.gemv(dev.from_numpy(x1), Wd).float()
    y2 = dev.gemv(dev.from_numpy(x2), Wd).float()
    y12 = dev.gemv(dev.from_numpy((x1 + x2).astype(np.float16)), Wd).float()
    assert torch.equal(y12, y1 + y2)


def test_split_k_workspace_shared_by_two_host_threads(dev):
    """Two host threads issue split-K GEMMs of growing size at the same time (the reference's Embedding::forward
    enters the backend from an OpenMP loop, tensorLib/src/nn/embedding.cpp:66-78).  Both use the one library-owned
    fp32 workspace, which has to grow several times meanwhile: a call keeps the buffer locked until its kernels are
    enqueued, so no thread can free it under another thread's queued kernel.  Every result is compared with the
    single-threaded one."""
    import threading
    K = 4096
    sizes = [(128, 1024), (96, 4096), (128, 8192), (128, 16384), (70, 2048), (128, 24576)]
    jobs = []
    dev.lib.tl_set_hgemm_splits(4)
    try:
        for i, (M, N) in enumerate(sizes):
            A = dev.from_numpy(synth.normal_f16(2300 + i, (M, K), 1.0))
            B = dev.from_numpy(synth.normal_f16(2400 + i, (N, K), 0.02))
            jobs.append((A, B, dev.hgemm(A, B).clone()))
    finally:
        dev.lib.tl_set_hgemm_splits(0)
    dev.synchronize()
    errors = []

    def worker(order):
        try:
            for _ in range(3):
                for j in order:
                    A, B, want = jobs[j]
                    C = dev.hgemm(A, B)
                    dev.synchronize()
                    if not torch.equal(C, want):
                        errors.append(f"job {j} differs")
        except Exception as e:   # noqa: BLE001
            errors.append(repr(e))

    dev.lib.tl_set_hgemm_splits(4)
    try:
        ts = [threading.Thread(target=worker, args=(o,)) for o in ([0, 1, 2, 3, 4, 5], [5, 3, 1, 4, 2, 0])]
        for t in ts:
            t.start()
        for t in ts:
            t.join()
    finally:
        dev.lib.tl_set_hgemm_splits(0)
    assert not errors, errors[:3]


# ---------------------------------------------------------------- split-K in one launch ----

SPLIT_IN_LAUNCH_CASES = [
    # (M, N, K), forced variant (None = dispatch), forced splits (0 = dispatch)
    ((128, 4096, 4096), None, 0),
    ((128, 4096, 11008), None, 0),
    ((512, 4096, 4096), None, 2),                  # the dispatch covers this one with 256 unsplit tiles
    ((512, 4096, 11008), None, 0),
    ((128, 11008, 4096), None, 0),
    ((130, 5128, 4096), None, 0),                  # partly filled last tiles in both directions
    ((64, 8200, 8192), None, 0),
    ((100, 1000, 1024), "p128x64x64w4x1s4", 3),    # splits that do not divide the K tiles evenly
    ((300, 1096, 1472), "p128x128x64w2x4s4", 5),
    ((512, 16640, 1024), "p128x256x64w2x4s3", 2),  # persistent kernel: 260 tiles on 256 workgroups, every tile ticketed
    ((512, 16640, 512), "p256x128x64w2x4s3", 2),
    ((256, 2048, 2048), "p128x128x64w2x2s4", 16),
]


@pytest.mark.parametrize("shape,variant,splits", SPLIT_IN_LAUNCH_CASES,
                         ids=lambda v: "x".join(map(str, v)) if isinstance(v, tuple) else str(v))
def test_hgemm_split_k_merged_inside_the_launch_equals_second_kernel(dev, oracle, shape, variant, splits):
    """The workgroup that finishes a C tile's last split adds the fp32 slabs in split order and writes fp16 C itself
    (per-tile tickets, device-coherent slabs; opt-in, the ordered second kernel is the faster default).  Same order, same
    rounding: the two must agree bit for bit on random data, on every call of a sequence (the tickets return to
    zero), and both must sit inside the gate against the oracle on sampled rows."""
    M, N, K = shape
    A = synth.normal_f16(8800 + M, (M, K), 1.0)
    B = synth.normal_f16(8801 + N % 97, (N, K), 0.02)
    Ad, Bd = dev.from_numpy(A), dev.from_numpy(B)
    names = dev.hgemm_variants()
    try:
        if variant:
            dev.set_hgemm_variant(names.index(variant))
        dev.lib.tl_set_hgemm_splits(splits)
        dev.lib.tl_set_hgemm_splitk_merge(2)
        want = dev.hgemm(Ad, Bd).clone()
        plan2 = dev.hgemm_last_plan()
        assert dev.lib.tl_hgemm_last_split_in_launch() == 0
        dev.lib.tl_set_hgemm_splitk_merge(1)
        for rep in range(3):
            got = dev.hgemm(Ad, Bd)
            assert dev.hgemm_last_plan() == plan2
            assert plan2[1] > 1, f"{shape}: the case is meant to split K, plan {plan2}"
            assert dev.lib.tl_hgemm_last_split_in_launch() == 1
            assert torch.equal(got, want), f"{shape} {plan2} call {rep}"
        # a smaller problem right behind it reuses the same tickets and slabs
        got2 = dev.hgemm(Ad[: max(2, M // 2)], Bd)
        dev.lib.tl_set_hgemm_splitk_merge(2)
        assert torch.equal(got2, dev.hgemm(Ad[: max(2, M // 2)], Bd))
    finally:
        dev.set_hgemm_variant(0)
        dev.lib.tl_set_hgemm_splits(0)
        dev.lib.tl_set_hgemm_splitk_merge(0)
    rng = np.random.default_rng(M + N)
    rows = np.unique(np.concatenate([[0, M - 1], rng.integers(0, M, 6)]))
    assert_close_f16(want.cpu().numpy()[rows], oracle.matmul2d(A[rows], B), RTOL, ATOL, f"split-K {shape}")


def test_hgemm_split_k_in_launch_integer_exact_and_reset(dev):
    """Small integers are exact whatever the split; tl_reset_scratch() between calls leaves the tickets usable."""
    for (M, N, K) in [(128, 4096, 4096), (96, 2048, 8192), (256, 4096, 11008)]:
        A = synth.small_ints_f16(8900 + M, (M, K), -2, 2)
        B = synth.small_ints_f16(8901 + N, (N, K), -1, 1)
        Ad, Bd = dev.from_numpy(A), dev.from_numpy(B)
        want = torch.from_numpy(A).cuda().double() @ torch.from_numpy(B).cuda().double().T
        assert float(want.abs().max()) <= 2048
        try:
            dev.lib.tl_set_hgemm_splitk_merge(1)
            for _ in range(2):
                C = dev.hgemm(Ad, Bd)
                assert dev.lib.tl_hgemm_last_split_in_launch() == 1, dev.hgemm_last_plan()
                assert torch.equal(C.double(), want)
                assert dev.lib.tl_reset_scratch() == 0
        finally:
            dev.lib.tl_set_hgemm_splitk_merge(0)
        C = dev.hgemm(Ad, Bd)
        assert dev.lib.tl_hgemm_last_split_in_launch() == 0 and torch.equal(C.double(), want)


def test_hgemm_split_k_falls_back_to_the_second_kernel(dev):
    """C rows that cannot take 8-byte stores (N % 8 != 0) keep the second kernel also when the in-launch merge is asked
    for; the result is the same sum."""
    M, N, K = 96, 1004, 4096
    A = synth.small_ints_f16(8950, (M, K), -2, 2)
    B = synth.small_ints_f16(8951, (N, K), -1, 1)
    try:
        dev.lib.tl_set_hgemm_splits(4)
        dev.lib.tl_set_hgemm_splitk_merge(1)
        C = dev.hgemm(dev.from_numpy(A), dev.from_numpy(B))
        assert dev.hgemm_last_plan()[1] == 4 and dev.lib.tl_hgemm_last_split_in_launch() == 0
    finally:
        dev.lib.tl_set_hgemm_splits(0)
        dev.lib.tl_set_hgemm_splitk_merge(0)
    want = A.astype(np.float64) @ B.astype(np.float64).T
    assert np.array_equal(C.cpu().numpy().astype(np.float64), want)


# ------------------------------------------------------- the dispatch of the benchmark shapes ----

BASELINE_PLANS = [
    # (M, N, K), (variant of the last launch, K splits): the twelve prefill shapes and the four projections of a 16-token
    # prompt on a 256-CU MI355X
    ((2048, 4096, 4096), ("a256x128x64w2x2", 1)),
    ((2048, 11008, 4096), ("a256x128x64w2x2", 1)),   # 8192 columns of 256x256 tiles first, this is the launch for the rest
    ((2048, 32000, 4096), ("a256x256x64w2x2", 1)),
    ((2048, 4096, 11008), ("a256x128x64w2x2", 1)),
    ((512, 4096, 4096), ("p128x64x64w4x1s4", 1)),
    ((512, 11008, 4096), ("p128x192x64w4x2s4", 1)),
    ((512, 32000, 4096), ("a256x256x64w2x2", 1)),
    ((512, 4096, 11008), ("p128x256x64w2x4s3", 4)),
    ((128, 4096, 4096), ("p128x64x64w4x1s4", 4)),
    ((128, 11008, 4096), ("p128x128x64w2x2s4", 2)),
    ((128, 32000, 4096), ("p128x128x64w2x2s4", 1)),
    ((128, 4096, 11008), ("p128x64x64w4x1s4", 4)),
    ((16, 12288, 4096), ("fewrows", 1)),
    ((16, 4096, 4096), ("fewrows", 1)),
    ((16, 22016, 4096), ("fewrows", 1)),
    ((16, 4096, 11008), ("p128x64x64w4x1s4", 4)),
]


@pytest.mark.parametrize("shape,plan", BASELINE_PLANS, ids=lambda v: "x".join(map(str, v)) if isinstance(v[0], int) else None)
def test_hgemm_dispatch_of_the_benchmark_shapes_is_pinned(dev, shape, plan):
    """The kernel variant and the K split the dispatch takes for every shape bench.py reports (the plans were measured
    on a 256-CU MI355X; a retune that moves one of them has to change this table and re-measure the shape)."""
    if dev.lib.tl_device_cu_count() != 256:
        pytest.skip("plans are pinned for 256 compute units")
    M, N, K = shape
    A = dev.from_numpy(synth.small_ints_f16(9100 + M, (M, K), -1, 1))
    B = dev.from_numpy(synth.small_ints_f16(9101 + N % 89, (N, K), -1, 1))
    C = dev.hgemm(A, B)
    assert dev.hgemm_last_plan() == plan
    rows = [0, M // 2, M - 1]
    want = A[rows].double() @ B.double().T
    assert float(want.abs().max()) <= 2048 and torch.equal(C[rows].double(), want)


@pytest.mark.parametrize("shape", [(256, 256, 256), (512, 768, 384), (2048, 40960, 512), (2560, 11008, 1024), (1024, 1024, 11008)],
                         ids=lambda s: "x".join(map(str, s)))
def test_hgemm_256x256_agpr_kernel_integer_exact(dev, shape):
    """hgemm_f16_big_kernel forced on whole-tile shapes: one tile, fewer tiles than compute units, several tiles per
    workgroup (the pipeline runs on into the next C tile), K walks rotated per tile and per XCD.  Small integers are
    exact whatever the order of the fp32 sums, so a K tile skipped, repeated or taken from the wrong C tile shows as a
    wrong bit."""
    M, N, K = shape
    A = dev.from_numpy(synth.small_ints_f16(9200 + M, (M, K), -2, 2))
    B = dev.from_numpy(synth.small_ints_f16(9201 + N % 83, (N, K), -2, 2))
    want = A.double() @ B.double().T
    assert float(want.abs().max()) <= 2048
    V = dev.hgemm_variants().index("a256x256x64w2x2")
    try:
        dev.set_hgemm_variant(V)
        for rot in ((-1, -1), (0, 0), (3, 5), (1000003, 17)):
            dev.lib.tl_set_hgemm_k_rotation(*rot)
            C = dev.hgemm(A, B)
            assert dev.hgemm_last_plan() == ("a256x256x64w2x2", 1)
            assert torch.equal(C.double(), want), (shape, rot)
    finally:
        dev.set_hgemm_variant(0)
        dev.lib.tl_set_hgemm_k_rotation(-1, -1)


@pytest.mark.parametrize("shape", [(256, 128, 192), (256, 128, 256), (512, 384, 320), (2048, 4096, 448), (2560, 11008, 1024),
                                   (256, 256, 11008)], ids=lambda s: "x".join(map(str, s)))
def test_hgemm_256x128_agpr_kernel_integer_exact(dev, shape):
    """hgemm_f16_mid_kernel forced on whole-tile shapes with 3, 4, 5, 7, 16 and 172 K tiles (every remainder of the
    three-stage ring's unrolled loop), one tile, more tiles than compute units, rotated K walks: small integers are
    exact whatever the order, so a K tile skipped, repeated or read from the wrong stage shows as a wrong bit."""
    M, N, K = shape
    A = dev.from_numpy(synth.small_ints_f16(9400 + M, (M, K), -2, 2))
    B = dev.from_numpy(synth.small_ints_f16(9401 + N % 83, (N, K), -2, 2))
    want = A.double() @ B.double().T
    assert float(want.abs().max()) <= 2048
    V = dev.hgemm_variants().index("a256x128x64w2x2")
    try:
        dev.set_hgemm_variant(V)
        for rot in ((-1, -1), (0, 0), (3, 5), (1000003, 17)):
            dev.lib.tl_set_hgemm_k_rotation(*rot)
            C = dev.hgemm(A, B)
            assert dev.hgemm_last_plan() == ("a256x128x64w2x2", 1)
            assert torch.equal(C.double(), want), (shape, rot)
    finally:
        dev.set_hgemm_variant(0)
        dev.lib.tl_set_hgemm_k_rotation(-1, -1)


def test_hgemm_agpr_kernels_drawn_whole_tile_shapes(dev):
    """Twenty drawn whole-tile shapes per AGPR kernel (1 .. 6 rows of tiles, 1 .. 12 columns, 3 .. 40 K tiles), each under
    a drawn tile band (the workgroup-to-tile map) and K rotation: small integers, exact."""
    rng = np.random.default_rng(20241125)
    names = dev.hgemm_variants()
    try:
        for name, bn, k_unit, k_min in (("a256x256x64w2x2", 256, 128, 256), ("a256x128x64w2x2", 128, 64, 192)):
            dev.set_hgemm_variant(names.index(name))
            for i in range(20):
                M = 256 * int(rng.integers(1, 7))
                N = bn * int(rng.integers(1, 13))
                K = max(k_min, k_unit * int(rng.integers(1, 2560 // k_unit + 1)))
                band = int(rng.choice([0, 1, 2, 3, 5, 8]))
                rot = (int(rng.integers(0, 50)), int(rng.integers(0, 50))) if i % 2 else (-1, -1)
                A = dev.from_numpy(synth.small_ints_f16(9700 + i, (M, K), -2, 2))
                B = dev.from_numpy(synth.small_ints_f16(9800 + i, (N, K), -2, 2))
                dev.lib.tl_set_hgemm_tile_band(band)
                dev.lib.tl_set_hgemm_k_rotation(*rot)
                C = dev.hgemm(A, B)
                assert dev.hgemm_last_plan() == (name, 1), (name, M, N, K)
                assert torch.equal(C.double(), A.double() @ B.double().T), (name, M, N, K, band, rot)
    finally:
        dev.set_hgemm_variant(0)
        dev.lib.tl_set_hgemm_tile_band(0)
        dev.lib.tl_set_hgemm_k_rotation(-1, -1)


def test_hgemm_agpr_kernels_can_be_switched_off(dev):
    """tl_set_hgemm_agpr_kernels(-1) hands the shapes back to the ring kernels; both give the exact integer result."""
    A = dev.from_numpy(synth.small_ints_f16(9500, (2048, 512), -2, 2))
    B = dev.from_numpy(synth.small_ints_f16(9501, (8192, 512), -2, 2))
    want = A.double() @ B.double().T
    try:
        C = dev.hgemm(A, B)
        assert dev.hgemm_last_plan()[0].startswith("a256x") and torch.equal(C.double(), want)
        dev.lib.tl_set_hgemm_agpr_kernels(-1)
        C = dev.hgemm(A, B)
        assert dev.hgemm_last_plan()[0].startswith("p") and torch.equal(C.double(), want)
    finally:
        dev.lib.tl_set_hgemm_agpr_kernels(0)


def test_hgemm_agpr_kernels_write_time_stamps_on_request(dev):
    """tl_set_hgemm_stamps: both AGPR kernels stamp start and end of every workgroup (end after start, all within a
    second of each other), leave the result alone, write nothing when the buffer is too small or switched off."""
    names = dev.hgemm_variants()
    A = dev.from_numpy(synth.small_ints_f16(9600, (512, 512), -2, 2))
    B = dev.from_numpy(synth.small_ints_f16(9601, (1024, 512), -2, 2))
    want = A.double() @ B.double().T
    try:
        for name, wgs in (("a256x256x64w2x2", 2 * 4), ("a256x128x64w2x2", 2 * 8)):
            dev.set_hgemm_variant(names.index(name))
            stamps = torch.zeros(2 * wgs + 6, dtype=torch.int64, device="cuda")
            dev.lib.tl_set_hgemm_stamps(stamps.data_ptr(), 2 * wgs + 6)
            C = dev.hgemm(A, B)
            assert dev.hgemm_last_plan()[0] == name and torch.equal(C.double(), want)
            t = stamps.cpu().numpy()
            assert (t[:2 * wgs] != 0).all() and (t[2 * wgs:] == 0).all(), name
            t = t[:2 * wgs].reshape(wgs, 2)
            assert (t[:, 1] > t[:, 0]).all() and t.max() - t.min() < 100_000_000, name
            small = torch.zeros(2 * wgs, dtype=torch.int64, device="cuda")
            dev.lib.tl_set_hgemm_stamps(small.data_ptr(), 2 * wgs - 2)     # does not hold every workgroup: untouched
            C = dev.hgemm(A, B)
            assert torch.equal(C.double(), want) and not bool(small.any())
            dev.lib.tl_set_hgemm_stamps(None, 0)
            stamps.zero_()
            dev.hgemm(A, B)
            assert not bool(stamps.any())
    finally:
        dev.lib.tl_set_hgemm_stamps(None, 0)
        dev.set_hgemm_variant(0)


def test_hgemm_256x256_agpr_kernel_falls_back_on_partial_tiles(dev, oracle):
    """Rows or columns that do not fill whole 256x256 tiles, a K that is not an even number of tiles: the forced variant
    hands the call to the ring kernel."""
    names = dev.hgemm_variants()
    try:
        for name in ("a256x256x64w2x2", "a256x128x64w2x2"):
            dev.set_hgemm_variant(names.index(name))
            for (M, N, K) in [(300, 512, 256), (512, 520, 256), (512, 512, 160), (256, 256, 128)]:
                A = synth.small_ints_f16(9300 + M, (M, K), -2, 2)
                B = synth.small_ints_f16(9301 + N, (N, K), -2, 2)
                C = dev.hgemm(dev.from_numpy(A), dev.from_numpy(B)).cpu().numpy()
                assert dev.hgemm_last_plan()[0] != name
                assert np.array_equal(C.view(np.uint16), oracle.matmul2d(A, B).view(np.uint16)), (name, M, N, K)
    finally:
        dev.set_hgemm_variant(0)
