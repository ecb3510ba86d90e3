"""GPU parity of the small kernels around the matmuls (RMSNorm, RoPE, softmax, SiLU,
elementwise, strided copies, argmax, embedding, mask, fused decode attention) against the
CPU oracle, through the C ABI.  Floating point: rtol 1e-2 / atol 1e-3 (north_star);
copies, argmax and embedding: bit-exact."""
import numpy as np
import pytest
import torch

from tensorlib_amd import synth
from tests.conftest import assert_close_f16, assert_close_scaled, assert_rope_equal, rope_cos_sin_differences

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-2, 1e-3


@pytest.mark.parametrize("tokens,hidden", [(1, 4096), (7, 4096), (128, 1024), (3, 100), (5, 8), (2, 11008)])
def test_rms_norm(dev, oracle, tokens, hidden):
    x = synth.normal_f16(10, (tokens, hidden), 1.0)
    w = synth.normal_f16(11, (hidden,), 1.0)
    got = dev.rms_norm(dev.from_numpy(x), dev.from_numpy(w), 1e-5).cpu().numpy()
    assert_close_f16(got, oracle.rms_norm(x, w, 1e-5, "fused"), RTOL, ATOL, "rms_norm vs fused semantics")
    assert_close_f16(got, oracle.rms_norm(x, w, 1e-5, "exact"), RTOL, ATOL, "rms_norm vs float64 definition")


def test_rms_norm_in_place(dev, oracle):
    x = synth.normal_f16(12, (4, 4096), 2.0)
    w = synth.normal_f16(13, (4096,), 1.0)
    xd = dev.from_numpy(x)
    dev.rms_norm(xd, dev.from_numpy(w), 1e-5, out=xd)
    assert_close_f16(xd.cpu().numpy(), oracle.rms_norm(x, w, 1e-5, "exact"), RTOL, ATOL, "rms_norm in place")


@pytest.mark.parametrize("B,T,H,D,start", [(1, 1, 32, 128, 0), (1, 1, 32, 128, 1023), (7, 9, 32, 128, 5),
                                           (1, 512, 32, 128, 0), (2, 3, 4, 64, 2047), (1, 2, 1, 2, 3)])
def test_rope(dev, oracle, B, T, H, D, start):
    x = synth.normal_f16(20, (B, T, H, D), 1.0)
    got = dev.apply_rotary_emb(dev.from_numpy(x), start).cpu().numpy()
    # every rounding of CPU.cpp:444-453 is reproduced, so the gate is bit equality
    assert_rope_equal(got, oracle.rope(x, start), rope_cos_sin_differences(dev, oracle, start + T, D), start, "rope")
    xd = dev.from_numpy(x)
    dev.apply_rotary_emb(xd, start, out=xd)  # in place, as Attention::forward does
    assert np.array_equal(xd.cpu().numpy().view(np.uint16), got.view(np.uint16))


@pytest.mark.parametrize("rows,cols", [(32, 1), (32, 1024), (32, 1025), (3, 5), (32 * 64, 512), (1, 32000), (4, 64),
                                       (4, 65), (2, 129)])
def test_softmax(dev, oracle, rows, cols):
    x = synth.normal_f16(30, (rows, cols), 2.0)
    got = dev.softmax(dev.from_numpy(x)).cpu().numpy()
    assert_close_f16(got, oracle.softmax(x), RTOL, ATOL, "softmax")
    s = got.astype(np.float64).sum(axis=1)
    assert np.all(np.abs(s - 1.0) < 5e-3)


def test_softmax_with_mask_rows(dev, oracle):
    """-inf entries (the causal mask) give exact zeros; in-place call."""
    x = synth.normal_f16(31, (16, 40), 1.0)
    x[:, 25:] = -np.inf
    xd = dev.from_numpy(x)
    dev.softmax(xd, out=xd)
    got = xd.cpu().numpy()
    assert np.all(got[:, 25:] == 0)
    assert_close_f16(got, oracle.softmax(x), RTOL, ATOL, "masked softmax")


@pytest.mark.parametrize("n", [1, 7, 8, 11008, 11008 * 3 + 5])
def test_silu_and_silu_mul(dev, oracle, n):
    a = synth.normal_f16(40, (n,), 3.0)
    b = synth.normal_f16(41, (n,), 1.0)
    assert_close_f16(dev.silu(dev.from_numpy(a)).cpu().numpy(), oracle.silu(a), RTOL, ATOL, "silu")
    assert_close_f16(dev.silu_mul(dev.from_numpy(a), dev.from_numpy(b)).cpu().numpy(), oracle.silu_mul(a, b), RTOL, ATOL,
                     "silu_mul")


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
def test_binary_bit_exact(dev, oracle, op):
    """One IEEE operation, one rounding: must equal the oracle bit for bit."""
    for n in (1, 9, 4096, 11008 + 3):
        a = synth.normal_f16(50, (n,), 2.0)
        b = synth.normal_f16(51, (n,), 2.0)
        got = dev.binary(dev.from_numpy(a), dev.from_numpy(b), op).cpu().numpy()
        assert np.array_equal(got.view(np.uint16), oracle.binary(a, b, op).view(np.uint16)), (op, n)
        s = float(np.float16(np.sqrt(128.0)))
        got = dev.binary(dev.from_numpy(a), s, op).cpu().numpy()
        assert np.array_equal(got.view(np.uint16), oracle.binary_scalar(a, s, op).view(np.uint16)), (op, n, "scalar")


def test_binary_unaligned(dev, oracle):
    a = synth.normal_f16(52, (1000,), 1.0)
    b = synth.normal_f16(53, (1000,), 1.0)
    ad, bd = dev.from_numpy(a), dev.from_numpy(b)
    out = dev.empty(1000)
    # unaligned pointers: slices of a larger buffer
    r = dev.add(ad[1:998], bd[3:1000], out=out[1:998])
    assert np.array_equal(r.cpu().numpy().view(np.uint16), oracle.binary(a[1:998], b[3:1000], "add").view(np.uint16))


def test_contiguous_and_set_item_kv_cache_patterns(dev, oracle):
    """The strided moves of Attention::forward (Transformer.cpp:49-80): cache write at a
    position, K gather to [H,T,D], V gather to [H,D,T], q/o transposes."""
    S, H, D, T = 64, 8, 128, 37
    cache = synth.normal_f16(60, (S, H, D), 1.0)
    cd = dev.from_numpy(cache)
    # keys: cache[:T] viewed [T,H,D] -> transpose(0,1) -> contiguous [H,T,D]
    got = dev.contiguous(cd, (H, T, D), (D, H * D, 1), 0).cpu().numpy()
    assert np.array_equal(got.view(np.uint16), np.ascontiguousarray(cache[:T].transpose(1, 0, 2)).view(np.uint16))
    assert np.array_equal(got.view(np.uint16), oracle.contiguous(cache, (H, T, D), (D, H * D, 1), 0).view(np.uint16))
    # values: -> [H,D,T] (last dim strided: scalar path)
    got = dev.contiguous(cd, (H, D, T), (D, 1, H * D), 0).cpu().numpy()
    assert np.array_equal(got.view(np.uint16), np.ascontiguousarray(cache[:T].transpose(1, 2, 0)).view(np.uint16))
    # offset + slice: rows 5..9 of the cache
    got = dev.contiguous(cd, (4, H, D), (H * D, D, 1), 5 * H * D).cpu().numpy()
    assert np.array_equal(got.view(np.uint16), cache[5:9].view(np.uint16))
    # setItem: write new k at positions [10, 13)
    src = synth.normal_f16(61, (3, H, D), 1.0)
    dev.set_item_ewise(cd, dev.from_numpy(src), (3, H, D), (H * D, D, 1), 10 * H * D)
    want = oracle.set_item_ewise(cache, src, (3, H, D), (H * D, D, 1), 10 * H * D)
    assert np.array_equal(cd.cpu().numpy().view(np.uint16), want.view(np.uint16))
    # odd sizes / broadcast stride 0
    base = synth.normal_f16(62, (5, 7), 1.0)
    got = dev.contiguous(dev.from_numpy(base), (3, 5, 7), (0, 7, 1), 0).cpu().numpy()
    assert np.array_equal(got.view(np.uint16), np.broadcast_to(base, (3, 5, 7)).copy().view(np.uint16))


def test_strided_rejects_bad_arguments(dev):
    from tensorlib_amd import TensorLibError
    base = dev.empty(64)
    with pytest.raises(TensorLibError):   # more than 8 dimensions
        dev.contiguous(base, (1,) * 9, (1,) * 9, 0)
    with pytest.raises(TensorLibError):   # negative stride
        dev.contiguous(base, (4,), (-1,), 8)


def test_argmax_first_max_wins(dev, oracle):
    x = synth.normal_f16(70, (5, 32000), 1.0)
    x[1, 100] = x[1, 31999] = 9.0     # tie: first index must win
    x[2, :] = 0.5                      # all equal -> 0
    x[3, 31999] = 20.0                 # max at the very end
    got = dev.argmax(dev.from_numpy(x)).cpu().numpy()
    want = oracle.argmax(x)
    assert np.array_equal(got, want)
    assert np.array_equal(got, np.argmax(x.astype(np.float32), axis=-1))
    small = synth.normal_f16(71, (300, 7), 1.0)
    assert np.array_equal(dev.argmax(dev.from_numpy(small)).cpu().numpy(), oracle.argmax(small))


def test_embedding(dev, oracle):
    table = synth.normal_f16(80, (1000, 4096), 1.0)
    ids = synth.token_ids(81, 33, 1000)
    got = dev.embedding(dev.from_numpy(table), dev.from_numpy(ids)).cpu().numpy()
    assert np.array_equal(got.view(np.uint16), oracle.embedding(table, ids).view(np.uint16))
    t2 = synth.normal_f16(82, (10, 13), 1.0)
    ids2 = np.array([9, 0, 3], np.int32)
    got = dev.embedding(dev.from_numpy(t2), dev.from_numpy(ids2)).cpu().numpy()
    assert np.array_equal(got.view(np.uint16), t2[ids2].view(np.uint16))


def test_full_and_causal_mask(dev):
    out = dev.empty(1001)
    dev.full(out, -2.5)
    assert torch.all(out == -2.5)
    m = dev.causal_mask(3, 4, 5).cpu().numpy().astype(np.float32)
    for i in range(4):
        for j in range(9):
            want = -np.inf if j > 5 + i else 0.0
            assert np.all(m[:, i, j] == want)


def _attention_chain_oracle(oracle, q, ck, cv, T):
    """Attention::forward at seqlen 1 composed from CPU-backend ops, in the reference's order
    (model/llama2_7b/src/Transformer.cpp:84-109): per-head q.K^T (matmul2d, rounded to half),
    ScalarDiv by half(sqrt(head_dim)), softmax, scores.V (matmul2d)."""
    H, D = q.shape
    keys = np.ascontiguousarray(ck[:T].transpose(1, 0, 2))      # [H,T,D]
    vals = np.ascontiguousarray(cv[:T].transpose(1, 2, 0))      # [H,D,T]
    sc = oracle.matmul2d_batched(q.reshape(H, 1, D), keys, H, 1, T, D, D, T * D).reshape(H, T)
    sc = oracle.binary_scalar(sc, np.sqrt(np.float32(D)), "div")
    p = oracle.softmax(sc)
    return oracle.matmul2d_batched(p.reshape(H, 1, T), vals, H, 1, D, T, T, D * T).reshape(H, D)


@pytest.mark.parametrize("T,H,D", [(1, 32, 128), (5, 32, 128), (64, 32, 128), (65, 32, 128), (1024, 32, 128),
                                   (2047, 32, 128), (300, 4, 64), (130, 2, 256),
                                   # either side of every switch of the chunk size (64 / 128 / 256 positions per workgroup)
                                   (128, 32, 128), (129, 32, 128), (192, 32, 128), (193, 32, 128), (1279, 8, 128),
                                   (1280, 8, 128), (100, 4, 64), (190, 4, 64), (1300, 4, 64)])
def test_decode_attention_fused_vs_chain(dev, oracle, T, H, D):
    S = max(T, 8)
    q = synth.normal_f16(90, (H, D), 1.0)
    ck = synth.normal_f16(91, (S, H, D), 1.0)
    cv = synth.normal_f16(92, (S, H, D), 1.0)
    got = dev.decode_attention(dev.from_numpy(q), dev.from_numpy(ck), dev.from_numpy(cv), T).cpu().numpy()
    want = _attention_chain_oracle(oracle, q, ck, cv, T)
    assert_close_f16(got, want, RTOL, ATOL, f"decode attention T={T}")


@pytest.mark.parametrize("tokens,hidden", [(1, 4096), (3, 264), (2, 100), (1, 11008), (5, 16384), (1, 20000)])
def test_add_rms_norm(dev, oracle, tokens, hidden):
    """EwiseAdd followed by RMSNorm in one launch; also with the aliasing the driver uses."""
    a = synth.normal_f16(100, (tokens, hidden), 1.0)
    b = synth.normal_f16(101, (tokens, hidden), 1.5)
    w = synth.normal_f16(102, (hidden,), 1.0)
    want_sum = oracle.binary(a, b, "add")
    want_norm = oracle.rms_norm(want_sum, w, 1e-5, "exact")
    s, n = dev.add_rms_norm(dev.from_numpy(a), dev.from_numpy(b), dev.from_numpy(w), 1e-5)
    assert np.array_equal(s.cpu().numpy().view(np.uint16), want_sum.view(np.uint16))
    assert_close_f16(n.cpu().numpy(), want_norm, RTOL, ATOL, "add_rms_norm")
    ad, bd = dev.from_numpy(a), dev.from_numpy(b)
    dev.add_rms_norm(ad, bd, dev.from_numpy(w), 1e-5, sum_out=ad, norm_out=bd)   # sum over a, norm over b
    assert np.array_equal(ad.cpu().numpy().view(np.uint16), want_sum.view(np.uint16))
    assert_close_f16(bd.cpu().numpy(), want_norm, RTOL, ATOL, "add_rms_norm aliased")


@pytest.mark.parametrize("H,D,pos", [(32, 128, 0), (32, 128, 1023), (4, 64, 17), (2, 256, 5)])
def test_rope_qk_store_kv(dev, oracle, H, D, pos):
    S = pos + 3
    qkv = synth.normal_f16(110, (3, H, D), 1.0)
    ck0 = synth.normal_f16(111, (S, H, D), 1.0)
    cv0 = synth.normal_f16(112, (S, H, D), 1.0)
    qd, kd, vd = dev.from_numpy(qkv), dev.from_numpy(ck0), dev.from_numpy(cv0)
    dev.rope_qk_store_kv(qd, kd, vd, pos)
    q_want = oracle.rope(qkv[0].reshape(1, 1, H, D), pos).reshape(H, D)
    k_want = oracle.rope(qkv[1].reshape(1, 1, H, D), pos).reshape(H, D)
    got = qd.cpu().numpy()
    differs = rope_cos_sin_differences(dev, oracle, pos + 1, D)
    assert_rope_equal(got[0][None], q_want[None], differs, pos, "q rope")
    assert np.array_equal(got[1:].view(np.uint16), qkv[1:].view(np.uint16))      # k, v inputs untouched
    ck, cv = kd.cpu().numpy(), vd.cpu().numpy()
    assert_rope_equal(ck[pos][None], k_want[None], differs, pos, "k rope into cache")
    assert np.array_equal(cv[pos].view(np.uint16), qkv[2].view(np.uint16))
    keep = np.arange(S) != pos
    assert np.array_equal(ck[keep].view(np.uint16), ck0[keep].view(np.uint16))
    assert np.array_equal(cv[keep].view(np.uint16), cv0[keep].view(np.uint16))


@pytest.mark.parametrize("pos,H,D", [(0, 32, 128), (63, 32, 128), (64, 32, 128), (1023, 32, 128), (100, 4, 64), (70, 2, 256)])
def test_decode_attention_rope_equals_separate_steps(dev, oracle, pos, H, D):
    """The fused launch must give exactly what rope_qk_store_kv followed by decode_attention gives,
    and leave the caches in the same state."""
    S = pos + 2
    qkv = synth.normal_f16(120, (3, H, D), 1.0)
    ck0 = synth.normal_f16(121, (S, H, D), 1.0)
    cv0 = synth.normal_f16(122, (S, H, D), 1.0)
    q1, k1, v1 = dev.from_numpy(qkv), dev.from_numpy(ck0), dev.from_numpy(cv0)
    dev.rope_qk_store_kv(q1, k1, v1, pos)
    want = dev.decode_attention(q1[0].contiguous(), k1, v1, pos + 1).cpu().numpy()
    q2, k2, v2 = dev.from_numpy(qkv), dev.from_numpy(ck0), dev.from_numpy(cv0)
    got = dev.decode_attention_rope(q2, k2, v2, pos).cpu().numpy()
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    assert torch.equal(k1, k2) and torch.equal(v1, v2)
    # with the precomputed (cos, sin) table: same bits again
    q3, k3, v3 = dev.from_numpy(qkv), dev.from_numpy(ck0), dev.from_numpy(cv0)
    got3 = dev.decode_attention_rope(q3, k3, v3, pos, rope_table=dev.rope_table(S, D)).cpu().numpy()
    assert np.array_equal(got3.view(np.uint16), want.view(np.uint16))
    assert torch.equal(k1, k3) and torch.equal(v1, v3)
    assert np.array_equal(q2.cpu().numpy().view(np.uint16), qkv.view(np.uint16))   # raw projections untouched
    # and against the CPU chain
    q_rot = oracle.rope(qkv[0].reshape(1, 1, H, D), pos).reshape(H, D)
    ck = ck0.copy(); cv = cv0.copy()
    ck[pos] = oracle.rope(qkv[1].reshape(1, 1, H, D), pos).reshape(H, D)
    cv[pos] = qkv[2]
    assert_close_f16(got, _attention_chain_oracle(oracle, q_rot, ck, cv, pos + 1), RTOL, ATOL, "fused rope attention")


@pytest.mark.parametrize("M,N,K", [(128, 4096, 4096), (128, 4096, 11008), (512, 4096, 4096), (1, 4096, 4096), (37, 264, 328),
                                   (128, 1000, 64), (2, 16384, 512)])
def test_hgemm_add_rms_norm(dev, oracle, M, N, K):
    """A projection, the residual add and the RMSNorm after it in one call: same bits as hgemm followed by
    add_rms_norm whether or not the GEMM split K (then its second pass runs inside the norm kernel), and within
    tolerance of the CPU chain."""
    A = synth.normal_f16(150, (M, K), 1.0)
    W = synth.normal_f16(151, (N, K), 0.02)
    res = synth.normal_f16(152, (M, N), 1.0)
    g = synth.normal_f16(153, (N,), 1.0)
    Ad, Wd, rd, gd = dev.from_numpy(A), dev.from_numpy(W), dev.from_numpy(res), dev.from_numpy(g)
    s_got, n_got = dev.hgemm_add_rms_norm(Ad, Wd, rd, gd, 1e-5)
    y = dev.hgemm(Ad, Wd) if M > 1 else dev.gemv(Ad.view(-1), Wd).view(1, N)
    s_want, n_want = dev.add_rms_norm(rd, y, gd, 1e-5)
    assert np.array_equal(s_got.cpu().numpy().view(np.uint16), s_want.cpu().numpy().view(np.uint16))
    assert np.array_equal(n_got.cpu().numpy().view(np.uint16), n_want.cpu().numpy().view(np.uint16))
    if M * N * K <= 128 * 4096 * 4096:
        s_cpu = oracle.binary(res, oracle.matmul2d(A, W), "add")
        assert_close_scaled(s_got.cpu().numpy(), s_cpu, 1e-2, 1e-2, "hgemm + residual")
        assert_close_scaled(n_got.cpu().numpy(), oracle.rms_norm(s_cpu, g, 1e-5, "fused"), 1e-2, 1e-2, "hgemm + residual + norm")


@pytest.mark.parametrize("N,K", [(4096, 11008), (300, 512), (64, 4096), (33, 12288), (10, 520)])
def test_gemv_silu_mul(dev, oracle, N, K):
    ab = synth.normal_f16(130, (2 * K,), 1.5)
    W = synth.normal_f16(131, (N, K), 0.02)
    got = dev.gemv_silu_mul(dev.from_numpy(ab), dev.from_numpy(W)).cpu().numpy()
    x2 = oracle.silu_mul(ab[:K], ab[K:])
    # silu*mul is rounded once on the GPU and twice on the CPU chain: compare on the output scale
    assert_close_scaled(got, oracle.matmul2d(x2[None, :], W)[0], 1e-2, 5e-3, "gemv with fused silu*mul")
    # identical bits to the two-step GPU path
    x2d = dev.silu_mul(dev.from_numpy(ab[:K]), dev.from_numpy(ab[K:]))
    two = dev.gemv(x2d, dev.from_numpy(W)).cpu().numpy()
    assert np.array_equal(got.view(np.uint16), two.view(np.uint16))


@pytest.mark.parametrize("N,K,with_addend", [(12288, 4096, True), (22016, 4096, True), (32000, 4096, True),
                                             (300, 512, True), (64, 4096, False), (33, 11008, True), (10, 520, True)])
def test_gemv_add_rms_norm(dev, oracle, N, K, with_addend):
    """Residual add + RMSNorm formed inside the GEMV's operand load: against the CPU chain
    (EwiseAdd -> RMSNorm -> matmul2d) and against the GPU's own three-step path."""
    h = synth.normal_f16(150, (K,), 1.0)
    d = synth.normal_f16(151, (K,), 0.7) if with_addend else None
    g = synth.normal_f16(152, (K,), 1.0)
    W = synth.normal_f16(153, (N, K), 0.02)
    eps = 1e-5
    want_sum = oracle.binary(h, d, "add") if with_addend else h
    want_norm = oracle.rms_norm(want_sum[None, :], g, eps, "exact")[0]
    want = oracle.matmul2d(want_norm[None, :], W)[0]
    hd, gd, Wd = dev.from_numpy(h), dev.from_numpy(g), dev.from_numpy(W)
    dd = dev.from_numpy(d) if with_addend else None
    y, s = dev.gemv_add_rms_norm(hd, dd, gd, eps, Wd)
    assert np.array_equal(s.cpu().numpy().view(np.uint16), want_sum.view(np.uint16))
    # the norm is rounded from a differently ordered fp32 sum of squares: compare on the output scale
    assert_close_scaled(y.cpu().numpy(), want, 1e-2, 5e-3, "gemv with fused add + rmsnorm")
    if with_addend:
        s2, n2 = dev.add_rms_norm(hd, dd, gd, eps)
    else:
        s2, n2 = hd, dev.rms_norm(hd.view(1, K), gd, eps).view(K)
    two = dev.gemv(n2, Wd).cpu().numpy()
    assert_close_scaled(y.cpu().numpy(), two, 1e-2, 2e-3, "fused vs three-step GPU path")
    assert np.array_equal(hd.cpu().numpy().view(np.uint16), h.view(np.uint16))       # inputs untouched
    y3, s3 = dev.gemv_add_rms_norm(hd, dd, gd, eps, Wd, want_sum=False)
    assert s3 is None and np.array_equal(y3.cpu().numpy().view(np.uint16), y.cpu().numpy().view(np.uint16))


def test_gemv_add_rms_norm_limits(dev):
    from tensorlib_amd import TensorLibError
    with pytest.raises(TensorLibError):
        dev.gemv_add_rms_norm(dev.empty(16384), None, dev.empty(16384), 1e-5, dev.empty(8, 16384))  # K too long
    with pytest.raises(TensorLibError):
        dev.gemv_add_rms_norm(dev.empty(100), None, dev.empty(100), 1e-5, dev.empty(8, 100))        # K % 8 != 0


def test_gemv_silu_mul_limits(dev):
    from tensorlib_amd import TensorLibError
    with pytest.raises(TensorLibError):
        dev.gemv_silu_mul(dev.empty(2 * 16384), dev.empty(8, 16384))     # K beyond the fused kernel's limit
    with pytest.raises(TensorLibError):
        dev.gemv_silu_mul(dev.empty(2 * 100), dev.empty(8, 100))         # K not a multiple of 8


def test_rope_table_values(dev):
    D, S = 128, 300
    tab = dev.rope_table(S, D).cpu().numpy().astype(np.float64)
    pos = np.arange(S)[:, None]
    th = pos * 10000.0 ** (-2.0 * np.arange(D // 2)[None, :] / D)
    assert np.abs(tab[..., 0] - np.cos(th)).max() < 1.5e-3 and np.abs(tab[..., 1] - np.sin(th)).max() < 1.5e-3
    assert np.all(tab[0, :, 0] == 1.0) and np.all(tab[0, :, 1] == 0.0)


@pytest.mark.parametrize("D", [128, 64])
def test_rope_table_bits_equal_the_cpu_loop(dev, oracle, D):
    """All 2048 positions of the largest context: the table holds the CPU loop's half(cos), half(sin) bit for bit,
    up to the handful of entries where the host libm is not correctly rounded (see rope_cos_sin_differences)."""
    differs = rope_cos_sin_differences(dev, oracle, 2048, D)
    assert differs.shape == (2048, D // 2) and not differs[0].any()


@pytest.mark.parametrize("S,H,D,K", [(128, 32, 128, 4096), (64, 32, 128, 4096), (100, 32, 128, 4096), (512, 32, 128, 4096),
                                     (2, 32, 128, 4096), (1, 8, 64, 512), (40, 8, 64, 8192), (300, 4, 128, 1024)])
def test_hgemm_prefill_rope_qkv_vt_equals_separate_calls(dev, S, H, D, K):
    """Projection + rotation in one call against tl_matmul2d_f16 followed by tl_prefill_rope_qkv_vt_f16: rotated q, both
    cache rows and the transposed values bit for bit, at prompt lengths where the GEMM splits K (the rotating kernel then
    reads the fp32 partial sums) and where it does not."""
    dim = H * D
    X = dev.from_numpy(synth.normal_f16(170 + S, (S, K), 1.0))
    W = dev.from_numpy(synth.normal_f16(171 + S, (3 * dim, K), 0.02))
    table = dev.rope_table(max(S, 8), D)
    qkv = dev.matmul2d(X, W)
    k1, v1 = dev.empty(S, H, D), dev.empty(S, H, D)
    q1, vT1 = dev.prefill_rope_qkv_vt(qkv[:, :dim], qkv[:, dim:2 * dim], qkv[:, 2 * dim:], k1, v1, table, H)
    split = dev.hgemm_last_plan()[1]
    k2, v2 = dev.empty(S, H, D), dev.empty(S, H, D)
    q2, vT2 = dev.hgemm_prefill_rope_qkv_vt(X, W, k2, v2, table, H)
    assert torch.equal(q2, q1) and torch.equal(k2, k1) and torch.equal(v2, v1) and torch.equal(vT2, vT1), f"splits {split}"


def test_hgemm_prefill_rope_qkv_vt_rejects_before_it_writes(dev):
    """Arguments of the second step (the rotation) are checked before the projection is launched: a call with an ldv
    that does not cover the tokens, or a missing output, fails and leaves the qkv buffer as it was."""
    TL_OK = 0
    S, H, D, K = 128, 8, 64, 512
    dim = H * D
    X = dev.from_numpy(synth.normal_f16(180, (S, K), 1.0))
    W = dev.from_numpy(synth.normal_f16(181, (3 * dim, K), 0.02))
    table = dev.rope_table(S, D)
    qkv = torch.full((S, 3 * dim), 7.0, dtype=torch.float16, device="cuda")
    q, kc, vc = dev.empty(H, S, D), dev.empty(S, H, D), dev.empty(S, H, D)
    vT = dev.empty(H, D, S)
    p = lambda t: t.data_ptr()
    lib = dev.lib
    rc = lib.tl_hgemm_prefill_rope_qkv_vt_f16(p(X), p(W), p(qkv), p(q), p(kc), p(vc), p(table), p(vT), 64, S, H, D, K)     # ldv < S
    assert rc != TL_OK
    rc = lib.tl_hgemm_prefill_rope_qkv_vt_f16(p(X), p(W), p(qkv), p(q), p(kc), p(vc), p(table), None, S, S, H, D, K)      # no vT
    assert rc != TL_OK
    rc = lib.tl_hgemm_prefill_rope_qkv_vt_f16(p(X), p(W), p(qkv), p(q) + 2, p(kc), p(vc), p(table), p(vT), S, S, H, D, K)  # unaligned q
    assert rc != TL_OK
    torch.cuda.synchronize()
    assert bool((qkv == 7.0).all())
    rc = lib.tl_hgemm_prefill_rope_qkv_vt_f16(p(X), p(W), p(qkv), p(q), p(kc), p(vc), p(table), p(vT), S, S, H, D, K)
    assert rc == TL_OK


@pytest.mark.parametrize("S", [128, 512, 33])
def test_hgemm_prefill_rope_qkv_vt_against_the_oracle(dev, oracle, S):
    """The fused projection + rotation entry against the CPU restatement directly: oracle.matmul2d of sampled token rows
    through wq, wk and wv, oracle.rope of the q and k rows at the tokens' positions.  The projection differs from the
    oracle's only in the order of the fp32 sum (gate of the GEMM tests); the rotation then acts on those fp16 values,
    so the rotated outputs are gated the same way and the v rows must equal the GEMM's own output bit for bit."""
    H, D, K = 32, 128, 4096
    dim = H * D
    X = synth.normal_f16(190 + S, (S, K), 1.0)
    W = synth.normal_f16(191 + S, (3 * dim, K), 0.02)
    Xd, Wd = dev.from_numpy(X), dev.from_numpy(W)
    table = dev.rope_table(max(S, 8), D)
    kc, vc = dev.empty(S, H, D), dev.empty(S, H, D)
    q, vT = dev.hgemm_prefill_rope_qkv_vt(Xd, Wd, kc, vc, table, H)            # q [H, S, D], vT [H, D, ldv]
    rng = np.random.default_rng(S)
    rows = np.unique(np.concatenate([[0, S - 1], rng.integers(0, S, 6)]))
    qkv = oracle.matmul2d(X[rows], W)                                           # [rows, 3 dim]
    qn, kn, vn, vTn = q.cpu().numpy(), kc.cpu().numpy(), vc.cpu().numpy(), vT.cpu().numpy()
    for i, t in enumerate(rows):
        want_q = oracle.rope(qkv[i, :dim].reshape(1, 1, H, D), int(t))[0, 0]
        want_k = oracle.rope(qkv[i, dim:2 * dim].reshape(1, 1, H, D), int(t))[0, 0]
        want_v = qkv[i, 2 * dim:].reshape(H, D)
        # a rotated value mixes two products of size |x|: gate on the pair's magnitude like the chain tests gate on rms
        assert_close_f16(qn[:, t, :], want_q, RTOL, 2 * ATOL, f"fused q row {t}")
        assert_close_f16(kn[t], want_k, RTOL, 2 * ATOL, f"fused k row {t}")
        assert_close_f16(vn[t], want_v, RTOL, ATOL, f"fused v row {t}")
        assert np.array_equal(vTn[:, :, t].view(np.uint16), vn[t].view(np.uint16))


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("chunk", [64, 128, 256])
def test_decode_attention_every_chunk_size_vs_chain(dev, oracle, chunk, D):
    """Each chunk size forced through the tuning hook, at contexts that end inside the first chunk, on a chunk boundary,
    one past it, and in a partly filled last chunk of several."""
    H = 6
    q = synth.normal_f16(160, (H, D), 1.0)
    ck = synth.normal_f16(161, (800, H, D), 1.0)
    cv = synth.normal_f16(162, (800, H, D), 1.0)
    qd, kd, vd = dev.from_numpy(q), dev.from_numpy(ck), dev.from_numpy(cv)
    try:
        dev.lib.tl_set_decode_attention_chunk(chunk)
        for T in (1, chunk - 1, chunk, chunk + 1, 2 * chunk, 2 * chunk + 37, 800):
            for mode in (1, 2):
                dev.lib.tl_set_decode_attention_merge(mode)
                got = dev.decode_attention(qd, kd, vd, T).cpu().numpy()
                assert_close_f16(got, _attention_chain_oracle(oracle, q, ck, cv, T), RTOL, ATOL,
                                 f"chunk {chunk} merge {mode} T={T}")
    finally:
        dev.lib.tl_set_decode_attention_chunk(0)
        dev.lib.tl_set_decode_attention_merge(0)


@pytest.mark.parametrize("T", [65, 200, 512, 513, 1500])
def test_decode_attention_merge_inside_the_launch_equals_second_launch(dev, T):
    """The chunk partials of a head are merged either by the workgroup that finishes the head's last chunk (tickets,
    device-coherent partials) or by a second launch: same chunk order, so the same bits; repeated calls show that
    the tickets return to zero."""
    H, D = 32, 128
    q = dev.from_numpy(synth.normal_f16(150, (H, D), 1.0))
    ck = dev.from_numpy(synth.normal_f16(151, (T, H, D), 1.0))
    cv = dev.from_numpy(synth.normal_f16(152, (T, H, D), 1.0))
    try:
        dev.lib.tl_set_decode_attention_merge(2)
        want = dev.decode_attention(q, ck, cv, T)
        dev.lib.tl_set_decode_attention_merge(1)
        for _ in range(3):
            assert torch.equal(dev.decode_attention(q, ck, cv, T), want)
        dev.lib.tl_set_decode_attention_merge(0)
        assert torch.equal(dev.decode_attention(q, ck, cv, T), want)
    finally:
        dev.lib.tl_set_decode_attention_merge(0)


def test_decode_attention_ticket_region_does_not_move_with_the_head_count(dev):
    """A call with few heads and several chunks leaves partial results in the scratch buffer; a later call with more
    heads must not find them where it keeps its tickets.  32 heads then 96 heads at 300 positions, through the entry
    with the grown-on-demand workspace and the one with the static array, against the second-launch merge; and the
    release/acquire form of the in-launch merge gives the same bits."""
    D, T = 128, 300
    for static in (False, True):
        for H in (32, 96, 32, 96):
            qkv = dev.from_numpy(synth.normal_f16(170 + H, (3, H, D), 1.0))
            ck0 = synth.normal_f16(171 + H, (T, H, D), 1.0)
            cv0 = synth.normal_f16(172 + H, (T, H, D), 1.0)
            table = dev.rope_table(T, D)
            outs = {}
            try:
                for mode in (2, 1, 3, 0):
                    dev.lib.tl_set_decode_attention_merge(mode)
                    ck, cv = dev.from_numpy(ck0), dev.from_numpy(cv0)
                    out = dev.empty(H, D)
                    dev.decode_attention_rope(qkv, ck, cv, T - 1, table, out=out, static_scratch=static)
                    outs[mode] = out.clone()
            finally:
                dev.lib.tl_set_decode_attention_merge(0)
            for mode in (1, 3, 0):
                assert torch.equal(outs[mode], outs[2]), (static, H, mode)


def test_decode_attention_more_heads_than_tickets_merges_with_the_second_kernel(dev, oracle):
    """More heads than the scratch buffer has ticket words: the launch takes the second-kernel merge by itself."""
    H, D, T = 1040, 64, 130
    q = synth.normal_f16(180, (H, D), 1.0)
    ck = synth.normal_f16(181, (T, H, D), 1.0)
    cv = synth.normal_f16(182, (T, H, D), 1.0)
    got = dev.decode_attention(dev.from_numpy(q), dev.from_numpy(ck), dev.from_numpy(cv), T).cpu().numpy()
    rows = [0, 63, 64, 1023, 1024, 1039]
    want = _attention_chain_oracle(oracle, q[rows], ck[:, rows], cv[:, rows], T)
    assert_close_f16(got[rows], want, RTOL, ATOL, "1040 heads")


def test_decode_attention_repeated_calls_reuse_counters(dev, oracle):
    """Many calls in a row with different numbers of chunks share one partials workspace: all of
    them have to agree with the CPU chain."""
    H, D = 8, 128
    q = synth.normal_f16(140, (H, D), 1.0)
    ck = synth.normal_f16(141, (700, H, D), 1.0)
    cv = synth.normal_f16(142, (700, H, D), 1.0)
    qd, kd, vd = dev.from_numpy(q), dev.from_numpy(ck), dev.from_numpy(cv)
    for T in (700, 65, 700, 130, 64, 129, 700):
        got = dev.decode_attention(qd, kd, vd, T).cpu().numpy()
        assert_close_f16(got, _attention_chain_oracle(oracle, q, ck, cv, T), RTOL, ATOL, f"repeat T={T}")


# ------------------------------------------------------------------- prefill glue ----

@pytest.mark.parametrize("S,H,D,start,fused_rows", [(128, 32, 128, 0, True), (17, 4, 64, 5, False), (3, 2, 256, 40, True)])
def test_prefill_rope_qkv(dev, oracle, S, H, D, start, fused_rows):
    """RoPE of q and k, cache writes and the q transpose in one launch, from separate projections or
    from the column blocks of one fused [S, 3*dim] projection."""
    dim = H * D
    qkv = synth.normal_f16(160, (S, 3 * dim), 1.0)
    q, k, v = qkv[:, :dim], qkv[:, dim:2 * dim], qkv[:, 2 * dim:]
    T = start + S + 2
    ck0 = synth.normal_f16(161, (T, H, D), 1.0)
    cv0 = synth.normal_f16(162, (T, H, D), 1.0)
    want_q = oracle.rope(np.ascontiguousarray(q).reshape(1, S, H, D), start)[0]      # [S, H, D]
    want_k = oracle.rope(np.ascontiguousarray(k).reshape(1, S, H, D), start)[0]
    kd, vd = dev.from_numpy(ck0), dev.from_numpy(cv0)
    table = dev.rope_table(T, D)
    if fused_rows:
        t = dev.from_numpy(qkv)
        qd, kk, vv = t[:, :dim], t[:, dim:2 * dim], t[:, 2 * dim:]
    else:
        qd, kk, vv = (dev.from_numpy(np.ascontiguousarray(a)) for a in (q, k, v))
    got_q = dev.prefill_rope_qkv(qd, kk, vv, kd, vd, table, start, H).cpu().numpy()   # [H, S, D]
    differs = rope_cos_sin_differences(dev, oracle, start + S, D)
    assert_rope_equal(np.ascontiguousarray(got_q.transpose(1, 0, 2)), want_q, differs, start, "prefill rope q")
    gk, gv = kd.cpu().numpy(), vd.cpu().numpy()
    assert_rope_equal(gk[start:start + S], want_k, differs, start, "prefill rope k -> cache")
    assert np.array_equal(gv[start:start + S].view(np.uint16), np.ascontiguousarray(v).reshape(S, H, D).view(np.uint16))
    keep = np.r_[0:start, start + S:T]                                                   # other cache rows untouched
    assert np.array_equal(gk[keep].view(np.uint16), ck0[keep].view(np.uint16))
    assert np.array_equal(gv[keep].view(np.uint16), cv0[keep].view(np.uint16))
    # identical bits to the per-op GPU path (apply_rotary_emb with the same half-rounded cos/sin)
    q4 = dev.from_numpy(np.ascontiguousarray(q).reshape(1, S, H, D))
    two = dev.apply_rotary_emb(q4, start).cpu().numpy()[0].transpose(1, 0, 2)
    assert np.array_equal(got_q.view(np.uint16), two.view(np.uint16))


@pytest.mark.parametrize("S,H,D,fused_rows", [(128, 32, 128, True), (70, 3, 128, True), (1, 2, 64, False), (200, 5, 64, True),
                                              (64, 4, 128, False)])
def test_prefill_rope_qkv_vt_equals_the_two_launches(dev, S, H, D, fused_rows):
    """The one-pass kernel for a fresh context against prefill_rope_qkv followed by gather_vt: rotated q, both
    cache rows and the transposed, zero-padded values, bit for bit (the pair is checked against the CPU above)."""
    dim = H * D
    qkv = synth.normal_f16(170, (S, 3 * dim), 1.0)
    ck0 = synth.normal_f16(171, (S + 2, H, D), 1.0)
    cv0 = synth.normal_f16(172, (S + 2, H, D), 1.0)
    table = dev.rope_table(S + 2, D)

    def inputs():
        if fused_rows:
            t = dev.from_numpy(qkv)
            return t[:, :dim], t[:, dim:2 * dim], t[:, 2 * dim:]
        return tuple(dev.from_numpy(np.ascontiguousarray(qkv[:, i * dim:(i + 1) * dim])) for i in range(3))

    k1, v1 = dev.from_numpy(ck0), dev.from_numpy(cv0)
    q1 = dev.prefill_rope_qkv(*inputs(), k1, v1, table, 0, H)
    ldv = (S + 63) // 64 * 64
    vT1 = dev.empty(H, D, ldv)
    from tensorlib_amd._lib import check
    check(dev.lib.tl_gather_vt_f16(vT1.data_ptr(), v1.data_ptr(), S, ldv, H, D), "tl_gather_vt_f16")
    k2, v2 = dev.from_numpy(ck0), dev.from_numpy(cv0)
    q2, vT2 = dev.prefill_rope_qkv_vt(*inputs(), k2, v2, table, H)
    assert torch.equal(q1, q2) and torch.equal(k1, k2) and torch.equal(v1, v2)
    assert torch.equal(vT1, vT2)
    assert vT2.shape[2] == ldv and (ldv == S or bool((vT2[:, :, S:] == 0).all()))


@pytest.mark.parametrize("H,S,start", [(32, 128, 0), (4, 17, 9), (2, 1, 300), (3, 70, 0)])
def test_scaled_causal_softmax(dev, oracle, H, S, start):
    """ScalarDiv, mask add and softmax of Attention::forward in one launch, against the three CPU ops."""
    T = start + S
    sc = synth.normal_f16(170, (H, S, T), 8.0)
    div = np.float16(np.sqrt(128.0))
    t = oracle.binary_scalar(sc, div, "div")
    mask = np.where(np.arange(T)[None, :] > start + np.arange(S)[:, None], -np.inf, 0.0).astype(np.float16)
    t = oracle.binary(t, np.broadcast_to(mask, (H, S, T)).copy(), "add")
    want = oracle.softmax(t.reshape(H * S, T)).reshape(H, S, T)
    got = dev.scaled_causal_softmax(dev.from_numpy(sc), float(div), start).cpu().numpy()
    assert_close_f16(got, want, RTOL, ATOL, "scaled causal softmax")
    assert np.all(got[:, np.arange(S)[:, None] + start < np.arange(T)[None, :]] == 0)   # masked columns are exactly 0
    # identical bits to the GPU's three-launch path
    d3 = dev.binary(dev.from_numpy(sc), float(div), "div")
    d3 = dev.binary(d3, dev.causal_mask(H, S, start).view(H, S, T), "add")
    three = dev.softmax(d3.view(H * S, T)).cpu().numpy().reshape(H, S, T)
    assert np.array_equal(got.view(np.uint16), three.view(np.uint16))


@pytest.mark.parametrize("rows,hidden", [(128, 11008), (3, 64), (1, 8)])
def test_silu_mul_rows(dev, oracle, rows, hidden):
    ab = synth.normal_f16(180, (rows, 2 * hidden), 1.5)
    want = oracle.silu_mul(np.ascontiguousarray(ab[:, :hidden]), np.ascontiguousarray(ab[:, hidden:]))
    got = dev.silu_mul_rows(dev.from_numpy(ab)).cpu().numpy()
    assert_close_f16(got, want, RTOL, ATOL, "silu_mul_rows")
    two = dev.silu_mul(dev.from_numpy(np.ascontiguousarray(ab[:, :hidden])), dev.from_numpy(np.ascontiguousarray(ab[:, hidden:])))
    assert np.array_equal(got.view(np.uint16), two.cpu().numpy().view(np.uint16))


@pytest.mark.parametrize("H,S,D,start", [(4, 128, 128, 0), (2, 70, 128, 9), (3, 33, 64, 100), (2, 1, 128, 40),
                                         (1, 32, 128, 0), (8, 512, 128, 0), (2, 200, 64, 313)])
def test_prefill_attention(dev, oracle, H, S, D, start):
    """Causal prefill attention in one launch (no score matrix in memory) against the CPU op chain."""
    T = start + S
    q = synth.normal_f16(190, (H, S, D), 1.0)
    ck = synth.normal_f16(191, (T + 3, H, D), 1.0)
    cv = synth.normal_f16(192, (T + 3, H, D), 1.0)
    want = oracle.attention_chain(q, ck, cv, start)
    got = dev.prefill_attention(dev.from_numpy(q), dev.from_numpy(ck), dev.from_numpy(cv), start).cpu().numpy()
    # probabilities are rounded to fp16 before (CPU: after) normalisation; measured worst case 0.7 of the gate
    assert_close_f16(got, want, RTOL, ATOL, f"prefill attention H={H} S={S} D={D} start={start}")
    # row 0 of a fresh context attends to position 0 only: the output is exactly v[0]
    if start == 0:
        assert np.array_equal(got[0].view(np.uint16), cv[0].view(np.uint16))


@pytest.mark.parametrize("H,S,start", [(2, 1, 0), (3, 130, 0), (2, 257, 70), (33, 384, 0), (2, 640, 129), (20, 1000, 24),
                                       (32, 2048, 0), (35, 1920, 37)])   # the last two: paired groups, even and odd count
def test_prefill_attention_tiled_kernel(dev, oracle, H, S, start):
    """The LDS-tiled kernel (workgroups of 128 query rows, key tiles of 64 staged once for four wavefronts; with many
    groups a workgroup takes a long and a short one) does per wavefront what the one-wavefront kernel does: it is
    checked against the CPU op chain where that is quick, and bit for bit against the other kernel everywhere."""
    D, T = 128, start + S
    q = synth.normal_f16(290, (H, S, D), 1.0)
    ck = synth.normal_f16(291, (T, H, D), 1.0)
    cv = synth.normal_f16(292, (T, H, D), 1.0)
    qd, kd, vd = dev.from_numpy(q), dev.from_numpy(ck), dev.from_numpy(cv)
    try:
        dev.lib.tl_set_prefill_attention_variant(1)
        one = dev.prefill_attention(qd, kd, vd, start).cpu().numpy()
        dev.lib.tl_set_prefill_attention_variant(2)
        tiled = dev.prefill_attention(qd, kd, vd, start).cpu().numpy()
    finally:
        dev.lib.tl_set_prefill_attention_variant(0)
    assert np.array_equal(one.view(np.uint16), tiled.view(np.uint16))
    if H * S * T <= 2 * 640 * 769:
        assert_close_f16(tiled, oracle.attention_chain(q, ck, cv, start), RTOL, ATOL, f"tiled prefill attention S={S} start={start}")
    if start == 0:
        assert np.array_equal(tiled[0].view(np.uint16), cv[0].view(np.uint16))


def test_prefill_attention_limits(dev):
    from tensorlib_amd import TensorLibError
    with pytest.raises(TensorLibError):
        dev.prefill_attention(dev.empty(2, 4, 256), dev.empty(8, 2, 256), dev.empty(8, 2, 256), 0)   # head_dim 256


def test_empty_inputs_are_accepted_and_touch_nothing(dev):
    """Zero rows / tokens / elements through the C ABI: every op returns success without a launch (the reference's
    Tensor layer can hand over empty views, e.g. a zero-length slice), and a canary buffer keeps its bits."""
    import ctypes
    from tensorlib_amd._lib import check
    lib = dev.lib
    canary = dev.from_numpy(synth.normal_f16(990, (64,), 1.0))
    before = canary.clone()
    p = ctypes.c_void_p(canary.data_ptr())
    ids = torch.zeros(4, dtype=torch.int32, device=canary.device)
    ip = ctypes.c_void_p(ids.data_ptr())
    check(lib.tl_rms_norm_f16(p, p, p, 1e-5, 64, 0), "rms_norm, no tokens")
    check(lib.tl_apply_rotary_emb_f16(p, p, 0, 1, 0, 2, 32), "rope, no positions")
    check(lib.tl_softmax_f16(p, p, 0, 64), "softmax, no rows")
    check(lib.tl_softmax_f16(p, p, 4, 0), "softmax, no columns")
    check(lib.tl_silu_f16(p, p, 0), "silu, no elements")
    check(lib.tl_silu_mul_f16(p, p, p, 0), "silu_mul, no elements")
    check(lib.tl_binary_f16(p, p, p, 0, 0), "binary, no elements")
    check(lib.tl_binary_scalar_f16(p, p, 0x3c00, 0, 3), "binary scalar, no elements")
    check(lib.tl_full_f16(p, 0x3c00, 0), "full, no elements")
    check(lib.tl_embedding_f16(p, p, ip, 0, 16, 4), "embedding, no tokens")
    check(lib.tl_gemv_f16(p, p, p, 0, 64), "gemv, no rows")
    check(lib.tl_causal_mask_f16(p, 0, 4, 0), "mask, no repetitions")
    check(lib.tl_add_rms_norm_f16(p, p, p, p, p, 1e-5, 64, 0), "add_rms_norm, no tokens")
    dev.synchronize()
    assert torch.equal(canary, before)
