"""Committed vectors (tests/golden/hotpath_vectors.npz, written by tests/golden/make_golden.py).
CPU: today's oracle must reproduce them bit for bit.  GPU: the kernels must match them within the
parity tolerance, through the C ABI."""
import os

import numpy as np
import pytest

from tests.conftest import assert_close_f16

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hotpath_vectors.npz")


@pytest.fixture(scope="module")
def gold():
    return dict(np.load(GOLD, allow_pickle=False))


def _same(a, b):
    return a.shape == b.shape and np.array_equal(a.view(np.uint16), b.view(np.uint16))


def test_oracle_reproduces_golden_vectors(oracle, gold):
    g = gold
    for tag in ("gemv_a", "gemv_b", "gemv_c"):
        assert _same(oracle.matmul2d(g[tag + "_x"], g[tag + "_W"]), g[tag + "_y"]), tag
    for tag in ("hgemm_a", "hgemm_b"):
        assert _same(oracle.matmul2d(g[tag + "_A"], g[tag + "_B"]), g[tag + "_C"]), tag
    assert _same(oracle.rope(g["rope_x"], int(g["rope_start"])), g["rope_y"])
    assert _same(oracle.softmax(g["softmax_x"]), g["softmax_y"])
    assert _same(oracle.rms_norm(g["rms_x"], g["rms_w"], 1e-5, "fused"), g["rms_y"])
    assert _same(oracle.silu(g["ew_a"]), g["silu_y"])
    assert _same(oracle.silu_mul(g["ew_a"], g["ew_b"]), g["silu_mul_y"])
    for op in ("add", "sub", "mul", "div"):
        assert _same(oracle.binary(g["ew_a"], g["ew_b"], op), g["bin_" + op]), op
    assert _same(oracle.binary_scalar(g["ew_a"], np.float16(11.3125), "div"), g["div_scalar"])
    assert np.array_equal(oracle.argmax(g["argmax_x"]), g["argmax_y"])
    assert _same(oracle.attention_chain(g["att_q"], g["att_k"], g["att_v"], int(g["att_start"])), g["att_prefill_y"])
    assert _same(oracle.attention_chain(g["att_q1"], g["att_k"], g["att_v"], 45), g["att_decode_y"])
    sm = oracle.binary(g["nrm_h"], g["nrm_d"], "add")
    assert _same(sm, g["nrm_sum"])
    assert _same(oracle.matmul2d(oracle.rms_norm(sm, g["nrm_g"], 1e-5, "exact"), g["nrm_W"]), g["nrm_y"])


def test_synthetic_inputs_are_stable(gold):
    from tensorlib_amd import synth
    assert _same(synth.normal_f16(1, (96, 520), 0.05), gold["gemv_a_W"])
    assert _same(synth.normal_f16(5, (2, 3, 4, 64), 1.0), gold["rope_x"])


@pytest.mark.gpu
def test_gpu_matches_golden_vectors(dev, gold):
    g = gold
    up = dev.from_numpy
    for tag in ("gemv_a", "gemv_b", "gemv_c"):
        y = dev.matmul2d(up(g[tag + "_x"]), up(g[tag + "_W"])).cpu().numpy()
        assert_close_f16(y, g[tag + "_y"], 1e-2, 1e-3, tag)
    for tag in ("hgemm_a", "hgemm_b"):
        c = dev.matmul2d(up(g[tag + "_A"]), up(g[tag + "_B"])).cpu().numpy()
        assert_close_f16(c, g[tag + "_C"], 1e-2, 1e-3, tag)
    from tests.conftest import assert_rope_equal, rope_cos_sin_differences
    from oracle import oracle
    start, T, D = int(g["rope_start"]), g["rope_x"].shape[1], g["rope_x"].shape[3]
    assert_rope_equal(dev.apply_rotary_emb(up(g["rope_x"]), start).cpu().numpy(), g["rope_y"],
                      rope_cos_sin_differences(dev, oracle, start + T, D), start, "rope")
    assert_close_f16(dev.softmax(up(g["softmax_x"])).cpu().numpy(), g["softmax_y"], 1e-2, 1e-3, "softmax")
    assert_close_f16(dev.rms_norm(up(g["rms_x"]), up(g["rms_w"]), 1e-5).cpu().numpy(), g["rms_y"], 1e-2, 1e-3, "rms_norm")
    assert_close_f16(dev.silu(up(g["ew_a"])).cpu().numpy(), g["silu_y"], 1e-2, 1e-3, "silu")
    assert_close_f16(dev.silu_mul(up(g["ew_a"]), up(g["ew_b"])).cpu().numpy(), g["silu_mul_y"], 1e-2, 1e-3, "silu_mul")
    for op in ("add", "sub", "mul", "div"):
        assert _same(dev.binary(up(g["ew_a"]), up(g["ew_b"]), op).cpu().numpy(), g["bin_" + op]), op
    assert _same(dev.div(up(g["ew_a"]), 11.3125).cpu().numpy(), g["div_scalar"])
    assert np.array_equal(dev.argmax(up(g["argmax_x"])).cpu().numpy(), g["argmax_y"])


@pytest.mark.gpu
def test_gpu_fused_kernels_match_golden_chains(dev, gold):
    """The fused kernels against the frozen outputs of the CPU op chains they replace."""
    from tests.conftest import assert_close_scaled
    g = gold
    up = dev.from_numpy
    start = int(g["att_start"])
    got = dev.prefill_attention(up(g["att_q"]), up(g["att_k"]), up(g["att_v"]), start).cpu().numpy()
    assert_close_f16(got, g["att_prefill_y"], 1e-2, 1e-3, "prefill attention")
    got = dev.decode_attention(up(np.ascontiguousarray(g["att_q1"][:, 0, :])), up(g["att_k"]), up(g["att_v"]), 46).cpu().numpy()
    assert_close_f16(got, g["att_decode_y"][0], 1e-2, 1e-3, "decode attention")
    y, s = dev.gemv_add_rms_norm(up(g["nrm_h"][0]), up(g["nrm_d"][0]), up(g["nrm_g"]), 1e-5, up(g["nrm_W"]))
    assert _same(s.cpu().numpy(), g["nrm_sum"][0])
    assert_close_scaled(y.cpu().numpy(), g["nrm_y"][0], 1e-2, 5e-3, "gemv with add + rmsnorm prologue")
