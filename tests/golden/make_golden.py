"""Writes tests/golden/hotpath_vectors.npz: small input/output vectors for every function on the path.

Origin of the expected outputs: the CPU oracle of this repository (oracle/tl_oracle.c) after it
passed tests/test_oracle_pins.py.  They are NOT outputs of the reference itself: the reference
holds no golden vectors for this path and its CPU backend cannot be compiled in the authoring
container (it includes <cuda_fp16.h>).  The fixture freezes today's oracle so that a later change
to the oracle, the synthetic-input generator or a GPU kernel that moves any of these numbers is
caught: the CPU suite checks the oracle against it bit for bit, the GPU suite checks the kernels
against it with the parity tolerance.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import oracle as o  # noqa: E402
from tensorlib_amd import synth  # noqa: E402


def build():
    v = {}
    # GEMV: aligned, ragged K, short rows
    for tag, (N, K) in {"gemv_a": (96, 520), "gemv_b": (33, 1001), "gemv_c": (40, 128)}.items():
        W, x = synth.normal_f16(1, (N, K), 0.05), synth.normal_f16(2, (1, K), 1.0)
        v[tag + "_W"], v[tag + "_x"], v[tag + "_y"] = W, x, o.matmul2d(x, W)
    # HGEMM: ragged M/N, K multiple of 64 and not
    for tag, (M, N, K) in {"hgemm_a": (70, 50, 192), "hgemm_b": (37, 65, 136)}.items():
        A, B = synth.normal_f16(3, (M, K), 1.0), synth.normal_f16(4, (N, K), 0.05)
        v[tag + "_A"], v[tag + "_B"], v[tag + "_C"] = A, B, o.matmul2d(A, B)
    x = synth.normal_f16(5, (2, 3, 4, 64), 1.0)
    v["rope_x"], v["rope_y"] = x, o.rope(x, 7)
    v["rope_start"] = np.array(7)
    s = synth.normal_f16(6, (9, 77), 2.0)
    v["softmax_x"], v["softmax_y"] = s, o.softmax(s)
    r, w = synth.normal_f16(7, (3, 264), 1.0), synth.normal_f16(8, (264,), 1.0)
    v["rms_x"], v["rms_w"], v["rms_y"] = r, w, o.rms_norm(r, w, 1e-5, "fused")
    a, b = synth.normal_f16(9, (515,), 2.0), synth.normal_f16(10, (515,), 2.0)
    v["ew_a"], v["ew_b"] = a, b
    v["silu_y"], v["silu_mul_y"] = o.silu(a), o.silu_mul(a, b)
    for op in ("add", "sub", "mul", "div"):
        v["bin_" + op] = o.binary(a, b, op)
    v["div_scalar"] = o.binary_scalar(a, np.float16(11.3125), "div")
    # attention (after RoPE): prefill of 40 tokens at position 5, and one decode row at position 45
    H, S, D, start = 2, 40, 64, 5
    q = synth.normal_f16(12, (H, S, D), 1.0)
    ck, cv = synth.normal_f16(13, (64, H, D), 1.0), synth.normal_f16(14, (64, H, D), 1.0)
    v["att_q"], v["att_k"], v["att_v"], v["att_start"] = q, ck, cv, np.array(start)
    v["att_prefill_y"] = o.attention_chain(q, ck, cv, start)
    q1 = synth.normal_f16(15, (H, 1, D), 1.0)
    v["att_q1"], v["att_decode_y"] = q1, o.attention_chain(q1, ck, cv, 45)
    # residual add -> RMSNorm -> projection (the chain the fused GEMV prologue replaces)
    hh, dd, gg = synth.normal_f16(16, (1, 512), 1.0), synth.normal_f16(17, (1, 512), 0.7), synth.normal_f16(18, (512,), 1.0)
    Wn = synth.normal_f16(19, (48, 512), 0.05)
    sm = o.binary(hh, dd, "add")
    v["nrm_h"], v["nrm_d"], v["nrm_g"], v["nrm_W"] = hh, dd, gg, Wn
    v["nrm_sum"], v["nrm_y"] = sm, o.matmul2d(o.rms_norm(sm, gg, 1e-5, "exact"), Wn)
    am = synth.normal_f16(11, (6, 300), 1.0)
    v["argmax_x"], v["argmax_y"] = am, o.argmax(am)
    return v


if __name__ == "__main__":
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hotpath_vectors.npz")
    np.savez_compressed(out, **build())
    print(out, os.path.getsize(out), "bytes")
