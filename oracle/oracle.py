"""ctypes front end of the CPU oracle (oracle/tl_oracle.c).

TEST INFRASTRUCTURE ONLY.  Imported by tests/, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py``; the product package never imports it.

All functions take and return numpy arrays; fp16 data is ``np.float16`` (reinterpreted as
uint16 bit patterns at the C boundary).  Each wrapper names the reference lines the C
function restates.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libtl_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile oracle/tl_oracle.c with gcc (see oracle/Makefile)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.tlo_max_threads.restype = ctypes.c_int
    return _lib


def max_threads() -> int:
    return int(lib().tlo_max_threads())


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def _h(a) -> np.ndarray:
    a = np.ascontiguousarray(a)
    if a.dtype != np.float16:
        raise TypeError(f"expected float16, got {a.dtype}")
    return a


_sz = ctypes.c_size_t


def h2f(bits: np.ndarray) -> np.ndarray:
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    out = np.empty(bits.shape, np.float32)
    lib().tlo_h2f(_p(bits), _p(out), _sz(bits.size))
    return out


def f2h(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().tlo_f2h(_p(x), _p(out), _sz(x.size))
    return out


def matmul2d(A: np.ndarray, B: np.ndarray) -> np.ndarray:
    """C[M,N] = A[M,K] . B[N,K]^T (tensorLib/src/device/cpu/CPU.cpp:76-89)."""
    A, B = _h(A), _h(B)
    M, K = A.shape
    N, K2 = B.shape
    assert K == K2
    C = np.empty((M, N), np.float16)
    lib().tlo_matmul2d_f16(_p(A), _p(B), _p(C), _sz(M), _sz(N), _sz(K))
    return C


def matmul2d_entries(A: np.ndarray, B: np.ndarray, ii: np.ndarray, jj: np.ndarray) -> np.ndarray:
    """Selected entries C[ii[e], jj[e]] with the same arithmetic as matmul2d."""
    A, B = _h(A), _h(B)
    ii = np.ascontiguousarray(ii, dtype=np.int64)
    jj = np.ascontiguousarray(jj, dtype=np.int64)
    out = np.empty(ii.shape, np.float16)
    lib().tlo_matmul2d_f16_entries(_p(A), _p(B), _p(out), _p(ii), _p(jj), _sz(ii.size), _sz(A.shape[1]))
    return out


def matmul2d_f32(A: np.ndarray, B: np.ndarray) -> np.ndarray:
    A = np.ascontiguousarray(A, dtype=np.float32)
    B = np.ascontiguousarray(B, dtype=np.float32)
    M, K = A.shape
    N = B.shape[0]
    C = np.empty((M, N), np.float32)
    lib().tlo_matmul2d_f32(_p(A), _p(B), _p(C), _sz(M), _sz(N), _sz(K))
    return C


def matmul2d_batched(A, B, batch, M, N, K, sA, sB) -> np.ndarray:
    """Batch loop of ops::matmul::call2 (tensorLib/src/ops/matmul.cpp:297-321)."""
    A, B = _h(A), _h(B)
    C = np.empty((batch, M, N), np.float16)
    lib().tlo_matmul2d_batched_f16(_p(A), _p(B), _p(C), _sz(M), _sz(N), _sz(K), _sz(batch),
                                   _sz(sA), _sz(sB), _sz(M * N))
    return C


def rope(x: np.ndarray, start_pos: int) -> np.ndarray:
    """x: [B,T,H,D] (tensorLib/src/device/cpu/CPU.cpp:427-461)."""
    x = _h(x)
    B, T, H, D = x.shape
    out = np.empty_like(x)
    lib().tlo_rope_f16(_p(x), _p(out), ctypes.c_int(start_pos), ctypes.c_int(B), ctypes.c_int(T),
                       ctypes.c_int(H), ctypes.c_int(D))
    return out


def softmax(x: np.ndarray, literal: bool = False) -> np.ndarray:
    """Row softmax of [rows, cols] (tensorLib/src/device/cpu/softmax.cpp:9-31)."""
    x = _h(x)
    rows, cols = x.shape
    out = np.empty_like(x)
    fn = lib().tlo_softmax_f16_literal if literal else lib().tlo_softmax_f16_f32
    fn(_p(x), _p(out), _sz(rows), _sz(cols))
    return out


def rms_norm(x: np.ndarray, w: np.ndarray, eps: float, variant: str = "fused") -> np.ndarray:
    """variant: 'fused' (tensorLib/src/device/cuda/rms_norm.cu:139-167), 'exact' (float64
    definition) or 'plain_literal' (tensorLib/src/nn/rmsNorm.cpp:14-56 via CPU half ops)."""
    x, w = _h(x), _h(w)
    tokens, hidden = x.shape
    out = np.empty_like(x)
    fn = {"fused": lib().tlo_rms_norm_f16_fused, "exact": lib().tlo_rms_norm_f16_exact,
          "plain_literal": lib().tlo_rms_norm_f16_plain_literal}[variant]
    fn(_p(x), _p(w), _p(out), ctypes.c_float(eps), ctypes.c_int(hidden), ctypes.c_int(tokens))
    return out


def silu(x: np.ndarray, cpu_literal: bool = False) -> np.ndarray:
    x = _h(x)
    out = np.empty_like(x)
    fn = lib().tlo_silu_f16_cpu_literal if cpu_literal else lib().tlo_silu_f16
    fn(_p(x), _p(out), _sz(x.size))
    return out


_OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3}


def binary(a: np.ndarray, b: np.ndarray, op: str) -> np.ndarray:
    a, b = _h(a), _h(b)
    assert a.shape == b.shape
    out = np.empty_like(a)
    lib().tlo_binary_f16(_p(a), _p(b), _p(out), _sz(a.size), ctypes.c_int(_OPS[op]))
    return out


def binary_scalar(a: np.ndarray, s, op: str) -> np.ndarray:
    a = _h(a)
    out = np.empty_like(a)
    bits = int(np.float16(s).view(np.uint16))
    lib().tlo_binary_scalar_f16(_p(a), ctypes.c_uint16(bits), _p(out), _sz(a.size), ctypes.c_int(_OPS[op]))
    return out


def silu_mul(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    a, b = _h(a), _h(b)
    out = np.empty_like(a)
    lib().tlo_silu_mul_f16(_p(a), _p(b), _p(out), _sz(a.size))
    return out


def attention_chain(q: np.ndarray, cache_k: np.ndarray, cache_v: np.ndarray, start_pos: int) -> np.ndarray:
    """Attention::forward after RoPE, composed from the CPU ops one for one
    (model/llama2_7b/src/Transformer.cpp:61-109): per head matmul2d(q, keys), ScalarDiv by
    half(sqrt(head_dim)), mask EwiseAdd (only when more than one token, Transformer.cpp:234), softmax(3),
    matmul2d(scores, values^T).  q: [H, S, D] rotated; caches [>= start_pos + S, H, D].
    Returns [S, H, D]."""
    q = _h(q)
    H, S, D = q.shape
    T = start_pos + S
    div = np.float16(np.sqrt(np.float32(D)))
    mask = np.where(np.arange(T)[None, :] > start_pos + np.arange(S)[:, None], -np.inf, 0.0).astype(np.float16)
    out = np.empty((S, H, D), np.float16)
    for h in range(H):
        k = np.ascontiguousarray(cache_k[:T, h, :])
        vt = np.ascontiguousarray(cache_v[:T, h, :].T)
        sc = binary_scalar(matmul2d(np.ascontiguousarray(q[h]), k), div, "div")
        if S > 1:
            sc = binary(sc, mask, "add")
        out[:, h, :] = matmul2d(softmax(sc), vt)
    return out


def _ints(v):
    return (ctypes.c_int * len(v))(*[int(i) for i in v])


def contiguous(base: np.ndarray, shape, stride, offset: int) -> np.ndarray:
    """tensorLib/src/device/cpu/CPU.cpp:127-139 (strides/offset in elements)."""
    base = _h(base)
    n = int(np.prod(shape))
    out = np.empty(tuple(shape), np.float16)
    lib().tlo_contiguous_f16(_p(base), _p(out), _ints(shape), _ints(stride), ctypes.c_int(len(shape)),
                             _sz(offset), _sz(n))
    return out


def set_item_ewise(base: np.ndarray, src: np.ndarray, shape, stride, offset: int) -> np.ndarray:
    """tensorLib/src/device/cpu/CPU.cpp:141-154; returns the updated copy of base."""
    base = _h(base).copy()
    src = _h(src)
    n = int(np.prod(shape))
    lib().tlo_set_item_ewise_f16(_p(base), _p(src), _ints(shape), _ints(stride), ctypes.c_int(len(shape)),
                                 _sz(offset), _sz(n))
    return base


def argmax(x: np.ndarray) -> np.ndarray:
    """Last-dim argmax, first maximum wins (tensorLib/src/device/cpu/CPU.cpp:356-372)."""
    x = _h(x)
    reduce_size = x.shape[-1]
    out = np.empty(x.size // reduce_size, np.int32)
    lib().tlo_argmax_f16(_p(x), _p(out), _sz(reduce_size), _sz(x.size))
    return out.reshape(x.shape[:-1])


def embedding(table: np.ndarray, ids: np.ndarray) -> np.ndarray:
    table = _h(table)
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    out = np.empty((ids.size, table.shape[1]), np.float16)
    lib().tlo_embedding_f16(_p(table), _p(ids), _p(out), ctypes.c_int(ids.size), ctypes.c_int(table.shape[1]))
    return out
