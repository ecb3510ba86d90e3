"""Python mirror of the reference's ``Device<half>`` interface over the C ABI.

Method names and argument meaning follow tensorLib/include/device/Device.hpp:13-101; the
``matmul`` method follows ``ops::matmul<dtype>::call2`` (tensorLib/src/ops/matmul.cpp:206-324)
including its error behaviour (``ValueError`` where the reference throws
``std::invalid_argument``).  Tensors are torch CUDA tensors used purely as device memory:
every computation happens in libtensorlib_amd.so.
"""
from __future__ import annotations

import ctypes
import math

import numpy as np
import torch

from ._lib import TensorLibError, check, lib

_OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3}


def _ptr(t: torch.Tensor) -> ctypes.c_void_p:
    return ctypes.c_void_p(t.data_ptr())


def _req(t: torch.Tensor, dtype=torch.float16, name="tensor") -> torch.Tensor:
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TensorLibError(f"{name} must be a CUDA(HIP) tensor; there is no CPU path")
    if t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    return t


def _ints(v):
    return (ctypes.c_int * len(v))(*[int(i) for i in v])


def half_bits(x: float) -> int:
    return int(np.float16(x).view(np.uint16))


def plan_matmul(a_shape, b_shape, out_shape=None):
    """Shape logic of ``ops::matmul<dtype>::call2`` (tensorLib/src/ops/matmul.cpp:209-286) for
    ``a[..., M, K] @ b[..., K, N]``: validates, right-aligns and broadcasts the batch dimensions.
    Returns ``(a_batch, b_batch, out_batch, M, N, K)`` with the batch shapes padded to equal rank.
    Raises ``ValueError`` where the reference throws ``std::invalid_argument``."""
    a_shape, b_shape = list(a_shape), list(b_shape)
    if len(a_shape) < 2 or len(b_shape) < 2:
        raise ValueError("Tensors must have at least 2 dimensions for matmul.")
    if a_shape[-1] != b_shape[-2]:
        raise ValueError("Shape mismatch: the number of columns in the first tensor must match the number "
                         "of rows in the second tensor.")
    M, K = a_shape[-2:]
    N = b_shape[-1]
    ab, bb = a_shape[:-2], b_shape[:-2]
    nb = max(len(ab), len(bb))
    ab = [1] * (nb - len(ab)) + ab
    bb = [1] * (nb - len(bb)) + bb
    ob = []
    for x, y in zip(ab, bb):
        if x != y and x != 1 and y != 1:
            raise ValueError("Shape mismatch: the batch dimensions must be broadcastable.")
        ob.append(max(x, y))
    if out_shape is not None and list(out_shape) != ob + [M, N]:
        raise ValueError("result shape does not match new_shape")
    return ab, bb, ob, M, N, K


class HipDevice:
    """One GPU; all work goes to the library's stream (torch's current stream by default)."""

    def __init__(self, ordinal: int = 0, bind_torch_stream: bool = True):
        if not torch.cuda.is_available():
            raise TensorLibError("no HIP device visible: tensorlib_amd has no CPU fallback")
        self.lib = lib()
        self.ordinal = ordinal
        torch.cuda.set_device(ordinal)
        check(self.lib.tl_init(ordinal), "tl_init")
        if bind_torch_stream:
            self.bind_stream(torch.cuda.current_stream())
        self.device = torch.device("cuda", ordinal)

    # -- runtime ---------------------------------------------------------------------
    def bind_stream(self, stream: "torch.cuda.Stream | None") -> None:
        raw = 0 if stream is None else stream.cuda_stream
        check(self.lib.tl_set_stream(ctypes.c_void_p(raw)), "tl_set_stream")

    def synchronize(self) -> None:
        check(self.lib.tl_synchronize(), "tl_synchronize")

    @property
    def cu_count(self) -> int:
        return int(self.lib.tl_device_cu_count())

    def empty(self, *shape, dtype=torch.float16) -> torch.Tensor:
        return torch.empty(*shape, dtype=dtype, device=self.device)

    def from_numpy(self, a: np.ndarray) -> torch.Tensor:
        return torch.from_numpy(np.ascontiguousarray(a)).to(self.device)

    # -- the hot path ----------------------------------------------------------------
    def matmul2d(self, A: torch.Tensor, B: torch.Tensor, C: torch.Tensor | None = None) -> torch.Tensor:
        """C[M,N] = A[M,K] . B[N,K]^T (Device.hpp:22)."""
        _req(A, name="A"), _req(B, name="B")
        M, K = A.shape
        N, K2 = B.shape
        if K != K2:
            raise ValueError("Shape mismatch: inner dimensions differ")
        if C is None:
            C = self.empty(M, N)
        _req(C, name="C")
        if tuple(C.shape) != (M, N):
            raise ValueError("result shape does not match new_shape")
        check(self.lib.tl_matmul2d_f16(_ptr(A), _ptr(B), _ptr(C), M, N, K), "tl_matmul2d_f16")
        return C

    def gemv(self, x: torch.Tensor, W: torch.Tensor, y: torch.Tensor | None = None) -> torch.Tensor:
        _req(x, name="x"), _req(W, name="W")
        N, K = W.shape
        if x.numel() != K:
            raise ValueError("Shape mismatch: x length differs from K")
        if y is None:
            y = self.empty(N)
        _req(y, name="y")
        check(self.lib.tl_gemv_f16(_ptr(x), _ptr(W), _ptr(y), N, K), "tl_gemv_f16")
        return y

    def hgemm(self, A: torch.Tensor, B: torch.Tensor, C: torch.Tensor | None = None) -> torch.Tensor:
        _req(A, name="A"), _req(B, name="B")
        M, K = A.shape
        N, K2 = B.shape
        if K != K2:
            raise ValueError("Shape mismatch: inner dimensions differ")
        if C is None:
            C = self.empty(M, N)
        _req(C, name="C")
        check(self.lib.tl_hgemm_f16(_ptr(A), _ptr(B), _ptr(C), M, N, K), "tl_hgemm_f16")
        return C

    def matmul2d_f32(self, A: torch.Tensor, B: torch.Tensor) -> torch.Tensor:
        _req(A, torch.float32, "A"), _req(B, torch.float32, "B")
        M, K = A.shape
        N, K2 = B.shape
        if K != K2:
            raise ValueError("Shape mismatch: inner dimensions differ")
        C = self.empty(M, N, dtype=torch.float32)
        check(self.lib.tl_matmul2d_f32(_ptr(A), _ptr(B), _ptr(C), M, N, K), "tl_matmul2d_f32")
        return C

    def matmul(self, a: torch.Tensor, b: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        """``Tensor::matmul`` semantics: a[..., M, K] @ b[..., K, N] with broadcast batch dims
        (tensorLib/src/ops/matmul.cpp:206-324).  ``b`` is transposed to the [N, K] operand the
        boundary wants; for a Linear weight passed as ``W.t()`` no copy is made."""
        if a.device != b.device:
            raise ValueError("Tensors must be on the same device.")
        for t, name in ((a, "a"), (b, "b")):          # strided views are fine here, dtype and device are not negotiable
            if not isinstance(t, torch.Tensor) or not t.is_cuda:
                raise TensorLibError(f"{name} must be a CUDA(HIP) tensor; there is no CPU path")
            if t.dtype != torch.float16:
                raise TypeError(f"{name} must be torch.float16, got {t.dtype}")
        ab, bb, obatch, M, N, K = plan_matmul(a.shape, b.shape, None if out is None else out.shape)
        # The temporaries below return to torch's caching allocator while the kernel may still be queued: that is
        # safe only because the library enqueues on the stream torch considers current, which is checked here.
        if (self.lib.tl_get_stream() or 0) != torch.cuda.current_stream().cuda_stream:
            raise TensorLibError("the library stream is not torch's current stream; call bind_stream(torch.cuda.current_stream()) first")
        A = a.contiguous()
        Bt = b.transpose(-2, -1).contiguous()  # [..., N, K]; a view of a Linear weight stays a view
        oshape = obatch + [M, N]
        if out is None:
            out = self.empty(*oshape)
        _req(out, name="out")
        batch = int(np.prod(obatch)) if obatch else 1
        if batch == 1:
            check(self.lib.tl_matmul2d_f16(_ptr(A), _ptr(Bt), _ptr(out), M, N, K), "tl_matmul2d_f16")
            return out
        # one batched launch when each operand is either fully batched or a single matrix
        a_full, b_full = int(np.prod(ab)) == batch, int(np.prod(bb)) == batch
        a_one, b_one = int(np.prod(ab)) == 1, int(np.prod(bb)) == 1
        if (a_full or a_one) and (b_full or b_one):
            check(self.lib.tl_matmul2d_batched_f16(_ptr(A), _ptr(Bt), _ptr(out), M, N, K, batch,
                                                   M * K if a_full else 0, N * K if b_full else 0, M * N),
                  "tl_matmul2d_batched_f16")
            return out
        # general broadcast: the reference's per-matrix loop (matmul.cpp:297-321)
        Ae = A.reshape(ab + [M, K]).expand(obatch + [M, K])
        Be = Bt.reshape(bb + [N, K]).expand(obatch + [N, K])
        o3 = out.view(batch, M, N)
        for i, idx in enumerate(np.ndindex(*obatch)):
            Ai, Bi = Ae[idx], Be[idx]
            esz = 2
            check(self.lib.tl_matmul2d_f16(ctypes.c_void_p(Ai.data_ptr()), ctypes.c_void_p(Bi.data_ptr()),
                                           ctypes.c_void_p(o3.data_ptr() + i * M * N * esz), M, N, K),
                  "tl_matmul2d_f16")
        return out

    # -- small ops --------------------------------------------------------------------
    def rms_norm(self, x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor | None = None):
        _req(x, name="x"), _req(weight, name="weight")
        hidden = x.shape[-1]
        tokens = x.numel() // hidden
        out = torch.empty_like(x) if out is None else _req(out, name="out")
        check(self.lib.tl_rms_norm_f16(_ptr(out), _ptr(x), _ptr(weight), eps, hidden, tokens), "tl_rms_norm_f16")
        return out

    def apply_rotary_emb(self, x: torch.Tensor, start_pos: int, out: torch.Tensor | None = None):
        _req(x, name="x")
        if x.dim() != 4:
            raise ValueError("apply_rotary_emb expects [B, T, n_heads, head_dim]")
        B, T, H, D = x.shape
        out = torch.empty_like(x) if out is None else _req(out, name="out")
        check(self.lib.tl_apply_rotary_emb_f16(_ptr(x), _ptr(out), start_pos, B, T, H, D), "tl_apply_rotary_emb_f16")
        return out

    def softmax(self, x: torch.Tensor, out: torch.Tensor | None = None):
        _req(x, name="x")
        cols = x.shape[-1]
        rows = x.numel() // cols if cols else 0
        out = torch.empty_like(x) if out is None else _req(out, name="out")
        check(self.lib.tl_softmax_f16(_ptr(out), _ptr(x), rows, cols), "tl_softmax_f16")
        return out

    def silu(self, x: torch.Tensor, out: torch.Tensor | None = None):
        _req(x, name="x")
        out = torch.empty_like(x) if out is None else _req(out, name="out")
        check(self.lib.tl_silu_f16(_ptr(out), _ptr(x), x.numel()), "tl_silu_f16")
        return out

    def silu_mul(self, a: torch.Tensor, b: torch.Tensor, out: torch.Tensor | None = None):
        _req(a, name="a"), _req(b, name="b")
        out = torch.empty_like(a) if out is None else _req(out, name="out")
        check(self.lib.tl_silu_mul_f16(_ptr(out), _ptr(a), _ptr(b), a.numel()), "tl_silu_mul_f16")
        return out

    def binary(self, a: torch.Tensor, b, op: str, out: torch.Tensor | None = None):
        _req(a, name="a")
        out = torch.empty_like(a) if out is None else _req(out, name="out")
        if isinstance(b, torch.Tensor):
            _req(b, name="b")
            if b.shape != a.shape:
                raise ValueError("Shape mismatch in elementwise op")
            check(self.lib.tl_binary_f16(_ptr(out), _ptr(a), _ptr(b), a.numel(), _OPS[op]), "tl_binary_f16")
        else:
            check(self.lib.tl_binary_scalar_f16(_ptr(out), _ptr(a), half_bits(b), a.numel(), _OPS[op]),
                  "tl_binary_scalar_f16")
        return out

    def add(self, a, b, out=None): return self.binary(a, b, "add", out)
    def sub(self, a, b, out=None): return self.binary(a, b, "sub", out)
    def mul(self, a, b, out=None): return self.binary(a, b, "mul", out)
    def div(self, a, b, out=None): return self.binary(a, b, "div", out)

    def contiguous(self, base: torch.Tensor, shape, stride, offset: int, out: torch.Tensor | None = None):
        _req(base, name="base")
        n = int(np.prod(shape))
        out = self.empty(*shape) if out is None else _req(out, name="out")
        check(self.lib.tl_contiguous_f16(_ptr(out), _ptr(base), _ints(shape), _ints(stride), len(shape), offset, n),
              "tl_contiguous_f16")
        return out

    def set_item_ewise(self, base: torch.Tensor, src: torch.Tensor, shape, stride, offset: int):
        _req(base, name="base"), _req(src, name="src")
        n = int(np.prod(shape))
        check(self.lib.tl_set_item_ewise_f16(_ptr(base), _ptr(src), _ints(shape), _ints(stride), len(shape), offset, n),
              "tl_set_item_ewise_f16")
        return base

    def argmax(self, x: torch.Tensor) -> torch.Tensor:
        _req(x, name="x")
        reduce_size = x.shape[-1]
        out = torch.empty(x.shape[:-1], dtype=torch.int32, device=self.device)
        check(self.lib.tl_argmax_f16(_ptr(out), _ptr(x), reduce_size, x.numel()), "tl_argmax_f16")
        return out

    def embedding(self, table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
        _req(table, name="table"), _req(ids, torch.int32, "ids")
        vocab, dim = table.shape
        out = self.empty(ids.numel(), dim)
        check(self.lib.tl_embedding_f16(_ptr(out), _ptr(table), _ptr(ids), ids.numel(), dim, vocab), "tl_embedding_f16")
        return out

    def full(self, out: torch.Tensor, value: float) -> torch.Tensor:
        _req(out, name="out")
        check(self.lib.tl_full_f16(_ptr(out), half_bits(value), out.numel()), "tl_full_f16")
        return out

    def causal_mask(self, reps: int, seqlen: int, start_pos: int) -> torch.Tensor:
        out = self.empty(reps, seqlen, start_pos + seqlen)
        check(self.lib.tl_causal_mask_f16(_ptr(out), reps, seqlen, start_pos), "tl_causal_mask_f16")
        return out

    def decode_attention(self, q: torch.Tensor, cache_k: torch.Tensor, cache_v: torch.Tensor, T: int):
        """q: [n_heads, head_dim]; caches: [max_seq, n_heads, head_dim]; attends to positions < T."""
        _req(q, name="q"), _req(cache_k, name="cache_k"), _req(cache_v, name="cache_v")
        H, D = q.shape
        if cache_k.shape[1:] != (H, D) or cache_v.shape != cache_k.shape or T > cache_k.shape[0]:
            raise ValueError("cache shape does not match q / T")
        out = torch.empty_like(q)
        check(self.lib.tl_decode_attention_f16(_ptr(out), _ptr(q), _ptr(cache_k), _ptr(cache_v), T, H, D),
              "tl_decode_attention_f16")
        return out

    def rope_table(self, max_seq: int, head_dim: int) -> torch.Tensor:
        t = self.empty(max_seq, head_dim // 2, 2)
        check(self.lib.tl_rope_table_f16(_ptr(t), max_seq, head_dim), "tl_rope_table_f16")
        return t

    def decode_attention_rope(self, qkv: torch.Tensor, cache_k: torch.Tensor, cache_v: torch.Tensor, pos: int,
                              rope_table: torch.Tensor | None = None, out: torch.Tensor | None = None,
                              static_scratch: bool = False):
        """qkv: [3, n_heads, head_dim] raw projections of the token at `pos`; writes cache rows `pos`.
        static_scratch: go through the entry point that allocates nothing (then pass `out` too)."""
        _req(qkv, name="qkv"), _req(cache_k, name="cache_k"), _req(cache_v, name="cache_v")
        _, H, D = qkv.shape
        if cache_k.shape[1:] != (H, D) or cache_v.shape != cache_k.shape or pos >= cache_k.shape[0]:
            raise ValueError("cache shape does not match qkv / pos")
        out = self.empty(H, D) if out is None else _req(out, name="out")
        tab = ctypes.c_void_p(0) if rope_table is None else _ptr(_req(rope_table, name="rope_table"))
        if static_scratch:
            check(self.lib.tl_decode_attention_rope_static_f16(_ptr(out), _ptr(qkv), _ptr(cache_k), _ptr(cache_v), tab,
                                                               pos, H, D), "tl_decode_attention_rope_static_f16")
        else:
            check(self.lib.tl_decode_attention_rope_f16(_ptr(out), _ptr(qkv), _ptr(cache_k), _ptr(cache_v), tab, pos, H, D),
                  "tl_decode_attention_rope_f16")
        return out

    def rope_qk_store_kv(self, qkv: torch.Tensor, cache_k: torch.Tensor, cache_v: torch.Tensor, pos: int):
        _req(qkv, name="qkv"), _req(cache_k, name="cache_k"), _req(cache_v, name="cache_v")
        _, H, D = qkv.shape
        check(self.lib.tl_rope_qk_store_kv_f16(_ptr(qkv), _ptr(cache_k), _ptr(cache_v), pos, H, D),
              "tl_rope_qk_store_kv_f16")

    def hgemm_add_rms_norm(self, A: torch.Tensor, W: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float):
        """(residual + A . W^T, rmsnorm of that sum * weight) for [M, K] rows: a projection, the residual add and the
        norm that follows it; a split-K GEMM's second pass happens inside the add + norm kernel."""
        _req(A, name="A"), _req(W, name="W"), _req(residual, name="residual"), _req(weight, name="weight")
        M, K = A.shape
        N = W.shape[0]
        if W.shape[1] != K or residual.shape != (M, N) or weight.numel() != N:
            raise ValueError("shape mismatch")
        s, n = self.empty(M, N), self.empty(M, N)
        check(self.lib.tl_hgemm_add_rms_norm_f16(_ptr(A), _ptr(W), _ptr(residual), _ptr(weight), eps, _ptr(s), _ptr(n), M, N, K),
              "tl_hgemm_add_rms_norm_f16")
        return s, n

    def add_rms_norm(self, a: torch.Tensor, b: torch.Tensor, weight: torch.Tensor, eps: float, sum_out=None, norm_out=None):
        _req(a, name="a"), _req(b, name="b"), _req(weight, name="weight")
        hidden = a.shape[-1]
        tokens = a.numel() // hidden
        sum_out = torch.empty_like(a) if sum_out is None else sum_out
        norm_out = torch.empty_like(a) if norm_out is None else norm_out
        check(self.lib.tl_add_rms_norm_f16(_ptr(sum_out), _ptr(norm_out), _ptr(a), _ptr(b), _ptr(weight), eps, hidden,
                                           tokens), "tl_add_rms_norm_f16")
        return sum_out, norm_out

    def gemv_silu_mul(self, ab: torch.Tensor, W: torch.Tensor) -> torch.Tensor:
        """y = W . (silu(ab[:K]) * ab[K:]) with W [N, K] and ab of 2*K halves."""
        _req(ab, name="ab"), _req(W, name="W")
        N, K = W.shape
        if ab.numel() != 2 * K:
            raise ValueError("ab must hold 2*K elements")
        y = self.empty(N)
        check(self.lib.tl_gemv_silu_mul_f16(_ptr(ab), _ptr(W), _ptr(y), N, K), "tl_gemv_silu_mul_f16")
        return y

    def gemv_add_rms_norm(self, x: torch.Tensor, addend, weight: torch.Tensor, eps: float, W: torch.Tensor,
                          want_sum: bool = True):
        """(y, x + addend) with y = W . (rmsnorm(x + addend) * weight); addend may be None."""
        _req(x, name="x"), _req(weight, name="weight"), _req(W, name="W")
        if addend is not None:
            _req(addend, name="addend")
        N, K = W.shape
        if x.numel() != K or weight.numel() != K or (addend is not None and addend.numel() != K):
            raise ValueError("x, addend and weight must hold K elements")
        y = self.empty(N)
        s = self.empty(K) if want_sum else None
        check(self.lib.tl_gemv_add_rms_norm_f16(_ptr(x), _ptr(addend) if addend is not None else None, _ptr(weight),
                                                float(eps), _ptr(W), _ptr(y), _ptr(s) if s is not None else None, N, K),
              "tl_gemv_add_rms_norm_f16")
        return y, s

    def prefill_rope_qkv(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cache_k: torch.Tensor,
                         cache_v: torch.Tensor, table: torch.Tensor, start_pos: int, n_heads: int) -> torch.Tensor:
        """q, k, v: [S, n_heads*head_dim] views sharing one row stride (e.g. column blocks of a fused
        [S, 3*dim] projection).  Returns rotated q as [n_heads, S, head_dim]; rotated k and v go into
        cache rows [start_pos, start_pos + S)."""
        for t, nm in ((q, "q"), (k, "k"), (v, "v")):
            if t.dtype != torch.float16 or not t.is_cuda or t.dim() != 2 or t.stride(1) != 1:
                raise ValueError(f"{nm} must be a 2-D fp16 device tensor with unit column stride")
        S, dim = q.shape
        ld = q.stride(0)
        if k.stride(0) != ld or v.stride(0) != ld or k.shape != q.shape or v.shape != q.shape:
            raise ValueError("q, k, v must share shape and row stride")
        D = dim // n_heads
        out = torch.empty((n_heads, S, D), dtype=torch.float16, device=q.device)
        check(self.lib.tl_prefill_rope_qkv_f16(_ptr(out), q.data_ptr(), k.data_ptr(), v.data_ptr(), ld, _ptr(cache_k),
                                               _ptr(cache_v), _ptr(table), start_pos, S, n_heads, D),
              "tl_prefill_rope_qkv_f16")
        return out


    def prefill_rope_qkv_vt(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cache_k: torch.Tensor,
                            cache_v: torch.Tensor, table: torch.Tensor, n_heads: int):
        """prefill_rope_qkv at start_pos 0 that also returns the transposed value operand of prefill_attention
        ([n_heads, head_dim, ldv], ldv = tokens rounded up to 64, zero padded)."""
        for t, nm in ((q, "q"), (k, "k"), (v, "v")):
            if t.dtype != torch.float16 or not t.is_cuda or t.dim() != 2 or t.stride(1) != 1:
                raise ValueError(f"{nm} must be a 2-D fp16 device tensor with unit column stride")
        S, dim = q.shape
        ld = q.stride(0)
        if k.stride(0) != ld or v.stride(0) != ld or k.shape != q.shape or v.shape != q.shape:
            raise ValueError("q, k, v must share shape and row stride")
        D = dim // n_heads
        ldv = (S + 63) // 64 * 64
        out = torch.empty((n_heads, S, D), dtype=torch.float16, device=q.device)
        vT = torch.empty((n_heads, D, ldv), dtype=torch.float16, device=q.device)
        check(self.lib.tl_prefill_rope_qkv_vt_f16(_ptr(out), q.data_ptr(), k.data_ptr(), v.data_ptr(), ld, _ptr(cache_k),
                                                  _ptr(cache_v), _ptr(table), _ptr(vT), ldv, S, n_heads, D),
              "tl_prefill_rope_qkv_vt_f16")
        return out, vT

    def hgemm_prefill_rope_qkv_vt(self, X: torch.Tensor, Wqkv: torch.Tensor, cache_k: torch.Tensor, cache_v: torch.Tensor,
                                  table: torch.Tensor, n_heads: int):
        """The fused q|k|v projection of a fresh context and prefill_rope_qkv_vt in one call (the rotating kernel adds
        up a split K itself).  X [S, K], Wqkv [3*dim, K].  Returns (q [n_heads, S, D], vT [n_heads, D, ldv])."""
        _req(X, name="X"), _req(Wqkv, name="Wqkv")
        S, K = X.shape
        N, K2 = Wqkv.shape
        if K != K2 or N % (3 * n_heads):
            raise ValueError("Shape mismatch: X [S, K] against Wqkv [3*n_heads*head_dim, K]")
        D = N // 3 // n_heads
        ldv = (S + 63) // 64 * 64
        qkv = torch.empty((S, N), dtype=torch.float16, device=X.device)
        out = torch.empty((n_heads, S, D), dtype=torch.float16, device=X.device)
        vT = torch.empty((n_heads, D, ldv), dtype=torch.float16, device=X.device)
        check(self.lib.tl_hgemm_prefill_rope_qkv_vt_f16(_ptr(X), _ptr(Wqkv), _ptr(qkv), _ptr(out), _ptr(cache_k), _ptr(cache_v),
                                                        _ptr(table), _ptr(vT), ldv, S, n_heads, D, K),
              "tl_hgemm_prefill_rope_qkv_vt_f16")
        return out, vT

    def scaled_causal_softmax(self, scores: torch.Tensor, divisor: float, start_pos: int) -> torch.Tensor:
        """In place on scores [n_heads, S, start_pos + S]: divide by half(divisor), causal mask, softmax."""
        _req(scores, name="scores")
        H, S, T = scores.shape
        if T != start_pos + S:
            raise ValueError("scores must be [n_heads, S, start_pos + S]")
        bits = int(np.array(divisor, dtype=np.float16).view(np.uint16))
        check(self.lib.tl_scaled_causal_softmax_f16(_ptr(scores), bits, H, S, start_pos), "tl_scaled_causal_softmax_f16")
        return scores

    def silu_mul_rows(self, ab: torch.Tensor) -> torch.Tensor:
        """ab: [rows, 2*hidden] -> silu(ab[:, :hidden]) * ab[:, hidden:]."""
        _req(ab, name="ab")
        rows, two_h = ab.shape
        out = torch.empty((rows, two_h // 2), dtype=torch.float16, device=ab.device)
        check(self.lib.tl_silu_mul_rows_f16(_ptr(out), _ptr(ab), rows, two_h // 2), "tl_silu_mul_rows_f16")
        return out

    def hgemm_silu_mul(self, X: torch.Tensor, W13: torch.Tensor, scratch: torch.Tensor | None = None) -> torch.Tensor:
        """silu(X @ W1.T) * (X @ W3.T) for W13 = [W1; W3] of shape [2*hidden, K]; one launch where the pipelined GEMM
        serves the shape, else GEMM into `scratch` ([M, 2*hidden], allocated here when not given) and the gate kernel."""
        _req(X, name="X"), _req(W13, name="W13")
        M, K = X.shape
        two_h, K2 = W13.shape
        if K != K2 or two_h % 2:
            raise ValueError("Shape mismatch: X [M, K] against W13 [2*hidden, K]")
        if scratch is None:
            scratch = torch.empty((M, two_h), dtype=torch.float16, device=X.device)
        _req(scratch, name="scratch")
        out = torch.empty((M, two_h // 2), dtype=torch.float16, device=X.device)
        check(self.lib.tl_hgemm_silu_mul_f16(_ptr(X), _ptr(W13), _ptr(scratch), _ptr(out), M, two_h // 2, K),
              "tl_hgemm_silu_mul_f16")
        return out

    def prefill_attention(self, q: torch.Tensor, cache_k: torch.Tensor, cache_v: torch.Tensor, start_pos: int):
        """q: [n_heads, S, head_dim] (rotated); caches [max_seq, n_heads, head_dim] holding positions
        < start_pos + S.  Returns [S, n_heads, head_dim]."""
        _req(q, name="q"), _req(cache_k, name="cache_k"), _req(cache_v, name="cache_v")
        H, S, D = q.shape
        T = start_pos + S
        ldv = (T + 63) // 64 * 64
        vT = self.empty(H, D, ldv)
        check(self.lib.tl_gather_vt_f16(_ptr(vT), _ptr(cache_v), T, ldv, H, D), "tl_gather_vt_f16")
        out = self.empty(S, H, D)
        check(self.lib.tl_prefill_attention_f16(_ptr(out), _ptr(q), _ptr(cache_k), _ptr(vT), ldv, start_pos, S, H, D),
              "tl_prefill_attention_f16")
        return out

    # -- tuning hooks -------------------------------------------------------------------
    def set_gemv_variant(self, v: int) -> None:
        check(self.lib.tl_set_gemv_variant(v), "tl_set_gemv_variant")

    def set_hgemm_variant(self, v: int) -> None:
        check(self.lib.tl_set_hgemm_variant(v), "tl_set_hgemm_variant")

    def gemv_variants(self) -> list[str]:
        out, i = [], 0
        while True:
            n = self.lib.tl_gemv_variant_name(i)
            if n is None:
                return out
            out.append(n.decode())
            i += 1

    def hgemm_last_plan(self) -> tuple[str, int]:
        """(kernel variant, K splits) of the most recent fp16 GEMM launch; the variant of the kernel for at most
        32 rows is reported as "fewrows"."""
        import ctypes
        v, s = ctypes.c_int(0), ctypes.c_int(0)
        check(self.lib.tl_hgemm_last_plan(ctypes.byref(v), ctypes.byref(s)), "tl_hgemm_last_plan")
        name = "fewrows" if v.value < 0 else self.lib.tl_hgemm_variant_name(v.value).decode()
        return name, s.value

    def hgemm_variants(self) -> list[str]:
        out, i = [], 0
        while True:
            n = self.lib.tl_hgemm_variant_name(i)
            if n is None:
                return out
            out.append(n.decode())
            i += 1
