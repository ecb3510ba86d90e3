"""CPU restatement of the reference's Llama2 forward pass, composed from the oracle's CPU-backend
ops (oracle/oracle.py).  TEST INFRASTRUCTURE ONLY.

Op order follows model/llama2_7b/src/Transformer.cpp:26-112 (Attention::forward), :132-145
(FeedForward::forward), :160-178 (TransformerBlock::forward), :263-299 (Transformer::forward),
with every intermediate rounded to fp16 as the reference stores it.  Two deliberate choices,
both forced by defects of the literal CPU path:
  * RMSNorm uses the semantics the model executes on the reference's GPU path
    (tensorLib/src/device/cuda/rms_norm.cu:139-167) and x_norm <- rmsnorm(x) is actually stored:
    the CPU forward_plain ignores its result buffer (tensorLib/src/nn/rmsNorm.cpp:36-56) so the
    literal CPU model reads stale data.
  * SiLU is x/(1+exp(-x)) (tensorLib/src/device/cuda/CUDA.cu:334-342); the CPU half branch has
    the exponent's sign flipped (tensorLib/src/device/cpu/CPU.cpp:216-219).
"""
from __future__ import annotations

import numpy as np

from . import oracle as o


class Llama2Oracle:
    def __init__(self, weights: dict, dim, hidden_dim, n_layers, n_heads, vocab_size, max_seq_len, eps=1e-5):
        self.w = weights
        self.dim, self.hidden, self.L, self.H = dim, hidden_dim, n_layers, n_heads
        self.D = dim // n_heads
        self.vocab, self.max_seq, self.eps = vocab_size, max_seq_len, eps
        self.cache_k = [np.zeros((max_seq_len, n_heads, self.D), np.float16) for _ in range(n_layers)]
        self.cache_v = [np.zeros((max_seq_len, n_heads, self.D), np.float16) for _ in range(n_layers)]

    def block(self, l: int, x: np.ndarray, start_pos: int) -> np.ndarray:
        w, H, D = self.w, self.H, self.D
        S = x.shape[0]
        T = start_pos + S
        x_norm = o.rms_norm(x, w[f"att_norm.{l}"], self.eps, "fused")
        xq = o.matmul2d(x_norm, w[f"wq.{l}"])
        xk = o.matmul2d(x_norm, w[f"wk.{l}"])
        xv = o.matmul2d(x_norm, w[f"wv.{l}"])
        xq = o.rope(xq.reshape(1, S, H, D), start_pos).reshape(S, H, D)
        xk = o.rope(xk.reshape(1, S, H, D), start_pos).reshape(S, H, D)
        self.cache_k[l][start_pos:T] = xk
        self.cache_v[l][start_pos:T] = xv.reshape(S, H, D)
        q_c = np.ascontiguousarray(xq.transpose(1, 0, 2))                 # [H,S,D]
        keys = np.ascontiguousarray(self.cache_k[l][:T].transpose(1, 0, 2))   # [H,T,D]
        vals = np.ascontiguousarray(self.cache_v[l][:T].transpose(1, 2, 0))   # [H,D,T]
        scores = o.matmul2d_batched(q_c, keys, H, S, T, D, S * D, T * D)       # [H,S,T]
        scores = o.binary_scalar(scores, np.sqrt(np.float32(D)), "div")
        if S > 1:
            j = np.arange(T)[None, :]
            i = np.arange(S)[:, None]
            mask = np.where(j > start_pos + i, -np.inf, 0.0).astype(np.float16)
            scores = o.binary(scores, np.broadcast_to(mask, scores.shape).copy(), "add")
        p = o.softmax(scores.reshape(H * S, T)).reshape(H, S, T)
        sv = o.matmul2d_batched(p, vals, H, S, D, T, S * T, D * T)             # [H,S,D]
        out = np.ascontiguousarray(sv.transpose(1, 0, 2)).reshape(S, self.dim)
        attn = o.matmul2d(out, w[f"wo.{l}"])
        h = o.binary(x, attn, "add")
        x_norm = o.rms_norm(h, w[f"ffn_norm.{l}"], self.eps, "fused")
        x1 = o.silu(o.matmul2d(x_norm, w[f"w1.{l}"]))
        x3 = o.matmul2d(x_norm, w[f"w3.{l}"])
        x2 = o.binary(x1, x3, "mul")
        ffn = o.matmul2d(x2, w[f"w2.{l}"])
        return o.binary(h, ffn, "add")

    def forward(self, tokens, start_pos: int, n_layers: int | None = None) -> np.ndarray:
        """Returns fp16 logits [n_tokens, vocab]."""
        x = o.embedding(self.w["tok_emb"], np.asarray(tokens, np.int32))
        for l in range(self.L if n_layers is None else n_layers):
            x = self.block(l, x, start_pos)
        self.last_hidden = x
        x_norm = o.rms_norm(x, self.w["final_norm"], self.eps, "fused")
        return o.matmul2d(x_norm, self.w["classifier"])
