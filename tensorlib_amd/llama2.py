"""ctypes binding of the C++ host-side Llama2 driver (libtensorlib_llama2.so,
include/tensorlib_llama2.h).  Weights are torch CUDA tensors used as device memory only."""
from __future__ import annotations

import ctypes
import os
from dataclasses import dataclass

import numpy as np
import torch

from ._lib import _PKG, TensorLibError, check, lib

LLAMA2_LIB_PATH = os.path.join(_PKG, "lib", "libtensorlib_llama2.so")

W_TOK_EMB, W_ATT_NORM, W_WQ, W_WK, W_WV, W_WO, W_FFN_NORM, W_W1, W_W2, W_W3, W_FINAL_NORM, W_CLASSIFIER = range(12)
MODE_REFERENCE_CHAIN, MODE_FUSED = 0, 1
BUF_X, BUF_LOGITS, BUF_CACHE_K, BUF_CACHE_V, BUF_NEXT_TOKEN = range(5)

_vp, _i, _f = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
_PROTOS = {
    "tlm_last_error": (ctypes.c_char_p, []),
    "tlm_create": (_i, [ctypes.POINTER(_vp), _i, _i, _i, _i, _i, _i, _f, _i]),
    "tlm_destroy": (_i, [_vp]),
    "tlm_set_weight": (_i, [_vp, _i, _i, _vp]),
    "tlm_forward": (_i, [_vp, _vp, _i, _i, _i, _i, ctypes.POINTER(_vp)]),
    "tlm_generate": (_i, [_vp, _vp, _i, _i, _i, _vp, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]),
    "tlm_text_completion": (_i, [_vp, _vp, ctypes.c_char_p, _i, ctypes.POINTER(_i), _i, _i, _vp, _vp, ctypes.POINTER(_i),
                                 ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]),
    "tlm_get_buffer": (_i, [_vp, _i, _i, ctypes.POINTER(_vp)]),
    "tlm_load_checkpoint": (_i, [ctypes.c_char_p, _i, _i, ctypes.POINTER(_vp)]),
    "tlm_get_config": (_i, [_vp, ctypes.POINTER(_i)]),
}
_PIECE_FN = ctypes.CFUNCTYPE(None, ctypes.POINTER(ctypes.c_char), ctypes.c_size_t, _i, _vp)
_llib = None


def llama2_lib() -> ctypes.CDLL:
    global _llib
    if _llib is None:
        lib()  # loads libtensorlib_amd.so first (RTLD_GLOBAL) so the driver binds to it
        if not os.path.exists(LLAMA2_LIB_PATH):
            raise TensorLibError(f"{LLAMA2_LIB_PATH} is missing: run `make -C tensorlib_amd/host`")
        h = ctypes.CDLL(LLAMA2_LIB_PATH)
        for name, (res, args) in _PROTOS.items():
            fn = getattr(h, name)
            fn.restype, fn.argtypes = res, args
        _llib = h
    return _llib


def _ck(status: int, what: str) -> None:
    if status != 0:
        raise TensorLibError(f"{what} failed: {llama2_lib().tlm_last_error().decode(errors='replace')}")


@dataclass
class Llama2Config:
    dim: int = 4096
    hidden_dim: int = 11008
    n_layers: int = 32
    n_heads: int = 32
    vocab_size: int = 32000
    max_seq_len: int = 2048
    norm_eps: float = 1e-5

    @property
    def head_dim(self) -> int:
        return self.dim // self.n_heads

    def weight_bytes_per_token(self) -> int:
        """fp16 weight bytes one decode step streams (all Linear weights + classifier)."""
        per_layer = 4 * self.dim * self.dim + 3 * self.hidden_dim * self.dim
        return 2 * (self.n_layers * per_layer + self.vocab_size * self.dim)


def write_checkpoint(path: str, cfg: Llama2Config, w: dict, shared_classifier: bool = False) -> None:
    """Write weights (name scheme of Llama2Model.set_weights) as a llama2.c legacy fp16 checkpoint:
    the layout script/export.py:138-190 produces and model/llama2_7b/src/main.cpp:36-228 reads.
    The rotary tables the format carries (seq_len * head_dim halves) are written as cos/sin of
    pos * 10000^(-2i/head_dim); readers of this format skip them."""
    import struct
    L = cfg.n_layers
    with open(path, "wb") as f:
        vocab = cfg.vocab_size if shared_classifier else -cfg.vocab_size
        f.write(struct.pack("iiiiiii", cfg.dim, cfg.hidden_dim, L, cfg.n_heads, cfg.n_heads, vocab, cfg.max_seq_len))

        def put(a):
            f.write(np.ascontiguousarray(a, dtype=np.float16).tobytes())
        put(w["tok_emb"])
        for name in ("att_norm", "wq", "wk", "wv", "wo", "ffn_norm", "w1", "w2", "w3"):
            for l in range(L):
                put(w[f"{name}.{l}"])
        put(w["final_norm"])
        half_d = cfg.head_dim // 2
        ang = np.outer(np.arange(cfg.max_seq_len), 10000.0 ** (-np.arange(half_d) * 2.0 / cfg.head_dim))
        put(np.cos(ang))
        put(np.sin(ang))
        if not shared_classifier:
            put(w["classifier"])


class Llama2Model:
    def __init__(self, dev, cfg: Llama2Config, max_tokens: int, _handle=None):
        self.dev, self.cfg, self.max_tokens = dev, cfg, max_tokens
        self.l = llama2_lib()
        self.weights = {}   # keeps the torch tensors alive
        if _handle is not None:
            self.h = _handle
            return
        h = _vp()
        _ck(self.l.tlm_create(ctypes.byref(h), cfg.dim, cfg.hidden_dim, cfg.n_layers, cfg.n_heads, cfg.vocab_size,
                              cfg.max_seq_len, cfg.norm_eps, max_tokens), "tlm_create")
        self.h = h

    @classmethod
    def from_checkpoint(cls, dev, path: str, max_tokens: int, max_seq_len: int = 0) -> "Llama2Model":
        """Load a llama2.c legacy fp16 .bin (the file the reference's read_checkpoint loads)."""
        l = llama2_lib()
        h = _vp()
        _ck(l.tlm_load_checkpoint(path.encode(), max_tokens, max_seq_len, ctypes.byref(h)), "tlm_load_checkpoint")
        c7 = (ctypes.c_int * 7)()
        _ck(l.tlm_get_config(h, c7), "tlm_get_config")
        cfg = Llama2Config(dim=c7[0], hidden_dim=c7[1], n_layers=c7[2], n_heads=c7[3], vocab_size=c7[4],
                           max_seq_len=c7[5])
        return cls(dev, cfg, c7[6], _handle=h)

    def close(self):
        if self.h:
            self.l.tlm_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _set(self, kind, layer, t: torch.Tensor):
        assert t.is_cuda and t.dtype == torch.float16 and t.is_contiguous()
        _ck(self.l.tlm_set_weight(self.h, kind, layer, _vp(t.data_ptr())), "tlm_set_weight")

    def set_weights(self, w: dict, fuse_layout: bool = True):
        """w: name -> np.float16 array, names as in the llama2.c export order
        (model/llama2_7b/src/main.cpp:36-190): tok_emb, final_norm, classifier and per layer l:
        att_norm.l, wq.l, wk.l, wv.l, wo.l, ffn_norm.l, w1.l, w2.l, w3.l.
        fuse_layout=True stores wq|wk|wv and w1|w3 adjacently so the fused mode can use one GEMV."""
        c, d = self.cfg, self.dev
        to = lambda a: d.from_numpy(a)  # noqa: E731
        self.weights["tok_emb"] = to(w["tok_emb"])
        self.weights["final_norm"] = to(w["final_norm"])
        self.weights["classifier"] = to(w["classifier"])
        self._set(W_TOK_EMB, 0, self.weights["tok_emb"])
        self._set(W_FINAL_NORM, 0, self.weights["final_norm"])
        self._set(W_CLASSIFIER, 0, self.weights["classifier"])
        for l in range(c.n_layers):
            if fuse_layout:
                qkv = to(np.concatenate([w[f"wq.{l}"], w[f"wk.{l}"], w[f"wv.{l}"]], axis=0))
                w13 = to(np.concatenate([w[f"w1.{l}"], w[f"w3.{l}"]], axis=0))
                wq, wk, wv = qkv[:c.dim], qkv[c.dim:2 * c.dim], qkv[2 * c.dim:]
                w1, w3 = w13[:c.hidden_dim], w13[c.hidden_dim:]
                self.weights[f"qkv.{l}"], self.weights[f"w13.{l}"] = qkv, w13
            else:
                wq, wk, wv, w1, w3 = (to(w[f"{n}.{l}"]) for n in ("wq", "wk", "wv", "w1", "w3"))
                self.weights[f"sep.{l}"] = (wq, wk, wv, w1, w3)
            rest = {n: to(w[f"{n}.{l}"]) for n in ("att_norm", "wo", "ffn_norm", "w2")}
            self.weights[f"rest.{l}"] = rest
            for kind, t in ((W_ATT_NORM, rest["att_norm"]), (W_WQ, wq), (W_WK, wk), (W_WV, wv), (W_WO, rest["wo"]),
                            (W_FFN_NORM, rest["ffn_norm"]), (W_W1, w1), (W_W2, rest["w2"]), (W_W3, w3)):
                self._set(kind, l, t)

    def random_init_on_device(self, seed: int = 0):
        """Random-init fp16 weights generated on the GPU (Linear ~ N(0, 0.02), norm weights ~ N(0,1)
        as nn::RMSNorm's constructor draws them, tensorLib/src/nn/rmsNorm.cpp:11; embedding ~ N(0,1))."""
        c = self.cfg
        g = torch.Generator(device="cuda")
        g.manual_seed(seed)

        def rn(shape, std):
            return (torch.randn(shape, generator=g, device="cuda", dtype=torch.float32) * std).to(torch.float16)
        self.weights["tok_emb"] = rn((c.vocab_size, c.dim), 1.0)
        self.weights["final_norm"] = rn((c.dim,), 1.0)
        self.weights["classifier"] = rn((c.vocab_size, c.dim), 0.02)
        self._set(W_TOK_EMB, 0, self.weights["tok_emb"])
        self._set(W_FINAL_NORM, 0, self.weights["final_norm"])
        self._set(W_CLASSIFIER, 0, self.weights["classifier"])
        for l in range(c.n_layers):
            qkv = rn((3 * c.dim, c.dim), 0.02)
            w13 = rn((2 * c.hidden_dim, c.dim), 0.02)
            rest = {"att_norm": rn((c.dim,), 1.0), "wo": rn((c.dim, c.dim), 0.02), "ffn_norm": rn((c.dim,), 1.0),
                    "w2": rn((c.dim, c.hidden_dim), 0.02)}
            self.weights[f"qkv.{l}"], self.weights[f"w13.{l}"], self.weights[f"rest.{l}"] = qkv, w13, rest
            for kind, t in ((W_ATT_NORM, rest["att_norm"]), (W_WQ, qkv[:c.dim]), (W_WK, qkv[c.dim:2 * c.dim]),
                            (W_WV, qkv[2 * c.dim:]), (W_WO, rest["wo"]), (W_FFN_NORM, rest["ffn_norm"]),
                            (W_W1, w13[:c.hidden_dim]), (W_W2, rest["w2"]), (W_W3, w13[c.hidden_dim:])):
                self._set(kind, l, t)

    def weights_to_numpy(self) -> dict:
        """Host copy of the weights in the name scheme of set_weights (for a host-side check)."""
        c = self.cfg
        out = {k: self.weights[k].cpu().numpy() for k in ("tok_emb", "final_norm", "classifier")}
        for l in range(c.n_layers):
            qkv, w13, rest = self.weights[f"qkv.{l}"], self.weights[f"w13.{l}"], self.weights[f"rest.{l}"]
            out[f"wq.{l}"], out[f"wk.{l}"], out[f"wv.{l}"] = (t.cpu().numpy() for t in qkv.split(c.dim))
            out[f"w1.{l}"], out[f"w3.{l}"] = (t.cpu().numpy() for t in w13.split(c.hidden_dim))
            for n in ("att_norm", "wo", "ffn_norm", "w2"):
                out[f"{n}.{l}"] = rest[n].cpu().numpy()
        return out

    def forward(self, tokens, start_pos: int, mode: int = MODE_FUSED, all_logits: bool = True) -> torch.Tensor:
        ids = torch.as_tensor(np.asarray(tokens, dtype=np.int32)).to(self.dev.device)
        n = ids.numel()
        ptr = _vp()
        _ck(self.l.tlm_forward(self.h, _vp(ids.data_ptr()), n, start_pos, mode, 1 if all_logits else 0,
                               ctypes.byref(ptr)), "tlm_forward")
        rows = n if all_logits else 1
        out = self.dev.empty(rows, self.cfg.vocab_size)
        check(self.dev.lib.tl_memcpy_d2d(_vp(out.data_ptr()), ptr, out.numel() * 2), "tl_memcpy_d2d")
        self.dev.synchronize()
        return out

    def get_buffer(self, which: int, layer: int, shape) -> torch.Tensor:
        ptr = _vp()
        _ck(self.l.tlm_get_buffer(self.h, which, layer, ctypes.byref(ptr)), "tlm_get_buffer")
        out = self.dev.empty(*shape)
        check(self.dev.lib.tl_memcpy_d2d(_vp(out.data_ptr()), ptr, out.numel() * 2), "tl_memcpy_d2d")
        self.dev.synchronize()
        return out

    def write_buffer(self, which: int, layer: int, a: np.ndarray) -> None:
        """Overwrite a driver buffer (e.g. pre-fill a KV cache) from a host fp16 array."""
        a = np.ascontiguousarray(a, dtype=np.float16)
        ptr = _vp()
        _ck(self.l.tlm_get_buffer(self.h, which, layer, ctypes.byref(ptr)), "tlm_get_buffer")
        check(self.dev.lib.tl_memcpy_h2d(ptr, a.ctypes.data_as(_vp), a.nbytes), "tl_memcpy_h2d")

    def generate(self, prompt, n_generate: int, mode: int = MODE_FUSED):
        prompt = np.ascontiguousarray(prompt, dtype=np.int32)
        out = np.empty(n_generate, np.int32)
        tp, td = ctypes.c_double(), ctypes.c_double()
        _ck(self.l.tlm_generate(self.h, prompt.ctypes.data_as(_vp), prompt.size, n_generate, mode,
                                out.ctypes.data_as(_vp), ctypes.byref(tp), ctypes.byref(td)), "tlm_generate")
        return out, tp.value, td.value


    def text_completion(self, tokenizer, text, position: int = 0, n_generate: int = 256, mode: int = MODE_FUSED,
                        chat_template: bool = False, on_piece=None):
        """Llama2::text_completion, or one chat turn with chat_template=True (model/llama2_7b/src/llama2.cpp:103-148).
        Returns (emitted token ids, their text as bytes, new position, decode steps run, prefill s, decode s);
        on_piece(bytes, token) is called as each token is produced."""
        raw = text.encode("utf-8") if isinstance(text, str) else bytes(text)
        tokens, chunks = [], []

        def _piece(ptr, n, token, _user):
            b = ctypes.string_at(ptr, n)
            tokens.append(int(token))
            chunks.append(b)
            if on_piece is not None:
                on_piece(b, int(token))

        cb = _PIECE_FN(_piece)
        pos, steps = _i(position), _i(0)
        tp, td = ctypes.c_double(), ctypes.c_double()
        _ck(self.l.tlm_text_completion(self.h, tokenizer.h, raw, int(chat_template), ctypes.byref(pos), n_generate, mode,
                                       ctypes.cast(cb, _vp), None, ctypes.byref(steps), ctypes.byref(tp),
                                       ctypes.byref(td)), "tlm_text_completion")
        return tokens, b"".join(chunks), pos.value, steps.value, tp.value, td.value


def bench_decode(dev, n_prompt: int = 128, n_generate: int = 256) -> dict:
    """Full Llama2-7B, random-init fp16 weights, 128-token random prompt,
    256 greedy steps, batch 1, max_seq 2048."""
    from . import synth
    cfg = Llama2Config()
    long_prompts = (512, 2048)
    m = Llama2Model(dev, cfg, max_tokens=max(long_prompts))
    m.random_init_on_device(seed=7)
    prompt = synth.token_ids(11, n_prompt, cfg.vocab_size)
    res = {"config": "Llama2-7B fp16 random-init, prompt 128, 256 greedy steps, batch 1",
           "parity": "tests/test_gpu_llama2.py: logits of the 32-layer model against the CPU restatement of the reference's op chain, normalised RMS "
                     "error <= 1e-2 (about 800 chained fp16 roundings; single kernels are gated at rtol 1e-2 / atol 1e-3)",
           "weight_bytes_per_token": cfg.weight_bytes_per_token()}
    ceiling = 8e12 / cfg.weight_bytes_per_token()
    for name, mode in (("fused", MODE_FUSED), ("reference_chain", MODE_REFERENCE_CHAIN)):
        m.generate(prompt, 4, mode)  # warm-up
        _, tp, td = m.generate(prompt, n_generate, mode)
        toks = (n_generate - 1) / td
        res[name] = {"decode_tok_s": round(toks, 2), "prefill_tok_s": round(n_prompt / tp, 1),
                     "frac_of_weight_streaming_ceiling": round(toks / ceiling, 4)}
    # prefill of longer prompts (fused mode; logits of the last token only, as generate computes them)
    import time
    res["prefill_long"] = {}
    for S in long_prompts:
        ids = synth.token_ids(12, S, cfg.vocab_size)
        m.forward(ids, 0, MODE_FUSED, all_logits=False)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        reps = 3
        for _ in range(reps):
            m.forward(ids, 0, MODE_FUSED, all_logits=False)
        torch.cuda.synchronize()
        res["prefill_long"][str(S)] = {"tok_s": round(S * reps / (time.perf_counter() - t0), 1)}
    m.close()
    return res
