"""Pins of the composed model oracle (oracle/llama2_oracle.py) on the CPU.

The checker here is a float64 Llama forward written from the textbook definition of the
architecture (the one script/model.py:94-203 of the reference states in PyTorch): RMSNorm ->
q,k,v -> rotary embedding on adjacent pairs -> causal softmax(Q K^T / sqrt(d)) V -> wo -> residual
-> RMSNorm -> w2(silu(w1 x) * (w3 x)) -> residual -> final norm -> classifier.  It shares no code
with the oracle: no fp16 rounding, no KV cache (the whole prefix is recomputed), complex
multiplication for the rotation, an explicit triangular mask.  The fp16 oracle must agree with it
to the accuracy that ~25 fp16 roundings per block allow, and must stop agreeing when a plausible
mistake is planted in the oracle (w1/w3 swapped, the second residual taken from x, the mask applied
to a single-token step, a wrong cache position), which the last tests prove.
"""
import numpy as np
import pytest

from tensorlib_amd import synth

DIM, HEADS, HIDDEN, LAYERS, VOCAB, MAX_SEQ, EPS = 64, 2, 176, 2, 97, 32, 1e-5


def _weights(seed, dim=DIM, hidden=HIDDEN, layers=LAYERS, vocab=VOCAB):
    # std 0.15 rather than 0.02: on a 64-wide toy model the branches must weigh something against the
    # residual stream, or a mistake inside a branch would drown in the embedding
    w = {"tok_emb": synth.normal_f16(seed, (vocab, dim), 1.0),
         "final_norm": synth.normal_f16(seed + 1, (dim,), 1.0),
         "classifier": synth.normal_f16(seed + 2, (vocab, dim), 0.15)}
    for l in range(layers):
        s = seed + 100 * (l + 1)
        w[f"att_norm.{l}"] = synth.normal_f16(s, (dim,), 1.0)
        w[f"ffn_norm.{l}"] = synth.normal_f16(s + 1, (dim,), 1.0)
        for i, n in enumerate(("wq", "wk", "wv", "wo")):
            w[f"{n}.{l}"] = synth.normal_f16(s + 2 + i, (dim, dim), 0.15)
        w[f"w1.{l}"] = synth.normal_f16(s + 6, (hidden, dim), 0.15)
        w[f"w3.{l}"] = synth.normal_f16(s + 7, (hidden, dim), 0.15)
        w[f"w2.{l}"] = synth.normal_f16(s + 8, (dim, hidden), 0.15)
    return w


def _oracle(w, **kw):
    from oracle.llama2_oracle import Llama2Oracle
    return Llama2Oracle(w, kw.get("dim", DIM), kw.get("hidden", HIDDEN), kw.get("layers", LAYERS),
                        kw.get("heads", HEADS), kw.get("vocab", VOCAB), MAX_SEQ, EPS)


# ------------------------------------------------------- the independent float64 model ----

def textbook_llama_f64(w, tokens, heads, layers, eps=EPS, theta=10000.0):
    """Logits [S, vocab] in float64 for the whole sequence `tokens` starting at position 0."""
    W = {k: np.asarray(v, np.float64) for k, v in w.items()}
    tokens = np.asarray(tokens)
    S, dim = len(tokens), W["tok_emb"].shape[1]
    d = dim // heads

    def norm(x, g):
        return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * g

    def rotate(x):                                    # x [S, heads, d]; pairs (2i, 2i+1) form a complex number
        z = x[..., 0::2] + 1j * x[..., 1::2]
        ang = np.arange(S)[:, None] * theta ** (-np.arange(0, d, 2) / d)[None, :]
        z = z * np.exp(1j * ang)[:, None, :]
        out = np.empty_like(x)
        out[..., 0::2], out[..., 1::2] = z.real, z.imag
        return out

    h = W["tok_emb"][tokens]
    for l in range(layers):
        xn = norm(h, W[f"att_norm.{l}"])
        q = rotate((xn @ W[f"wq.{l}"].T).reshape(S, heads, d))
        k = rotate((xn @ W[f"wk.{l}"].T).reshape(S, heads, d))
        v = (xn @ W[f"wv.{l}"].T).reshape(S, heads, d)
        att = np.einsum("shd,thd->hst", q, k) / np.sqrt(d)
        att = np.where(np.triu(np.ones((S, S), bool), 1)[None], -np.inf, att)
        att = np.exp(att - att.max(-1, keepdims=True))
        att /= att.sum(-1, keepdims=True)
        o = np.einsum("hst,thd->shd", att, v).reshape(S, dim)
        h = h + o @ W[f"wo.{l}"].T
        xn = norm(h, W[f"ffn_norm.{l}"])
        a = xn @ W[f"w1.{l}"].T
        h = h + ((a / (1.0 + np.exp(-a))) * (xn @ W[f"w3.{l}"].T)) @ W[f"w2.{l}"].T
    return norm(h, W["final_norm"]) @ W["classifier"].T


def nrmse(got, want):
    g, t = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return float(np.sqrt(np.mean((g - t) ** 2)) / np.sqrt(np.mean(t ** 2)))


# fp16 chain against float64: measured 1.2e-3..1.6e-3 on this toy model; every planted mistake below
# lands above 0.2
GATE = 4e-3


# ------------------------------------------------------------------------------ pins ----

@pytest.mark.parametrize("seed", [11, 12, 13])
def test_prefill_logits_match_textbook_float64(oracle, seed):
    w = _weights(seed)
    toks = synth.token_ids(seed, 12, VOCAB)
    got = _oracle(w).forward(toks, 0)
    want = textbook_llama_f64(w, toks, HEADS, LAYERS)
    assert got.dtype == np.float16 and got.shape == (12, VOCAB)
    assert nrmse(got, want) < GATE


def test_prefill_then_single_token_steps_match_textbook(oracle):
    """KV-cache positions and the rotary start position: a 5-token prefill followed by 7 single-token steps
    must give the rows the cache-free float64 model gives for the whole 12-token sequence."""
    w = _weights(21)
    toks = synth.token_ids(21, 12, VOCAB)
    want = textbook_llama_f64(w, toks, HEADS, LAYERS)
    m = _oracle(w)
    rows = [m.forward(toks[:5], 0)]
    for pos in range(5, 12):
        rows.append(m.forward(toks[pos:pos + 1], pos))
    got = np.concatenate(rows)
    assert nrmse(got, want) < GATE
    assert max(nrmse(got[i], want[i]) for i in range(12)) < 2 * GATE


def test_prefill_equals_token_by_token(oracle):
    """The same oracle run as one prefill and as S single-token steps: identical op chain per row apart from
    the masked columns, so the logits agree far inside the float64 gate, and the caches hold the same rows."""
    w = _weights(31)
    toks = synth.token_ids(31, 9, VOCAB)
    a = _oracle(w)
    full = a.forward(toks, 0)
    b = _oracle(w)
    step = np.concatenate([b.forward(toks[i:i + 1], i) for i in range(9)])
    assert nrmse(step, full) < 2e-3
    for l in range(LAYERS):
        assert np.array_equal(a.cache_k[l][:9], b.cache_k[l][:9])   # k rows do not depend on other positions
        assert np.array_equal(a.cache_v[l][:9], b.cache_v[l][:9])
        assert not a.cache_k[l][9:].any() and not b.cache_v[l][9:].any()


def test_zero_branch_weights_pass_the_residual_through(oracle):
    """wo = w2 = 0 switches both branches off: the block returns its input bit for bit and the logits are
    classifier(rmsnorm(embedding)), computable in float64 directly."""
    w = _weights(41)
    for l in range(LAYERS):
        w[f"wo.{l}"][:] = 0
        w[f"w2.{l}"][:] = 0
    toks = synth.token_ids(41, 6, VOCAB)
    m = _oracle(w)
    got = m.forward(toks, 0)
    assert np.array_equal(m.last_hidden, w["tok_emb"][toks])
    e = w["tok_emb"][toks].astype(np.float64)
    want = (e / np.sqrt(np.mean(e * e, -1, keepdims=True) + EPS) * w["final_norm"].astype(np.float64)) \
        @ w["classifier"].astype(np.float64).T
    assert nrmse(got, want) < 2e-3


def test_single_head_uniform_attention_closed_form(oracle):
    """wq = 0 makes every score 0, so the attention output at row s is the plain mean of the value rows 0..s
    (the causal prefix); with wo = identity and the FFN off the block output is x + that mean."""
    dim, heads = 32, 1
    w = _weights(51, dim=dim, hidden=48, layers=1)
    w["wq.0"][:] = 0
    w["wo.0"] = np.eye(dim, dtype=np.float16)
    w["w2.0"][:] = 0
    toks = synth.token_ids(51, 8, VOCAB)
    m = _oracle(w, dim=dim, hidden=48, layers=1, heads=heads)
    m.forward(toks, 0)
    x = w["tok_emb"][toks].astype(np.float64)
    xn = x / np.sqrt(np.mean(x * x, -1, keepdims=True) + EPS) * w["att_norm.0"].astype(np.float64)
    v = xn @ w["wv.0"].astype(np.float64).T
    want = x + np.cumsum(v, 0) / np.arange(1, 9)[:, None]
    assert nrmse(m.last_hidden, want) < 2e-3


# ------------------------------------------------- the gate bites: planted mistakes fail ----

def _mutant(name):
    """A copy of the oracle class with one plausible mistake planted by editing its source text."""
    import inspect
    import textwrap
    from oracle import llama2_oracle as lo
    src = textwrap.dedent(inspect.getsource(lo.Llama2Oracle))
    swaps = {
        "w1_w3_swapped": ('x1 = o.silu(o.matmul2d(x_norm, w[f"w1.{l}"]))\n        x3 = o.matmul2d(x_norm, w[f"w3.{l}"])',
                          'x1 = o.silu(o.matmul2d(x_norm, w[f"w3.{l}"]))\n        x3 = o.matmul2d(x_norm, w[f"w1.{l}"])'),
        "second_residual_from_x": ('return o.binary(h, ffn, "add")', 'return o.binary(x, ffn, "add")'),
        # (the correct mask is all zero on a single-token step, get_mask at Transformer.cpp:233 only skips the
        # work; what must fail is a mask that is applied there and, as a [S, S] triangle, forgets the prefix)
        "mask_on_single_token_ignoring_prefix": ("if S > 1:\n            j = np.arange(T)[None, :]\n            i = np.arange(S)[:, None]\n            mask = np.where(j > start_pos + i,",
                                                 "if S >= 1:\n            j = np.arange(T)[None, :]\n            i = np.arange(S)[:, None]\n            mask = np.where(j > i,"),
        "mask_off_by_one": ("j > start_pos + i", "j >= start_pos + i + 2"),
        "cache_written_at_zero": ("self.cache_k[l][start_pos:T] = xk", "self.cache_k[l][0:S] = xk"),
        "rope_start_ignored": ("xk = o.rope(xk.reshape(1, S, H, D), start_pos)", "xk = o.rope(xk.reshape(1, S, H, D), 0)"),
        "ffn_norm_of_x": ('x_norm = o.rms_norm(h, w[f"ffn_norm.{l}"]', 'x_norm = o.rms_norm(x, w[f"ffn_norm.{l}"]'),
        "no_score_scale": ('scores = o.binary_scalar(scores, np.sqrt(np.float32(D)), "div")', "pass"),
    }
    old, new = swaps[name]
    assert src.count(old) == 1, f"mutation site for {name} not found exactly once"
    ns = {"np": np, "o": lo.o, "annotations": None}
    exec("from __future__ import annotations\n" + src.replace(old, new), ns)
    return ns["Llama2Oracle"]


def _run(cls, w, toks, split):
    m = cls(w, DIM, HIDDEN, LAYERS, HEADS, VOCAB, MAX_SEQ, EPS)
    rows = [m.forward(toks[:split], 0)]
    for pos in range(split, len(toks)):
        rows.append(m.forward(toks[pos:pos + 1], pos))
    return np.concatenate(rows)


@pytest.mark.parametrize("name", ["w1_w3_swapped", "second_residual_from_x", "mask_on_single_token_ignoring_prefix", "mask_off_by_one",
                                  "cache_written_at_zero", "rope_start_ignored", "ffn_norm_of_x", "no_score_scale"])
def test_planted_mistake_fails_the_float64_gate(oracle, name):
    from oracle.llama2_oracle import Llama2Oracle
    w = _weights(61)
    toks = synth.token_ids(61, 12, VOCAB)
    want = textbook_llama_f64(w, toks, HEADS, LAYERS)
    assert nrmse(_run(Llama2Oracle, w, toks, 5), want) < GATE          # the real oracle passes on this very input
    got = _run(_mutant(name), w, toks, 5)
    with np.errstate(invalid="ignore"):
        err = nrmse(np.nan_to_num(got.astype(np.float64), nan=1e4), want)
    assert err > 5 * GATE, f"{name}: nrmse {err} would pass the gate"
