"""CPU check of the llama2.c legacy fp16 checkpoint writer against the layout the reference reads
(model/llama2_7b/src/main.cpp:26-34,36-190; script/export.py:138-190): header fields, the sign of
vocab_size, tensor order and the size of the skipped rotary tables."""
import struct

import numpy as np

from tensorlib_amd import synth
from tensorlib_amd.llama2 import Llama2Config, write_checkpoint


def _w(cfg):
    w = {"tok_emb": synth.normal_f16(1, (cfg.vocab_size, cfg.dim)), "final_norm": synth.normal_f16(2, (cfg.dim,)),
         "classifier": synth.normal_f16(3, (cfg.vocab_size, cfg.dim))}
    for l in range(cfg.n_layers):
        for i, (n, shp) in enumerate([("att_norm", (cfg.dim,)), ("wq", (cfg.dim, cfg.dim)), ("wk", (cfg.dim, cfg.dim)),
                                      ("wv", (cfg.dim, cfg.dim)), ("wo", (cfg.dim, cfg.dim)), ("ffn_norm", (cfg.dim,)),
                                      ("w1", (cfg.hidden_dim, cfg.dim)), ("w2", (cfg.dim, cfg.hidden_dim)),
                                      ("w3", (cfg.hidden_dim, cfg.dim))]):
            w[f"{n}.{l}"] = synth.normal_f16(10 * l + i + 4, shp)
    return w


def test_layout_matches_the_reference_reader(tmp_path):
    cfg = Llama2Config(dim=16, hidden_dim=40, n_layers=2, n_heads=2, vocab_size=11, max_seq_len=8)
    w = _w(cfg)
    p = str(tmp_path / "m.bin")
    write_checkpoint(p, cfg, w, shared_classifier=False)
    raw = open(p, "rb").read()
    hdr = struct.unpack("iiiiiii", raw[:28])
    assert hdr == (16, 40, 2, 2, 2, -11, 8)          # negative vocab: classifier is stored separately
    body = np.frombuffer(raw[28:], dtype=np.float16)
    order = ["att_norm", "wq", "wk", "wv", "wo", "ffn_norm", "w1", "w2", "w3"]
    off = 0

    def take(a):
        nonlocal off
        got = body[off:off + a.size]
        off += a.size
        assert np.array_equal(got.view(np.uint16), a.ravel().view(np.uint16))
    take(w["tok_emb"])
    for n in order:
        for l in range(cfg.n_layers):
            take(w[f"{n}.{l}"])
    take(w["final_norm"])
    off += cfg.max_seq_len * cfg.head_dim                # freqs_cos + freqs_sin, skipped by the reader
    take(w["classifier"])
    assert off == body.size
    write_checkpoint(p, cfg, w, shared_classifier=True)
    raw2 = open(p, "rb").read()
    assert struct.unpack("iiiiiii", raw2[:28])[5] == 11
    assert len(raw2) == len(raw) - 2 * cfg.vocab_size * cfg.dim
