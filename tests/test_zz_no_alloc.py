"""The entry point that allocates nothing (tl_decode_attention_rope_static_f16) against the entry point it is a
variant of (tl_decode_attention_rope_f16), through the C ABI: same kernels, so outputs and the written cache rows must
be bit-identical.  Two calls in a row share the static scratch array, the second with a smaller input, so stale partial
results of the first call would show; then a size beyond the array's limit must be refused with a clear error."""
import numpy as np
import pytest
import torch

from tensorlib_amd import synth

pytestmark = pytest.mark.gpu


def _case(dev, seed, pos, H, D, with_table):
    S = pos + 2
    qkv = synth.normal_f16(seed, (3, H, D), 1.0)
    ck = synth.normal_f16(seed + 1, (S, H, D), 1.0)
    cv = synth.normal_f16(seed + 2, (S, H, D), 1.0)
    table = dev.rope_table(S, D) if with_table else None
    return qkv, ck, cv, table


@pytest.mark.parametrize("with_table", [True, False])
def test_static_scratch_entry_matches_workspace_entry_twice_in_a_row(dev, with_table):
    H, D = 32, 128
    results = []
    for seed, pos in ((300, 1500), (310, 200)):            # 24 chunks per head, then 4: the second call is smaller
        qkv, ck, cv, table = _case(dev, seed, pos, H, D, with_table)
        q1, k1, v1 = dev.from_numpy(qkv), dev.from_numpy(ck), dev.from_numpy(cv)
        want = dev.decode_attention_rope(q1, k1, v1, pos, rope_table=table)
        q2, k2, v2 = dev.from_numpy(qkv), dev.from_numpy(ck), dev.from_numpy(cv)
        out = dev.empty(H, D)                                # allocated by the caller, before the call
        results.append((want, k1, v1, out, k2, v2, q2, pos, table))
    # the two static calls back to back, nothing in between
    for want, k1, v1, out, k2, v2, q2, pos, table in results:
        dev.decode_attention_rope(q2, k2, v2, pos, rope_table=table, out=out, static_scratch=True)
    dev.synchronize()
    for want, k1, v1, out, k2, v2, q2, pos, table in results:
        assert torch.equal(out, want), f"pos {pos}: output differs from tl_decode_attention_rope_f16"
        assert torch.equal(k1, k2) and torch.equal(v1, v2), f"pos {pos}: cache rows differ"


def test_static_scratch_entry_single_chunk_and_small_heads(dev):
    for seed, pos, H, D in ((320, 40, 4, 64), (330, 700, 8, 128), (340, 0, 2, 256), (350, 129, 2, 256)):
        qkv, ck, cv, table = _case(dev, seed, pos, H, D, True)
        q1, k1, v1 = dev.from_numpy(qkv), dev.from_numpy(ck), dev.from_numpy(cv)
        want = dev.decode_attention_rope(q1, k1, v1, pos, rope_table=table)
        q2, k2, v2 = dev.from_numpy(qkv), dev.from_numpy(ck), dev.from_numpy(cv)
        got = dev.decode_attention_rope(q2, k2, v2, pos, rope_table=table, out=dev.empty(H, D), static_scratch=True)
        assert torch.equal(got, want) and torch.equal(k1, k2) and torch.equal(v1, v2)


def test_static_scratch_entry_refuses_sizes_beyond_its_array(dev):
    from tensorlib_amd import TensorLibError
    H, D = 64, 256                          # 64 heads x 64 chunks x 258 floats = 1056768 > 2^20
    pos = 64 * 64 - 1
    cache = dev.empty(pos + 1, H, D)
    cache.zero_()
    qkv = dev.from_numpy(synth.normal_f16(360, (3, H, D), 1.0))
    with pytest.raises(TensorLibError, match="exceed the static scratch"):
        dev.decode_attention_rope(qkv, cache, cache.clone(), pos, out=dev.empty(H, D), static_scratch=True)
    # one chunk fewer fits
    dev.decode_attention_rope(qkv, cache, cache.clone(), pos - 64, out=dev.empty(H, D), static_scratch=True)
    dev.synchronize()
