"""The decode step with the q|k|v projection, the attention and the o projection of a layer in one launch, against the
same step with three launches: the same arithmetic operation for operation, so logits, tokens and KV rows must be
bit-identical (the two-launch form is what the other tests hold against the oracle)."""
import numpy as np
import pytest

import oracle as orc
import llm_weights
from conftest import max_err_rel_to_max
from test_gpu_decoder import SHORT_CACHE, dev_weights

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def g():
    import gpu_util

    return gpu_util


def pair(g, cfg, weights):
    """(fused executor, two-launch executor) over the same weights, each with its own KV cache"""
    two = g.mynn.Decoder(cfg, weights, unfused_decode=True)
    one = g.mynn.Decoder(cfg, weights)
    assert one.stats()["graph"] and two.stats()["graph"]
    assert one.stats()["launches_per_step"] == two.stats()["launches_per_step"] - 2 * cfg["n_layers"] - 2
    return one, two


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("D,max_seq,n", [(64, 512, 140), (128, 256, 140), (64, 2048, 1100), (128, 1024, 600)])
def test_fused_step_bit_identical_to_two_launches(g, dt, D, max_seq, n):
    cfg, w = llm_weights.synthetic_int8(dict(SHORT_CACHE[D], max_seq=max_seq), dt, seed=31 + D)
    one, two = pair(g, cfg, dev_weights(g, w, dt))
    toks = np.random.default_rng(D + dt).integers(0, cfg["vocab"], n)
    for i, t in enumerate(toks):
        a, la = one.step([t], [i], i, i + 1, want_logits=True)
        b, lb = two.step([t], [i], i, i + 1, want_logits=True)
        assert np.array_equal(la, lb), i
        assert a[0] == b[0], i
    for l in range(cfg["n_layers"]):
        for j in range(2):
            assert np.array_equal(g.to_host(one.kv[l][j]), g.to_host(two.kv[l][j])), (l, j)
    # the device-resident loop (graph replays) continues identically from here
    first = int(a[0])
    assert one.decode_loop(first, n, 40) == two.decode_loop(first, n, 40)
    one.close(), two.close()


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
def test_fused_step_vs_oracle(g, dt):
    """Held against the oracle directly as well: three layers, ragged ffn and vocabulary, a negative token id."""
    cfg, w = llm_weights.synthetic_int8(dict(SHORT_CACHE[64], n_layers=3, ffn=1136, vocab=1003), dt, seed=5)
    ref = orc.Model(cfg, w)
    dec = g.mynn.Decoder(cfg, dev_weights(g, w, dt))
    assert dec.stats()["launches_per_step"] == 3 * 3 + 1
    toks = [7, -1, 1002, 0, 511, -1003 + 4]
    for i, t in enumerate(toks):
        want = ref.forward([t % cfg["vocab"]], [i], i, i + 1, False)
        nxt, got = dec.step([t], [i], i, i + 1, want_logits=True)
        assert max_err_rel_to_max(g.f32(got, dt), g.f32(want, dt)) <= 1e-2, i
        assert nxt[0] == orc.argmax_last(got[0], dt)
    dec.close()


def test_fused_step_full_size_tinyllama_shape(g):
    """The benchmark's model: both executors, the same 24 steps, bit-identical logits, then the replayed loop."""
    import os
    import sys
    import torch

    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import bench

    dt = orc.F16
    cfg = dict(bench.TINYLLAMA, dtype=dt, max_seq=384)
    weights = bench.make_weights(cfg, dt, 1234)
    torch.cuda.synchronize()
    one, two = pair(g, cfg, weights)
    assert one.stats()["launches_per_step"] == 67
    toks = np.random.default_rng(3).integers(0, cfg["vocab"], 24)
    for i, t in enumerate(toks):
        a, la = one.step([t], [i], i, i + 1, want_logits=True)
        b, lb = two.step([t], [i], i, i + 1, want_logits=True)
        assert np.array_equal(la, lb), i
        assert a[0] == b[0]
    first = int(a[0])
    assert one.decode_loop(first, 24, 64) == two.decode_loop(first, 24, 64)
    one.close(), two.close()
