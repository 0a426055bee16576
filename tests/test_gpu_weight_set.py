"""One weight set per session: the executors of a session (decode, prefill chunk, few-row, batched) built on one
mynn_weight_set share the library's derived weight copies -- each copy exists once, the results are bit-for-bit those
of executors with private copies, and the set lives until its last holder lets go.  The reference's LlmSession likewise
uploads the initializers once and hands the same device buffers to its decode and its prefill session
(crates/llm/src/session.rs:201-224, initializer_buffers)."""
import numpy as np
import pytest

import oracle as orc
import llm_weights

pytestmark = pytest.mark.gpu

SMALL = dict(n_layers=3, hidden=256, n_heads=8, n_kv_heads=2, head_dim=32, ffn=704, vocab=1000, max_seq=96,
             eps=1e-5, rope_theta=10000.0)
FEWROWS = dict(SMALL, ffn=768)  # every K a multiple of 128: 16..64 rows take the tiled int8 copy


@pytest.fixture(scope="module")
def g():
    import gpu_util

    return gpu_util


def dev_weights(g, w, dt):
    out = {}
    for k, v in w.items():
        out[k] = (g.to_dev(v[0]), g.to_dev(v[1], dt)) if isinstance(v, tuple) else g.to_dev(v, dt)
    return out


def run_chunks(dec, cfg, rows, batch, seed, chunks=2):
    rng = np.random.default_rng(seed)
    out, past = [], 0
    for _ in range(chunks):
        ids = rng.integers(0, cfg["vocab"], rows * batch)
        pos = np.arange(past, past + rows)
        nxt, logits = dec.step(ids, pos, past, past + rows, want_logits=True)
        out.append((list(nxt), logits.copy()))
        past += rows
    return out


def expected_repack_bytes(cfg, eb):
    H, F = cfg["hidden"], cfg["ffn"]
    QD, KD = cfg["n_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"]
    per_layer = (QD + 2 * KD) * H + (QD + 2 * KD) * eb + 2 * F * H + 2 * F * eb
    return cfg["n_layers"] * per_layer


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
def test_executors_on_one_weight_set_equal_private_copies_bit_for_bit(g, dt):
    cfg, w = llm_weights.synthetic_int8(SMALL, dt, seed=77)
    dw = dev_weights(g, w, dt)
    wset = g.mynn.WeightSet(cfg, dw)
    st = wset.stats()
    assert st["holders"] == 1 and st["repack_bytes"] == 0 and st["resident16_bytes"] == 0

    shapes = [dict(seq_q=1), dict(seq_q=32), dict(seq_q=1, batch=4), dict(seq_q=16)]
    shared = [g.mynn.Decoder(cfg, dw, weight_set=wset, **s) for s in shapes]
    st = wset.stats()
    assert st["holders"] == 1 + len(shapes)
    assert st["repack_bytes"] == expected_repack_bytes(cfg, 2)  # the q|k|v and gate/up repacks: once, not per executor
    H, F, V = cfg["hidden"], cfg["ffn"], cfg["vocab"]
    QD, KD = cfg["n_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"]
    weights = cfg["n_layers"] * ((QD + 2 * KD) * H + H * QD + 2 * F * H + H * F) + V * H
    # the 16-bit resident copy of the matrix-core path (rows >= 16): one for the 32-row and the 16-row executor
    # together (rows are padded to whole 8-element groups, so allow a little over 2 bytes per weight)
    assert 2 * weights <= st["resident16_bytes"] <= 2 * weights * 1.1
    assert st["tiled_int8_bytes"] == 0 and st["w8a8_interleave_bytes"] == 0

    for s, dec in zip(shapes, shared):
        own = g.mynn.Decoder(cfg, dw, **s)
        rows, batch = s["seq_q"], s.get("batch", 1)
        a = run_chunks(dec, cfg, rows, batch, seed=rows + batch)
        b = run_chunks(own, cfg, rows, batch, seed=rows + batch)
        for (na, la), (nb, lb) in zip(a, b):
            assert na == nb
            assert np.array_equal(la, lb), s
        own.close()
    assert wset.stats() == st  # private executors leave the set alone

    # the caller lets go first: the executors keep the copies alive and still give the same results
    before = run_chunks(shared[1], cfg, 32, 1, seed=5, chunks=1)
    wset.close()
    after = run_chunks(shared[1], cfg, 32, 1, seed=5, chunks=1)
    assert before[0][0] == after[0][0] and np.array_equal(before[0][1], after[0][1])
    for dec in shared:
        dec.close()


def test_few_row_executor_adds_the_tiled_int8_copy_once(g):
    dt = orc.F16
    cfg, w = llm_weights.synthetic_int8(FEWROWS, dt, seed=78)
    dw = dev_weights(g, w, dt)
    wset = g.mynn.WeightSet(cfg, dw)
    a = g.mynn.Decoder(cfg, dw, seq_q=32, weight_set=wset)
    one = wset.stats()
    assert one["tiled_int8_bytes"] > 0 and one["resident16_bytes"] == 0
    b = g.mynn.Decoder(cfg, dw, seq_q=16, weight_set=wset)
    c = g.mynn.Decoder(cfg, dw, seq_q=1, weight_set=wset)
    two = wset.stats()
    assert two["tiled_int8_bytes"] == one["tiled_int8_bytes"] and two["repack_bytes"] == one["repack_bytes"]
    assert two["holders"] == 4
    ref = orc.Model(cfg, w)
    ids = np.arange(32) % cfg["vocab"]
    want = ref.forward(ids, np.arange(32), 0, 32, True)
    _, got = a.step(ids, np.arange(32), 0, 32, want_logits=True)
    from conftest import max_err_rel_to_max

    assert max_err_rel_to_max(g.f32(got, dt), g.f32(want, dt)) <= 1e-2
    a.close(), b.close()
    assert wset.stats()["holders"] == 2
    c.close(), wset.close()


def test_weight_set_refuses_other_shapes(g):
    dt = orc.F16
    cfg, w = llm_weights.synthetic_int8(SMALL, dt, seed=79)
    dw = dev_weights(g, w, dt)
    wset = g.mynn.WeightSet(cfg, dw)
    other, w2 = llm_weights.synthetic_int8(dict(SMALL, ffn=640), dt, seed=79)
    with pytest.raises(g.mynn.MynnError, match="other shapes"):
        g.mynn.Decoder(other, dev_weights(g, w2, dt), weight_set=wset)
    with pytest.raises(g.mynn.MynnError, match="other shapes"):
        g.mynn.Decoder(dict(cfg, dtype=orc.BF16), dw, weight_set=wset)
    assert wset.stats()["holders"] == 1
    wset.close()
