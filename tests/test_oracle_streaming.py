"""Pins for the oracle's streaming-KV mode (sink + ring cache), including steps past sink + window.

The mechanism exists only in the reference's CUDA backend (src/codegen/cuda/cpp/common.cuh:55-60,
kvcache_update.cuh:12-26, quantizing_kvcache_update.cuh:24-36, attention.cuh:100-200, 386-420, 495-606) and its
session (crates/llm/src/session.rs:539-635); the reference's own tests past the window assert only that generation
runs (crates/llm/tests/tinyllama_random.rs:157-315).  What pins the restatement here:
  * up to sink + window the streaming graph is arithmetically the plain graph (bit-equal logits with a 16-bit cache);
  * slot, rank and kv_position tables for sink 4 / window 16 written out by hand from the reference's formulas;
  * the ring attention against an f64 brute force over hand-listed rows, and against the numpy restatement that
    gathers rows first (a second, independent code path);
  * the whole streaming decoder against a numpy composition of the operator-level functions, step by step."""
import numpy as np
import pytest

import oracle as orc
import llm_weights
from conftest import max_err_rel_to_max
from oracle_compose import compose_step

TINY = dict(n_layers=2, hidden=64, n_heads=4, n_kv_heads=2, head_dim=16, ffn=96, vocab=97, max_seq=32,
            eps=1e-5, rope_theta=10000.0)
SINK, WINDOW = 4, 16

# ---- tables written out by hand -------------------------------------------------------------------------------------
# Decode step at stream position p >= sink + window = 20: the session passes ring_start = (p - 4) % 16 and the update
# kernel maps rank = offset = p through ring_phys_index: slot = 4 + (ring_start + (p - 4)) % 16.
#   p = 20: ring_start 0,  rel = 0 + 16 = 16 -> 0  -> slot 4        p = 21: ring_start 1, rel = 1 + 17 = 18 -> 2 -> slot 6
#   p = 22: ring_start 2,  rel = 2 + 18 = 20 -> 4  -> slot 8        p = 23: 3 + 19 = 22 -> 6  -> slot 10
#   p = 24: 4 + 20 = 24 -> 8 -> slot 12                             p = 25: 5 + 21 = 26 -> 10 -> slot 14
#   p = 26: 6 + 22 = 28 -> 12 -> slot 16                            p = 27: 7 + 23 = 30 -> 14 -> slot 18
#   p = 28: 8 + 24 = 32 -> 0 -> slot 4   ... the odd ring slots 5, 7, .., 19 are never written again
SLOT_OF_POSITION = {20: 4, 21: 6, 22: 8, 23: 10, 24: 12, 25: 14, 26: 16, 27: 18,
                    28: 4, 29: 6, 30: 8, 31: 10, 32: 12, 33: 14, 34: 16, 35: 18,
                    36: 4, 37: 6, 38: 8, 39: 10, 40: 12, 41: 14, 42: 16, 43: 18, 44: 4}
# The attention of the step at p = 21 (ring_start 1, 20 active keys) reads rank -> slot
RANK_TO_SLOT_P21 = [0, 1, 2, 3, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 17, 18, 19, 4]
# and at p = 30 (ring_start (30 - 4) % 16 = 10)
RANK_TO_SLOT_P30 = [0, 1, 2, 3, 14, 15, 16, 17, 18, 19, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13]
# kv_position by SLOT at p = 21 (streaming_kv_position: ring slot s has age (s - 4 + 16 - 1) % 16, position 4 + age;
# slots past sink + window keep their index)
KV_POSITION_P21 = [0, 1, 2, 3, 19, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 17, 18] + list(range(20, 32))


def ring_start_of(p):
    return 0 if p < SINK + WINDOW else (p - SINK) % WINDOW


def test_slot_rank_and_position_tables_by_hand():
    for p, slot in SLOT_OF_POSITION.items():
        assert orc.ring_phys_index(p, SINK, WINDOW, ring_start_of(p)) == slot, p
    assert [orc.ring_phys_index(r, SINK, WINDOW, 1) for r in range(20)] == RANK_TO_SLOT_P21
    assert [orc.ring_phys_index(r, SINK, WINDOW, 10) for r in range(20)] == RANK_TO_SLOT_P30
    assert list(orc.streaming_kv_position(SINK, WINDOW, 21, 32)) == KV_POSITION_P21
    # below the window nothing moves: slot = position, kv_position = slot
    for p in range(20):
        assert orc.ring_phys_index(p, SINK, WINDOW, ring_start_of(p)) == p
        assert list(orc.streaming_kv_position(SINK, WINDOW, p, 32)) == list(range(32))


@pytest.mark.parametrize("dt", [orc.F32, orc.BF16, orc.F16])
def test_streaming_graph_equals_plain_graph_up_to_the_window(dt):
    """Slot = position and the key is rotated by its own position when read instead of when written: the same
    products and the same single rounding, so logits are bit-equal; the cache holds the un-rotated keys."""
    cfg, w = llm_weights.synthetic_int8(TINY, dt, seed=3)
    plain, strm = orc.Model(cfg, w), orc.Model(cfg, w)
    strm.set_streaming(SINK, WINDOW)
    rng = np.random.default_rng(0)
    for p, t in enumerate(rng.integers(0, cfg["vocab"], SINK + WINDOW)):
        want = plain.forward([t], [p], p, p + 1, False)
        kvp = orc.streaming_kv_position(SINK, WINDOW, p, cfg["max_seq"])
        got = strm.forward_streaming([t], [p], p, p + 1, False, SINK, WINDOW, 0, kvp)
        assert np.array_equal(got, want), p
    cos, sin = orc.rope_table(cfg["max_seq"], cfg["head_dim"], cfg["rope_theta"], dt)
    for l in range(cfg["n_layers"]):
        k_raw, v_raw = strm.kv_cache(l)
        k_ref, v_ref = plain.kv_cache(l)
        assert np.array_equal(orc.rope(k_raw, cos, sin, np.arange(cfg["max_seq"]), dt)[:, :20], k_ref[:, :20])
        assert np.array_equal(v_raw, v_ref)
    # and through the session loop: same ids, prefill chunks included
    a, b = orc.Model(cfg, w), orc.Model(cfg, w)
    b.set_streaming(SINK, WINDOW)
    prompt = [int(t) for t in rng.integers(0, cfg["vocab"], 7)]
    assert a.generate(prompt, 10, prefill_len=4) == b.generate(prompt, 10, prefill_len=4)


@pytest.mark.parametrize("kv8", [False, True])
def test_update_lands_in_the_hand_listed_slot_past_the_window(kv8):
    """Each decode step changes exactly one cache row per layer and head: the slot of the hand-written table."""
    dt = orc.F16
    cfg, w = llm_weights.synthetic_int8(TINY, dt, seed=5)
    m = orc.Model(cfg, w)
    m.set_options(quant_kv_cache=kv8)
    m.set_streaming(SINK, WINDOW)
    rng = np.random.default_rng(1)
    toks = rng.integers(0, cfg["vocab"], 45)
    for p in range(45):
        before = [m.kv_cache(l) for l in range(cfg["n_layers"])]
        m.decode_step(int(toks[p]))
        assert m.past_len == p + 1
        for l in range(cfg["n_layers"]):
            k, v = m.kv_cache(l)
            for new, old in ((k, before[l][0]), (v, before[l][1])):
                changed = sorted(set(np.nonzero((new != old).any(axis=(0, 2)))[0]))
                want = [SLOT_OF_POSITION[p]] if p >= 20 else [p]
                assert changed == want, (p, l, changed)


def attention_f64_over_rows(q, k, v, rows, scale, dt, past, k_scale=None, v_scale=None, rope=None):
    """Brute force in f64 over an explicit list of cache rows (one per rank); causal: rank <= past + query row."""
    B, Hq, Sq, D = q.shape
    Hkv = k.shape[1]
    qf = orc.to_f32(q, dt).astype(np.float64)
    kf = (k.astype(np.float64) * orc.to_f32(k_scale, dt)[..., None]) if k.dtype == np.int8 else orc.to_f32(k, dt).astype(np.float64)
    vf = (v.astype(np.float64) * orc.to_f32(v_scale, dt)[..., None]) if v.dtype == np.int8 else orc.to_f32(v, dt).astype(np.float64)
    out = np.zeros(q.shape)
    half = D // 2
    for b in range(B):
        for h in range(Hq):
            g = h // (Hq // Hkv)
            for s in range(Sq):
                n = min(len(rows), past + s + 1) if past is not None else len(rows)
                sc = np.zeros(n)
                for r in range(n):
                    key = kf[b, g, rows[r]].copy()
                    if rope is not None:
                        c = orc.to_f32(rope[0], dt)[rope[2][r]].astype(np.float64)
                        sn = orc.to_f32(rope[1], dt)[rope[2][r]].astype(np.float64)
                        pair = np.concatenate([-key[half:], key[:half]])
                        key = key * c + pair * sn
                    sc[r] = qf[b, h, s] @ key * scale
                p = np.exp(sc - sc.max())
                p /= p.sum()
                out[b, h, s] = sum(p[r] * vf[b, g, rows[r]] for r in range(n))
    return out


@pytest.mark.parametrize("dt", [orc.F32, orc.F16, orc.BF16])
@pytest.mark.parametrize("kv8,rope_on", [(False, False), (True, True), (False, True), (True, False)])
@pytest.mark.parametrize("Sq", [1, 3])
def test_ring_attention_vs_f64_over_hand_listed_rows(dt, kv8, rope_on, Sq):
    rng = np.random.default_rng(7)
    B, Hq, Hkv, D, Sk = 2, 4, 2, 16, 32
    q = orc.to_storage(rng.standard_normal((B, Hq, Sq, D)), dt)
    if kv8:
        k = rng.integers(-127, 128, (B, Hkv, Sk, D)).astype(np.int8)
        v = rng.integers(-127, 128, (B, Hkv, Sk, D)).astype(np.int8)
        ks = orc.to_storage(rng.uniform(0.005, 0.02, (B, Hkv, Sk)), dt)
        vs = orc.to_storage(rng.uniform(0.005, 0.02, (B, Hkv, Sk)), dt)
    else:
        k = orc.to_storage(rng.standard_normal((B, Hkv, Sk, D)), dt)
        v = orc.to_storage(rng.standard_normal((B, Hkv, Sk, D)), dt)
        ks = vs = None
    cos, sin = orc.rope_table(Sk, D, 10000.0, dt)
    kvp = np.array(KV_POSITION_P21, np.int64)
    rope = (cos, sin, kvp) if rope_on else None
    got = orc.attention_ring(q, k, v, dt, 0.25, Sq > 1, 20, SINK, WINDOW, 1, ks, vs, rope)
    # rank-indexed kv_position, as the reference's kernels read it
    want = attention_f64_over_rows(q, k, v, RANK_TO_SLOT_P21, 0.25, dt, 20 - Sq if Sq > 1 else None, ks, vs,
                                   (cos, sin, KV_POSITION_P21) if rope_on else None)
    tol = {orc.F32: 2e-5, orc.F16: 2e-3, orc.BF16: 1e-2}[dt]
    assert max_err_rel_to_max(orc.to_f32(got, dt), want) <= tol
    # the gather-first numpy restatement is a second code path for the same operator
    other = orc.attention_streaming(q, k, v, dt, 0.25, Sq > 1, 20, SINK, WINDOW, 1, ks, vs, rope)
    assert max_err_rel_to_max(orc.to_f32(got, dt), orc.to_f32(other, dt)) <= tol
    if not kv8 and not rope_on:
        assert np.array_equal(got, other)  # same loop order over the same rows


def numpy_streaming_step(cfg, w, caches, ids, positions, past, active, causal, ring_start, kvp, dt, kv8):
    return compose_step(cfg, w, caches, ids, positions, past, active, causal, dt, kv8=kv8, ring=(SINK, WINDOW, ring_start, kvp))


@pytest.mark.parametrize("dt", [orc.F32, orc.F16])
@pytest.mark.parametrize("kv8", [False, True])
@pytest.mark.parametrize("prefill_len", [0, 4])
def test_streaming_decoder_past_the_window_vs_operator_composition(dt, kv8, prefill_len):
    """45 tokens through the streaming session of the C decoder (decode-only, or prefill chunks of 4 and then decode
    steps) against the same inputs composed in numpy from the operator-level functions: 16-bit KV bit-equal (same
    arithmetic in the same order), int8 KV within f32 re-association of the in-operator rotation."""
    cfg, w = llm_weights.synthetic_int8(TINY, dt, seed=11)
    m = orc.Model(cfg, w)
    m.set_options(quant_kv_cache=kv8)
    m.set_streaming(SINK, WINDOW)
    Hkv, D, MS, L = cfg["n_kv_heads"], cfg["head_dim"], cfg["max_seq"], cfg["n_layers"]
    if kv8:
        caches = [[np.zeros((1, Hkv, MS, D), np.int8), np.zeros((1, Hkv, MS, D), np.int8),
                   np.zeros((1, Hkv, MS), orc.np_dtype(dt)), np.zeros((1, Hkv, MS), orc.np_dtype(dt))] for _ in range(L)]
    else:
        caches = [[np.zeros((1, Hkv, MS, D), orc.np_dtype(dt)), np.zeros((1, Hkv, MS, D), orc.np_dtype(dt))] for _ in range(L)]
    rng = np.random.default_rng(2)
    toks = [int(t) for t in rng.integers(0, cfg["vocab"], 45)]
    max_active = SINK + WINDOW
    past = 0
    worst = 0.0

    def check(got, want, where):
        nonlocal worst
        if kv8:
            worst = max(worst, max_err_rel_to_max(orc.to_f32(got, dt), orc.to_f32(want, dt)))
        else:
            assert np.array_equal(got, want), where

    if prefill_len:
        # two prompts of 6 tokens = chunks of 4 + 2 (padded), the second one past the window
        for start in (0, 30):
            while past < start:  # decode steps up to the second prompt
                sp = past
                kvp = orc.streaming_kv_position(SINK, WINDOW, sp, MS)
                want = numpy_streaming_step(cfg, w, caches, [toks[sp]], [min(sp, max_active - 1)], sp, min(sp + 1, max_active),
                                            False, ring_start_of(sp), kvp, dt, kv8)
                got = m.forward_streaming([toks[sp]], [min(sp, max_active - 1)], sp, min(sp + 1, max_active), False, SINK,
                                          WINDOW, ring_start_of(sp), kvp)
                check(got, want, ("decode", sp))
                past += 1
                m.past_len = past
            for chunk in (4, 2):
                sp, after = past, past + prefill_len
                ids = toks[sp:sp + chunk] + [0] * (prefill_len - chunk)
                pos = [min(sp + i, max_active - 1) for i in range(prefill_len)]
                rs = 0 if after <= max_active else (after - SINK) % WINDOW
                kvp = orc.streaming_kv_position(SINK, WINDOW, after, MS)
                want = numpy_streaming_step(cfg, w, caches, ids, pos, sp, min(after, max_active), True, rs, kvp, dt, kv8)
                got = m.forward_streaming(ids, pos, sp, min(after, max_active), True, SINK, WINDOW, rs, kvp)
                check(got, want, ("prefill", sp))
                past += chunk
                m.past_len = past
    while past < 45:
        sp = past
        kvp = orc.streaming_kv_position(SINK, WINDOW, sp, MS)
        want = numpy_streaming_step(cfg, w, caches, [toks[sp]], [min(sp, max_active - 1)], sp, min(sp + 1, max_active), False,
                                    ring_start_of(sp), kvp, dt, kv8)
        # through the session entry: it builds these very inputs itself
        before = m.past_len
        m.decode_step(toks[sp])
        assert m.past_len == before + 1
        m.past_len = before
        got = m.forward_streaming([toks[sp]], [min(sp, max_active - 1)], sp, min(sp + 1, max_active), False, SINK, WINDOW,
                                  ring_start_of(sp), kvp)
        check(got, want, ("decode", sp))
        past += 1
        m.past_len = past
    if kv8:
        assert worst <= 2e-3, worst
    for l in range(L):
        k, v = m.kv_cache(l)
        assert np.array_equal(k, caches[l][0][0]) and np.array_equal(v, caches[l][1][0])


@pytest.mark.parametrize("kv8", [False, True])
@pytest.mark.parametrize("prefill_len", [0, 4])
def test_session_runs_past_the_window(kv8, prefill_len):
    """The four scenarios of crates/llm/tests/tinyllama_random.rs:157-315 on the oracle: max_seq 32, sink 4,
    window 16, want = sink + window + 10 new ids, past_len ends beyond sink + window (and no PromptTooLong)."""
    cfg, w, golden = llm_weights.tiny_llama_random(orc.BF16, max_seq=32)
    m = orc.Model(cfg, w)
    m.set_options(quant_kv_cache=kv8)
    m.set_streaming(SINK, WINDOW)
    want = SINK + WINDOW + 10
    ids = m.generate(golden["prompt_ids"], want, prefill_len=prefill_len)
    assert len(ids) == want and m.past_len > SINK + WINDOW
    # a second turn far past max_seq_len still runs
    ids2 = m.generate([5, 6, 7, 8, 9], 4, prefill_len=prefill_len)
    assert len(ids2) == 4 and m.past_len > cfg["max_seq"]
