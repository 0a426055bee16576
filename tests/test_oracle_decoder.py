"""Whole-decoder pins for the oracle: the reference's exact greedy ids on its tiny random Llama
(crates/llm/tests/tinyllama_random.rs:20-24) and the generate-loop bookkeeping."""
import numpy as np
import pytest

import oracle as orc
import llm_weights


@pytest.mark.parametrize("dt", [orc.F32, orc.BF16, orc.F16])
def test_tiny_llama_random_golden_ids(dt):
    cfg, w, golden = llm_weights.tiny_llama_random(dt, max_seq=golden_max_seq())
    m = orc.Model(cfg, w)
    ids = m.generate(golden["prompt_ids"], len(golden["expected_new_ids"]))
    assert ids == golden["expected_new_ids"]
    # every prompt token and every generated token but the last is fed through one decode step
    # (crates/llm/tests/mock_decode.rs:44-52: 3 prompt ids + 5 new -> past_len 7)
    assert m.past_len == len(golden["prompt_ids"]) + len(ids) - 1
    m.close()


def golden_max_seq():
    return 4 + 28  # STREAM_SINK + STREAM_WINDOW of the reference test


@pytest.mark.parametrize("lanes", [1, 4, 64])
def test_tiny_llama_random_ids_do_not_depend_on_summation_order(lanes):
    orc.set_lanes(lanes)
    try:
        cfg, w, golden = llm_weights.tiny_llama_random(orc.BF16)
        m = orc.Model(cfg, w)
        assert m.generate(golden["prompt_ids"], 8) == golden["expected_new_ids"]
    finally:
        orc.set_lanes(16)


def test_prefill_matches_decode_only():
    """crates/llm/tests/tinyllama_random.rs cpu_multi_turn_prefill_matches_decode_only: a chunked,
    zero-padded prefill gives the same ids as feeding the prompt token by token."""
    cfg, w, golden = llm_weights.tiny_llama_random(orc.F32)
    prompt = [15043, 29892, 590, 1024, 338, 29871, 13, 450, 4996, 17354, 1701]
    a = orc.Model(cfg, w)
    ids_decode = a.generate(prompt, 6)
    b = orc.Model(cfg, w)
    ids_prefill = b.generate(prompt, 6, prefill_len=4)
    assert ids_decode == ids_prefill
    assert a.past_len == b.past_len == len(prompt) + 6 - 1
    # second turn on top of the kept KV cache
    assert a.generate([3038, 25190], 3) == b.generate([3038, 25190], 3, prefill_len=4)


def test_prompt_too_long_and_max_seq_stop():
    cfg, w, _ = llm_weights.tiny_llama_random(orc.F32, max_seq=8)
    m = orc.Model(cfg, w)
    with pytest.raises(ValueError):
        m.generate(list(range(9)), 1)
    with pytest.raises(ValueError):  # 5 tokens padded to 2 chunks of 4 = 8 fits, 9 padded to 12 does not
        m.generate(list(range(9)), 1, prefill_len=4)
    m.reset()
    ids = m.generate([1, 2, 3, 4, 5], 10)  # stops when past_len reaches max_seq
    assert m.past_len == 8 and len(ids) == 4, (m.past_len, ids)
    assert m.generate([], 5) == []


def test_forward_rows_are_causal():
    """Row s of a prefill run only sees tokens <= s: logits of a prefix do not change when the
    suffix does."""
    cfg, w, _ = llm_weights.tiny_llama_random(orc.F32)
    m = orc.Model(cfg, w)
    ids = np.array([5, 77, 3001, 12, 9], np.int64)
    pos = np.arange(5)
    a = m.forward(ids, pos, 0, 5, True)
    ids2 = ids.copy()
    ids2[3:] = [31999, 4]
    b = m.forward(ids2, pos, 0, 5, True)
    assert np.array_equal(a[:3], b[:3]) and not np.array_equal(a[3], b[3])


@pytest.mark.parametrize("dt", [orc.F32, orc.BF16])
def test_quant_kv_cache_and_quantize_activations_options_stay_close_to_the_plain_model(dt):
    """The two int8 options change storage/arithmetic precision, not the function: an int8 KV cache
    (127 levels per token row) and W8A8 linears (127 levels per activation row) must leave the logits
    within a few percent of the plain model's, the caches must dequantise to the plain caches within
    half a quantisation step, and the options must actually change the arithmetic."""
    cfg = dict(n_layers=2, hidden=64, n_heads=4, n_kv_heads=2, head_dim=16, ffn=96, vocab=200, max_seq=24,
               eps=1e-5, rope_theta=10000.0)
    cfg, w = llm_weights.synthetic_int8(cfg, dt, seed=2)
    ids = np.random.default_rng(0).integers(0, cfg["vocab"], 10)
    pos = np.arange(10)
    plain = orc.Model(cfg, w)
    base = orc.to_f32(plain.forward(ids, pos, 0, 10, True), dt)
    for kv8, w8a8 in [(True, False), (False, True), (True, True)]:
        m = orc.Model(cfg, w)
        m.set_options(quant_kv_cache=kv8, quantize_activations=w8a8)
        got = orc.to_f32(m.forward(ids, pos, 0, 10, True), dt)
        err = np.abs(got - base).max() / np.abs(base).max()
        assert 0 < err < 0.08, (kv8, w8a8, err)
        if kv8 and not w8a8:
            for l in range(cfg["n_layers"]):
                kq, vq = m.kv_cache(l)
                ks, vs = m.kv_scales(l)
                kp, vp = plain.kv_cache(l)
                assert kq.dtype == np.int8
                kd = kq[:, :10].astype(np.float32) * orc.to_f32(ks, dt)[:, :10, None]
                if l == 0:  # layer 0 sees identical inputs in both models
                    step = orc.to_f32(ks, dt)[:, :10, None]
                    # half a step from the rounding, plus 127 codes times the rounding of the stored scale
                    slack = 0.5 * 1.02 + (127 * 2.0 ** -8 if dt == orc.BF16 else 0.0)
                    assert np.all(np.abs(kd - orc.to_f32(kp, dt)[:, :10]) <= slack * step + 1e-6)
                assert np.abs(kq[:, :10]).max() == 127 and not kq[:, 10:].any()


# ------------------------------------------------------------------ q / k / v projection bias (qwen2)
def decoder_f64(cfg, w, ids):
    """Independent float64 statement of the decoder over a whole prompt (textbook form: y = x W^T + b, rotate-half
    RoPE, causal softmax attention with grouped kv heads, SwiGLU), plain float weights; returns logits [S, vocab]."""
    H, Hq, Hkv, D = cfg["hidden"], cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    S = len(ids)
    f = lambda a: np.asarray(a, np.float64)
    rms = lambda x, g: x / np.sqrt((x * x).mean(-1, keepdims=True) + cfg["eps"]) * f(g)
    inv = cfg["rope_theta"] ** (-np.arange(0, D, 2, dtype=np.float64) / D)
    ang = np.arange(S, dtype=np.float64)[:, None] * inv[None, :]
    cos, sin = np.cos(np.concatenate([ang, ang], -1)), np.sin(np.concatenate([ang, ang], -1))
    rot = lambda t: np.concatenate([-t[..., D // 2:], t[..., :D // 2]], -1)
    x = f(w["embed"])[ids]
    for l in range(cfg["n_layers"]):
        g = lambda nm: f(w["layers.%d.%s" % (l, nm)])
        b = lambda nm: f(w.get("layers.%d.%s.bias" % (l, nm), 0.0))
        n = rms(x, w["layers.%d.norm1" % l])
        q = (n @ g("q").T + b("q")).reshape(S, Hq, D)
        k = (n @ g("k").T + b("k")).reshape(S, Hkv, D)
        v = (n @ g("v").T + b("v")).reshape(S, Hkv, D)
        q = q * cos[:, None] + rot(q) * sin[:, None]
        k = k * cos[:, None] + rot(k) * sin[:, None]
        o = np.zeros((S, Hq, D))
        for h in range(Hq):
            kh = h // (Hq // Hkv)
            sc = q[:, h] @ k[:, kh].T / np.sqrt(D)
            sc = np.where(np.tril(np.ones((S, S), bool)), sc, -np.inf)
            p = np.exp(sc - sc.max(-1, keepdims=True))
            o[:, h] = (p / p.sum(-1, keepdims=True)) @ v[:, kh]
        x = x + o.reshape(S, Hq * D) @ g("o").T
        n = rms(x, w["layers.%d.norm2" % l])
        a, u = n @ g("gate").T, n @ g("up").T
        x = x + (a / (1 + np.exp(-a)) * u) @ g("down").T
    return rms(x, w["final_norm"]) @ f(w["lm_head"]).T


BIAS_CFG = dict(n_layers=2, hidden=64, n_heads=4, n_kv_heads=2, head_dim=16, ffn=96, vocab=50, max_seq=16, eps=1e-5,
                rope_theta=10000.0)


def plain_f32_weights(cfg, seed):
    rng = np.random.default_rng(seed)
    H, F, V = cfg["hidden"], cfg["ffn"], cfg["vocab"]
    QD, KD = cfg["n_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"]
    r = lambda *s: (rng.standard_normal(s) * 0.2).astype(np.float32)
    w = {"embed": r(V, H), "lm_head": r(V, H), "final_norm": (1 + 0.1 * rng.standard_normal(H)).astype(np.float32)}
    for l in range(cfg["n_layers"]):
        for nm, (n, k) in {"q": (QD, H), "k": (KD, H), "v": (KD, H), "o": (H, QD), "gate": (F, H), "up": (F, H), "down": (H, F)}.items():
            w["layers.%d.%s" % (l, nm)] = r(n, k)
        w["layers.%d.norm1" % l] = (1 + 0.1 * rng.standard_normal(H)).astype(np.float32)
        w["layers.%d.norm2" % l] = (1 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    return w


def test_qkv_bias_against_an_independent_f64_decoder():
    """The bias path of decoder.rs:167-184 has no fixture in the reference (its only checkpoint is a Llama): the oracle's
    f32 model with biases must follow a float64 textbook decoder, with one bias at a time and with all three -- a bias
    added after RoPE, to the wrong projection, or scaled, would miss by the size of the bias's effect, which the test
    shows to be orders of magnitude above the bound."""
    cfg = dict(BIAS_CFG, dtype=orc.F32)
    w = plain_f32_weights(cfg, 3)
    wb = llm_weights.add_qkv_bias(cfg, w, orc.F32, seed=4)
    ids = np.array([3, 41, 7, 7, 19, 0, 33], np.int64)
    base = decoder_f64(cfg, w, ids)
    assert np.max(np.abs(orc.Model(cfg, w).forward(ids, np.arange(len(ids)), 0, len(ids), True) - base)) <= 1e-4 * np.max(np.abs(base))
    for which in (("q",), ("k",), ("v",), ("q", "k", "v")):
        wsel = {k: v for k, v in wb.items() if not k.endswith(".bias") or k.split(".")[-2] in which}
        want = decoder_f64(cfg, wsel, ids)
        got = orc.Model(cfg, wsel).forward(ids, np.arange(len(ids)), 0, len(ids), True)
        assert np.max(np.abs(got - want)) <= 1e-4 * np.max(np.abs(want)), which
        if which != ("k",):  # (a k bias alone shifts every score of a query by nearly the same amount: its effect is small)
            assert np.max(np.abs(want - base)) >= 1e-2 * np.max(np.abs(base)), which


@pytest.mark.parametrize("dt", [orc.F32, orc.BF16, orc.F16])
def test_zero_qkv_bias_changes_no_bit_and_decode_equals_prefill(dt):
    cfg, w, golden = llm_weights.tiny_llama_random(dt)
    zero = {k: orc.to_storage(np.zeros_like(orc.to_f32(v, dt)), dt) for k, v in llm_weights.add_qkv_bias(cfg, w, dt).items()
            if k.endswith(".bias")}
    m = orc.Model(cfg, dict(w, **zero))
    assert m.generate(golden["prompt_ids"], 8) == golden["expected_new_ids"]
    # with real biases: feeding a prompt token by token and as one prefill give the same rows (f32: to rounding)
    wb = llm_weights.add_qkv_bias(cfg, w, dt, std=0.1)
    a, b = orc.Model(cfg, wb), orc.Model(cfg, wb)
    ids = np.array(golden["prompt_ids"] + [7, 99], np.int64)
    full = a.forward(ids, np.arange(len(ids)), 0, len(ids), True)
    for i, t in enumerate(ids):
        row = b.forward([t], [i], i, i + 1, False)
    fl, rl = orc.to_f32(full[-1], dt), orc.to_f32(row[0], dt)
    assert np.max(np.abs(fl - rl)) <= (1e-5 if dt == orc.F32 else 3e-2) * np.max(np.abs(fl))


@pytest.mark.parametrize("dt", [orc.F32, orc.BF16, orc.F16])
@pytest.mark.parametrize("kv8,w8a8", [(False, False), (True, False), (False, True), (True, True)])
def test_decoder_options_equal_the_composition_of_the_pinned_operators(dt, kv8, w8a8):
    """BuildOptions::quant_kv_cache and Options::quantize_activations in the C decoder against the same graph composed
    in numpy from the operator-level functions (DynamicQuantizeLinear + QuantizedMatMul for every int8 linear with
    K % 32 == 0, RoPE before the quantising cache update, scales into the attention): bit-equal logits and caches over
    a 12-token causal prefill chunk and 10 decode steps of a 2-layer model."""
    from oracle_compose import compose_step, empty_caches

    shape = dict(n_layers=2, hidden=64, n_heads=4, n_kv_heads=2, head_dim=16, ffn=96, vocab=97, max_seq=32, eps=1e-5,
                 rope_theta=10000.0)
    cfg, w = llm_weights.synthetic_int8(shape, dt, seed=21)
    m = orc.Model(cfg, w)
    m.set_options(quant_kv_cache=kv8, quantize_activations=w8a8)
    caches = empty_caches(cfg, dt, kv8)
    rng = np.random.default_rng(3)
    ids = [int(t) for t in rng.integers(0, cfg["vocab"], 12)]
    want = compose_step(cfg, w, caches, ids, list(range(12)), 0, 12, True, dt, kv8=kv8, w8a8=w8a8)
    assert np.array_equal(m.forward(ids, np.arange(12), 0, 12, True), want)
    for p in range(12, 22):
        t = int(rng.integers(0, cfg["vocab"]))
        want = compose_step(cfg, w, caches, [t], [p], p, p + 1, False, dt, kv8=kv8, w8a8=w8a8)
        assert np.array_equal(m.forward([t], [p], p, p + 1, False), want), p
    for l in range(cfg["n_layers"]):
        k, v = m.kv_cache(l)
        assert np.array_equal(k, caches[l][0][0]) and np.array_equal(v, caches[l][1][0])
        if kv8:
            ks, vs = m.kv_scales(l)
            assert np.array_equal(ks, caches[l][2][0]) and np.array_equal(vs, caches[l][3][0])
