"""Pins what the golden vectors leave open with closed forms, known answers of the reference's
own tests, invariants and brute force (chosen so a dropped term, wrong sign/index or transposed
operand fails)."""
import numpy as np
import pytest

import oracle as orc
from conftest import close_either, max_abs_rel

DT = [orc.F32, orc.BF16, orc.F16]


def test_f16_conversion_matches_numpy_exhaustively():
    bits = np.arange(65536, dtype=np.uint16)
    f = orc.to_f32(bits, orc.F16)
    want = bits.view(np.float16).astype(np.float32)
    assert np.array_equal(f.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(200000).astype(np.float32) * s for s in (1e-7, 1e-4, 1, 300, 7e4)])
    # exact ties and near-ties around every f16 boundary
    h = bits[(bits & 0x7C00) != 0x7C00].view(np.float16).astype(np.float32)
    nxt = np.nextafter(h.astype(np.float16), np.float16(np.inf)).astype(np.float32)
    mid = ((h.astype(np.float64) + nxt.astype(np.float64)) / 2).astype(np.float32)
    x = np.concatenate([x, mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf))])
    got = orc.to_storage(x, orc.F16)
    with np.errstate(over="ignore"):
        want16 = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want16)


def test_bf16_rne_formula():
    # crates/llm/src/quantize.rs:74-81: (bits + 0x7fff + ((bits >> 16) & 1)) >> 16
    rng = np.random.default_rng(1)
    x = rng.standard_normal(100000).astype(np.float32) * 37
    got = orc.to_storage(x, orc.BF16)
    b = x.view(np.uint32).astype(np.uint64)
    want = ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16)
    assert np.array_equal(got, want)


def test_rope_basic_known_answer():
    # crates/llm/tests/builder_ops.rs:264-287
    x = np.array([1, 2, 3, 4], np.float32).reshape(1, 1, 1, 4)
    cos = np.full((1, 4), 0.5, np.float32)
    sin = np.ones((1, 4), np.float32)
    got = orc.rope(x, cos, sin, [0], orc.F32)
    assert np.allclose(got.ravel(), [-2.5, -3.0, 2.5, 4.0], atol=1e-6)


def test_rope_table_known_answer():
    # crates/llm/tests/builder_ops.rs:289-336
    cos, sin = orc.rope_table(2, 4, 10000.0, orc.F32)
    c1, s1, c01, s01 = np.cos(1.0), np.sin(1.0), np.cos(0.01), np.sin(0.01)
    assert np.allclose(cos[1], [c1, c01, c1, c01], atol=1e-7)
    assert np.allclose(sin[1], [s1, s01, s1, s01], atol=1e-7)
    assert np.allclose(cos[0], 1) and np.allclose(sin[0], 0)
    x = np.array([1, 2, 3, 4], np.float32).reshape(1, 1, 1, 4)
    got = orc.rope(x, cos, sin, [1], orc.F32).ravel()
    want = [1 * c1 - 3 * s1, 2 * c01 - 4 * s01, 3 * c1 + 1 * s1, 4 * c01 + 2 * s01]
    ok, md = close_either(got, want, 1e-6)
    assert ok, md


def test_rope_table_bf16_is_truncated_f32():
    # src/session.rs:171-175 narrows f64 initializers with `(x as f32).to_bits() >> 16`
    cos, sin = orc.rope_table(64, 64, 10000.0, orc.BF16)
    p = np.arange(64, dtype=np.float64)[:, None]
    inv = 1.0 / np.power(10000.0, 2.0 * (np.arange(64) % 32) / 64.0)[None, :]
    want = (np.cos(p * inv).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    assert np.array_equal(cos, want)


@pytest.mark.parametrize("dt", DT)
def test_rope_is_a_rotation_and_matches_hf_rotate_half(dt):
    rng = np.random.default_rng(2)
    D, S, H = 64, 5, 3
    x = orc.to_storage(rng.standard_normal((1, H, S, D)), dt)
    cos, sin = orc.rope_table(16, D, 10000.0, dt)
    pos = np.array([3, 0, 7, 15, 1])
    got = orc.to_f32(orc.rope(x, cos, sin, pos, dt), dt).astype(np.float64)
    xf = orc.to_f32(x, dt).astype(np.float64)
    c = orc.to_f32(cos, dt).astype(np.float64)[pos][None, None]
    s = orc.to_f32(sin, dt).astype(np.float64)[pos][None, None]
    rot = np.concatenate([-xf[..., D // 2:], xf[..., :D // 2]], -1)
    want = xf * c + rot * s
    tol = {orc.F32: 1e-6, orc.BF16: 2.0 ** -7, orc.F16: 2.0 ** -10}[dt]
    ok, md = close_either(got, want, tol)
    assert ok, md
    if dt == orc.F32:  # norm preserved per (lo, hi) pair
        n0 = xf[..., :D // 2] ** 2 + xf[..., D // 2:] ** 2
        n1 = got[..., :D // 2] ** 2 + got[..., D // 2:] ** 2
        assert np.allclose(n0, n1, rtol=1e-5)
    assert np.array_equal(orc.rope(x, cos, sin, [0] * S, dt), x)  # position 0 is the identity


def test_rms_norm_known_answer():
    # crates/llm/tests/builder_ops.rs:103-128
    x = np.array([[1, 2, 3, 4]], np.float32)
    w = np.full(4, 0.5, np.float32)
    inv = 1.0 / np.sqrt(7.5 + 1e-5)
    got = orc.rms_norm(x, w, 1e-5, orc.F32)
    ok, md = close_either(got.ravel(), 0.5 * np.array([1, 2, 3, 4]) * inv, 1e-5)
    assert ok, md


@pytest.mark.parametrize("dt", DT)
def test_rms_norm_matches_torch(dt):
    import torch

    rng = np.random.default_rng(3)
    x = orc.to_storage(rng.standard_normal((7, 2048)) * 3, dt)
    w = orc.to_storage(rng.standard_normal(2048), dt)
    got = orc.to_f32(orc.rms_norm(x, w, 1e-5, dt), dt)
    want = torch.nn.functional.rms_norm(torch.from_numpy(orc.to_f32(x, dt)).double(), (2048,),
                                        torch.from_numpy(orc.to_f32(w, dt)).double(), 1e-5).numpy()
    tol = {orc.F32: 1e-5, orc.BF16: 2.0 ** -7, orc.F16: 2.0 ** -10}[dt]
    ok, md = close_either(got, want, tol)
    assert ok, md


def test_silu_known_answer_and_swiglu():
    # crates/llm/tests/builder_ops.rs:240-262: silu(x) = x * sigmoid(x)
    x = np.array([-2.0, -0.5, 0.0, 0.5, 3.0], np.float32)
    want = x / (1 + np.exp(-x.astype(np.float64)))
    ok, md = close_either(orc.swish(x, orc.F32), want, 1e-6)
    assert ok, md
    u = np.array([2.0, -1.0, 5.0, 0.25, -3.0], np.float32)
    ok, md = close_either(orc.swiglu(x, u, orc.F32), want * u, 1e-6)
    assert ok, md


def test_quantizer_known_answers():
    # crates/llm/tests/quantize.rs:106-159
    w = np.array([[127, -127, 0, 64], [2, -1, 0, 0.5], [0, 0, 0, 0]], np.float32)
    q, s = orc.quantize_per_channel(w, orc.BF16)
    sf = orc.to_f32(s, orc.BF16)
    assert np.allclose(sf, [1.0, 2 / 127, 1.0], atol=1e-3)
    assert list(q[0]) == [127, -127, 0, 64]
    assert list(q[1]) == [127, -64, 0, 32]  # -63.5 and 31.75: round half away from zero
    assert list(q[2]) == [0, 0, 0, 0]
    rng = np.random.default_rng(4)
    w = rng.standard_normal((33, 257)).astype(np.float32)
    q, s = orc.quantize_per_channel(w, orc.F32)
    amax = np.abs(w).max(1)
    assert np.allclose(s, amax / 127, rtol=1e-6)
    assert np.all(np.abs(q.astype(np.float32) * s[:, None] - w) <= (amax / 127)[:, None] * 0.5001)
    assert np.all(np.abs(q).max(1) == 127)


@pytest.mark.parametrize("lanes", [1, 16])
def test_gemv_cfg1_shape_against_f64_closed_form(lanes):
    """y[n] = s[n] * sum_k x[k] W[n,k], K=2048 N=5632 f32 (the single DequantizeLinear->MatMul
    subgraph of the first benchmark config); expected error ~ K * 2^-24 relative to |x|.|w|."""
    orc.set_lanes(lanes)
    try:
        rng = np.random.default_rng(5)
        K, N = 2048, 5632
        x = rng.standard_normal((1, K)).astype(np.float32)
        W = rng.integers(-127, 128, (N, K)).astype(np.int8)
        s = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
        got = orc.dequant_matmul(x, W, s, orc.F32, orc.F32, mode=-1)
        want = (W.astype(np.float64) @ x[0].astype(np.float64)) * s.astype(np.float64)
        bound = (np.abs(W).astype(np.float64) @ np.abs(x[0]).astype(np.float64)) * s * K * 2.0 ** -24
        assert np.all(np.abs(got[0] - want) <= bound)
        # a transposed operand or dropped scale cannot hide: compare one row computed by hand
        n = 1234
        assert abs(got[0, n] - s[n] * float(np.dot(W[n].astype(np.float64), x[0]))) <= bound[n]
    finally:
        orc.set_lanes(16)


@pytest.mark.parametrize("dt", [orc.BF16, orc.F16])
def test_dequant_matmul_modes_on_random_16bit(dt):
    rng = np.random.default_rng(6)
    M, N, K = 5, 96, 320
    act = orc.to_storage(rng.standard_normal((M, K)), dt)
    W = rng.integers(-127, 128, (N, K)).astype(np.int8)
    s = orc.to_storage(rng.uniform(5e-3, 1.2e-2, N), dt)
    a = orc.to_f32(act, dt).astype(np.float64)
    sf = orc.to_f32(s, dt).astype(np.float64)
    exact = (a @ W.astype(np.float64).T) * sf[None, :]
    tol = {orc.BF16: 2.0 ** -8, orc.F16: 2.0 ** -10}[dt]
    for mode in (0, 1):
        got = orc.to_f32(orc.dequant_matmul(act, W, s, dt, dt, mode=mode), dt)
        ok, md = close_either(got, exact, tol)
        assert ok, (mode, md)
    # mode 2 rounds the scaled weight first: closed form with that rounding applied
    wr = orc.to_f32(orc.to_storage((W.astype(np.float32) * orc.to_f32(s, dt)[:, None]), dt), dt).astype(np.float64)
    got = orc.to_f32(orc.dequant_matmul(act, W, s, dt, dt, mode=2), dt)
    ok, md = close_either(got, a @ wr.T, tol)
    assert ok, md


def test_quantized_matmul_extremes_are_exact():
    # accumulators at the int8 extremes: K * 128 * 128 must not wrap or lose bits
    K = 4096
    lhs = np.full((2, K), -128, np.int8)
    rhs = np.stack([np.full(K, -128, np.int8), np.full(K, 127, np.int8)])
    ones = np.ones(2, np.float32)
    out, acc = orc.quantized_matmul(lhs, ones, rhs, ones, orc.F32)
    assert acc.tolist() == [[K * 16384, -K * 16256]] * 2
    assert out.tolist() == [[float(K * 16384), float(-K * 16256)]] * 2


def test_dynquant_rule():
    x = np.array([[0.0, 0.0, 0.0], [1.0, -2.54, 0.5 * 2.54 / 127], [3.0, 1.5, -3.0]], np.float32)
    y, s = orc.dynquant_i8(x, orc.F32)
    assert s[0] == 1.0 and list(y[0]) == [0, 0, 0]  # zero row guard
    assert np.isclose(s[1], 2.54 / 127)
    assert list(y[1]) == [50, -127, 1]  # 0.5 rounds away from zero
    assert list(y[2]) == [127, 64, -127]  # 63.5 -> 64


@pytest.mark.parametrize("dt", DT)
def test_attention_invariants(dt):
    rng = np.random.default_rng(7)
    B, Hq, Hkv, L, D = 2, 8, 2, 37, 16
    q = orc.to_storage(rng.standard_normal((B, Hq, 1, D)), dt)
    k = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
    v = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
    tol = {orc.F32: 2e-6, orc.BF16: 2.0 ** -7, orc.F16: 2.0 ** -10}[dt]
    out = orc.to_f32(orc.attention(q, k, v, dt, 0.25), dt)
    ok, md = close_either(out, orc.attention_f64(q, k, v, dt, 0.25), tol)
    assert ok, md
    # active = 1 -> the first V row of the mapped kv head
    out1 = orc.attention(q, k, v, dt, 0.25, active=1)
    vf = v.reshape(B, Hkv, L, D)
    for h in range(Hq):
        assert np.array_equal(out1[:, h, 0], vf[:, h // (Hq // Hkv), 0])
    # GQA == MHA with K/V heads repeated
    kr, vr = np.repeat(k, Hq // Hkv, 1), np.repeat(v, Hq // Hkv, 1)
    assert np.array_equal(orc.attention(q, kr, vr, dt, 0.25), orc.attention(q, k, v, dt, 0.25))
    # uniform keys -> mean of V
    ku = np.repeat(k[:, :, :1], L, 2)
    outu = orc.to_f32(orc.attention(q, ku, v, dt, 0.25), dt)
    meanv = orc.to_f32(v, dt).astype(np.float64).mean(2)
    ok, md = close_either(outu[:, :, 0], np.repeat(meanv, Hq // Hkv, 1), tol * 4)
    assert ok, md
    # output is a convex combination of V rows
    vf32 = orc.to_f32(v, dt)
    lo = np.repeat(vf32.min(2), Hq // Hkv, 1)
    hi = np.repeat(vf32.max(2), Hq // Hkv, 1)
    assert np.all(out[:, :, 0] >= lo - 1e-2) and np.all(out[:, :, 0] <= hi + 1e-2)


def test_attention_causal_prefill_equals_stepwise_decode():
    rng = np.random.default_rng(8)
    Hq, Hkv, S, D, past = 4, 2, 6, 8, 3
    L = 16
    q = rng.standard_normal((1, Hq, S, D)).astype(np.float32)
    k = rng.standard_normal((1, Hkv, L, D)).astype(np.float32)
    v = rng.standard_normal((1, Hkv, L, D)).astype(np.float32)
    full = orc.attention(q, k, v, orc.F32, 0.3, True, past + S)
    for s in range(S):
        step = orc.attention(q[:, :, s:s + 1], k, v, orc.F32, 0.3, False, past + s + 1)
        assert np.allclose(full[:, :, s], step[:, :, 0], atol=1e-6)


def test_session_state_kv_attention_three_steps():
    """tests/session_state.rs:154-229: KVCacheUpdate + decode attention over 3 runs with the
    closed-form inputs sin(0.31 i + 1.7 step + 2.4 kind)/2, checked by f64 brute force."""
    B, H, S_MAX, D = 1, 2, 8, 4
    kc = np.zeros((B, H, S_MAX, D), np.float32)
    vc = np.zeros((B, H, S_MAX, D), np.float32)

    def data(step, kind):
        i = np.arange(B * H * D, dtype=np.float64)
        return np.clip(np.sin(i * 0.31 + step * 1.7 + kind * 2.4) * 0.5, -1, 1).astype(np.float32).reshape(B, H, 1, D)

    for step in range(3):
        q, sk, sv = data(step, 0), data(step, 1), data(step, 2)
        orc.kv_cache_update(kc, sk, step)
        orc.kv_cache_update(vc, sv, step)
        got = orc.attention(q, kc, vc, orc.F32, 1 / np.sqrt(D), False, step + 1)
        # brute force in numpy f64
        want = np.zeros((B, H, 1, D))
        for h in range(H):
            lg = (kc[0, h, :step + 1].astype(np.float64) @ q[0, h, 0].astype(np.float64)) / np.sqrt(D)
            p = np.exp(lg - lg.max())
            p /= p.sum()
            want[0, h, 0] = p @ vc[0, h, :step + 1].astype(np.float64)
        ok, md = close_either(got, want, 1e-4)
        assert ok, (step, md)


def test_quantizing_kv_update_rule_and_int8_attention():
    rng = np.random.default_rng(9)
    B, H, L, D = 1, 2, 8, 16
    cache = np.zeros((B, H, L, D), np.int8)
    scale = np.zeros((B, H, L), np.float32)
    new = rng.standard_normal((B, H, 3, D)).astype(np.float32)
    new[0, 1, 1] = 0  # zero row: scale 0, all zeros
    orc.quantizing_kv_cache_update(cache, scale, new, 2, orc.F32)
    amax = np.abs(new).max(-1)
    assert np.allclose(scale[:, :, 2:5], amax / 127, rtol=1e-6)
    assert np.all(cache[:, :, :2] == 0) and np.all(cache[:, :, 5:] == 0)
    deq = cache[:, :, 2:5].astype(np.float32) * scale[:, :, 2:5, None]
    assert np.all(np.abs(deq - new) <= (amax / 127)[..., None] * 0.501 + 1e-7)
    assert np.all(cache[0, 1, 3] == 0) and scale[0, 1, 3] == 0
    # int8-KV attention == float attention over the dequantised cache
    q = rng.standard_normal((B, 4, 1, D)).astype(np.float32)
    vc, vs = cache.copy(), scale.copy()
    got = orc.attention(q, cache, vc, orc.F32, 0.25, False, 5, k_scale=scale, v_scale=vs)
    full = cache.astype(np.float32) * scale[..., None]
    want = orc.attention_f64(q, full, full, orc.F32, 0.25, False, 5)
    ok, md = close_either(got, want, 1e-5)
    assert ok, md


def test_argmax_last_max_wins():
    # crates/llm/src/session.rs:683-690: Iterator::max_by returns the last maximum
    assert orc.argmax_last(np.array([1, 5, 3, 5, 2], np.float32), orc.F32) == 3
    assert orc.argmax_last(np.array([7, 7, 7], np.float32), orc.F32) == 2
    assert orc.argmax_last(orc.to_storage(np.array([0.1, -3, 0.1001]), orc.BF16), orc.BF16) == 2


def test_ring_index_and_streaming_positions():
    # cuda common.cuh:55-60
    assert [orc.ring_phys_index(r, 4, 0, 0) for r in range(6)] == list(range(6))
    assert [orc.ring_phys_index(r, 2, 4, 3) for r in range(6)] == [0, 1, 5, 2, 3, 4]
    # crates/llm/src/session.rs:604-635: unsaturated ring -> identity
    assert orc.streaming_kv_position(4, 28, 9, 32).tolist() == list(range(32))
    # saturated: sink 2, window 4, stream_pos 9 -> ring_start (9-2)%4 = 3; slot 2+3 is the oldest
    pos = orc.streaming_kv_position(2, 4, 9, 8).tolist()
    assert pos == [0, 1, 3, 4, 5, 2, 6, 7]


def test_ring_phys_index_is_the_sink_plus_ring_map():
    """common.cuh:55-60 against a hand-kept ring: ranks below the sink are fixed, the next `window` ranks are a
    bijection onto the ring rows starting at ring_start, window 0 is the identity."""
    for sink, window in [(0, 4), (4, 16), (3, 5), (4, 28)]:
        for start in range(window):
            ring = [sink + (start + i) % window for i in range(window)]  # row of the i-th oldest ring entry
            rows = [orc.ring_phys_index(r, sink, window, start) for r in range(sink + window)]
            assert rows[:sink] == list(range(sink))
            assert rows[sink:] == ring and sorted(rows) == list(range(sink + window))
    assert [orc.ring_phys_index(r, 4, 0, 3) for r in range(10)] == list(range(10))


def test_kv_cache_update_streaming_reduces_to_plain_update_and_wraps():
    rng = np.random.default_rng(0)
    B, H, L, D, sink, window = 2, 3, 24, 8, 4, 16
    new = rng.standard_normal((B, H, 5, D)).astype(np.float32)
    a = np.zeros((B, H, L, D), np.float32)
    b = np.zeros_like(a)
    # before the ring wraps (ring_start 0, rows below sink + window) it is the plain update
    orc.kv_cache_update_streaming(a, new, 9, sink, window, 0)
    orc.kv_cache_update(b, new, 9)
    assert np.array_equal(a, b)
    # wrapping: rows land at sink + (start + rank - sink) % window, later rows overwrite earlier ones
    c = np.zeros_like(a)
    orc.kv_cache_update_streaming(c, new, 17, sink, window, 6)
    want = np.zeros_like(a)
    for t in range(5):
        want[:, :, sink + (6 + 17 + t - sink) % window] = new[:, :, t]
    assert np.array_equal(c, want)
    assert not c[:, :, sink + window:].any() and not c[:, :, :sink].any()


@pytest.mark.parametrize("dt", [orc.F32, orc.F16])
@pytest.mark.parametrize("causal,Sq", [(False, 1), (True, 6)])
def test_attention_streaming_equals_attention_over_rank_ordered_rows(dt, causal, Sq):
    """Keys written in rank order into a cache through the ring map, then read back by the streaming attention,
    must give the attention over the rank-ordered rows themselves (f64 brute force): the two maps are inverse."""
    rng = np.random.default_rng(3)
    B, Hq, Hkv, D, L, sink, window, start, active = 2, 4, 2, 16, 32, 4, 16, 11, 19
    q = orc.to_storage(rng.standard_normal((B, Hq, Sq, D)), dt)
    k_rank = orc.to_storage(rng.standard_normal((B, Hkv, active, D)), dt)
    v_rank = orc.to_storage(rng.standard_normal((B, Hkv, active, D)), dt)
    k = orc.to_storage(np.full((B, Hkv, L, D), np.nan), dt)
    v = orc.to_storage(np.full((B, Hkv, L, D), np.nan), dt)
    for r in range(active):
        row = sink + (start + r - sink) % window if r >= sink else r
        k[:, :, row] = k_rank[:, :, r]
        v[:, :, row] = v_rank[:, :, r]
    got = orc.attention_streaming(q, k, v, dt, D ** -0.5, causal, active, sink, window, start)
    exact = orc.attention_f64(q, k_rank, v_rank, dt, D ** -0.5, causal, active)
    assert max_abs_rel(orc.to_f32(got, dt), exact) <= (1e-4 if dt == orc.F32 else 2e-3)



def test_quantizing_kv_cache_update_streaming_is_the_plain_rule_at_ring_rows():
    rng = np.random.default_rng(1)
    B, H, L, D, sink, window, start, offset = 1, 2, 24, 8, 4, 16, 5, 18
    new = orc.to_storage(rng.standard_normal((B, H, 3, D)), orc.BF16)
    c, s = np.zeros((B, H, L, D), np.int8), np.zeros((B, H, L), np.uint16)
    orc.quantizing_kv_cache_update_streaming(c, s, new, offset, sink, window, start, orc.BF16)
    pc, ps = np.zeros((B, H, L, D), np.int8), np.zeros((B, H, L), np.uint16)
    orc.quantizing_kv_cache_update(pc, ps, new, 0, orc.BF16)
    for t in range(3):
        row = sink + (start + offset + t - sink) % window
        assert np.array_equal(c[:, :, row], pc[:, :, t]) and np.array_equal(s[:, :, row], ps[:, :, t])
    assert np.count_nonzero(s) == 3 * H
