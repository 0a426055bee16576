"""GPU parity of the GQA attention kernels against the oracle, the reference's golden vectors
and the f64 brute force of the reference's own state test (tests/session_state.rs:122-229)."""
import os

import numpy as np
import pytest

import oracle as orc
import pbreader
from conftest import GOLDEN, close_either, max_abs_rel, max_err_rel_to_max

pytestmark = pytest.mark.gpu
SO = os.path.join(GOLDEN, "single_op")


@pytest.fixture(scope="module")
def g():
    import gpu_util

    return gpu_util


@pytest.mark.parametrize("name,causal,scale,active_slot", [
    ("attention_decode", False, 8 ** -0.5, None),
    ("attention_decode_gqa", False, 8 ** -0.5, None),
    ("attention_decode_runtime_kv", False, 0.5, 3),
    ("attention_causal", True, 8 ** -0.5, None),
    ("attention_no_causal", False, 8 ** -0.5, None),
])
def test_attention_golden(g, name, causal, scale, active_slot):
    ins, (o,) = pbreader.read_case(os.path.join(SO, name))
    q, k, v = ins[0], ins[1], ins[2]
    active = int(ins[active_slot].array) if active_slot is not None else None
    got = g.to_host(g.mynn.attention(g.to_dev(q.array), g.to_dev(k.array), g.to_dev(v.array), scale, causal, active))
    ok, md = close_either(got, o.array, 1e-4)
    assert ok, md


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("B,L", [(1, 512), (4, 2048), (16, 512), (2, 4096), (1, 37), (3, 1), (1, 2048), (1, 4096), (4, 512),
                                 (4, 4096), (16, 2048), (16, 4096)])
def test_decode_attention_vs_oracle_cfg2_shapes(g, dt, B, L):
    """GQA decode attention op of the second benchmark config: 32 query heads, 4 KV heads,
    head_dim 64, softmax scale 1/8, no mask beyond the cache length."""
    rng = np.random.default_rng(B * 10007 + L)
    Hq, Hkv, D = 32, 4, 64
    q = orc.to_storage(rng.standard_normal((B, Hq, 1, D)), dt)
    k = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
    v = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
    want = orc.attention(q, k, v, dt, 0.125)
    got = g.to_host(g.mynn.attention(g.to_dev(q, dt), g.to_dev(k, dt), g.to_dev(v, dt), 0.125))
    assert max_abs_rel(g.f32(got, dt), g.f32(want, dt)) <= 1e-2
    exact = orc.attention_f64(q, k, v, dt, 0.125)
    assert max_abs_rel(g.f32(got, dt), exact) <= 1e-2


@pytest.mark.parametrize("dt", [orc.F32, orc.F16])
@pytest.mark.parametrize("Hq,Hkv,D", [(8, 8, 128), (32, 8, 128), (4, 2, 8), (6, 3, 32), (4, 1, 16)])
def test_decode_attention_head_shapes_and_active_length(g, dt, Hq, Hkv, D):
    import torch

    rng = np.random.default_rng(Hq * 100 + D)
    B, L, active = 2, 300, 173
    q = orc.to_storage(rng.standard_normal((B, Hq, 1, D)), dt)
    k = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
    v = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
    want = orc.attention(q, k, v, dt, D ** -0.5, False, active)
    tol = 1e-4 if dt == orc.F32 else 1e-2
    got = g.to_host(g.mynn.attention(g.to_dev(q, dt), g.to_dev(k, dt), g.to_dev(v, dt), D ** -0.5, False, active))
    assert max_abs_rel(g.f32(got, dt), g.f32(want, dt)) <= tol
    # the same with the active length read on the device (what a captured graph replays)
    d_active = torch.tensor([active], dtype=torch.int32, device="cuda")
    got2 = g.to_host(g.mynn.attention(g.to_dev(q, dt), g.to_dev(k, dt), g.to_dev(v, dt), D ** -0.5, False,
                                      active=L, d_active=d_active))
    assert max_abs_rel(g.f32(got2, dt), g.f32(want, dt)) <= tol
    # rows beyond `active` are never read: poison them
    k2, v2 = k.copy(), v.copy()
    k2[:, :, active:] = orc.to_storage(np.full((B, Hkv, L - active, D), np.nan), dt)
    v2[:, :, active:] = orc.to_storage(np.full((B, Hkv, L - active, D), np.nan), dt)
    got3 = g.to_host(g.mynn.attention(g.to_dev(q, dt), g.to_dev(k2, dt), g.to_dev(v2, dt), D ** -0.5, False, active))
    assert np.array_equal(got3, got)


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("B,Hq,Hkv,D,L,active", [(8, 32, 8, 128, 1100, 1037), (16, 32, 4, 64, 700, 613),
                                                 (8, 8, 8, 64, 600, 600), (4, 16, 8, 64, 1200, 1111),
                                                 (32, 32, 8, 128, 160, 129)])
def test_streaming_decode_attention_vs_oracle(g, dt, B, Hq, Hkv, D, L, active):
    """Batch x context products large enough for the streaming kernel (matrix-core scores, online
    softmax, key ranges merged by the last workgroup): ragged active lengths, the length read on the
    device, and rows beyond it poisoned."""
    import torch

    assert B * Hkv * min(active, L) >= 8192 or B * Hkv * L >= 8192
    rng = np.random.default_rng(B * 31 + D + active)
    q = orc.to_storage(rng.standard_normal((B, Hq, 1, D)), dt)
    k = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
    v = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
    k[:, :, active:] = orc.to_storage(np.full((B, Hkv, L - active, D), np.nan), dt)
    v[:, :, active:] = orc.to_storage(np.full((B, Hkv, L - active, D), np.nan), dt)
    want = orc.attention(q, k, v, dt, D ** -0.5, False, active)
    exact = orc.attention_f64(q, k, v, dt, D ** -0.5, False, active)
    dq, dk, dv = g.to_dev(q, dt), g.to_dev(k, dt), g.to_dev(v, dt)
    d_active = torch.tensor([active], dtype=torch.int32, device="cuda")
    for rep in range(2):  # the second call finds the merge counters as the first left them
        got = g.to_host(g.mynn.attention(dq, dk, dv, D ** -0.5, False, active=L, d_active=d_active))
        assert max_abs_rel(g.f32(got, dt), g.f32(want, dt)) <= 1e-2, rep
        assert max_abs_rel(g.f32(got, dt), exact) <= 1e-2, rep
    if B * Hkv * active >= 8192:
        got = g.to_host(g.mynn.attention(dq, dk, dv, D ** -0.5, False, active))
        assert max_abs_rel(g.f32(got, dt), exact) <= 1e-2


def test_decode_attention_seeded_shape_sweep(g):
    """48 seeded shapes across the dispatch boundaries of the decode kernels (caches of 1..700 rows, shorter
    and longer than a 32-key tile; batch x heads x context on either side of the streaming kernel's threshold;
    1..8 query heads per kv head; head dims 32/64/128; the length passed by value or read on the device; the
    tail of the cache poisoned) against the f64 formula."""
    import torch

    rng = np.random.default_rng(2024)
    for case in range(48):
        dt = [orc.F16, orc.BF16][case % 2]
        D = [32, 64, 128][int(rng.integers(0, 3))]
        Hkv = int(rng.choice([1, 2, 4, 8]))
        G = int(rng.choice([1, 2, 4, 8]))
        Hq = Hkv * G
        L = int(rng.choice([1, 3, 17, 31, 32, 33, 64, 100, 257, 512, 700]))
        B = int(rng.choice([1, 2, 5, 16, 40])) if L * Hkv < 3000 else int(rng.choice([1, 3, 12]))
        active = int(rng.integers(1, L + 1))
        q = orc.to_storage(rng.standard_normal((B, Hq, 1, D)), dt)
        k = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
        v = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
        if active < L:
            k[:, :, active:] = orc.to_storage(np.full((B, Hkv, L - active, D), np.nan), dt)
            v[:, :, active:] = orc.to_storage(np.full((B, Hkv, L - active, D), np.nan), dt)
        exact = orc.attention_f64(q, k, v, dt, D ** -0.5, False, active)
        dq, dk, dv = g.to_dev(q, dt), g.to_dev(k, dt), g.to_dev(v, dt)
        if case % 3 == 0:
            d_active = torch.tensor([active], dtype=torch.int32, device="cuda")
            got = g.mynn.attention(dq, dk, dv, D ** -0.5, False, active=L, d_active=d_active)
        else:
            got = g.mynn.attention(dq, dk, dv, D ** -0.5, False, active)
        got = g.f32(g.to_host(got), dt)
        assert not np.isnan(got).any(), (case, B, Hq, Hkv, D, L, active)
        assert max_err_rel_to_max(got, exact) <= (4e-3 if dt == orc.BF16 else 1e-3), (case, B, Hq, Hkv, D, L, active)


@pytest.mark.parametrize("dt", [orc.F32, orc.F16, orc.BF16])
def test_attention_invariants_on_gpu(g, dt):
    rng = np.random.default_rng(11)
    B, Hq, Hkv, L, D = 2, 8, 2, 200, 64
    q = orc.to_storage(rng.standard_normal((B, Hq, 1, D)), dt)
    k = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
    v = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
    dq, dk, dv = g.to_dev(q, dt), g.to_dev(k, dt), g.to_dev(v, dt)
    # active = 1 -> exactly the first V row of the mapped kv head
    out1 = g.to_host(g.mynn.attention(dq, dk, dv, 0.125, False, 1))
    for h in range(Hq):
        assert np.array_equal(out1[:, h, 0], v[:, h // (Hq // Hkv), 0])
    # uniform keys -> mean of V
    ku = np.repeat(k[:, :, :1], L, 2)
    outu = g.f32(g.to_host(g.mynn.attention(dq, g.to_dev(ku, dt), dv, 0.125)), dt)
    meanv = np.repeat(g.f32(v, dt).astype(np.float64).mean(2), Hq // Hkv, 1)
    tol = 1e-5 if dt == orc.F32 else 1e-2
    assert max_abs_rel(outu[:, :, 0], meanv) <= tol
    # GQA == MHA with K/V heads repeated
    kr, vr = np.repeat(k, Hq // Hkv, 1), np.repeat(v, Hq // Hkv, 1)
    a = g.to_host(g.mynn.attention(dq, dk, dv, 0.125))
    b = g.to_host(g.mynn.attention(dq, g.to_dev(kr, dt), g.to_dev(vr, dt), 0.125))
    assert max_abs_rel(g.f32(a, dt), g.f32(b, dt)) <= tol


@pytest.mark.parametrize("dt", [orc.F32, orc.F16])
def test_causal_rows_plain_path(g, dt):
    """Sq > 1 with a past: row sq sees keys [0, past + sq + 1)."""
    rng = np.random.default_rng(12)
    Hq, Hkv, S, D, past, L = 8, 2, 9, 64, 5, 32
    q = orc.to_storage(rng.standard_normal((1, Hq, S, D)), dt)
    k = orc.to_storage(rng.standard_normal((1, Hkv, L, D)), dt)
    v = orc.to_storage(rng.standard_normal((1, Hkv, L, D)), dt)
    want = orc.attention(q, k, v, dt, 0.125, True, past + S)
    got = g.to_host(g.mynn.attention(g.to_dev(q, dt), g.to_dev(k, dt), g.to_dev(v, dt), 0.125, True, past + S))
    assert max_abs_rel(g.f32(got, dt), g.f32(want, dt)) <= (1e-4 if dt == orc.F32 else 1e-2)


def test_session_state_three_steps_on_gpu(g):
    B, H, S_MAX, D = 1, 2, 8, 4
    kc = g.to_dev(np.zeros((B, H, S_MAX, D), np.float32))
    vc = g.to_dev(np.zeros((B, H, S_MAX, D), np.float32))
    kh = np.zeros((B, H, S_MAX, D), np.float32)
    vh = np.zeros((B, H, S_MAX, D), np.float32)

    def data(step, kind):
        i = np.arange(B * H * D, dtype=np.float64)
        return np.clip(np.sin(i * 0.31 + step * 1.7 + kind * 2.4) * 0.5, -1, 1).astype(np.float32).reshape(B, H, 1, D)

    for step in range(3):
        q, sk, sv = data(step, 0), data(step, 1), data(step, 2)
        g.mynn.kvcache_update(kc, g.to_dev(sk), step)
        g.mynn.kvcache_update(vc, g.to_dev(sv), step)
        kh[:, :, step], vh[:, :, step] = sk[:, :, 0], sv[:, :, 0]
        got = g.to_host(g.mynn.attention(g.to_dev(q), kc, vc, 1 / np.sqrt(D), False, step + 1))
        want = orc.attention_f64(q, kh, vh, orc.F32, 1 / np.sqrt(D), False, step + 1)
        ok, md = close_either(got, want, 1e-4)
        assert ok, (step, md)


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
def test_int8_kv_attention(g, dt):
    rng = np.random.default_rng(13)
    B, Hq, Hkv, L, D = 2, 32, 4, 257, 64
    q = orc.to_storage(rng.standard_normal((B, Hq, 1, D)), dt)
    kc = np.zeros((B, Hkv, L, D), np.int8)
    vc = np.zeros((B, Hkv, L, D), np.int8)
    ks = orc.to_storage(np.zeros((B, Hkv, L)), dt)
    vs = orc.to_storage(np.zeros((B, Hkv, L)), dt)
    orc.quantizing_kv_cache_update(kc, ks, orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt), 0, dt)
    orc.quantizing_kv_cache_update(vc, vs, orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt), 0, dt)
    want = orc.attention(q, kc, vc, dt, 0.125, False, 200, k_scale=ks, v_scale=vs)
    got = g.to_host(g.mynn.attention(g.to_dev(q, dt), g.to_dev(kc), g.to_dev(vc), 0.125, False, 200,
                                     k_scale=g.to_dev(ks, dt), v_scale=g.to_dev(vs, dt)))
    assert max_abs_rel(g.f32(got, dt), g.f32(want, dt)) <= 1e-2


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("B,Hq,Hkv,D,L,active", [(16, 32, 4, 64, 700, 613), (8, 32, 8, 128, 1100, 1037)])
def test_streaming_decode_attention_int8_kv(g, dt, B, Hq, Hkv, D, L, active):
    """The streaming kernel over an int8 cache with per-token scales (k scale on the score, v scale on p),
    rows beyond the active length poisoned with the most negative code and a NaN scale."""
    rng = np.random.default_rng(active + D)
    q = orc.to_storage(rng.standard_normal((B, Hq, 1, D)), dt)
    kc = np.zeros((B, Hkv, L, D), np.int8)
    vc = np.zeros((B, Hkv, L, D), np.int8)
    ks = orc.to_storage(np.zeros((B, Hkv, L)), dt)
    vs = orc.to_storage(np.zeros((B, Hkv, L)), dt)
    orc.quantizing_kv_cache_update(kc, ks, orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt), 0, dt)
    orc.quantizing_kv_cache_update(vc, vs, orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt), 0, dt)
    kc[:, :, active:] = -128
    vc[:, :, active:] = -128
    ks[:, :, active:] = orc.to_storage(np.full((B, Hkv, L - active), np.nan), dt)
    vs[:, :, active:] = orc.to_storage(np.full((B, Hkv, L - active), np.nan), dt)
    want = orc.attention(q, kc, vc, dt, D ** -0.5, False, active, k_scale=ks, v_scale=vs)
    got = g.to_host(g.mynn.attention(g.to_dev(q, dt), g.to_dev(kc), g.to_dev(vc), D ** -0.5, False, active,
                                     k_scale=g.to_dev(ks, dt), v_scale=g.to_dev(vs, dt)))
    assert max_abs_rel(g.f32(got, dt), g.f32(want, dt)) <= 1e-2


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("B,Hq,Hkv,S,D,past,causal", [
    (1, 8, 2, 128, 64, 0, True),
    (2, 4, 4, 100, 64, 0, True),      # ragged: rows past the last 128-row block, MHA
    (1, 32, 4, 257, 64, 31, True),    # TinyLlama heads, a past, odd length
    (1, 8, 8, 64, 128, 0, True),      # head_dim 128
    (2, 16, 2, 96, 128, 40, True),    # 8 query heads per kv head, D=128
    (1, 4, 2, 130, 64, 0, False),     # full (non-causal) attention
    (1, 2, 1, 16, 64, 5, True),       # the smallest shape the matrix-core kernel takes
])
def test_prefill_attention_matrix_cores_vs_oracle(g, dt, B, Hq, Hkv, S, D, past, causal):
    rng = np.random.default_rng(S * 131 + D + past)
    L = past + S + 7  # cache longer than the active prefix
    q = orc.to_storage(rng.standard_normal((B, Hq, S, D)), dt)
    k = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
    v = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
    # rows beyond the active prefix must never be read
    k[:, :, past + S:] = orc.to_storage(np.full((B, Hkv, L - past - S, D), np.nan), dt)
    v[:, :, past + S:] = orc.to_storage(np.full((B, Hkv, L - past - S, D), np.nan), dt)
    scale = D ** -0.5
    want = orc.attention_f64(q, k, v, dt, scale, causal, past + S)
    got = g.to_host(g.mynn.attention(g.to_dev(q, dt), g.to_dev(k, dt), g.to_dev(v, dt), scale, causal, past + S))
    assert not np.isnan(g.f32(got, dt)).any()
    # The probabilities enter the second product in the 16-bit type (as in the reference's
    # tensor-core kernel, attention.cuh:45-314), so the error is set by the tensor's scale, not by
    # each element's: an output near zero that is the sum of +-v terms carries the same absolute
    # error as a large one.  Bound: error / max|out| <= 1e-2 (measured: ~1e-3 bf16, ~1e-4 f16).
    assert max_err_rel_to_max(g.f32(got, dt), want) <= (3e-3 if dt == orc.BF16 else 5e-4)
    ref = orc.attention(q, k, v, dt, scale, causal, past + S)
    assert max_err_rel_to_max(g.f32(got, dt), g.f32(ref, dt)) <= 1e-2
    if dt == orc.F16:
        assert max_abs_rel(g.f32(got, dt), want) <= 1e-2  # elementwise too at fp16 resolution


def test_prefill_attention_rows_equal_decode_rows(g):
    """Size-independent property at the full prefill length (1024 rows, TinyLlama heads): each
    causal row equals a decode call with that row's prefix."""
    dt = orc.F16
    rng = np.random.default_rng(77)
    Hq, Hkv, S, D = 32, 4, 1024, 64
    q = orc.to_storage(rng.standard_normal((1, Hq, S, D)), dt)
    k = orc.to_storage(rng.standard_normal((1, Hkv, S, D)), dt)
    v = orc.to_storage(rng.standard_normal((1, Hkv, S, D)), dt)
    dq, dk, dv = g.to_dev(q, dt), g.to_dev(k, dt), g.to_dev(v, dt)
    full = g.f32(g.to_host(g.mynn.attention(dq, dk, dv, 0.125, True, S)), dt)
    for row in (0, 1, 31, 32, 500, 1023):
        one = g.mynn.attention(dq[:, :, row:row + 1].contiguous(), dk, dv, 0.125, False, row + 1)
        assert max_err_rel_to_max(full[:, :, row], g.f32(g.to_host(one), dt)[:, :, 0]) <= 2e-3, row
    assert np.array_equal(full[:, :, 0], np.repeat(g.f32(v, dt)[:, :, 0], Hq // Hkv, 1))  # first row sees one key


# ---- streaming KV (sink + ring cache): the slot map of common.cuh:55-60 in KVCacheUpdate and Attention
@pytest.mark.parametrize("kind", ["f16", "f32", "i8"])
@pytest.mark.parametrize("offset,S_new,sink,window,start", [
    (9, 5, 4, 16, 0),      # not wrapped: the plain update
    (17, 5, 4, 16, 6),     # wraps inside the ring
    (2, 7, 4, 16, 3),      # rows on both sides of the sink boundary
    (20, 40, 4, 16, 9),    # more rows than ring slots: later rows win
    (3, 6, 0, 0, 0),       # ring switched off
])
def test_kvcache_update_streaming_bit_exact(g, kind, offset, S_new, sink, window, start):
    import torch

    rng = np.random.default_rng(offset * 7 + S_new)
    B, H, L, D = 2, 3, 64, 32
    npdt = {"f16": np.uint16, "f32": np.float32, "i8": np.int8}[kind]
    if kind == "f32":
        cache = rng.standard_normal((B, H, L, D)).astype(np.float32)
        new = rng.standard_normal((B, H, S_new, D)).astype(np.float32)
    else:
        hi = 65536 if kind == "f16" else 128
        lo = 0 if kind == "f16" else -128
        cache = rng.integers(lo, hi, (B, H, L, D)).astype(npdt)
        new = rng.integers(lo, hi, (B, H, S_new, D)).astype(npdt)
    want = orc.kv_cache_update_streaming(cache.copy(), new, offset, sink, window, start)
    tdt = {"f16": torch.float16, "f32": torch.float32, "i8": torch.int8}[kind]
    dc = torch.from_numpy(cache.view(np.int16) if kind == "f16" else cache).cuda()
    dn = torch.from_numpy(new.view(np.int16) if kind == "f16" else new).cuda()
    if kind == "f16":
        dc, dn = dc.view(tdt), dn.view(tdt)
    g.mynn.kvcache_update_streaming(dc, dn, offset, sink, window, start)
    got = dc.view(torch.int16).cpu().numpy().view(np.uint16) if kind == "f16" else dc.cpu().numpy()
    assert np.array_equal(got, want)


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("Sq,causal,sink,window,start,active,D", [
    (1, False, 4, 16, 11, 19, 64),    # decode over a wrapped ring
    (1, False, 4, 28, 0, 9, 32),      # ring not full yet
    (1, False, 0, 8, 5, 8, 128),      # no sink
    (1, False, 4, 16, 3, 20, 64),     # the whole ring
    (24, True, 4, 40, 17, 44, 64),    # causal prefill chunk over ranks (matrix-core kernel)
    (6, True, 2, 16, 9, 13, 32),      # causal, per-row kernel
    (1, False, 3, 0, 0, 12, 64),      # ring switched off: plain attention
])
def test_attention_streaming_vs_oracle(g, dt, Sq, causal, sink, window, start, active, D):
    """Keys enumerated by recency rank through the ring map; rows that no rank maps to are poisoned."""
    rng = np.random.default_rng(active * 13 + D + Sq)
    B, Hq, Hkv, L = 2, 8, 2, 64
    q = orc.to_storage(rng.standard_normal((B, Hq, Sq, D)), dt)
    k = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
    v = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
    used = {orc.ring_phys_index(r, sink, window, start) for r in range(active)}
    for row in range(L):
        if row not in used:
            k[:, :, row] = orc.to_storage(np.full((B, Hkv, D), np.nan), dt)
            v[:, :, row] = orc.to_storage(np.full((B, Hkv, D), np.nan), dt)
    want = orc.attention_streaming(q, k, v, dt, D ** -0.5, causal, active, sink, window, start)
    got = g.to_host(g.mynn.attention_streaming(g.to_dev(q, dt), g.to_dev(k, dt), g.to_dev(v, dt), D ** -0.5, causal, active,
                                               sink, window, start))
    assert not np.isnan(g.f32(got, dt)).any()
    assert max_err_rel_to_max(g.f32(got, dt), g.f32(want, dt)) <= 1e-2
    # and against the f64 attention over the rank-ordered rows
    rows = [orc.ring_phys_index(r, sink, window, start) for r in range(active)]
    exact = orc.attention_f64(q, np.ascontiguousarray(k[:, :, rows]), np.ascontiguousarray(v[:, :, rows]), dt, D ** -0.5, causal, active)
    assert max_err_rel_to_max(g.f32(got, dt), exact) <= (4e-3 if dt == orc.BF16 else 1e-3)


def test_attention_streaming_int8_kv(g):
    dt = orc.F16
    rng = np.random.default_rng(8)
    B, Hq, Hkv, L, D, sink, window, start, active = 2, 8, 2, 64, 64, 4, 32, 21, 30
    q = orc.to_storage(rng.standard_normal((B, Hq, 1, D)), dt)
    k = rng.integers(-127, 128, (B, Hkv, L, D)).astype(np.int8)
    v = rng.integers(-127, 128, (B, Hkv, L, D)).astype(np.int8)
    ks = orc.to_storage(rng.uniform(1e-3, 2e-2, (B, Hkv, L)), dt)
    vs = orc.to_storage(rng.uniform(1e-3, 2e-2, (B, Hkv, L)), dt)
    want = orc.attention_streaming(q, k, v, dt, D ** -0.5, False, active, sink, window, start, ks, vs)
    got = g.to_host(g.mynn.attention_streaming(g.to_dev(q, dt), g.to_dev(k), g.to_dev(v), D ** -0.5, False, active, sink, window,
                                               start, k_scale=g.to_dev(ks, dt), v_scale=g.to_dev(vs, dt)))
    assert max_err_rel_to_max(g.f32(got, dt), g.f32(want, dt)) <= 1e-2


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("offset,S_new,sink,window,start", [(9, 5, 4, 16, 0), (17, 5, 4, 16, 6), (20, 40, 4, 16, 9), (3, 6, 0, 0, 0)])
def test_quantizing_kvcache_update_streaming_bit_exact(g, dt, offset, S_new, sink, window, start):
    rng = np.random.default_rng(offset + S_new)
    B, H, L, D = 2, 3, 64, 32
    new = orc.to_storage(rng.standard_normal((B, H, S_new, D)) * 3, dt)
    cache = rng.integers(-128, 128, (B, H, L, D)).astype(np.int8)
    scale = orc.to_storage(rng.uniform(0.01, 0.1, (B, H, L)), dt)
    want_c, want_s = orc.quantizing_kv_cache_update_streaming(cache.copy(), scale.copy(), new, offset, sink, window, start, dt)
    dc, ds = g.to_dev(cache), g.to_dev(scale, dt)
    g.mynn.quantizing_kvcache_update_streaming(dc, ds, g.to_dev(new, dt), offset, sink, window, start)
    assert np.array_equal(g.to_host(dc), want_c) and np.array_equal(g.to_host(ds), want_s)


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16, orc.F32])
@pytest.mark.parametrize("kv8,Sq,causal,window", [(True, 1, False, 16), (False, 1, False, 16), (True, 5, True, 16), (True, 1, False, 0)])
def test_attention_streaming_with_k_rotation_inside_the_operator(g, dt, kv8, Sq, causal, window):
    """Operator slots 10-12: the dequantised key of rank r is rotated by table row kv_position[r] (ranks, as the
    reference's kernels index it), f32 throughout.  Against the oracle and, for the decode row, an explicit f64 loop."""
    import torch

    if kv8 and dt == orc.F32:
        pytest.skip("int8 KV comes with 16-bit scales")
    rng = np.random.default_rng(17 + Sq + window)
    B, Hq, Hkv, L, D, sink, start, active = 2, 4, 2, 48, 32, 4, 7 if window else 0, 15
    q = orc.to_storage(rng.standard_normal((B, Hq, Sq, D)), dt)
    if kv8:
        k = rng.integers(-127, 128, (B, Hkv, L, D)).astype(np.int8)
        v = rng.integers(-127, 128, (B, Hkv, L, D)).astype(np.int8)
        ks = orc.to_storage(rng.uniform(1e-3, 2e-2, (B, Hkv, L)), dt)
        vs = orc.to_storage(rng.uniform(1e-3, 2e-2, (B, Hkv, L)), dt)
    else:
        k = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
        v = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
        ks = vs = None
    cos_t, sin_t = orc.rope_table(L, D, 10000.0, dt)
    kvpos = rng.integers(0, L, L).astype(np.int64)
    want = orc.attention_streaming(q, k, v, dt, D ** -0.5, causal, active, sink, window, start, ks, vs, rope=(cos_t, sin_t, kvpos))
    dev = lambda a: g.to_dev(a, dt) if a is not None and a.dtype != np.int8 else (g.to_dev(a) if a is not None else None)
    got = g.to_host(g.mynn.attention_streaming(dev(q), dev(k), dev(v), D ** -0.5, causal, active, sink, window, start,
                                               k_scale=dev(ks), v_scale=dev(vs),
                                               rope=(dev(cos_t), dev(sin_t), torch.from_numpy(kvpos).cuda())))
    assert max_err_rel_to_max(g.f32(got, dt), g.f32(want, dt)) <= (1e-2 if dt != orc.F32 else 1e-5)
    if Sq == 1:
        qf, cf, sf = [orc.to_f32(a, dt).astype(np.float64) for a in (q, cos_t, sin_t)]
        out = np.zeros((B, Hq, 1, D))
        for b in range(B):
            for h in range(Hq):
                hk = h // (Hq // Hkv)
                sc, vv = [], []
                for r in range(active):
                    slot = orc.ring_phys_index(r, sink, window, start)
                    if kv8:
                        kk = k[b, hk, slot].astype(np.float64) * float(orc.to_f32(ks[b, hk, slot:slot + 1], dt)[0])
                        vr = v[b, hk, slot].astype(np.float64) * float(orc.to_f32(vs[b, hk, slot:slot + 1], dt)[0])
                    else:
                        kk = orc.to_f32(k[b, hk, slot], dt).astype(np.float64)
                        vr = orc.to_f32(v[b, hk, slot], dt).astype(np.float64)
                    p = int(kvpos[r])
                    rot = np.concatenate([kk[:D // 2] * cf[p, :D // 2] - kk[D // 2:] * sf[p, :D // 2],
                                          kk[D // 2:] * cf[p, D // 2:] + kk[:D // 2] * sf[p, D // 2:]])
                    sc.append(float(qf[b, h, 0] @ rot) * D ** -0.5)
                    vv.append(vr)
                sc = np.array(sc)
                w = np.exp(sc - sc.max())
                out[b, h, 0] = (w / w.sum()) @ np.array(vv)
        assert max_err_rel_to_max(g.f32(got, dt), out) <= (4e-3 if dt == orc.BF16 else 1e-3 if dt == orc.F16 else 1e-5)


@pytest.mark.parametrize("B,Hq,Hkv,D,L", [(2, 32, 8, 64, 2176), (4, 16, 4, 128, 1664), (1, 8, 8, 64, 4096)])
def test_workspace_size_holds_for_every_active_length(g, B, Hq, Hkv, D, L):
    """mynn_attention_workspace_bytes is asked once, for the cache; the number of key ranges a call is planned with
    is not monotonic in its active length (2176 rows over 16 (sequence, kv head) pairs: 9 ranges, 2048 rows: 16), so
    the reported size must cover every length: a workspace of exactly that size serves active = 1 .. L."""
    import torch

    dt = orc.F16
    rng = np.random.default_rng(L)
    q = g.to_dev(orc.to_storage(rng.standard_normal((B, Hq, 1, D)), dt), dt)
    k = g.to_dev(orc.to_storage(rng.standard_normal((B, Hkv, L, D), dtype=np.float32), dt), dt)
    v = g.to_dev(orc.to_storage(rng.standard_normal((B, Hkv, L, D), dtype=np.float32), dt), dt)
    lib = g.mynn.lib()
    need = lib.mynn_attention_workspace_bytes(B, 1, L, Hq, Hkv, D, dt, 0)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    out = torch.empty_like(q)
    lengths = sorted(set(list(range(1, L + 1, 97)) + list(range(128, L + 1, 128)) + [L - 1, L]))
    for active in lengths:
        g.mynn.check(lib.mynn_attention_ws(out.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), None, 0, 0, None, None,
                                           D ** -0.5, 0, B, 1, active, None, L, active - 1, Hq, Hkv, D, dt, 0, ws.data_ptr(), need,
                                           torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    # the last call (the full cache) against the library-scratch entry point
    assert torch.equal(out, g.mynn.attention(q, k, v, D ** -0.5, False, L))
