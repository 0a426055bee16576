"""GPU parity: every kernel of the C ABI against the CPU oracle on the same seeded inputs, and
against the reference's golden vectors.  Integer/byte/index results are bit-exact; float
results are within the stated max-abs-rel (1e-2 for 16-bit outputs, the bound the target states)."""
import glob
import os

import numpy as np
import pytest

import oracle as orc
import pbreader
from conftest import GOLDEN, close_either, max_abs_rel

pytestmark = pytest.mark.gpu

SO = os.path.join(GOLDEN, "single_op")
DT = [orc.F32, orc.BF16, orc.F16]
DT16 = [orc.BF16, orc.F16]


@pytest.fixture(scope="module")
def g():
    import gpu_util

    info = gpu_util.mynn.device_info()
    assert info["wave_size"] == 64 and info["arch"].startswith("gfx950"), info
    return gpu_util


def case(name):
    return pbreader.read_case(os.path.join(SO, name))


# ------------------------------------------------------------------ GEMV
@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("N,K", [(5632, 2048), (2048, 5632), (2560, 2048), (32000, 2048), (7, 16), (130, 4096)])
def test_dequant_gemv_vs_oracle(g, dt, N, K):
    rng = np.random.default_rng(N * 31 + K)
    act = orc.to_storage(rng.standard_normal((1, K)), dt)
    W = rng.integers(-127, 128, (N, K)).astype(np.int8)
    sc = orc.to_storage(rng.uniform(1e-3, 1e-2, N), dt)
    want = orc.dequant_matmul(act, W, sc, dt, dt, mode=0)[0]
    got = g.to_host(g.mynn.dequant_gemv(g.to_dev(act, dt), g.to_dev(W), g.to_dev(sc, dt)))
    assert max_abs_rel(g.f32(got, dt), g.f32(want, dt)) <= g.TOL[dt]
    # f64 closed form: the kernel's own f32 error stays inside K * 2^-24 * sum|a||w| (+ one rounding)
    exact = (W.astype(np.float64) @ g.f32(act, dt)[0].astype(np.float64)) * g.f32(sc, dt)
    bound = (np.abs(W).astype(np.float64) @ np.abs(g.f32(act, dt)[0])) * g.f32(sc, dt) * K * 2.0 ** -24
    ulp = {orc.F32: 2.0 ** -23, orc.BF16: 2.0 ** -8, orc.F16: 2.0 ** -10}[dt]
    assert np.all(np.abs(g.f32(got, dt) - exact) <= bound + np.abs(exact) * ulp + 1e-30)
    if dt != orc.F32:  # most elements agree with the oracle bit for bit; the rest are 1 ulp apart
        assert np.mean(got == want) > 0.95


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("N,K", [(2048, 5632), (4096, 14336), (11264, 2048)])
@pytest.mark.parametrize("mean", [0.0, 0.5, 1.0, 3.0])
def test_dequant_gemv_accumulation_noise_with_non_zero_mean_activations(g, dt, N, K, mean):
    """The fp16 decode GEMV multiplies biased weights (1152 + w for even elements, w - 1151 for odd ones) and takes the
    bias back out of the f32 sums; activations with a non-zero mean (SwiGLU outputs into down_proj, attention outputs
    into o_proj, long rows) must not turn that into cancellation error.  With a power-of-two scale the stored value is
    the f32 sum rounded once, so the distance to the exact sum is the accumulation noise plus one 16-bit rounding: the
    noise stays below 1/16 of half a 16-bit spacing of the row's largest output, for every mean (the plain
    convert-and-FMA path of bf16 models is held to the same bound)."""
    rng = np.random.default_rng(K + int(mean * 10))
    W = rng.integers(-127, 128, (N, K)).astype(np.int8)
    x = orc.to_storage(rng.standard_normal(K) * 0.5 + mean, dt)
    sc = orc.to_storage(np.full(N, 2.0 ** -7), dt)
    exact = (W.astype(np.float64) @ g.f32(x, dt).astype(np.float64)) * 2.0 ** -7
    got = g.f32(g.to_host(g.mynn.dequant_gemv(g.to_dev(x, dt), g.to_dev(W), g.to_dev(sc, dt))), dt).astype(np.float64)
    mant = 10 if dt == orc.F16 else 7
    half_ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(exact), 1e-30))) - mant - 1)
    noise = np.maximum(np.abs(got - exact) - half_ulp, 0.0)  # what is left after one correct rounding
    top = float(np.max(np.abs(exact)))
    assert noise.max() <= 2.0 ** -(mant + 2 + 4) * top, (noise.max() / top, mean)
    # the large outputs (the ones a greedy choice is made among) are the correctly rounded sums
    big = np.abs(exact) >= top / 4
    ideal = g.f32(orc.to_storage(exact.astype(np.float32), dt), dt)
    assert np.mean(got[big] == ideal[big]) >= 0.98


def test_dequant_gemv_mixed_types_cfg1(g):
    """First benchmark config: f32 x, int8 W [5632,2048], f32 scale, f32 out."""
    rng = np.random.default_rng(1)
    K, N = 2048, 5632
    x = rng.standard_normal((1, K)).astype(np.float32)
    W = rng.integers(-127, 128, (N, K)).astype(np.int8)
    s = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    got = g.to_host(g.mynn.dequant_gemv(g.to_dev(x), g.to_dev(W), g.to_dev(s)))
    want = orc.dequant_matmul(x, W, s, orc.F32, orc.F32)[0]
    assert max_abs_rel(got, want) <= 2e-5


def test_dequant_gemv_rejects_bad_arguments(g):
    import torch

    W = torch.zeros((8, 24), dtype=torch.int8, device="cuda")  # K % 16 != 0
    a = torch.zeros((24,), dtype=torch.float16, device="cuda")
    s = torch.zeros((8,), dtype=torch.float16, device="cuda")
    with pytest.raises(g.mynn.MynnError):
        g.mynn.dequant_gemv(a, W, s)


@pytest.mark.parametrize("dt", DT16)
@pytest.mark.parametrize("M", [2, 3, 7, 15])
def test_dequant_matmul_small_m_scale_after_sum(g, dt, M):
    rng = np.random.default_rng(M)
    N, K = 96, 320
    act = orc.to_storage(rng.standard_normal((M, K)), dt)
    W = rng.integers(-127, 128, (N, K)).astype(np.int8)
    sc = orc.to_storage(rng.uniform(5e-3, 1.2e-2, N), dt)
    want = orc.dequant_matmul(act, W, sc, dt, dt, mode=0)
    got = g.to_host(g.mynn.dequant_matmul(g.to_dev(act, dt), g.to_dev(W), g.to_dev(sc, dt)))
    assert max_abs_rel(g.f32(got, dt), g.f32(want, dt)) <= g.TOL[dt]


def test_dequant_matmul_small_golden(g):
    (act, wq, scale), (out,) = case("dequant_matmul")  # M = 3: the scale-after-sum kernel
    got = g.to_host(g.mynn.dequant_matmul(g.to_dev(act.array, orc.BF16), g.to_dev(wq.array), g.to_dev(scale.array, orc.BF16)))
    assert np.array_equal(got, out.array)


# ------------------------------------------------------------------ small operators
@pytest.mark.parametrize("dt", DT)
def test_rms_norm(g, dt):
    rng = np.random.default_rng(3)
    x = orc.to_storage(rng.standard_normal((5, 2048)) * 2, dt)
    w = orc.to_storage(rng.standard_normal(2048), dt)
    want = orc.rms_norm(x, w, 1e-5, dt)
    got = g.to_host(g.mynn.rms_norm(g.to_dev(x, dt), g.to_dev(w, dt), 1e-5))
    assert max_abs_rel(g.f32(got, dt), g.f32(want, dt)) <= g.TOL[dt]


@pytest.mark.parametrize("dt", DT)
def test_rope_bit_exact(g, dt):
    import torch

    rng = np.random.default_rng(4)
    D, S, H = 64, 5, 6
    x = orc.to_storage(rng.standard_normal((1, H, S, D)), dt)
    cos, sin = orc.rope_table(64, D, 10000.0, dt)
    pos = np.array([3, 0, 7, 63, 1], np.int64)
    want = orc.rope(x, cos, sin, pos, dt)
    got = g.to_host(g.mynn.rope(g.to_dev(x, dt), g.to_dev(cos, dt), g.to_dev(sin, dt), torch.from_numpy(pos).cuda()))
    assert np.array_equal(got, want)  # two products, one sum, one rounding: no freedom


def test_rope_known_answer(g):
    import torch

    x = np.array([1, 2, 3, 4], np.float32).reshape(1, 1, 1, 4)
    cos = np.full((1, 4), 0.5, np.float32)
    sin = np.ones((1, 4), np.float32)
    got = g.to_host(g.mynn.rope(g.to_dev(x), g.to_dev(cos), g.to_dev(sin), torch.zeros(1, dtype=torch.int64, device="cuda")))
    assert np.allclose(got.ravel(), [-2.5, -3.0, 2.5, 4.0], atol=1e-6)


def test_kv_cache_update_golden_and_persistence(g):
    (cache, src, off), (out,) = case("kv_cache_update")
    c = g.to_dev(cache.array.copy())
    g.mynn.kvcache_update(c, g.to_dev(src.array), int(off.array))
    upd = g.to_host(c)
    ok, md = close_either(1 / (1 + np.exp(-upd.astype(np.float64))), out.array, 1e-5)
    assert ok, md
    assert np.array_equal(upd, orc.kv_cache_update(cache.array.copy(), src.array, int(off.array)))
    # three successive scatters accumulate in the same buffer (tests/session_state.rs:64-120)
    B, H, S_MAX, D = 1, 2, 8, 4
    dev = g.to_dev(np.zeros((B, H, S_MAX, D), np.float32))
    ref = np.zeros((B, H, S_MAX, D), np.float32)
    for step in range(3):
        srcv = (np.arange(B * H * D) * 0.1 + step + 1).astype(np.float32).reshape(B, H, 1, D)
        g.mynn.kvcache_update(dev, g.to_dev(srcv), step)
        orc.kv_cache_update(ref, srcv, step)
        assert np.array_equal(g.to_host(dev), ref)


@pytest.mark.parametrize("dt", DT16)
def test_kv_cache_update_16bit(g, dt):
    rng = np.random.default_rng(5)
    cache = orc.to_storage(rng.standard_normal((2, 4, 16, 64)), dt)
    new = orc.to_storage(rng.standard_normal((2, 4, 3, 64)), dt)
    c = g.to_dev(cache.copy(), dt)
    g.mynn.kvcache_update(c, g.to_dev(new, dt), 11)
    assert np.array_equal(g.to_host(c), orc.kv_cache_update(cache.copy(), new, 11))
    with pytest.raises(g.mynn.MynnError):
        g.mynn.kvcache_update(c, g.to_dev(new, dt), 14)  # would run past max_seq


def test_quantizing_kvcache_update_golden(g):
    (cache, scale, new, off), (out,) = case("quantizing_kvcache_update")
    c, s = g.to_dev(cache.array.copy()), g.to_dev(scale.array.copy(), orc.BF16)
    g.mynn.quantizing_kvcache_update(c, s, g.to_dev(new.array, orc.BF16), int(off.array))
    assert np.array_equal(g.to_host(c), out.array)
    rc, rs = orc.quantizing_kv_cache_update(cache.array.copy(), scale.array.copy(), new.array, int(off.array), orc.BF16)
    assert np.array_equal(g.to_host(s), rs)


@pytest.mark.parametrize("dt", DT)
def test_quantizing_kvcache_update_random(g, dt):
    rng = np.random.default_rng(6)
    B, H, L, D = 2, 4, 32, 64
    cache = np.zeros((B, H, L, D), np.int8)
    scale = orc.to_storage(np.zeros((B, H, L)), dt)
    new = orc.to_storage(rng.standard_normal((B, H, 5, D)) * 3, dt)
    new.reshape(-1, D)[7] = 0  # a zero row
    c, s = g.to_dev(cache.copy()), g.to_dev(scale.copy(), dt)
    g.mynn.quantizing_kvcache_update(c, s, g.to_dev(new, dt), 9)
    rc, rs = orc.quantizing_kv_cache_update(cache.copy(), scale.copy(), new, 9, dt)
    assert np.array_equal(g.to_host(c), rc) and np.array_equal(g.to_host(s), rs)


def test_dequantize_linear_golden(g):
    (x, s), (y,) = case("dequantize_linear")
    got = g.to_host(g.mynn.dequantize_linear(g.to_dev(x.array), g.to_dev(s.array, orc.BF16)))
    assert np.array_equal(got, y.array)


@pytest.mark.parametrize("name", ["gather_default_axis", "gather_negative_indices"])
def test_gather_golden(g, name):
    import torch

    (data, idx), (out,) = case(name)
    got = g.to_host(g.mynn.gather_rows(g.to_dev(data.array), torch.from_numpy(idx.array).cuda()))
    assert np.array_equal(got.reshape(out.array.shape), out.array)


@pytest.mark.parametrize("dt", DT)
def test_swiglu_and_add(g, dt):
    rng = np.random.default_rng(7)
    a = orc.to_storage(rng.standard_normal(5632) * 3, dt)
    b = orc.to_storage(rng.standard_normal(5632), dt)
    got = g.to_host(g.mynn.swiglu(g.to_dev(a, dt), g.to_dev(b, dt)))
    assert max_abs_rel(g.f32(got, dt), g.f32(orc.swiglu(a, b, dt), dt)) <= g.TOL[dt]
    got = g.to_host(g.mynn.add(g.to_dev(a, dt), g.to_dev(b, dt)))
    assert np.array_equal(got, orc.add(a, b, dt))  # one exact-ish sum, one rounding


def test_swish_golden_via_swiglu(g):
    (x,), (y,) = case("swish")
    ones = np.ones_like(x.array)
    got = g.to_host(g.mynn.swiglu(g.to_dev(x.array), g.to_dev(ones)))
    ok, md = close_either(got, y.array, 1e-5)
    assert ok, md


@pytest.mark.parametrize("name,sym", [("dyn_quantize_linear_sym_per_row", True), ("dyn_quantize_linear_asym_per_row", False)])
def test_dynquant_golden(g, name, sym):
    (x,), (y, s, zp) = case(name)
    gy, gs, gz = g.mynn.dynamic_quantize_linear(g.to_dev(x.array, orc.BF16), symmetric=sym)
    assert np.array_equal(g.to_host(gy), y.array)
    assert np.array_equal(g.to_host(gz), zp.array)
    ok, md = close_either(g.f32(g.to_host(gs), orc.BF16), s.f32(), 1e-3)
    assert ok, md


@pytest.mark.parametrize("name,sym", [("dyn_quantize_linear_sym_per_tensor", True), ("dyn_quantize_linear_asym_per_tensor", False)])
def test_dynquant_per_tensor_golden(g, name, sym):
    """The per-tensor fixtures: one quantisation slice over the whole tensor (axis_dim 1)."""
    (x,), (y, s, zp) = case(name)
    flat = g.to_dev(x.array.reshape(1, -1), orc.BF16)
    gy, gs, gz = g.mynn.dynamic_quantize_linear(flat, symmetric=sym)
    assert np.array_equal(g.to_host(gy).reshape(y.array.shape), y.array)
    assert int(g.to_host(gz)[0]) == int(np.asarray(zp.array).reshape(-1)[0])
    ok, md = close_either(g.f32(g.to_host(gs), orc.BF16), s.f32().reshape(1), 1e-3)
    assert ok, md
    if sym:
        wy, ws = orc.dynquant_i8_per_tensor(x.array, orc.BF16)
        assert np.array_equal(g.to_host(gy).reshape(wy.shape), wy) and np.array_equal(g.to_host(gs).reshape(-1), np.asarray(ws).reshape(-1))


@pytest.mark.parametrize("dt", DT)
def test_dynquant_random_bit_exact(g, dt):
    rng = np.random.default_rng(8)
    x = orc.to_storage(rng.standard_normal((33, 2048)) * 4, dt)
    x[5] = 0
    gy, gs, _ = g.mynn.dynamic_quantize_linear(g.to_dev(x, dt), symmetric=True)
    wy, ws = orc.dynquant_i8(x, dt)
    assert np.array_equal(g.to_host(gy), wy) and np.array_equal(g.to_host(gs), ws)


@pytest.mark.parametrize("dt", DT)
def test_argmax_last_wins(g, dt):
    rng = np.random.default_rng(9)
    v = rng.standard_normal(32000).astype(np.float32)
    v[[17, 4242, 31999]] = 9.0  # three equal maxima: the last index wins
    s = orc.to_storage(v, dt)
    assert int(g.to_host(g.mynn.argmax_last(g.to_dev(s, dt)))[0]) == 31999 == orc.argmax_last(s, dt)
    v[31999] = 0
    s = orc.to_storage(v, dt)
    assert int(g.to_host(g.mynn.argmax_last(g.to_dev(s, dt)))[0]) == 4242
    s = orc.to_storage(np.full(1000, -3.0), dt)
    assert int(g.to_host(g.mynn.argmax_last(g.to_dev(s, dt)))[0]) == 999
