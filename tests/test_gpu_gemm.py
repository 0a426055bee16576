"""GPU parity of the matrix-core paths: DequantMatMul (M >= 16) and QuantizedMatMul against the
reference's golden vectors and the oracle.  int32 accumulators are bit-exact."""
import glob
import os

import numpy as np
import pytest

import oracle as orc
import pbreader
from conftest import GOLDEN, close_either, max_abs_rel

pytestmark = pytest.mark.gpu
SO = os.path.join(GOLDEN, "single_op")


@pytest.fixture(scope="module")
def g():
    import gpu_util

    return gpu_util


DQMM = sorted(os.path.basename(p) for p in glob.glob(os.path.join(SO, "dequant_matmul_*")))


@pytest.mark.parametrize("name", DQMM)
def test_dequant_matmul_goldens(g, name):
    """tests/single_op.rs dequant_matmul_MxNxK fixtures (eps 1e-1 there).  Shapes the reference
    sends to its tensor-core kernel (M >= 16, K % 8 == 0) must reproduce the goldens to the bit
    except where f32 accumulation order crosses a bf16 rounding boundary."""
    (act, wq, scale), (out,) = pbreader.read_case(os.path.join(SO, name))
    got = g.to_host(g.mynn.dequant_matmul(g.to_dev(act.array, orc.BF16), g.to_dev(wq.array), g.to_dev(scale.array, orc.BF16)))
    ok, md = close_either(g.f32(got, orc.BF16), out.f32(), 1e-1)
    assert ok, md
    M, K = act.array.shape
    if M >= 16 and K % 8 == 0:
        mism = np.count_nonzero(got != out.array)
        assert mism <= max(2, out.array.size // 200), "%d of %d differ from the golden bits" % (mism, out.array.size)


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("M,N,K", [(16, 128, 32), (200, 300, 512), (129, 127, 40), (515, 385, 96), (128, 2560, 2048), (64, 2048, 5632),
                                   (4096, 4096, 64), (4000, 4090, 72)])
def test_dequant_matmul_mfma_vs_oracle(g, dt, M, N, K):
    rng = np.random.default_rng(M * 7 + N * 3 + K)
    act = orc.to_storage(rng.standard_normal((M, K)), dt)
    W = rng.integers(-127, 128, (N, K)).astype(np.int8)
    sc = orc.to_storage(rng.uniform(1e-3, 1e-2, N), dt)
    want = orc.dequant_matmul(act, W, sc, dt, dt, mode=2)  # W rounded to the 16-bit type first
    got = g.to_host(g.mynn.dequant_matmul(g.to_dev(act, dt), g.to_dev(W), g.to_dev(sc, dt)))
    assert max_abs_rel(g.f32(got, dt), g.f32(want, dt)) <= 1e-2
    assert np.mean(got == want) > 0.97
    # closed form in f64 over the rounded weights
    wr = g.f32(orc.to_storage(W.astype(np.float32) * g.f32(sc, dt)[:, None], dt), dt).astype(np.float64)
    exact = g.f32(act, dt).astype(np.float64) @ wr.T
    assert max_abs_rel(g.f32(got, dt), exact) <= 1e-2


def test_dequant_matmul_seeded_shape_sweep(g):
    """40 seeded shapes across the kernel choices of DequantMatMul (one row, a few rows, 16 and more rows on the
    matrix cores; K a multiple of 8 or not, shorter and longer than a K step; N with tails in every tile width)
    against the f64 closed form of the kernel each shape takes (scale after the sum below 16 rows or for odd K,
    weights rounded to the storage type first otherwise)."""
    rng = np.random.default_rng(77)
    for case in range(40):
        dt = [orc.F16, orc.BF16][case % 2]
        M = int(rng.choice([1, 2, 3, 7, 15, 16, 17, 33, 64, 65, 130, 260]))
        N = int(rng.choice([1, 5, 31, 64, 100, 129, 255, 256, 257, 320, 700, 1030]))
        K = int(rng.choice([8, 16, 24, 40, 64, 72, 128, 200, 512, 1032, 2048, 12, 100]))
        act = orc.to_storage(rng.standard_normal((M, K)), dt)
        W = rng.integers(-127, 128, (N, K)).astype(np.int8)
        sc = orc.to_storage(rng.uniform(1e-3, 1e-2, N), dt)
        got = g.f32(g.to_host(g.mynn.dequant_matmul(g.to_dev(act, dt), g.to_dev(W), g.to_dev(sc, dt))), dt)
        a64, s64 = g.f32(act, dt).astype(np.float64), g.f32(sc, dt).astype(np.float64)
        if M >= 16 and K % 8 == 0:
            wr = g.f32(orc.to_storage(W.astype(np.float32) * g.f32(sc, dt)[:, None], dt), dt).astype(np.float64)
            exact = a64 @ wr.T
        else:
            exact = (a64 @ W.astype(np.float64).T) * s64[None, :]
        assert got.shape == (M, N) and not np.isnan(got).any(), (case, M, N, K)
        assert max_abs_rel(got, exact) <= 1e-2, (case, M, N, K)


@pytest.mark.parametrize("tile", [1, 2, 3, 4])
@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("M,N,K", [(200, 300, 512), (700, 520, 128), (128, 2560, 2048), (300, 650, 64), (257, 321, 192)])
def test_dequant_matmul_every_workgroup_tile(g, dt, M, N, K, tile):
    """Each workgroup tile / load scheme of the matrix-core GEMM (256x128 and 256x256 staged through
    registers; 256x256 and 256x320 with direct-to-LDS loads and swizzled tiles) on shapes with row and
    column tails and 1, 2, 3, 8 and 32 K steps."""
    rng = np.random.default_rng(M + N + K)
    act = orc.to_storage(rng.standard_normal((M, K)), dt)
    W = rng.integers(-127, 128, (N, K)).astype(np.int8)
    sc = orc.to_storage(rng.uniform(1e-3, 1e-2, N), dt)
    want = orc.dequant_matmul(act, W, sc, dt, dt, mode=2)
    da, dw, ds = g.to_dev(act, dt), g.to_dev(W), g.to_dev(sc, dt)
    got = g.to_host(g.mynn.dequant_matmul_ws(da, dw, ds, gemm_tile=tile))
    assert max_abs_rel(g.f32(got, dt), g.f32(want, dt)) <= 1e-2
    assert np.mean(got == want) > 0.97
    # prepare once / multiply many gives the values of the per-call dequantisation
    wt = g.mynn.dequant_weight_prepare(dw, ds)
    assert np.array_equal(g.to_host(g.mynn.dequant_matmul_prepared(da, wt, N, gemm_tile=tile)), got)


def test_dequant_matmul_linearity_at_prefill_size(g):
    """Size-independent property at the prefill shape (M = 8192): rows are independent, so any
    row block of the big product equals the product of that block alone."""
    import torch

    dt = orc.F16
    rng = np.random.default_rng(0)
    M, N, K = 8192, 2560, 2048
    act = orc.to_storage(rng.standard_normal((M, K)), dt)
    W = rng.integers(-127, 128, (N, K)).astype(np.int8)
    sc = orc.to_storage(rng.uniform(1e-3, 1e-2, N), dt)
    da, dw, ds = g.to_dev(act, dt), g.to_dev(W), g.to_dev(sc, dt)
    full = g.mynn.dequant_matmul(da, dw, ds)
    part = g.mynn.dequant_matmul(da[4096 + 128:4096 + 384].contiguous(), dw, ds)
    assert torch.equal(full[4096 + 128:4096 + 384], part)
    want = orc.dequant_matmul(act[:32], W, sc, dt, dt, mode=2)
    assert max_abs_rel(g.f32(g.to_host(full[:32]), dt), g.f32(want, dt)) <= 1e-2


QMM = sorted(os.path.basename(p) for p in glob.glob(os.path.join(SO, "quantized_matmul_*")))


@pytest.mark.parametrize("name", QMM)
def test_quantized_matmul_goldens(g, name):
    (lhs, ls, rhs, rs), (y,) = pbreader.read_case(os.path.join(SO, name))
    out, acc = g.mynn.quantized_matmul(g.to_dev(lhs.array), g.to_dev(ls.array, orc.BF16), g.to_dev(rhs.array),
                                       g.to_dev(rs.array, orc.BF16))
    want_acc = lhs.array.astype(np.int64) @ rhs.array.astype(np.int64).T
    assert np.array_equal(g.to_host(acc).astype(np.int64), want_acc)  # bit-exact int32
    ok, md = close_either(g.f32(g.to_host(out), orc.BF16), y.f32(), 1e-1)
    assert ok, md
    ref_out, ref_acc = orc.quantized_matmul(lhs.array, ls.array, rhs.array, rs.array, orc.BF16)
    assert np.array_equal(g.to_host(out), ref_out)  # same three f32 operations, same rounding


@pytest.mark.parametrize("dt", [orc.F32, orc.BF16, orc.F16])
@pytest.mark.parametrize("M,N,K", [(1, 2048, 2048), (5, 300, 64), (15, 77, 5632), (16, 64, 32), (130, 257, 2048),
                                   (256, 5632, 2048)])
def test_quantized_matmul_bit_exact(g, dt, M, N, K):
    rng = np.random.default_rng(M + N + K)
    lhs = rng.integers(-128, 128, (M, K)).astype(np.int8)
    rhs = rng.integers(-128, 128, (N, K)).astype(np.int8)
    ls = orc.to_storage(rng.uniform(1e-3, 1e-1, M), dt)
    rs = orc.to_storage(rng.uniform(1e-3, 1e-2, N), dt)
    out, acc = g.mynn.quantized_matmul(g.to_dev(lhs), g.to_dev(ls, dt), g.to_dev(rhs), g.to_dev(rs, dt))
    want_out, want_acc = orc.quantized_matmul(lhs, ls, rhs, rs, dt)
    assert np.array_equal(g.to_host(acc), want_acc)
    assert np.array_equal(g.to_host(out), want_out)


@pytest.mark.parametrize("dt", [orc.BF16, orc.F16])
@pytest.mark.parametrize("M,N,K", [(4096, 2048, 128), (4000, 2100, 384), (8192, 2560, 256)])
def test_quantized_matmul_large_tiles_bit_exact(g, dt, M, N, K):
    """Grids of at least half a round of 256-row tiles take the direct-to-LDS int8 kernel (256x256 and, for
    N = 2560, 256x320 tiles; 1, 3 and 2 K steps; row and column tails): int32 sums and scaled output bit
    for bit against the oracle."""
    rng = np.random.default_rng(M + N + K)
    lhs = rng.integers(-128, 128, (M, K)).astype(np.int8)
    rhs = rng.integers(-128, 128, (N, K)).astype(np.int8)
    ls = orc.to_storage(rng.uniform(1e-3, 1e-1, M), dt)
    rs = orc.to_storage(rng.uniform(1e-3, 1e-2, N), dt)
    out, acc = g.mynn.quantized_matmul(g.to_dev(lhs), g.to_dev(ls, dt), g.to_dev(rhs), g.to_dev(rs, dt))
    want_acc = (lhs.astype(np.float64) @ rhs.astype(np.float64).T).astype(np.int32)  # exact: |sum| < 2^53
    assert np.array_equal(g.to_host(acc), want_acc)
    want_out = orc.to_storage((want_acc.astype(np.float32) * g.f32(ls, dt)[:, None]) * g.f32(rs, dt)[None, :], dt)
    assert np.array_equal(g.to_host(out), want_out)
    sub = slice(0, 64)
    ref_out, ref_acc = orc.quantized_matmul(lhs[sub], ls[sub], rhs, rs, dt)
    assert np.array_equal(want_acc[sub], ref_acc) and np.array_equal(want_out[sub], ref_out)


def test_quantized_matmul_extremes(g):
    K = 4096
    lhs = np.full((32, K), -128, np.int8)
    rhs = np.stack([np.full(K, -128, np.int8), np.full(K, 127, np.int8)] * 16)
    ones = np.ones(32, np.float32)
    out, acc = g.mynn.quantized_matmul(g.to_dev(lhs), g.to_dev(ones), g.to_dev(rhs), g.to_dev(ones))
    a = g.to_host(acc)
    assert np.all(a[:, 0::2] == K * 16384) and np.all(a[:, 1::2] == -K * 16256)
    with pytest.raises(g.mynn.MynnError):
        g.mynn.quantized_matmul(g.to_dev(lhs[:, :48].copy()), g.to_dev(ones), g.to_dev(rhs[:, :48].copy()), g.to_dev(ones))


def test_w8a8_linear_pipeline(g):
    """DynamicQuantizeLinear -> QuantizedMatMul (Options.quantize_activations in the reference):
    the product is checked against the oracle's two steps, bit for bit."""
    dt = orc.BF16
    rng = np.random.default_rng(3)
    M, N, K = 24, 512, 2048
    x = orc.to_storage(rng.standard_normal((M, K)), dt)
    W = rng.integers(-127, 128, (N, K)).astype(np.int8)
    ws = orc.to_storage(rng.uniform(1e-3, 1e-2, N), dt)
    xq, xs, _ = g.mynn.dynamic_quantize_linear(g.to_dev(x, dt), symmetric=True)
    out, _ = g.mynn.quantized_matmul(xq, xs, g.to_dev(W), g.to_dev(ws, dt))
    rq, rs = orc.dynquant_i8(x, dt)
    want, _ = orc.quantized_matmul(rq, rs, W, ws, dt)
    assert np.array_equal(g.to_host(out), want)
