"""Paged KV cache on the GPU: the attention kernels reading K/V through a page table, the cache update into a pool,
the pool / page-set bookkeeping, and executors whose caches are pools.

The reference has no paged cache (its buffers are contiguous [B,Hkv,max_seq,D], crates/llm/src/session.rs:284-394), so
the expected values are those of the contiguous path on the same rows: the oracle's attention on the gathered cache, and
-- where both take the same kernel -- the bits of the library's own contiguous call."""
import numpy as np
import pytest

import oracle as orc
import llm_weights
from conftest import max_abs_rel, max_err_rel_to_max
from test_gpu_decoder import SMALL_D64, dev_weights

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def g():
    import gpu_util

    return gpu_util


def scatter_to_pool(cache, P, rng, spare=3, fill=0xFFFF):
    """contiguous [B,Hkv,L,...] (L a multiple of P) -> (pool [n_pages,Hkv,P,...], table int32 [B, L/P]) with the pages
    handed out in a random order and every row of an unused page set to `fill` (NaN bit pattern for 16-bit types)."""
    B, Hkv, L = cache.shape[:3]
    pps = L // P
    n_pages = B * pps + spare
    table = rng.permutation(n_pages)[:B * pps].astype(np.int32).reshape(B, pps)
    pool = np.full((n_pages, Hkv, P) + cache.shape[3:], fill, cache.dtype)
    for b in range(B):
        for s in range(pps):
            pool[table[b, s]] = cache[b, :, s * P:(s + 1) * P]
    return pool, table


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("B,Hq,Hkv,D,L,active,P", [
    (8, 32, 8, 128, 1024, 1001, 256),   # the batched-serving head shape, streaming kernel on both sides
    (16, 32, 4, 64, 768, 613, 128),     # TinyLlama heads
    (4, 16, 8, 64, 1280, 1111, 32),     # a page per tile
    (32, 32, 8, 128, 256, 129, 64),
    (2, 8, 8, 64, 512, 77, 64),         # small: the contiguous call takes another kernel
    (1, 32, 4, 64, 2048, 2048, 1024),   # batch 1, full cache, two pages
    (3, 8, 2, 128, 96, 33, 32),
])
def test_paged_decode_attention_vs_oracle_and_contiguous(g, dt, B, Hq, Hkv, D, L, active, P):
    import torch

    rng = np.random.default_rng(B * 131 + L + P)
    q = orc.to_storage(rng.standard_normal((B, Hq, 1, D)), dt)
    k = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
    v = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
    # rows at and beyond the active length: NaN (never read)
    k[:, :, active:] = 0xFFFF
    v[:, :, active:] = 0xFFFF
    want = orc.attention(q, k, v, dt, D ** -0.5, False, active)
    exact = orc.attention_f64(q, k, v, dt, D ** -0.5, False, active)
    kp, table = scatter_to_pool(k, P, rng)
    vp = np.full_like(kp, 0xFFFF)  # (V shares K's table)
    for b in range(B):
        for s in range(L // P):
            vp[table[b, s]] = v[b, :, s * P:(s + 1) * P]
    # pages no active row falls into are not mapped at all
    first_unused = (active + P - 1) // P
    table_dev = table.copy()
    table_dev[:, first_unused:] = -1
    dq, dkp, dvp = g.to_dev(q, dt), g.to_dev(kp, dt), g.to_dev(vp, dt)
    dtab = torch.from_numpy(table_dev).cuda()
    got = g.to_host(g.mynn.attention_paged(dq, dkp, dvp, dtab, P, D ** -0.5, False, active))
    assert max_abs_rel(g.f32(got, dt), g.f32(want, dt)) <= 1e-2
    assert max_abs_rel(g.f32(got, dt), exact) <= 1e-2
    # the active length read on the device (graph replay): the plan is made for the whole cache
    d_active = torch.tensor([active], dtype=torch.int32, device="cuda")
    got_d = g.to_host(g.mynn.attention_paged(dq, dkp, dvp, dtab, P, D ** -0.5, False, L, d_active=d_active))
    assert max_abs_rel(g.f32(got_d, dt), exact) <= 1e-2
    # the contiguous call on the same rows: the same bits when it takes the streaming kernel too
    dk, dv = g.to_dev(k, dt), g.to_dev(v, dt)
    plain = g.to_host(g.mynn.attention(dq, dk, dv, D ** -0.5, False, active))
    if B * Hkv * active >= 8192:
        assert np.array_equal(got, plain)
    else:
        assert max_abs_rel(g.f32(got, dt), g.f32(plain, dt)) <= 1e-2


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("B,Hq,Hkv,D,L,active,P", [(8, 32, 8, 128, 768, 600, 128), (16, 32, 4, 64, 768, 613, 256)])
def test_paged_decode_attention_int8_kv_vs_contiguous(g, dt, B, Hq, Hkv, D, L, active, P):
    """int8 K/V with one scale per token row: code pools and scale pools share the table."""
    import torch

    rng = np.random.default_rng(L + P)
    q = orc.to_storage(rng.standard_normal((B, Hq, 1, D)), dt)
    k = rng.integers(-127, 128, (B, Hkv, L, D)).astype(np.int8)
    v = rng.integers(-127, 128, (B, Hkv, L, D)).astype(np.int8)
    ks = orc.to_storage(rng.uniform(0.005, 0.02, (B, Hkv, L)), dt)
    vs = orc.to_storage(rng.uniform(0.005, 0.02, (B, Hkv, L)), dt)
    want = orc.attention(q, k, v, dt, D ** -0.5, False, active, ks, vs)
    kp, table = scatter_to_pool(k, P, rng, fill=0)
    pools = []
    for a, fill in ((v, 0), (ks, 0xFFFF), (vs, 0xFFFF)):
        pl = np.full((kp.shape[0], Hkv, P) + a.shape[3:], fill, a.dtype)
        for b in range(B):
            for s in range(L // P):
                pl[table[b, s]] = a[b, :, s * P:(s + 1) * P]
        pools.append(pl)
    dq = g.to_dev(q, dt)
    dtab = torch.from_numpy(table).cuda()
    got = g.to_host(g.mynn.attention_paged(dq, g.to_dev(kp), g.to_dev(pools[0]), dtab, P, D ** -0.5, False, active,
                                           k_scale_pool=g.to_dev(pools[1], dt), v_scale_pool=g.to_dev(pools[2], dt)))
    assert max_abs_rel(g.f32(got, dt), g.f32(want, dt)) <= 1e-2
    plain = g.to_host(g.mynn.attention(dq, g.to_dev(k), g.to_dev(v), D ** -0.5, False, active,
                                       k_scale=g.to_dev(ks, dt), v_scale=g.to_dev(vs, dt)))
    assert B * Hkv * active >= 8192 and np.array_equal(got, plain)


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("B,Hq,Hkv,D,Sq,past,P,pps", [
    (2, 8, 2, 64, 200, 0, 64, 4),      # causal prefill from an empty cache, ragged last tile
    (1, 8, 4, 128, 96, 160, 128, 2),   # a chunk behind 160 cached rows
    (3, 4, 4, 64, 17, 47, 64, 1),      # a few rows, one page
    (1, 32, 4, 64, 512, 512, 256, 4),  # TinyLlama heads
])
def test_paged_prefill_attention_vs_oracle_and_contiguous(g, dt, B, Hq, Hkv, D, Sq, past, P, pps):
    import torch

    L = P * pps
    active = past + Sq
    assert active <= L
    rng = np.random.default_rng(Sq + past)
    q = orc.to_storage(rng.standard_normal((B, Hq, Sq, D)), dt)
    k = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
    v = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
    k[:, :, active:] = 0xFFFF
    v[:, :, active:] = 0xFFFF
    # the oracle's causal rule puts query row i at position Sk - Sq + i: hand it the active rows only
    want = orc.attention(q, np.ascontiguousarray(k[:, :, :active]), np.ascontiguousarray(v[:, :, :active]), dt, D ** -0.5, True)
    kp, table = scatter_to_pool(k, P, rng)
    vp = np.full_like(kp, 0xFFFF)
    for b in range(B):
        for s in range(pps):
            vp[table[b, s]] = v[b, :, s * P:(s + 1) * P]
    dq = g.to_dev(q, dt)
    dtab = torch.from_numpy(table).cuda()
    got = g.to_host(g.mynn.attention_paged(dq, g.to_dev(kp, dt), g.to_dev(vp, dt), dtab, P, D ** -0.5, True, active, q_pos_offset=past))
    # (the bound of the contiguous kernel's own test: bf16 P carries 8 bits into the second product)
    assert max_err_rel_to_max(g.f32(got, dt), g.f32(want, dt)) <= 1e-2
    if Sq >= 16:  # the contiguous call takes the same matrix-core kernel: the same bits
        plain = g.to_host(g.mynn.attention(dq, g.to_dev(k, dt), g.to_dev(v, dt), D ** -0.5, True, active, q_pos_offset=past))
        assert np.array_equal(got, plain)


def test_paged_attention_seeded_shape_sweep(g):
    """60 seeded shapes: 1..40 sequences, 1 / 2 / 4 / 8 query heads per kv head, head_dim 64 / 128, pages of 32..512 rows, 1..12
    pages per sequence in a shuffled pool, ragged active lengths (first row of a page, last row, one row), one query row
    (streaming kernel, with and without key ranges to merge) or a causal block of query rows behind a prefix (prefill
    kernel), fp16 and bf16 -- against the f64 formula on the gathered rows; unused pages and rows hold NaN."""
    import torch

    rng = np.random.default_rng(2024)
    for case in range(60):
        dt = orc.F16 if case % 2 == 0 else orc.BF16
        D = int(rng.choice([64, 128]))
        G = int(rng.choice([1, 2, 4, 8]))
        Hkv = int(rng.choice([1, 2, 4, 8]))
        prefill = case % 5 == 4
        P = int(rng.choice([64, 128, 256] if prefill else [32, 64, 128, 256, 512]))
        pps = int(rng.integers(1, 7 if prefill else 13))
        B = int(rng.integers(1, 4 if prefill else 41))
        L = P * pps
        while B * Hkv * L * D > 24e6:  # keep the host-side f64 loop short
            B = max(1, B // 2)
        Sq = int(rng.integers(2, min(L, 96) + 1)) if prefill else 1
        kind = case % 4
        active = L if kind == 0 else max(Sq, (L - 1) // P * P + 1) if kind == 1 else Sq if kind == 2 else int(rng.integers(Sq, L + 1))
        Hq = G * Hkv
        q = orc.to_storage(rng.standard_normal((B, Hq, Sq, D)), dt)
        k = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
        v = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
        k[:, :, active:] = 0xFFFF
        v[:, :, active:] = 0xFFFF
        exact = orc.attention_f64(q, np.ascontiguousarray(k[:, :, :active]), np.ascontiguousarray(v[:, :, :active]), dt, D ** -0.5, prefill)
        kp, table = scatter_to_pool(k, P, rng, spare=int(rng.integers(0, 5)))
        vp = np.full_like(kp, 0xFFFF)
        for b in range(B):
            for s_ in range(pps):
                vp[table[b, s_]] = v[b, :, s_ * P:(s_ + 1) * P]
        tab = table.copy()
        tab[:, (active + P - 1) // P:] = -1
        got = g.to_host(g.mynn.attention_paged(g.to_dev(q, dt), g.to_dev(kp, dt), g.to_dev(vp, dt), torch.from_numpy(tab).cuda(), P,
                                               D ** -0.5, prefill, active, q_pos_offset=active - Sq))
        err = max_err_rel_to_max(g.f32(got, dt), exact) if prefill else max_abs_rel(g.f32(got, dt), exact)
        assert err <= 1e-2, (case, dt, B, Hq, Hkv, D, Sq, L, active, P, err)


def test_paged_attention_rejects_bad_arguments_with_a_status(g):
    """Shapes and page geometries the paged kernels have no form for come back as errors before anything is launched."""
    import torch

    q = torch.zeros((1, 8, 1, 64), dtype=torch.float16, device="cuda")
    pool = torch.zeros((4, 2, 64, 64), dtype=torch.float16, device="cuda")
    tab = torch.zeros((1, 2), dtype=torch.int32, device="cuda")
    ok = g.mynn.attention_paged(q, pool, pool, tab, 64, 0.125, False, 100)
    assert ok.shape == q.shape
    lib = g.mynn.lib()

    def call(**kw):
        a = dict(out=ok, q=q, k=pool, v=pool, ks=None, vs=None, tab=tab, pps=2, P=64, scale=0.125, causal=0, B=1, Sq=1, active=100,
                 d_active=None, qoff=0, Hq=8, Hkv=2, D=64, dt=g.mynn.F16, kv8=0)
        a.update(kw)
        p = lambda t: None if t is None else t.data_ptr()
        return lib.mynn_attention_paged(p(a["out"]), p(a["q"]), p(a["k"]), p(a["v"]), p(a["ks"]), p(a["vs"]), p(a["tab"]), a["pps"], a["P"],
                                        a["scale"], a["causal"], a["B"], a["Sq"], a["active"], p(a["d_active"]), a["qoff"], a["Hq"], a["Hkv"],
                                        a["D"], a["dt"], a["kv8"], None, 0, None)

    assert call() == 0
    assert call(tab=None) == -1
    assert call(P=48) == -1 and call(P=16) == -1          # not a power of two / below a tile
    assert call(kv8=1) == -1                              # int8 pools without scale pools
    assert call(active=0) == -1
    assert call(dt=g.mynn.F32) == -2
    assert call(Hq=7) == -1                               # not a multiple of the kv heads
    assert call(Hq=6) == -2                               # 3 query heads per kv head: no form
    assert call(D=32) == -2
    q16 = torch.zeros((1, 8, 16, 64), dtype=torch.float16, device="cuda")
    out16 = torch.zeros_like(q16)
    assert call(out=out16, q=q16, Sq=16, causal=1, active=16) == 0
    assert call(out=out16, q=q16, Sq=16, causal=1, active=16, P=32, pps=4) == -2   # a prefill tile is 64 keys
    assert call(out=out16, q=q16, Sq=16, causal=1, active=16, kv8=1, ks=pool, vs=pool) == -2
    big_tab = torch.zeros((1, 65), dtype=torch.int32, device="cuda")
    assert call(out=out16, q=q16, Sq=16, causal=1, active=16, tab=big_tab, pps=65) == -2
    torch.cuda.synchronize()


def test_kvcache_update_paged_scatters_rows_through_the_table(g):
    import torch

    rng = np.random.default_rng(3)
    B, Hkv, D, P, pps = 3, 2, 64, 32, 4
    n_pages = B * pps + 2
    table = rng.permutation(n_pages)[:B * pps].astype(np.int32).reshape(B, pps)
    pool = torch.zeros((n_pages, Hkv, P, D), dtype=torch.float16, device="cuda")
    dtab = torch.from_numpy(table).cuda()
    want = np.zeros((B, Hkv, P * pps, D), np.float16)
    for offset, S_new in ((0, 5), (5, 40), (45, 1), (46, 82)):  # crossing page borders, up to the last row
        new = rng.standard_normal((B, Hkv, S_new, D)).astype(np.float16)
        want[:, :, offset:offset + S_new] = new
        g.mynn.kvcache_update_paged(pool, torch.from_numpy(new).cuda(), offset, dtab, P)
    got = pool.cpu().numpy()
    for b in range(B):
        for s in range(pps):
            assert np.array_equal(got[table[b, s]], want[b, :, s * P:(s + 1) * P]), (b, s)
    used = set(table.ravel().tolist())
    for pg in range(n_pages):
        if pg not in used:
            assert not got[pg].any()
    with pytest.raises(g.mynn.MynnError):
        g.mynn.kvcache_update_paged(pool, torch.zeros((B, Hkv, 2, D), dtype=torch.float16, device="cuda"), P * pps - 1, dtab, P)


def test_pool_and_page_sets_bookkeeping(g):
    """Pages go out on demand, sets on one pool never share a page, a dry pool refuses without taking anything, a
    released set's pages can be taken by another."""
    pool = g.mynn.KvPool(10, 64)
    a = g.mynn.KvPages(pool, 2, 256)   # 2 sequences, up to 4 pages each
    b = g.mynn.KvPages(pool, 1, 512)   # 1 sequence, up to 8 pages
    assert pool.free_pages == 10 and a.pages_per_seq == 4 and b.pages_per_seq == 8 and a.mapped_rows == 0
    assert (a.table() == -1).all()
    a.reserve(1)
    assert a.mapped_rows == 64 and pool.free_pages == 8
    a.reserve(64)  # already there
    assert pool.free_pages == 8
    b.reserve(130)
    assert b.mapped_rows == 192 and pool.free_pages == 5
    a.reserve(65)
    assert pool.free_pages == 3
    ta, tb = a.table(), b.table()
    mapped = [p for p in list(ta.ravel()) + list(tb.ravel()) if p >= 0]
    assert len(mapped) == 7 and len(set(mapped)) == 7 and all(0 <= p < 10 for p in mapped)
    assert (ta[:, :2] >= 0).all() and (ta[:, 2:] == -1).all() and (tb[0, :3] >= 0).all() and (tb[0, 3:] == -1).all()
    # the device table is the host table
    import torch

    dev = torch.empty((2, 4), dtype=torch.int32, device="cuda")
    g.mynn.lib().model_memcpy(dev.data_ptr(), a.table_ptr, 2 * 4 * 4, 3)
    assert np.array_equal(dev.cpu().numpy(), ta)
    # 4 pages wanted, 3 free: refused, nothing taken
    with pytest.raises(g.mynn.MynnError) as e:
        a.reserve(256)
    assert "mynn error -5" in str(e.value) and pool.free_pages == 3 and np.array_equal(a.table(), ta)
    with pytest.raises(g.mynn.MynnError) as e:
        a.reserve(257)  # beyond the set's max_seq
    assert "mynn error -4" in str(e.value)
    b.release()
    assert pool.free_pages == 6 and (b.table() == -1).all() and b.mapped_rows == 0
    a.reserve(256)
    assert pool.free_pages == 2 and (a.table() >= 0).all() and len(set(a.table().ravel().tolist())) == 8
    with pytest.raises(g.mynn.MynnError):
        pool.close()  # sets still alive
    a.close(), b.close()
    assert pool.free_pages == 10
    pool.close()
    for bad in ((0, 64), (4, 48), (4, 16)):
        with pytest.raises(g.mynn.MynnError):
            g.mynn.KvPool(*bad)


PAGED_D64 = dict(SMALL_D64, max_seq=256, ffn=768)  # (every K a multiple of 128: 16..64 rows take the few-row int8 GEMM)


def _sessions(g, cfg, dw, dt, pool, kvbufs, batch, prefill_rows=0, **kw):
    pages = g.mynn.KvPages(pool, batch, cfg["max_seq"])
    dec = g.mynn.Decoder(cfg, dw, batch=batch, kv=kvbufs, kv_pages=pages, **kw)
    pre = g.mynn.Decoder(cfg, dw, batch=batch, seq_q=prefill_rows, kv=kvbufs, kv_pages=pages, **kw) if prefill_rows else None
    return pages, dec, pre


def gather_cache(g, pool_t, table, P):
    """pool tensor [n_pages,Hkv,P,D] -> numpy [B,Hkv,mapped rows,D] in sequence order"""
    pool_np = g.to_host(pool_t)
    B, pps = table.shape
    n = int((table[0] >= 0).sum())
    return np.stack([np.concatenate([pool_np[table[b, s]] for s in range(n)], axis=1) for b in range(B)])


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
def test_paged_executor_prefill_then_batched_decode_equals_contiguous(g, dt):
    """Two sessions of different lengths share one pool; each prefills its prompt chunk by chunk and then decodes.
    Logits, tokens and every cached row are those of an executor pair with contiguous caches, bit for bit (both take
    the same kernels for 16 rows per launch), and pages are taken only as the sequences reach them."""
    import torch

    # (16 sequences x 2 kv heads x 1024 rows: the contiguous decode executor takes the streaming attention kernel too)
    cfg, w = llm_weights.synthetic_int8(dict(PAGED_D64, max_seq=1024), dt, seed=17)
    dw = dev_weights(g, w, dt)
    tdt = g.torch_dtype(dt)
    P = 64
    pool = g.mynn.KvPool(3 * 16 * 4, P)
    kvbufs = pool.buffers(cfg["n_layers"], cfg["n_kv_heads"], cfg["head_dim"], tdt, fill=float("nan"))
    rng = np.random.default_rng(5)
    B = 16
    sessions = []
    for si, (chunk, n_chunks, n_decode) in enumerate(((16, 3, 30), (16, 5, 9))):
        pages, dec, pre = _sessions(g, cfg, dw, dt, pool, kvbufs, B, prefill_rows=chunk)
        ref_dec = g.mynn.Decoder(cfg, dw, batch=B)
        ref_pre = g.mynn.Decoder(cfg, dw, batch=B, seq_q=chunk, kv=ref_dec.kv)
        sessions.append((pages, dec, pre, ref_dec, ref_pre, chunk, n_chunks, n_decode))
    # interleave the two sessions' work so that their pages interleave in the pool
    progress = [0, 0]
    toks = [None, None]
    for rnd in range(40):
        for si, (pages, dec, pre, ref_dec, ref_pre, chunk, n_chunks, n_decode) in enumerate(sessions):
            past = progress[si]
            if past < chunk * n_chunks:
                ids = rng.integers(0, cfg["vocab"], (B, chunk))
                pos = np.arange(past, past + chunk)
                a, la = pre.step(ids, pos, past, past + chunk, want_logits=True)
                b, lb = ref_pre.step(ids, pos, past, past + chunk, want_logits=True)
                assert np.array_equal(la, lb) and a == b, (si, past)
                progress[si] = past + chunk
                toks[si] = a
            elif past < chunk * n_chunks + n_decode:
                a, la = dec.step(toks[si], [past], past, past + 1, want_logits=True)
                b, lb = ref_dec.step(toks[si], [past], past, past + 1, want_logits=True)
                assert np.array_equal(la, lb) and a == b, (si, past)
                progress[si] = past + 1
                toks[si] = a
            assert pages.mapped_rows == (progress[si] + P - 1) // P * P
    assert progress == [48 + 30, 80 + 9]
    assert pool.free_pages == 3 * 16 * 4 - 16 * (2 + 2)
    t0, t1 = sessions[0][0].table(), sessions[1][0].table()
    assert not set(t0[t0 >= 0].tolist()) & set(t1[t1 >= 0].tolist())
    for si, (pages, dec, pre, ref_dec, ref_pre, *_rest) in enumerate(sessions):
        table = pages.table()
        for l in range(cfg["n_layers"]):
            for j in range(2):
                got = gather_cache(g, kvbufs[l][j], table, P)
                want = g.to_host(ref_dec.kv[l][j])
                n = progress[si]
                assert np.array_equal(got[:, :, :n], want[:, :, :n]), (si, l, j)
    # a finished session gives its pages back; the other goes on undisturbed
    pages0, dec0 = sessions[0][0], sessions[0][1]
    pages0.release()
    assert pool.free_pages == 3 * 16 * 4 - 16 * 2
    pages, dec, pre, ref_dec, ref_pre, *_ = sessions[1]
    past = progress[1]
    a, la = dec.step(toks[1], [past], past, past + 1, want_logits=True)
    b, lb = ref_dec.step(toks[1], [past], past, past + 1, want_logits=True)
    assert np.array_equal(la, lb)
    for s in sessions:
        for d in s[1:5]:
            d.close()
        s[0].close()
    pool.close()


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
def test_paged_executor_batch1_decode_vs_oracle(g, dt):
    """Batch-1 decode over a paged cache (hipGraph replay, the device-resident loop included) against the oracle: as
    with a contiguous cache, projection, attention and o projection of a layer are one launch that finds its rows
    through the page table."""
    cfg, w = llm_weights.synthetic_int8(PAGED_D64, dt, seed=23)
    dw = dev_weights(g, w, dt)
    ref = orc.Model(cfg, w)
    P = 64
    pool = g.mynn.KvPool(5, P)
    kvbufs = pool.buffers(cfg["n_layers"], cfg["n_kv_heads"], cfg["head_dim"], g.torch_dtype(dt), fill=float("nan"))
    # take and return a page first so that the session's pages are not 0, 1, 2 ...
    other = g.mynn.KvPages(pool, 1, cfg["max_seq"])
    other.reserve(1)
    pages, dec, _ = _sessions(g, cfg, dw, dt, pool, kvbufs, 1)
    st = dec.stats()
    assert st["graph"] and st["launches_per_step"] == 3 * cfg["n_layers"] + 1
    rng = np.random.default_rng(2)
    n = 70  # crosses the first page border
    toks = rng.integers(0, cfg["vocab"], n)
    for i, t in enumerate(toks):
        want = ref.forward([t], [i], i, i + 1, False)
        nxt, got = dec.step([t], [i], i, i + 1, want_logits=True)
        assert max_err_rel_to_max(g.f32(got, dt), g.f32(want, dt)) <= 1e-2, i
        assert nxt[0] == orc.argmax_last(got[0], dt)
    assert pages.mapped_rows == 128 and pool.free_pages == 2
    table = pages.table()
    assert table[0, 0] != 0
    for l in range(cfg["n_layers"]):
        k_ref, v_ref = ref.kv_cache(l)
        for j, want in ((0, k_ref), (1, v_ref)):
            got = gather_cache(g, kvbufs[l][j], table, P)[0]
            assert max_err_rel_to_max(g.f32(got[:, :n], dt), g.f32(want[:, :n], dt)) <= 1e-2
    # the device-resident loop reserves its rows up front: 70 + 100 rows = 3 pages; then the pool is dry
    out = dec.decode_loop(int(toks[-1]), n - 1, 100)
    assert pages.mapped_rows == 192 and pool.free_pages == 1
    again = dec.decode_loop(int(toks[-1]), n - 1, 100)
    assert out == again
    # ... and step by step gives the same tokens
    t = int(toks[-1])
    for i in range(5):
        nxt, _ = dec.step([t], [n - 1 + i], n - 1 + i, n + i)
        assert nxt[0] == out[i], i
        t = nxt[0]
    other.reserve(65)  # the last free page goes to the other set
    with pytest.raises(g.mynn.MynnError) as e:
        dec.decode_loop(int(toks[-1]), n - 1, 150)
    assert "mynn error -5" in str(e.value)
    with pytest.raises(g.mynn.MynnError) as e:
        dec.step([1], [200], 200, 201)
    assert "mynn error -5" in str(e.value)
    dec.close(), pages.close(), other.close(), pool.close()


@pytest.mark.parametrize("kv8", [False, True], ids=["kv16", "kv_int8"])
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
def test_paged_batch1_single_launch_layer_equals_contiguous(g, dt, D, kv8):
    """The single-launch layer (q|k|v projection, RoPE + append + attention, o projection) over a paged cache reads and
    writes the same rows in the same order as over a contiguous one: logits, tokens and cached rows bit for bit, step
    by step across page borders and inside the device-resident loop; one op per launch (unfused_decode: the streaming
    attention kernel) agrees with it within the 16-bit tolerance."""
    from test_gpu_decoder import SHORT_CACHE

    cfg, w = llm_weights.synthetic_int8(SHORT_CACHE[D], dt, seed=37)
    dw = dev_weights(g, w, dt)
    P = 64
    pool = g.mynn.KvPool(2 * cfg["max_seq"] // P + 3, P)
    tdt = g.torch_dtype(dt)
    other = g.mynn.KvPages(pool, 1, cfg["max_seq"])
    other.reserve(P + 1)  # (the session's pages then are not 0, 1, 2 ...)
    plain = g.mynn.Decoder(cfg, dw, quant_kv_cache=kv8)
    kv_a = pool.buffers(cfg["n_layers"], cfg["n_kv_heads"], cfg["head_dim"], tdt, fill=float("nan"), kv_int8=kv8)
    pages_a = g.mynn.KvPages(pool, 1, cfg["max_seq"])
    paged = g.mynn.Decoder(cfg, dw, kv=kv_a, kv_pages=pages_a, quant_kv_cache=kv8)
    pages_b = g.mynn.KvPages(pool, 1, cfg["max_seq"])
    single = g.mynn.Decoder(cfg, dw, kv=kv_a, kv_pages=pages_b, quant_kv_cache=kv8, unfused_decode=True)
    L = cfg["n_layers"]
    assert plain.stats()["launches_per_step"] == paged.stats()["launches_per_step"] == 3 * L + 1
    assert single.stats()["launches_per_step"] > 3 * L + 1
    rng = np.random.default_rng(D)
    n = 2 * P + 7
    toks = rng.integers(0, cfg["vocab"], n)
    for i, t in enumerate(toks):
        a, la = plain.step([t], [i], i, i + 1, want_logits=True)
        b, lb = paged.step([t], [i], i, i + 1, want_logits=True)
        assert a == b and np.array_equal(la, lb), i
        if i % 16 == 5 or i >= n - 3:
            _, lc = single.step([t], [i], i, i + 1, want_logits=True)
            assert max_err_rel_to_max(g.f32(lc, dt), g.f32(la, dt)) <= (3e-2 if kv8 else 1e-2), i
        else:
            single.step([t], [i], i, i + 1)
    table = pages_a.table()
    assert table[0, 0] >= 2 and pages_a.mapped_rows == 3 * P
    for l in range(L):
        for j in range(len(plain.kv[l])):  # (int8 KV: codes, then per-row scales)
            got = gather_cache(g, kv_a[l][j] if kv_a[l][j].dim() == 4 else kv_a[l][j].unsqueeze(-1), table, P)[0]
            want = g.to_host(plain.kv[l][j])[0]
            want = want if want.ndim == 3 else want[..., None]
            assert np.array_equal(got[:, :n], want[:, :n]), (l, j)
    # the device-resident loop
    assert paged.decode_loop(int(toks[-1]), n - 1, 40) == plain.decode_loop(int(toks[-1]), n - 1, 40)
    for d in (plain, paged, single):
        d.close()
    pages_a.close(), pages_b.close(), other.close(), pool.close()


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
def test_paged_int8_kv_decode_executor_equals_contiguous(g, dt):
    """quant_kv_cache over pools (code pools + scale pools, decode models): 16 sequences fed token by token write and read
    the same codes and scales as the executor with contiguous int8 caches, and return the same logits, bit for bit."""
    cfg, w = llm_weights.synthetic_int8(dict(PAGED_D64, max_seq=1024), dt, seed=29)
    dw = dev_weights(g, w, dt)
    P, B = 64, 16
    pool = g.mynn.KvPool(B * 3, P)
    kvbufs = pool.buffers(cfg["n_layers"], cfg["n_kv_heads"], cfg["head_dim"], g.torch_dtype(dt), fill=float("nan"), kv_int8=True)
    pages = g.mynn.KvPages(pool, B, cfg["max_seq"])
    dec = g.mynn.Decoder(cfg, dw, batch=B, kv=kvbufs, kv_pages=pages, quant_kv_cache=True)
    ref = g.mynn.Decoder(cfg, dw, batch=B, quant_kv_cache=True)
    rng = np.random.default_rng(12)
    n = 70
    for i in range(n):
        toks = rng.integers(0, cfg["vocab"], B)
        a, la = dec.step(toks, [i], i, i + 1, want_logits=True)
        b, lb = ref.step(toks, [i], i, i + 1, want_logits=True)
        assert np.array_equal(la, lb) and a == b, i
    assert pages.mapped_rows == 128 and pool.free_pages == B
    table = pages.table()
    for l in range(cfg["n_layers"]):
        for j in range(4):
            got = gather_cache(g, kvbufs[l][j], table, P)
            want = g.to_host(ref.kv[l][j])
            assert np.array_equal(got[:, :, :n], want[:, :, :n]), (l, j)
    with pytest.raises(g.mynn.MynnError):  # a prefill model over int8 pages: no kernel
        g.mynn.Decoder(cfg, dw, batch=B, seq_q=16, kv=kvbufs, kv_pages=pages, quant_kv_cache=True)
    dec.close(), ref.close(), pages.close(), pool.close()


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("opt", ["w8a8", "qkv_bias", "unfused", "kv_int8_w8a8"])
def test_paged_batch1_decode_with_other_options_vs_oracle(g, dt, opt):
    """The paged cache under the executor's other options (int8 activations, projection biases, one op per launch,
    int8 cache + int8 activations): batch-1 decode across a page border against the oracle with the same options."""
    cfg, w = llm_weights.synthetic_int8(PAGED_D64, dt, seed=37)
    if opt == "qkv_bias":
        w = llm_weights.add_qkv_bias(cfg, w, dt, seed=38, std=0.05)
    w8a8, kv8 = "w8a8" in opt, "kv_int8" in opt
    ref = orc.Model(cfg, w)
    ref.set_options(quant_kv_cache=kv8, quantize_activations=w8a8)
    P = 64
    pool = g.mynn.KvPool(4, P)
    kvbufs = pool.buffers(cfg["n_layers"], cfg["n_kv_heads"], cfg["head_dim"], g.torch_dtype(dt), fill=float("nan"), kv_int8=kv8)
    pages = g.mynn.KvPages(pool, 1, cfg["max_seq"])
    dec = g.mynn.Decoder(cfg, dev_weights(g, w, dt), kv=kvbufs, kv_pages=pages, quantize_activations=w8a8, quant_kv_cache=kv8,
                         unfused_decode=opt == "unfused")
    tol = 3e-2 if w8a8 else 1e-2
    rng = np.random.default_rng(3)
    for i, t in enumerate(rng.integers(0, cfg["vocab"], 68)):
        want = ref.forward([t], [i], i, i + 1, False)
        nxt, got = dec.step([t], [i], i, i + 1, want_logits=True)
        assert max_err_rel_to_max(g.f32(got, dt), g.f32(want, dt)) <= tol, i
        assert nxt[0] == orc.argmax_last(got[0], dt)
    assert pages.mapped_rows == 128
    dec.close(), pages.close(), pool.close()


def test_generate_loop_over_a_paged_cache_and_reset_gives_the_pages_back(g):
    """LlmSession (chunked zero-padded prefill, then greedy decode) over models with a paged cache produces the ids of the
    same session over contiguous caches; reset returns the pages to the pool and a second run reproduces the first."""
    dt = orc.F16
    cfg, w = llm_weights.synthetic_int8(PAGED_D64, dt, seed=53)
    dw = dev_weights(g, w, dt)
    pool = g.mynn.KvPool(4, 64)
    kvbufs = pool.buffers(cfg["n_layers"], cfg["n_kv_heads"], cfg["head_dim"], g.torch_dtype(dt), fill=float("nan"))
    pages, dec, pre = _sessions(g, cfg, dw, dt, pool, kvbufs, 1, prefill_rows=16)
    ref_dec = g.mynn.Decoder(cfg, dw, unfused_decode=True)
    ref_pre = g.mynn.Decoder(cfg, dw, seq_q=16, kv=ref_dec.kv)
    prompt = np.random.default_rng(9).integers(0, cfg["vocab"], 37).tolist()
    a = g.mynn.LlmSession(dec, prefill=pre)
    b = g.mynn.LlmSession(ref_dec, prefill=ref_pre)
    ids = a.generate_ids(prompt, 40)
    want = b.generate_ids(prompt, 40)
    # the paged decode attention runs in another kernel than the contiguous executor's: equal ids up to ties the oracle confirms
    if ids != want:
        first = next(i for i in range(40) if ids[i] != want[i])
        ok, verdicts = g.both_acceptable(cfg, w, prompt + want[:first], [ids[first], want[first]], dt)
        assert ok, (first, verdicts)
    assert a.past_len == len(prompt) + 40 - 1 and pages.mapped_rows == 128 and pool.free_pages == 2
    a.reset()
    assert a.past_len == 0 and pages.mapped_rows == 0 and pool.free_pages == 4
    assert a.generate_ids(prompt, 40) == ids
    a.close(), b.close()
    for d in (dec, pre, ref_dec, ref_pre):
        d.close()
    pages.close(), pool.close()


def test_paged_executor_rejects_what_it_has_no_kernel_for(g):
    dt = orc.F16
    cfg, w = llm_weights.synthetic_int8(PAGED_D64, dt, seed=1)
    dw = dev_weights(g, w, dt)
    pool = g.mynn.KvPool(8, 64)
    kvbufs = pool.buffers(cfg["n_layers"], cfg["n_kv_heads"], cfg["head_dim"], g.torch_dtype(dt))
    pages = g.mynn.KvPages(pool, 1, cfg["max_seq"])
    for kw in (dict(streaming_kv=True), dict(batch=2)):
        with pytest.raises(g.mynn.MynnError):
            g.mynn.Decoder(cfg, dw, kv=kvbufs, kv_pages=pages, **kw)
    pool32 = g.mynn.KvPool(8, 32)  # pages smaller than a prefill tile
    pages32 = g.mynn.KvPages(pool32, 1, cfg["max_seq"])
    with pytest.raises(g.mynn.MynnError):
        g.mynn.Decoder(cfg, dw, kv=kvbufs, kv_pages=pages32)
    pages32.close(), pool32.close(), pages.close(), pool.close()


def test_paged_decode_key_range_longer_than_62_pages_is_cut(g):
    """Batch 32 x 8 kv heads fills the CUs with one key range per (sequence, kv head); at 4096 rows in pages of 64 that
    range would span 64 pages, more than the one register of page numbers a workgroup carries (62): the plan cuts it
    into two ranges and merges them.  Result against the oracle and the contiguous call."""
    import torch

    dt = orc.F16
    B, Hq, Hkv, D, L, active, P = 32, 32, 8, 64, 4096, 4001, 64
    rng = np.random.default_rng(77)
    q = orc.to_storage(rng.standard_normal((B, Hq, 1, D)), dt)
    k = orc.to_storage(rng.standard_normal((B, Hkv, L, D), dtype=np.float32), dt)
    v = orc.to_storage(rng.standard_normal((B, Hkv, L, D), dtype=np.float32), dt)
    k[:, :, active:] = 0xFFFF
    v[:, :, active:] = 0xFFFF
    kp, table = scatter_to_pool(k, P, rng)
    vp = np.full_like(kp, 0xFFFF)
    for b in range(B):
        for s in range(L // P):
            vp[table[b, s]] = v[b, :, s * P:(s + 1) * P]
    dq, dtab = g.to_dev(q, dt), torch.from_numpy(table).cuda()
    got = g.to_host(g.mynn.attention_paged(dq, g.to_dev(kp, dt), g.to_dev(vp, dt), dtab, P, D ** -0.5, False, active))
    del kp, vp
    plain = g.to_host(g.mynn.attention(dq, g.to_dev(k, dt), g.to_dev(v, dt), D ** -0.5, False, active))
    assert max_abs_rel(g.f32(got, dt), g.f32(plain, dt)) <= 1e-2
    want = orc.attention(q[:2], k[:2], v[:2], dt, D ** -0.5, False, active)
    assert max_abs_rel(g.f32(got[:2], dt), g.f32(want, dt)) <= 1e-2
