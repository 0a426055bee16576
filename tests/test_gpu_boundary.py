"""The boundary's own contracts on the GPU: the KV row a decode step writes, recovery when a shared launch's
hand-over gives up, the additive attention mask (operator slot 3), caller-owned workspaces and prepared weights,
the executor's own weight workspace, the streaming-KV graph up to sink + window (past it: test_gpu_streaming.py)."""
import os

import numpy as np
import pytest

import oracle as orc
import llm_weights
import pbreader
from conftest import GOLDEN, close_either, max_abs_rel, max_err_rel_to_max
from test_gpu_decoder import SHORT_CACHE, SMALL, dev_weights

pytestmark = pytest.mark.gpu
SO = os.path.join(GOLDEN, "single_op")


@pytest.fixture(scope="module")
def g():
    import gpu_util

    return gpu_util


# ------------------------------------------------------------------ KVCacheUpdate(offset = past_len)
@pytest.mark.parametrize("kind", ["shared_launches", "one_op_per_launch", "generic_head_dim_32"])
def test_decode_step_appends_at_past_len_whatever_active_says(g, kind):
    """The reference's decode graph writes the new K/V row at `past_len` (KVCacheUpdate's offset) and attends to
    rows [0, active_seq_kv); LlmSession always passes active = past + 1, a Session caller may not.  Every batch-1
    executor must do the same: a step that rewrites row 3 while attending to 6 rows, and one whose new row lies
    beyond the attended range."""
    dt = orc.F16
    shape = SMALL if kind == "generic_head_dim_32" else SHORT_CACHE[64]
    cfg, w = llm_weights.synthetic_int8(shape, dt, seed=101)
    ref = orc.Model(cfg, w)
    dec = g.mynn.Decoder(cfg, dev_weights(g, w, dt), unfused_decode=(kind == "one_op_per_launch"))
    if kind == "shared_launches":
        assert dec.stats()["launches_per_step"] == 3 * cfg["n_layers"] + 1
    steps = [(5, 0, 0, 1), (17, 1, 1, 2), (99, 2, 2, 3), (4, 3, 3, 4), (250, 4, 4, 5), (31, 5, 5, 6),
             (77, 3, 3, 6),   # rewrites row 3, attends to rows 0..5
             (12, 6, 6, 5),   # appends row 6, attends to rows 0..4 only
             (8, 6, 6, 7)]    # and the ordinary next step over what those left
    for tok, pos, past, active in steps:
        want = ref.forward([tok], [pos], past, active, False)
        nxt, got = dec.step([tok], [pos], past, active, want_logits=True)
        assert max_err_rel_to_max(g.f32(got, dt), g.f32(want, dt)) <= 1e-2, (tok, past, active)
        assert nxt[0] == orc.argmax_last(got[0], dt)
    for l in range(cfg["n_layers"]):
        k_ref, v_ref = ref.kv_cache(l)
        k_gpu, v_gpu = g.to_host(dec.kv[l][0])[0], g.to_host(dec.kv[l][1])[0]
        assert max_err_rel_to_max(g.f32(k_gpu[:, :7], dt), g.f32(k_ref[:, :7], dt)) <= 1e-2
        assert max_err_rel_to_max(g.f32(v_gpu[:, :7], dt), g.f32(v_ref[:, :7], dt)) <= 1e-2
        assert not k_gpu[:, 7:].any() and not v_gpu[:, 7:].any()
    dec.close()


# ------------------------------------------------------------------ hand-over give-up and recovery
@pytest.mark.parametrize("kv8", [False, True], ids=["kv16", "kv_int8"])
@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
def test_handover_give_up_falls_back_to_one_op_per_launch(g, dt, kv8):
    """A consumer role that gives up at once (handover_spin_limit = -1) raises the error word; every kernel still
    exits normally.  The executor then discards the step, rebuilds itself with one op per launch and repeats the
    step: the caller sees the results of the un-fused executor, bit for bit, and a failure count of 1."""
    cfg, w = llm_weights.synthetic_int8(SHORT_CACHE[64], dt, seed=71)
    dw = dev_weights(g, w, dt)
    plain = g.mynn.Decoder(cfg, dw, unfused_decode=True, quant_kv_cache=kv8)
    quick = g.mynn.Decoder(cfg, dw, handover_spin_limit=-1, quant_kv_cache=kv8)
    assert quick.stats()["launches_per_step"] == 3 * cfg["n_layers"] + 1 and quick.handover_failures == 0
    toks = np.random.default_rng(1).integers(0, cfg["vocab"], 12)
    for i, t in enumerate(toks):
        a, la = quick.step([t], [i], i, i + 1, want_logits=True)
        b, lb = plain.step([t], [i], i, i + 1, want_logits=True)
        assert np.array_equal(la, lb) and a == b, i
    assert quick.handover_failures == 1, "producers cannot have finished before the consumers' first look"
    assert quick.stats()["launches_per_step"] == plain.stats()["launches_per_step"] and quick.stats()["graph"]
    for l in range(cfg["n_layers"]):
        for j in range(len(plain.kv[l])):  # (int8 KV: codes and per-row scales)
            assert np.array_equal(g.to_host(quick.kv[l][j]), g.to_host(plain.kv[l][j]))
    quick.close()
    # the same inside the device-resident loop: the whole loop is repeated after the rebuild
    loop = g.mynn.Decoder(cfg, dw, handover_spin_limit=-1, quant_kv_cache=kv8)
    n = len(toks)
    for i, t in enumerate(toks):
        first, _ = plain.step([t], [i], i, i + 1)  # (plain's cache already holds these rows: same values again)
    for l in range(cfg["n_layers"]):
        for j in range(len(plain.kv[l])):
            loop.kv[l][j].copy_(plain.kv[l][j])
    assert loop.decode_loop(first[0], n, 20) == plain.decode_loop(first[0], n, 20)
    assert loop.handover_failures == 1
    loop.close(), plain.close()


@pytest.mark.parametrize("dt", [orc.F16])
def test_handover_fallback_rearms_after_clean_steps(g, dt):
    """A model that fell back goes back to the shared launches after the given number of clean steps.  With a consumer
    that always gives up at once the first shared step after the re-arm fails again (and doubles the wait), so the
    failure count shows where the re-arms happened; every step's results stay those of the un-fused executor."""
    cfg, w = llm_weights.synthetic_int8(SHORT_CACHE[64], dt, seed=72)
    dw = dev_weights(g, w, dt)
    plain = g.mynn.Decoder(cfg, dw, unfused_decode=True)
    quick = g.mynn.Decoder(cfg, dw, handover_spin_limit=-1)
    quick.set_handover_rearm(3)
    shared, single = quick.stats()["launches_per_step"], plain.stats()["launches_per_step"]
    toks = np.random.default_rng(2).integers(0, cfg["vocab"], 14)
    failures, launches = [], []
    for i, t in enumerate(toks):
        a, la = quick.step([t], [i], i, i + 1, want_logits=True)
        b, lb = plain.step([t], [i], i, i + 1, want_logits=True)
        assert np.array_equal(la, lb) and a == b, i
        failures.append(quick.handover_failures)
        launches.append(quick.stats()["launches_per_step"])
    # step 0 gives up (1); clean steps 1-3 re-arm; step 4 gives up (2) and the wait doubles to 6: clean steps
    # 5-10 re-arm; step 11 gives up (3); the wait is 12 from there
    assert failures == [1, 1, 1, 1, 2, 2, 2, 2, 2, 2, 2, 3, 3, 3]
    assert launches == [single] * 3 + [shared] + [single] * 6 + [shared] + [single] * 3
    # never again once switched off
    quick.set_handover_rearm(0)
    for i in range(14, 40):
        quick.step([int(toks[i % 14])], [i], i, i + 1)
    assert quick.handover_failures == 3 and quick.stats()["launches_per_step"] == single
    quick.close(), plain.close()


# ------------------------------------------------------------------ additive mask (operator slot 3)
def test_attention_causal_golden_as_explicit_mask(g):
    """The reference's `attention_causal` fixture with the causal rule written as an additive mask (0 on and below
    the diagonal, -inf above) and is_causal off: the same output."""
    ins, (o,) = pbreader.read_case(os.path.join(SO, "attention_causal"))
    q, k, v = ins[0].array, ins[1].array, ins[2].array
    S = q.shape[2]
    mask = np.triu(np.full((S, S), -np.inf, np.float32), 1)
    got = g.to_host(g.mynn.attention_ws(g.to_dev(q), g.to_dev(k), g.to_dev(v), 8 ** -0.5, False, mask=g.to_dev(mask)))
    ok, md = close_either(got, o.array, 1e-4)
    assert ok, md
    plain = g.to_host(g.mynn.attention(g.to_dev(q), g.to_dev(k), g.to_dev(v), 8 ** -0.5, True))
    ok, md = close_either(got, plain, 1e-6)  # masked-out keys weigh exactly 0; only the order of the sums may differ
    assert ok, md


def masked_attention_f64(q, k, v, mask, scale, causal, active, dt):
    """f64 restatement with the reference's order: score * scale + mask, then softmax over the admitted keys
    (attention.cuh:436-451)."""
    qf, kf, vf = orc.to_f32(q, dt).astype(np.float64), orc.to_f32(k, dt).astype(np.float64), orc.to_f32(v, dt).astype(np.float64)
    B, Hq, Sq, D = qf.shape
    Hkv = kf.shape[1]
    out = np.zeros_like(qf)
    mf = np.broadcast_to(orc.to_f32(mask, dt).astype(np.float64), (B, Hq, Sq, kf.shape[2])) if mask.ndim == 4 else None
    for b in range(B):
        for h in range(Hq):
            kk, vv = kf[b, h // (Hq // Hkv)], vf[b, h // (Hq // Hkv)]
            for s in range(Sq):
                n = min(active, active - Sq + s + 1) if causal else active
                sc = kk[:n] @ qf[b, h, s] * scale + mf[b, h, s, :n]
                p = np.exp(sc - sc.max())
                out[b, h, s] = (p / p.sum()) @ vv[:n]
    return out


@pytest.mark.parametrize("dt", [orc.F32, orc.F16, orc.BF16])
@pytest.mark.parametrize("B,Hq,Hkv,D,Sq,L,active,mshape", [
    (2, 4, 2, 8, 4, 4, 4, (2, 4, 4, 4)),          # one mask slice per (batch, head)
    (2, 4, 2, 32, 3, 40, 33, (1, 1, 3, 40)),      # broadcast over batch and heads
    (1, 8, 2, 64, 1, 3000, 2777, (1, 1, 1, 3000)),  # decode over a cache several workgroups share; one mask row
    (2, 8, 4, 64, 5, 700, 700, (2, 8, 1, 700)),   # the same row for every query position
])
def test_attention_additive_mask_vs_f64(g, dt, B, Hq, Hkv, D, Sq, L, active, mshape):
    rng = np.random.default_rng(B * 1000 + L + Sq)
    q = orc.to_storage(rng.standard_normal((B, Hq, Sq, D)), dt)
    k = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
    v = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
    mask = orc.to_storage(rng.standard_normal(mshape) * 2, dt)
    for causal in (False, True):
        want = masked_attention_f64(q, k, v, mask, D ** -0.5, causal, active, dt)
        got = g.to_host(g.mynn.attention_ws(g.to_dev(q, dt), g.to_dev(k, dt), g.to_dev(v, dt), D ** -0.5, causal, active,
                                            mask=g.to_dev(mask, dt)))
        assert max_abs_rel(g.f32(got, dt), want) <= (1e-4 if dt == orc.F32 else 1e-2), causal


# ------------------------------------------------------------------ workspaces, prepared weights
def test_attention_and_matmul_with_caller_workspace_equal_the_library_scratch_forms(g):
    import torch

    dt = orc.F16
    rng = np.random.default_rng(12)
    B, Hq, Hkv, D, L = 2, 32, 4, 64, 4096
    assert g.mynn.lib().mynn_attention_workspace_bytes(B, 1, L, Hq, Hkv, D, dt, 0) > 0
    q = g.to_dev(orc.to_storage(rng.standard_normal((B, Hq, 1, D)), dt), dt)
    k = g.to_dev(orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt), dt)
    v = g.to_dev(orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt), dt)
    assert torch.equal(g.mynn.attention_ws(q, k, v, 0.125, active=3999), g.mynn.attention(q, k, v, 0.125, active=3999))
    # a workspace that is too small is refused, not overrun
    out = torch.empty_like(q)
    ws = torch.empty(64, dtype=torch.uint8, device="cuda")
    rc = g.mynn.lib().mynn_attention_ws(out.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), None, 0, 0, None, None, 0.125, 0,
                                        B, 1, 3999, None, L, 3998, Hq, Hkv, D, dt, 0, ws.data_ptr(), 64, None)
    assert rc == -1 and b"workspace" in g.mynn.lib().mynn_last_error()
    M, N, K = 48, 520, 256
    act = g.to_dev(orc.to_storage(rng.standard_normal((M, K)), dt), dt)
    W = g.to_dev(rng.integers(-127, 128, (N, K)).astype(np.int8))
    sc = g.to_dev(orc.to_storage(rng.uniform(1e-3, 1e-2, N), dt), dt)
    assert g.mynn.lib().mynn_dequant_matmul_workspace_bytes(M, N, K, dt, dt) >= N * K * 2
    assert g.mynn.lib().mynn_dequant_matmul_workspace_bytes(8, N, K, dt, dt) == 0
    assert torch.equal(g.mynn.dequant_matmul_ws(act, W, sc), g.mynn.dequant_matmul(act, W, sc))


def test_dequant_matmul_on_two_streams_keeps_two_workspaces(g):
    """Calls on different streams get different library workspaces: two products in flight at once, each many
    times, each against its own weight."""
    import torch

    dt = orc.F16
    rng = np.random.default_rng(5)
    M, N, K = 256, 1024, 1024
    acts = [g.to_dev(orc.to_storage(rng.standard_normal((M, K)), dt), dt) for _ in range(2)]
    Ws = [g.to_dev(rng.integers(-127, 128, (N, K)).astype(np.int8)) for _ in range(2)]
    scs = [g.to_dev(orc.to_storage(rng.uniform(1e-3, 1e-2, N), dt), dt) for _ in range(2)]
    want = [g.mynn.dequant_matmul_ws(acts[i], Ws[i], scs[i]) for i in range(2)]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [[], []]
    for rep in range(20):
        for i in range(2):
            with torch.cuda.stream(streams[i]):
                outs[i].append(g.mynn.dequant_matmul(acts[i], Ws[i], scs[i]))
    torch.cuda.synchronize()
    for i in range(2):
        for o in outs[i]:
            assert torch.equal(o, want[i])


def test_workspace_variant_replays_from_a_captured_graph(g):
    """mynn_dequant_matmul_ws touches nothing global, so a caller may capture it: replayed three times with new
    activations and eager work in between, every replay equals the eager call."""
    import torch

    dt = orc.F16
    rng = np.random.default_rng(6)
    M, N, K = 64, 512, 512
    act = g.to_dev(orc.to_storage(rng.standard_normal((M, K)), dt), dt)
    W = g.to_dev(rng.integers(-127, 128, (N, K)).astype(np.int8))
    sc = g.to_dev(orc.to_storage(rng.uniform(1e-3, 1e-2, N), dt), dt)
    lib = g.mynn.lib()
    need = lib.mynn_dequant_matmul_workspace_bytes(M, N, K, dt, dt)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    out = torch.empty((M, N), dtype=torch.float16, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        g.mynn.check(lib.mynn_dequant_matmul_ws(out.data_ptr(), act.data_ptr(), W.data_ptr(), sc.data_ptr(), M, N, K, dt, dt,
                                                ws.data_ptr(), need, 0, side.cuda_stream))  # warm-up: function attributes are set
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g.mynn.check(lib.mynn_dequant_matmul_ws(out.data_ptr(), act.data_ptr(), W.data_ptr(), sc.data_ptr(), M, N, K, dt, dt,
                                                ws.data_ptr(), need, 0, torch.cuda.current_stream().cuda_stream))
    for rep in range(3):
        new = g.to_dev(orc.to_storage(rng.standard_normal((M, K)), dt), dt)
        act.copy_(new)
        want = g.mynn.dequant_matmul(new, W, sc)
        torch.cuda.synchronize()
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), rep


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
def test_prefill_executor_with_its_own_weight_workspace(g, dt):
    """A prefill executor whose shapes take neither the resident 16-bit weights nor the few-row kernel (ffn not a
    multiple of 32) dequantises each weight per call into a workspace it owns: two of them alive at once, run
    alternately, each against the oracle."""
    shape = dict(SMALL, ffn=712)
    cfg, w = llm_weights.synthetic_int8(shape, dt, seed=91)
    cfg2, w2 = llm_weights.synthetic_int8(dict(shape, hidden=128, n_heads=4, n_kv_heads=2), dt, seed=92)
    refs = [orc.Model(cfg, w), orc.Model(cfg2, w2)]
    for r in refs:
        r.set_gemm_mode(2)
    decs = [g.mynn.Decoder(cfg, dev_weights(g, w, dt), seq_q=24), g.mynn.Decoder(cfg2, dev_weights(g, w2, dt), seq_q=24)]
    assert "dequant_weight" in [n for n, _, _, _ in decs[0].profile(np.zeros(24, np.int64), np.arange(24), 0, 24)]
    rng = np.random.default_rng(2)
    for chunk in range(2):
        for d, r, c in zip(decs, refs, (cfg, cfg2)):
            ids = rng.integers(0, c["vocab"], 24)
            pos = np.arange(24 * chunk, 24 * chunk + 24)
            want = r.forward(ids, pos, 24 * chunk, 24 * chunk + 24, True)
            _, got = d.step(ids, pos, 24 * chunk, 24 * chunk + 24, want_logits=True)
            assert max_err_rel_to_max(g.f32(got, dt), g.f32(want, dt)) <= 1e-2
    for d in decs:
        d.close()


# ------------------------------------------------------------------ streaming KV in the executor
@pytest.mark.parametrize("dt", [orc.BF16, orc.F16])
@pytest.mark.parametrize("prefill_len", [0, 4])
def test_streaming_kv_executor_reproduces_the_reference_ids(g, dt, prefill_len):
    """crates/llm/tests/tinyllama_random.rs:20-60: the reference's known answer is produced with
    BuildOptions::streaming_kv, sink 4 + window 28 = max_seq_len 32, LlmSession::for_llama_streaming -- the same
    configuration here (and, as its multi-turn test, with a prefill session in front)."""
    cfg, w, golden = llm_weights.tiny_llama_random(dt, max_seq=32)
    dw = dev_weights(g, w, dt)
    dec = g.mynn.Decoder(cfg, dw, streaming_kv=True)
    pre = g.mynn.Decoder(cfg, dw, seq_q=prefill_len, kv=dec.kv, streaming_kv=True) if prefill_len else None
    llm = g.mynn.LlmSession(dec, prefill=pre, eos=1, streaming=(4, 28))
    ids = llm.generate_ids(golden["prompt_ids"], len(golden["expected_new_ids"]))
    assert ids == golden["expected_new_ids"]
    assert not dec.stats()["graph"]  # the ring inputs are read at launch time, as the reference's kernels do
    llm.close(), dec.close()
    if pre:
        pre.close()


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("kv8", [False, True])
def test_streaming_kv_executor_steps_vs_oracle(g, dt, kv8):
    """Up to sink + window the streaming graph computes what the plain graph computes -- the key of position p sits
    in slot p and is rotated by p when it is read instead of when it is written -- so logits follow the oracle's
    plain decoder; the cache itself holds the UN-ROTATED keys (rotating them by their positions gives the plain
    graph's cache).  With an int8 cache the key is quantised before the rotation instead of after it, which is a
    different (equally valid) rounding: logits within the quantisation noise of that path."""
    shape = dict(SMALL, max_seq=48)
    cfg, w = llm_weights.synthetic_int8(shape, dt, seed=17)
    ref = orc.Model(cfg, w)
    ref.set_options(quant_kv_cache=kv8, quantize_activations=False)
    ref.set_gemm_mode(2)
    dw = dev_weights(g, w, dt)
    sink, window = 4, 40
    dec = g.mynn.Decoder(cfg, dw, streaming_kv=True, quant_kv_cache=kv8)
    pre = g.mynn.Decoder(cfg, dw, seq_q=16, kv=dec.kv, streaming_kv=True, quant_kv_cache=kv8)
    tol = 3e-2 if kv8 else 1e-2
    rng = np.random.default_rng(8)
    ids = rng.integers(0, cfg["vocab"], 16)
    kvpos = orc.streaming_kv_position(sink, window, 16, cfg["max_seq"])
    want = ref.forward(ids, np.arange(16), 0, 16, True)
    _, got = pre.step_streaming(ids, np.arange(16), 0, 16, sink, window, 0, kvpos, want_logits=True)
    assert max_err_rel_to_max(g.f32(got, dt), g.f32(want, dt)) <= tol
    past = 16
    for t in [7, 500, 31, 999, 2]:
        kvpos = orc.streaming_kv_position(sink, window, past, cfg["max_seq"])
        want = ref.forward([t], [past], past, past + 1, False)
        if past % 2:
            nxt, got = dec.step_streaming([t], [past], past, past + 1, sink, window, 0, kvpos, want_logits=True)
        else:  # the reference ABI with its eight inputs
            got = dec.model([t], [past], past, past + 1, ring=(sink, window, 0, kvpos))
        assert max_err_rel_to_max(g.f32(got, dt), g.f32(want, dt)) <= tol, past
        past += 1
    if not kv8:
        cos, sin = orc.rope_table(cfg["max_seq"], cfg["head_dim"], cfg["rope_theta"], dt)
        for l in range(cfg["n_layers"]):
            k_raw = g.to_host(dec.kv[l][0])[0][:, :past]
            k_rot = orc.rope(k_raw, cos, sin, np.arange(past), dt)
            k_ref, v_ref = ref.kv_cache(l)
            assert max_err_rel_to_max(g.f32(k_rot, dt), g.f32(k_ref[:, :past], dt)) <= 1e-2
            assert max_err_rel_to_max(g.f32(g.to_host(dec.kv[l][1])[0][:, :past], dt), g.f32(v_ref[:, :past], dt)) <= 1e-2
    # a plain step on a streaming model, and ring inputs on a plain model, are refused
    with pytest.raises(g.mynn.MynnError):
        dec.step([1], [past], past, past + 1)
    # (steps past sink + window: tests/test_gpu_streaming.py)
    dec.close(), pre.close()
