"""Streaming KV (sink + ring cache) through the executor and the session, including steps past sink + window.

The reference serves those steps on its CUDA backend only (src/codegen/cuda/cpp/kvcache_update.cuh:21,
quantizing_kvcache_update.cuh:24-36, attention.cuh:386-420, 495-606, crates/llm/src/session.rs:539-635) and its tests
assert that generation runs (crates/llm/tests/tinyllama_random.rs:157-315: cuda_streaming_runs_past_window and its
three variants).  Here the same four scenarios run through the library, and on top of them every step's logits are
compared with the oracle's restatement of those kernels (pinned in tests/test_oracle_streaming.py)."""
import numpy as np
import pytest

import oracle as orc
import llm_weights
from conftest import max_err_rel_to_max
from test_gpu_decoder import SHORT_CACHE, SMALL, dev_weights

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def g():
    import gpu_util

    return gpu_util


def decode_inputs(sp, sink, window, max_seq):
    """streaming_decode_inputs (session.rs:571-597)"""
    max_active = sink + window
    rs = 0 if sp < max_active else (sp - sink) % window
    return [min(sp, max_active - 1)], sp, min(sp + 1, max_active), rs, orc.streaming_kv_position(sink, window, sp, max_seq)


def prefill_inputs(sp, P, sink, window, max_seq):
    """streaming_prefill_inputs (session.rs:539-569)"""
    max_active = sink + window
    after = sp + P
    rs = 0 if after <= max_active else (after - sink) % window
    pos = [min(sp + i, max_active - 1) for i in range(P)]
    return pos, sp, min(after, max_active), rs, orc.streaming_kv_position(sink, window, after, max_seq)


@pytest.mark.parametrize("kv8", [False, True], ids=["kv16", "kv_int8"])
@pytest.mark.parametrize("prefill_len", [0, 4], ids=["decode_only", "with_prefill"])
def test_reference_scenarios_run_past_the_window(g, kv8, prefill_len):
    """tinyllama_random.rs:157-315: max_seq_len 32, sink 4, window 16, prompt "Hello", want = sink + window + 10 new
    ids; assert_eq!(new_ids.len(), want) and max_active < past_len.  Then the same token stream step by step against
    the oracle: logits within 1e-2 (3e-2 with the int8 cache, whose codes may differ by one at a rounding tie) of
    the oracle's at every step, before and past the window."""
    dt = orc.BF16
    sink, window, max_seq = 4, 16, 32
    cfg, w, golden = llm_weights.tiny_llama_random(dt, max_seq=max_seq)
    dw = dev_weights(g, w, dt)
    dec = g.mynn.Decoder(cfg, dw, streaming_kv=True, quant_kv_cache=kv8)
    pre = g.mynn.Decoder(cfg, dw, seq_q=prefill_len, kv=dec.kv, streaming_kv=True, quant_kv_cache=kv8) if prefill_len else None
    llm = g.mynn.LlmSession(dec, prefill=pre, eos=-1, streaming=(sink, window))
    want = sink + window + 10
    prompt = golden["prompt_ids"]
    ids = llm.generate_ids(prompt, want)
    assert len(ids) == want
    assert llm.past_len > sink + window
    assert llm.past_len == len(prompt) + want - 1
    # a second turn, now past max_seq_len as well (streaming sessions never report PromptTooLong, session.rs:357)
    ids2 = llm.generate_ids([5, 6, 7, 8, 9], 6)
    assert len(ids2) == 6 and llm.past_len > max_seq
    llm.close(), dec.close()
    if pre:
        pre.close()

    # ---- the same stream, step by step, against the oracle
    ref = orc.Model(cfg, w)
    ref.set_options(quant_kv_cache=kv8)
    dec = g.mynn.Decoder(cfg, dw, streaming_kv=True, quant_kv_cache=kv8)
    pre = g.mynn.Decoder(cfg, dw, seq_q=prefill_len, kv=dec.kv, streaming_kv=True, quant_kv_cache=kv8) if prefill_len else None
    tol = 3e-2 if kv8 else 1e-2
    stream = list(prompt) + ids[:-1] + [5, 6, 7, 8, 9] + ids2[:-1]
    turns = [(0, len(prompt)), (len(prompt) + want - 1, 5)]  # (stream position, prompt tokens) of the two prompts
    sp, worst, past_window = 0, 0.0, 0
    got_ids = []
    while sp < len(stream):
        turn = [t for t in turns if t[0] == sp]
        if pre and turn:
            n = turn[0][1]
            while n > 0:
                chunk = min(n, prefill_len)
                toks = stream[sp:sp + chunk] + [0] * (prefill_len - chunk)
                pos, past, active, rs, kvp = prefill_inputs(sp, prefill_len, sink, window, max_seq)
                wl = ref.forward_streaming(toks, pos, past, active, True, sink, window, rs, kvp)
                _, gl = pre.step_streaming(toks, pos, past, active, sink, window, rs, kvp, want_logits=True)
                worst = max(worst, max_err_rel_to_max(g.f32(gl[:chunk], dt), g.f32(wl[:chunk], dt)))
                sp += chunk
                n -= chunk
            got_ids.append(orc.argmax_last(gl[chunk - 1], dt))
            continue
        pos, past, active, rs, kvp = decode_inputs(sp, sink, window, max_seq)
        wl = ref.forward_streaming([stream[sp]], pos, past, active, False, sink, window, rs, kvp)
        nxt, gl = dec.step_streaming([stream[sp]], pos, past, active, sink, window, rs, kvp, want_logits=True)
        err = max_err_rel_to_max(g.f32(gl, dt), g.f32(wl, dt))
        assert err <= tol, (sp, err)
        worst = max(worst, err)
        past_window += sp >= sink + window
        assert nxt[0] == orc.argmax_last(gl[0], dt)
        sp += 1
    assert worst <= tol, worst
    assert past_window >= 15
    # cache contents: the same slots hold the same rows
    for l in range(cfg["n_layers"]):
        k_ref, v_ref = ref.kv_cache(l)
        k_gpu, v_gpu = g.to_host(dec.kv[l][0])[0], g.to_host(dec.kv[l][1])[0]
        if kv8:
            assert np.max(np.abs(k_gpu.astype(np.int32) - k_ref)) <= 1 and np.max(np.abs(v_gpu.astype(np.int32) - v_ref)) <= 1
        else:
            assert max_err_rel_to_max(g.f32(k_gpu, dt), g.f32(k_ref, dt)) <= 1e-2
            assert max_err_rel_to_max(g.f32(v_gpu, dt), g.f32(v_ref, dt)) <= 1e-2
    dec.close()
    if pre:
        pre.close()


STREAM_SHAPES = {
    "d32": dict(SMALL, max_seq=48),
    "d64": dict(SHORT_CACHE[64], max_seq=64),    # the widths the single-launch attention block is built for:
    "d128": dict(SHORT_CACHE[128], max_seq=64),  # a streaming model must not take it
}


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("kv8", [False, True], ids=["kv16", "kv_int8"])
@pytest.mark.parametrize("shape", ["d32", "d64", "d128"])
def test_streaming_executor_int8_weights_past_the_window_vs_oracle(g, dt, kv8, shape):
    """Int8-weight models at head_dim 32 / 64 / 128 (the last two are the shapes whose plain decode step shares
    launches; the streaming graph runs op by op), sink 4 + window 24 in a cache of 48 / 64 rows: a 12-token prefill
    chunk, then 50 decode steps -- 34 of them past the window -- each against the oracle."""
    cfg, w = llm_weights.synthetic_int8(STREAM_SHAPES[shape], dt, seed=23)
    sink, window, ms = 4, 24, cfg["max_seq"]
    ref = orc.Model(cfg, w)
    ref.set_options(quant_kv_cache=kv8)
    ref.set_gemm_mode(2)
    dw = dev_weights(g, w, dt)
    dec = g.mynn.Decoder(cfg, dw, streaming_kv=True, quant_kv_cache=kv8)
    pre = g.mynn.Decoder(cfg, dw, seq_q=12, kv=dec.kv, streaming_kv=True, quant_kv_cache=kv8)
    assert not dec.stats()["graph"]
    tol = 3e-2 if kv8 else 1e-2
    rng = np.random.default_rng(4)
    toks = [int(t) for t in rng.integers(0, cfg["vocab"], 12)]
    pos, past, active, rs, kvp = prefill_inputs(0, 12, sink, window, ms)
    wl = ref.forward_streaming(toks, pos, past, active, True, sink, window, rs, kvp)
    _, gl = pre.step_streaming(toks, pos, past, active, sink, window, rs, kvp, want_logits=True)
    assert max_err_rel_to_max(g.f32(gl, dt), g.f32(wl, dt)) <= tol
    tok = orc.argmax_last(gl[-1], dt)
    for sp in range(12, 62):
        pos, past, active, rs, kvp = decode_inputs(sp, sink, window, ms)
        wl = ref.forward_streaming([tok], pos, past, active, False, sink, window, rs, kvp)
        if sp % 3 == 0:  # the reference ABI with its eight inputs
            gl = dec.model([tok], pos, past, active, ring=(sink, window, rs, kvp))
            tok = orc.argmax_last(gl[0], dt)
        else:
            nxt, gl = dec.step_streaming([tok], pos, past, active, sink, window, rs, kvp, want_logits=True)
            tok = nxt[0]
        assert max_err_rel_to_max(g.f32(gl, dt), g.f32(wl, dt)) <= tol, sp
    # a prefill chunk past the window (second turn of a session)
    toks = [int(t) for t in rng.integers(0, cfg["vocab"], 12)]
    pos, past, active, rs, kvp = prefill_inputs(62, 12, sink, window, ms)
    wl = ref.forward_streaming(toks, pos, past, active, True, sink, window, rs, kvp)
    _, gl = pre.step_streaming(toks, pos, past, active, sink, window, rs, kvp, want_logits=True)
    assert max_err_rel_to_max(g.f32(gl, dt), g.f32(wl, dt)) <= tol
    dec.close(), pre.close()


def test_two_streaming_models_on_their_own_streams(g):
    """Each streaming executor gathers into memory of its own: two models of different shapes stepped alternately
    (their launches interleave on two streams) give what each gives alone."""
    dt = orc.F16
    sink, window = 4, 24
    models = []
    for shape, seed in (("d64", 5), ("d32", 6)):
        cfg, w = llm_weights.synthetic_int8(STREAM_SHAPES[shape], dt, seed=seed)
        dw = dev_weights(g, w, dt)
        models.append((cfg, dw))
    rng = np.random.default_rng(9)
    toks = rng.integers(0, 1000, 40)

    def run(decs):
        outs = [[] for _ in decs]
        for sp in range(40):
            for i, (d, cfg) in enumerate(decs):
                pos, past, active, rs, kvp = decode_inputs(sp, sink, window, cfg["max_seq"])
                _, gl = d.step_streaming([int(toks[sp])], pos, past, active, sink, window, rs, kvp, want_logits=True)
                outs[i].append(gl.copy())
        return outs

    alone = []
    for cfg, dw in models:
        d = g.mynn.Decoder(cfg, dw, streaming_kv=True)
        alone.append(run([(d, cfg)])[0])
        d.close()
    both = [(g.mynn.Decoder(cfg, dw, streaming_kv=True), cfg) for cfg, dw in models]
    together = run(both)
    for i in range(2):
        for a, b in zip(alone[i], together[i]):
            assert np.array_equal(a, b)
    for d, _ in both:
        d.close()


def test_attention_streaming_with_the_callers_workspace(g):
    """mynn_attention_streaming_ws: same bits as mynn_attention_streaming, for every active length, from a
    workspace sized once for the cache."""
    import torch

    dt = orc.F16
    rng = np.random.default_rng(3)
    B, Hq, Hkv, D, L = 1, 8, 2, 64, 160
    q = g.to_dev(orc.to_storage(rng.standard_normal((B, Hq, 1, D)), dt), dt)
    k = g.to_dev(orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt), dt)
    v = g.to_dev(orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt), dt)
    need = g.mynn.lib().mynn_attention_streaming_workspace_bytes(B, 1, L, Hq, Hkv, D, dt, 0, 0)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    for active, sink, window, start in [(1, 4, 100, 0), (77, 4, 100, 0), (104, 4, 100, 37), (160, 32, 128, 127), (50, 0, 160, 3)]:
        a = g.mynn.attention_streaming(q, k, v, 0.125, False, active, sink, window, start)
        b = g.mynn.attention_streaming(q, k, v, 0.125, False, active, sink, window, start, workspace=ws)
        assert torch.equal(a, b)
        want = orc.attention_ring(g.to_host(q), g.to_host(k), g.to_host(v), dt, 0.125, False, active, sink, window, start)
        assert max_err_rel_to_max(g.f32(g.to_host(b), dt), g.f32(want, dt)) <= 1e-2
    with pytest.raises(g.mynn.MynnError, match="workspace"):
        g.mynn.attention_streaming(q, k, v, 0.125, False, 100, 4, 100, 0, workspace=ws[:256])
