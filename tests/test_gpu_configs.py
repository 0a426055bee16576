"""The benchmark configurations at their stated sizes, each against the oracle: the full 128 + 256 token greedy
decode of the TinyLlama-shape model, the 8 x 1024 prefill pass, and the Llama-3-8B-shape batch-32 decode at its
real widths."""
import os
import sys

import numpy as np
import pytest

import oracle as orc
from conftest import ROOT, max_err_rel_to_max

pytestmark = pytest.mark.gpu
sys.path.insert(0, ROOT)


@pytest.fixture(scope="module")
def g():
    import gpu_util

    return gpu_util


@pytest.fixture(scope="module")
def bench():
    import bench as b

    return b


@pytest.fixture(scope="module")
def tinyllama(g, bench):
    """The benchmark's model: TinyLlama-1.1B shape, int8 weights, fp16 activations, seed 1234."""
    import torch

    dt = orc.F16
    cfg = dict(bench.TINYLLAMA, dtype=dt)
    weights = bench.make_weights(cfg, dt, 1234)
    torch.cuda.synchronize()
    host = bench.to_host_weights(weights)
    return cfg, weights, host


def test_config2_full_greedy_decode_128_prompt_256_generated_vs_oracle(g, bench, tinyllama):
    """configs[2] at full length: 128 prompt tokens through the decode path, then 256 greedy tokens, through
    LlmSession and through the device-resident loop the benchmark times (the same ids).  The oracle follows the
    GPU's token stream step by step (so both always see the same context) and its own greedy choice is compared at
    each of the 256 generated positions.  The reference leaves the order of its f32 sums open, and with random-init
    weights the two best logits are sometimes closer than two orders differ: the oracle therefore runs under four
    summation orders (16, 8, 32, 64 lanes + tree; one KV cache each; a disputed step again under 1, 2 and 4), and a token
    that is not the first order's choice is accepted only where the oracle's own arithmetic does not separate the two tokens: the GPU's
    token is the choice under another order, the orders disagree among themselves, or the oracle's gap between the
    two is inside the shifts its orders show among themselves at that step (oracle.SummationOrders.judge) -- anything
    else fails.  Measured on MI355X, seed 1234: 2 of 256 (positions 149 and 186), both flipped by another order."""
    cfg, weights, host = tinyllama
    dt = cfg["dtype"]
    prompt = np.random.default_rng(1234).integers(0, cfg["vocab"], bench.PROMPT_LEN).tolist()
    n_new = 256
    dec = g.mynn.Decoder(cfg, weights)
    assert dec.stats()["graph"] and dec.stats()["launches_per_step"] == 3 * cfg["n_layers"] + 1
    llm = g.mynn.LlmSession(dec)
    got = llm.generate_ids(prompt, n_new)
    assert len(got) == n_new and llm.past_len == len(prompt) + n_new - 1
    llm.close()
    # the device-resident loop produces the same ids
    first_tok = None
    for i, t in enumerate(prompt):
        first_tok, _ = dec.step([t], [i], i, i + 1)
    assert [first_tok[0]] + dec.decode_loop(first_tok[0], len(prompt), n_new - 1) == got
    dec.close()
    # ... and so does the same model over a paged cache (the single-launch layer finds its rows through the page
    # table), built on a weight set it shares with a second executor
    wset = g.mynn.WeightSet(cfg, weights)
    pool = g.mynn.KvPool(cfg["max_seq"] // 128 + 2, 128)
    other = g.mynn.KvPages(pool, 1, cfg["max_seq"])
    other.reserve(129)  # (two pages gone: the session's pages are not 0, 1, 2)
    pages = g.mynn.KvPages(pool, 1, cfg["max_seq"])
    kv = pool.buffers(cfg["n_layers"], cfg["n_kv_heads"], cfg["head_dim"], g.torch_dtype(dt))
    paged = g.mynn.Decoder(cfg, weights, kv=kv, kv_pages=pages, weight_set=wset)
    twin = g.mynn.Decoder(cfg, weights, weight_set=wset)
    assert paged.stats()["launches_per_step"] == 3 * cfg["n_layers"] + 1 and wset.stats()["holders"] == 3
    for d in (paged, twin):
        for i, t in enumerate(prompt):
            first_tok, _ = d.step([t], [i], i, i + 1)
        assert [first_tok[0]] + d.decode_loop(first_tok[0], len(prompt), n_new - 1) == got
    paged.close(), twin.close(), wset.close(), pages.close(), other.close(), pool.close()
    ref = orc.SummationOrders(cfg, host)
    stream = prompt + got[:-1]
    undecided, wrong = [], []
    for i, t in enumerate(stream):
        rows = [l[0] for l in ref.forward([t], [i], i, i + 1, False)]
        j = i - (len(prompt) - 1)
        if j < 0:
            continue
        verdict, choices = ref.judge(rows, got[j])
        if verdict != "identical":
            lf = orc.to_f32(rows[0], dt)
            gap = float(lf[choices[0]] - lf[got[j]]) / (2.0 ** -11 * abs(float(lf[choices[0]])))
            (wrong if verdict == "different" else undecided).append((j, verdict, sorted(set(choices)), got[j], round(gap, 2)))
    ref.close()
    print("config2: %d of %d generated tokens are not the first summation order's choice; undecided by the oracle: %s; different: %s"
          % (len(undecided) + len(wrong), n_new, undecided, wrong))
    assert not wrong, wrong
    assert len(undecided) <= 8, undecided


def test_config3_prefill_8x1024_executor_vs_oracle(g, bench, tinyllama):
    """configs[3] at full size: 8 prompts x 1024 tokens through the prefill executor (M = 8192 on the matrix cores,
    causal attention at S = 1024).  Causality makes the first rows of a prompt independent of the rest, so logits
    rows and KV rows of a 96-token prefix of three of the prompts are held against the oracle's prefill of that
    prefix; deeper rows are held against the decode path of the same library (rows == decode rows)."""
    cfg, weights, host = tinyllama
    dt = cfg["dtype"]
    B, S, n = bench.PREFILL_BATCH, bench.PREFILL_LEN, 96
    cfg = dict(cfg, max_seq=S)
    pre = g.mynn.Decoder(cfg, weights, seq_q=S, batch=B)
    rng = np.random.default_rng(77)
    ids = rng.integers(0, cfg["vocab"], B * S)
    nxt, got = pre.step(ids, np.arange(S), 0, S, want_logits=True)
    got = got.reshape(B, S, -1)
    ref = orc.Model(dict(cfg), host)
    ref.set_gemm_mode(2)  # the matrix-core kernel choice: weights dequantised to fp16 first
    for b in (0, 3, 7):
        ref.reset()
        want = ref.forward(ids[b * S:b * S + n], np.arange(n), 0, n, True)
        assert max_err_rel_to_max(g.f32(got[b, :n], dt), g.f32(want, dt)) <= 1e-2, b
        for l in (0, 10, 21):
            k_ref, v_ref = ref.kv_cache(l)
            k_gpu, v_gpu = g.to_host(pre.kv[l][0])[b], g.to_host(pre.kv[l][1])[b]
            assert max_err_rel_to_max(g.f32(k_gpu[:, :n], dt), g.f32(k_ref[:, :n], dt)) <= 1e-2, (b, l)
            assert max_err_rel_to_max(g.f32(v_gpu[:, :n], dt), g.f32(v_ref[:, :n], dt)) <= 1e-2, (b, l)
    # the greedy token of every prompt is the argmax of its last row
    for b in range(B):
        assert nxt[b] == orc.argmax_last(got[b, S - 1], dt)
    # the last row of a prompt equals a decode step over that prompt's cache (another kernel family, same values
    # up to summation order): feed token S-1 of prompt 5 again at position S-1 through a decode executor that
    # shares prompt 5's cache rows
    import torch

    b = 5
    dcfg = dict(cfg)
    kv = [(pre.kv[l][0][b:b + 1].clone(), pre.kv[l][1][b:b + 1].clone()) for l in range(cfg["n_layers"])]
    dec = g.mynn.Decoder(dcfg, weights, kv=kv)
    _, last = dec.step([ids[b * S + S - 1]], [S - 1], S - 1, S, want_logits=True)
    assert max_err_rel_to_max(g.f32(last[0], dt), g.f32(got[b, S - 1], dt)) <= 2e-2
    dec.close(), pre.close()
    torch.cuda.empty_cache()


LLAMA3_WIDTHS = dict(n_layers=2, hidden=4096, n_heads=32, n_kv_heads=8, head_dim=128, ffn=14336, vocab=128256, max_seq=64,
                     eps=1e-5, rope_theta=500000.0)


def test_config4_llama3_8b_widths_batch32_decode_vs_per_sequence_oracles(g, bench):
    """configs[4] at its real widths (hidden 4096, 32 / 8 heads of 128, ffn 14336, vocab 128256; two layers instead
    of 32 -- the layers are identical in shape): 32 sequences decoded together for 24 steps, three of them followed
    step by step by their own batch-1 oracle.  The few-row int8 GEMM, the RoPE + append in its reducing launch and
    the decode attention at D = 128 run at the shapes the benchmark times."""
    import torch

    dt = orc.F16
    cfg = dict(LLAMA3_WIDTHS, dtype=dt)
    weights = bench.make_weights(cfg, dt, 4321)
    torch.cuda.synchronize()
    host = bench.to_host_weights(weights)
    B, steps = 32, 24
    dec = g.mynn.Decoder(cfg, weights, batch=B)
    names = [k[0] for k in dec.profile(np.zeros(B, np.int64), [0], 0, 1)]
    assert "linear_gateup_swiglu" in names and "swiglu" not in names  # the few-row int8 GEMM path
    for kv in dec.kv:  # (the profile run wrote row 0)
        kv[0].zero_(), kv[1].zero_()
    follow = (0, 13, 31)
    refs = {b: orc.Model(dict(cfg), host) for b in follow}
    rng = np.random.default_rng(99)
    toks = rng.integers(0, cfg["vocab"], B).tolist()
    for step in range(steps):
        nxt, got = dec.step(toks, [step], step, step + 1, want_logits=True)
        for b in follow:
            want = refs[b].forward([toks[b]], [step], step, step + 1, False)
            assert max_err_rel_to_max(g.f32(got[b:b + 1], dt), g.f32(want, dt)) <= 1e-2, (step, b)
        for b in range(B):
            assert nxt[b] == orc.argmax_last(got[b], dt), (step, b)
        toks = nxt
    for l in range(cfg["n_layers"]):
        for b in follow:
            k_ref, v_ref = refs[b].kv_cache(l)
            k_gpu, v_gpu = g.to_host(dec.kv[l][0])[b], g.to_host(dec.kv[l][1])[b]
            assert max_err_rel_to_max(g.f32(k_gpu[:, :steps], dt), g.f32(k_ref[:, :steps], dt)) <= 1e-2
            assert max_err_rel_to_max(g.f32(v_gpu[:, :steps], dt), g.f32(v_ref[:, :steps], dt)) <= 1e-2
    dec.close()
    del weights
    torch.cuda.empty_cache()


@pytest.mark.parametrize("variant", ["default", "kv_int8", "w8a8", "unfused"])
def test_llama3_8b_widths_batch1_decode_vs_oracle(g, bench, variant):
    """The Llama-3-8B widths at batch 1 (two layers; max_seq 512 so that the D = 128 short attention covers the cache):
    the shared-launch decode step at hidden 4096 / ffn 14336 / vocab 128256 -- four 1024-element chunks per lane in the
    projection roles, fourteen in the down projection, 16 k candidate words in the lm_head launch -- and the same model
    with the int8 KV cache, with int8 activations and as one op per launch, each against the oracle with the same
    options, 12 steps."""
    import torch

    dt = orc.F16
    cfg = dict(LLAMA3_WIDTHS, dtype=dt, max_seq=512)
    weights = bench.make_weights(cfg, dt, 777)
    torch.cuda.synchronize()
    host = bench.to_host_weights(weights)
    kw = dict(default={}, kv_int8=dict(quant_kv_cache=True), w8a8=dict(quantize_activations=True), unfused=dict(unfused_decode=True))[variant]
    dec = g.mynn.Decoder(cfg, weights, **kw)
    L = cfg["n_layers"]
    want_launches = dict(default=3 * L + 1, kv_int8=3 * L + 1, w8a8=5 * L + 3, unfused=5 * L + 3)[variant]
    assert dec.stats()["graph"] and dec.stats()["launches_per_step"] == want_launches, dec.stats()
    ref = orc.Model(dict(cfg), host)
    ref.set_options(quant_kv_cache=variant == "kv_int8", quantize_activations=variant == "w8a8")
    tol = 2e-2 if variant in ("kv_int8", "w8a8") else 1e-2
    tok = 12345
    for step in range(12):
        want = ref.forward([tok], [step], step, step + 1, False)
        nxt, got = dec.step([tok], [step], step, step + 1, want_logits=True)
        assert max_err_rel_to_max(g.f32(got, dt), g.f32(want, dt)) <= tol, step
        assert nxt[0] == orc.argmax_last(got[0], dt), step
        tok = int(nxt[0])
    # the device-resident loop continues the same stream
    more = dec.decode_loop(tok, 12, 4)
    assert len(more) == 4
    dec.close()
    del weights
    torch.cuda.empty_cache()


def test_config4_streaming_decode_attention_at_batch32_context_2048(g):
    """The attention of configs[4] at the benchmarked size: 32 sequences, 32 / 8 heads of 128 dims, 2048 cached
    keys of a 2304-row cache, fp16 and int8 caches, against the oracle and f64."""
    import torch

    dt = orc.F16
    B, Hq, Hkv, D, L, active = 32, 32, 8, 128, 2304, 2048
    rng = np.random.default_rng(2048)
    q = orc.to_storage(rng.standard_normal((B, Hq, 1, D)), dt)
    k = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
    v = orc.to_storage(rng.standard_normal((B, Hkv, L, D)), dt)
    want = orc.attention(q, k, v, dt, D ** -0.5, False, active)
    exact = orc.attention_f64(q, k, v, dt, D ** -0.5, False, active)
    d_active = torch.tensor([active], dtype=torch.int32, device="cuda")
    got = g.to_host(g.mynn.attention(g.to_dev(q, dt), g.to_dev(k, dt), g.to_dev(v, dt), D ** -0.5, False, active=L, d_active=d_active))
    from conftest import max_abs_rel

    assert max_abs_rel(g.f32(got, dt), g.f32(want, dt)) <= 1e-2
    assert max_abs_rel(g.f32(got, dt), exact) <= 1e-2
