"""End-to-end parity of the decoder executor (model_init / model / LlmSession) against the
oracle and the reference's own known answer on its tiny random Llama."""
import numpy as np
import pytest

import oracle as orc
import llm_weights
from conftest import max_abs_rel, max_err_rel_to_max

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def g():
    import gpu_util

    return gpu_util


def dev_weights(g, w, dt):
    out = {}
    for k, v in w.items():
        out[k] = (g.to_dev(v[0]), g.to_dev(v[1], dt)) if isinstance(v, tuple) else g.to_dev(v, dt)
    return out


SMALL = dict(n_layers=3, hidden=256, n_heads=8, n_kv_heads=2, head_dim=32, ffn=704, vocab=1000, max_seq=96,
             eps=1e-5, rope_theta=10000.0)


@pytest.mark.parametrize("dt", [orc.BF16, orc.F16])
def test_tiny_llama_random_golden_ids_on_gpu(g, dt):
    """crates/llm/tests/tinyllama_random.rs:20-24: prompt "Hello" -> 8 exact ids (un-quantised
    checkpoint, narrowed to the 16-bit type)."""
    cfg, w, golden = llm_weights.tiny_llama_random(dt)
    dec = g.mynn.Decoder(cfg, dev_weights(g, w, dt))
    llm = g.mynn.LlmSession(dec, eos=1)
    ids = llm.generate_ids(golden["prompt_ids"], len(golden["expected_new_ids"]))
    assert ids == golden["expected_new_ids"]
    assert llm.past_len == len(golden["prompt_ids"]) + len(ids) - 1
    llm.close(), dec.close()


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
def test_int8_decoder_step_logits_and_kv_vs_oracle(g, dt):
    cfg, w = llm_weights.synthetic_int8(SMALL, dt, seed=7)
    ref = orc.Model(cfg, w)
    dec = g.mynn.Decoder(cfg, dev_weights(g, w, dt), reference_abi=True)  # mynn_model_configure + model_init
    st = dec.stats()
    assert st["graph"], "the decode step must replay a captured hipGraph"
    assert st["launches_per_step"] <= 2 + 6 * cfg["n_layers"] + 3
    toks = [5, 999, 123, 0, 77]
    for i, t in enumerate(toks):
        want = ref.forward([t], [i], i, i + 1, False)
        nxt, got = dec.step([t], [i], i, i + 1, want_logits=True)
        assert max_err_rel_to_max(g.f32(got, dt), g.f32(want, dt)) <= 1e-2, i
        assert nxt[0] == orc.argmax_last(got[0], dt)
    # KV rows written by the fused RoPE + append kernel
    for l in range(cfg["n_layers"]):
        k_ref, v_ref = ref.kv_cache(l)
        k_gpu, v_gpu = g.to_host(dec.kv[l][0])[0], g.to_host(dec.kv[l][1])[0]
        n = len(toks)
        assert max_err_rel_to_max(g.f32(k_gpu[:, :n], dt), g.f32(k_ref[:, :n], dt)) <= 1e-2
        assert max_err_rel_to_max(g.f32(v_gpu[:, :n], dt), g.f32(v_ref[:, :n], dt)) <= 1e-2
        assert not k_gpu[:, n:].any() and not v_gpu[:, n:].any()
    # the reference ABI entry point returns the same logits
    l2 = dec.model([3], [5], 5, 6)
    _, l3 = dec.step([3], [5], 5, 6, want_logits=True)
    assert np.array_equal(l2, l3)
    dec.close()


SHORT_CACHE = {
    64: dict(SMALL, n_layers=2, hidden=256, n_heads=4, n_kv_heads=2, head_dim=64, max_seq=512),
    128: dict(SMALL, n_layers=2, hidden=256, n_heads=2, n_kv_heads=1, head_dim=128, max_seq=256),
}
# the same form walks a longer cache in rounds of 512 / 256 rows (up to four)
LONGER_CACHE = {
    64: dict(SHORT_CACHE[64], max_seq=1300),
    128: dict(SHORT_CACHE[128], max_seq=1024),
}


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("rounds", [1, 4], ids=["one_round", "several_rounds"])
def test_decode_attention_short_cache_every_pass_vs_oracle(g, dt, D, rounds):
    """Head dims 64 and 128 with a cache one workgroup covers (512 / 256 rows a round, up to four rounds): the
    decode step's attention keeps a round's keys in registers, a lane group per key and pass.  Token by token
    through most of the cache, so that every round, pass and wave gets keys, and the rows the kernel appends,
    against the oracle."""
    cfg, w = llm_weights.synthetic_int8((SHORT_CACHE if rounds == 1 else LONGER_CACHE)[D], dt, seed=13 + D)
    ref = orc.Model(cfg, w)
    dec = g.mynn.Decoder(cfg, dev_weights(g, w, dt))
    n = cfg["max_seq"] - 5
    toks = np.random.default_rng(D).integers(0, cfg["vocab"], n)
    for i, t in enumerate(toks):
        want = ref.forward([t], [i], i, i + 1, False)
        if i % 37 == 0 or i >= n - 3:
            nxt, got = dec.step([t], [i], i, i + 1, want_logits=True)
            assert max_err_rel_to_max(g.f32(got, dt), g.f32(want, dt)) <= 1e-2, i
            assert nxt[0] == orc.argmax_last(got[0], dt)
        else:
            dec.step([t], [i], i, i + 1)
    for l in range(cfg["n_layers"]):
        k_ref, v_ref = ref.kv_cache(l)
        k_gpu, v_gpu = g.to_host(dec.kv[l][0])[0], g.to_host(dec.kv[l][1])[0]
        assert max_err_rel_to_max(g.f32(k_gpu[:, :n], dt), g.f32(k_ref[:, :n], dt)) <= 1e-2
        assert max_err_rel_to_max(g.f32(v_gpu[:, :n], dt), g.f32(v_ref[:, :n], dt)) <= 1e-2
        assert not k_gpu[:, n:].any() and not v_gpu[:, n:].any()
    dec.close()


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
def test_int8_greedy_tokens_vs_oracle_small(g, dt):
    """Greedy ids of the HIP path against the oracle on a small int8 model.  The oracle is
    teacher-forced with the GPU's tokens and runs under several f32 summation orders; a step where
    the GPU's token is not the first order's choice must be one where the oracle's own arithmetic
    does not separate the two tokens (oracle.SummationOrders.judge; the reference leaves the order
    of its sums open)."""
    cfg, w = llm_weights.synthetic_int8(SMALL, dt, seed=11)
    rng = np.random.default_rng(5)
    prompt = rng.integers(0, cfg["vocab"], 24).tolist()
    dec = g.mynn.Decoder(cfg, dev_weights(g, w, dt))
    got, want, undecided, different = g.greedy_compare(cfg, w, dec, prompt, 48, dt)
    assert not different, different
    assert len(undecided) <= 4, undecided
    # LlmSession drives the same steps; the device-resident decode loop repeats them
    llm = g.mynn.LlmSession(dec)
    assert llm.generate_ids(prompt, 48) == got
    assert llm.past_len == len(prompt) + 48 - 1
    first = None
    for i, t in enumerate(prompt):
        first, _ = dec.step([t], [i], i, i + 1)
    loop = dec.decode_loop(first[0], len(prompt), 47)
    assert [first[0]] + loop == got
    llm.close(), dec.close()


def test_generate_bookkeeping_and_errors(g):
    dt = orc.F16
    cfg, w = llm_weights.synthetic_int8(dict(SMALL, max_seq=16), dt, seed=3)
    dec = g.mynn.Decoder(cfg, dev_weights(g, w, dt))
    llm = g.mynn.LlmSession(dec)
    with pytest.raises(g.mynn.MynnError):  # PromptTooLong
        llm.generate_ids(list(range(17)), 1)
    assert llm.generate_ids([], 4) == []
    ids = llm.generate_ids([1, 2, 3, 4, 5], 100)  # stops when the cache is full
    assert llm.past_len == 16 and len(ids) == 12
    llm.reset()
    assert llm.past_len == 0
    with pytest.raises(g.mynn.MynnError):
        dec.step([cfg["vocab"]], [0], 0, 1)  # token outside the vocabulary
    with pytest.raises(g.mynn.MynnError):
        dec.step([1], [16], 0, 1)  # position outside the RoPE table
    llm.close(), dec.close()


@pytest.mark.parametrize("shape", ["generic_head_dim_32", "single_launch_layer"])
def test_generate_runs_of_steps_on_the_device_equal_step_by_step(g, shape):
    """LlmSession.generate_ids serves decode steps in runs of the executor's device-resident loop.  Ids, the stop at
    the end-of-sequence id in the middle of a run, past_len and a following turn (which overwrites the rows the run
    computed past the stop) are those of feeding one token per call (session.rs:508-537, 612-640)."""
    dt = orc.F16
    cfg, w = llm_weights.synthetic_int8(SMALL if shape == "generic_head_dim_32" else SHORT_CACHE[64], dt, seed=13)
    dw = dev_weights(g, w, dt)
    prompt = [7, 8, 9, 10, 11]

    def by_steps(dec, past, feed, n_new, eos):
        out, nxt = [], None
        for t in feed:
            nxt, _ = dec.step([t], [past], past, past + 1)
            past += 1
        out.append(nxt[0])
        while len(out) < n_new and out[-1] != eos:
            nxt, _ = dec.step([out[-1]], [past], past, past + 1)
            past += 1
            out.append(nxt[0])
        return out, past

    dec, ref = g.mynn.Decoder(cfg, dw), g.mynn.Decoder(cfg, dw)
    free, _ = by_steps(ref, 0, prompt, 60, -1)
    llm = g.mynn.LlmSession(dec, eos=-1)
    assert llm.generate_ids(prompt, 60) == free and llm.past_len == len(prompt) + 59
    llm.close()
    # an end-of-sequence id that first shows up inside a run
    j0 = next(j for j in range(10, 60) if free[j] not in free[:j])
    eos = free[j0]
    llm = g.mynn.LlmSession(dec, eos=eos)
    assert llm.generate_ids(prompt, 60) == free[:j0 + 1]
    assert llm.past_len == len(prompt) + j0
    want2, past2 = by_steps(ref, len(prompt) + j0, [3, 4], 12, eos)
    assert llm.generate_ids([3, 4], 12) == want2 and llm.past_len == past2
    llm.close(), dec.close(), ref.close()


@pytest.fixture(params=[0, 1, 2, 3, 4], ids=["tile_auto", "tile_256x128", "tile_256x256", "tile_256x256_direct_lds", "tile_256x320_direct_lds"])
def gemm_tile(request):
    return request.param


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("P", [4, 32])
def test_prefill_model_logits_and_kv_vs_oracle(g, dt, P, gemm_tile):
    """Mode::Prefill{len}: one graph run over P tokens writes P cache rows and returns [P, vocab]
    logits; rows < 16 take the scale-after-sum kernels, rows >= 16 the matrix cores, exactly as
    the reference dispatches (src/codegen/cuda.rs:1518-1652)."""
    cfg, w = llm_weights.synthetic_int8(SMALL, dt, seed=21)
    ref = orc.Model(cfg, w)
    ref.set_gemm_mode(2)  # the CUDA backend's kernel choice, which the HIP path reproduces
    dec = g.mynn.Decoder(cfg, dev_weights(g, w, dt), seq_q=P, gemm_tile=gemm_tile)
    rng = np.random.default_rng(P)
    past = 0
    for chunk in range(2):
        ids = rng.integers(0, cfg["vocab"], P)
        pos = np.arange(past, past + P)
        want = ref.forward(ids, pos, past, past + P, True)
        nxt, got = dec.step(ids, pos, past, past + P, want_logits=True)
        assert max_err_rel_to_max(g.f32(got, dt), g.f32(want, dt)) <= 1e-2, chunk
        assert nxt[0] == orc.argmax_last(got[-1], dt)
        past += P
    for l in range(cfg["n_layers"]):
        k_ref, v_ref = ref.kv_cache(l)
        k_gpu, v_gpu = g.to_host(dec.kv[l][0])[0], g.to_host(dec.kv[l][1])[0]
        assert max_err_rel_to_max(g.f32(k_gpu[:, :past], dt), g.f32(k_ref[:, :past], dt)) <= 1e-2
        assert max_err_rel_to_max(g.f32(v_gpu[:, :past], dt), g.f32(v_ref[:, :past], dt)) <= 1e-2
    dec.close()


@pytest.mark.parametrize("dt", [orc.F16])
def test_prefill_then_decode_shares_kv_and_matches_decode_only(g, dt):
    """crates/llm/tests/tinyllama_random.rs cpu_multi_turn_prefill_matches_decode_only on the GPU:
    a prefill session and a decode session over the same weights and KV buffers (PersistentBuffers);
    chunked zero-padded prefill then greedy decode gives the ids of feeding the prompt token by token
    (up to ties at 16-bit resolution, checked against the oracle's logits)."""
    cfg, w = llm_weights.synthetic_int8(SMALL, dt, seed=31)
    dw = dev_weights(g, w, dt)
    dec = g.mynn.Decoder(cfg, dw)
    pre = g.mynn.Decoder(cfg, dw, seq_q=16, kv=dec.kv)
    rng = np.random.default_rng(9)
    prompt = rng.integers(0, cfg["vocab"], 37).tolist()  # 2 full chunks + a padded one
    a = g.mynn.LlmSession(dec, prefill=pre)
    ids_prefill = a.generate_ids(prompt, 20)
    assert a.past_len == len(prompt) + 20 - 1
    a.close()
    dec2 = g.mynn.Decoder(cfg, dw)
    b = g.mynn.LlmSession(dec2)
    ids_decode = b.generate_ids(prompt, 20)
    # the two paths use different kernels for the prompt (GEMM vs GEMV numerics), so compare
    # through the oracle when they part
    if ids_prefill != ids_decode:
        first = next(i for i in range(20) if ids_prefill[i] != ids_decode[i])
        ok, verdicts = g.both_acceptable(cfg, w, prompt + ids_decode[:first], [ids_prefill[first], ids_decode[first]], dt)
        assert ok, (first, verdicts)
    with pytest.raises(g.mynn.MynnError):  # padded prompt does not fit: PromptTooLong
        c = g.mynn.LlmSession(dec2, prefill=pre)
        c.generate_ids(list(range(100)), 1)
    b.close(), dec.close(), pre.close(), dec2.close()


SMALL_D64 = dict(SMALL, n_heads=4, n_kv_heads=2, head_dim=64)


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("shape", ["d32", "d64"])
@pytest.mark.parametrize("kv8,w8a8", [(True, False), (False, True), (True, True)])
def test_int8_kv_cache_and_w8a8_executor_vs_oracle(g, dt, kv8, w8a8, shape):
    """BuildOptions::quant_kv_cache (int8 caches + per-token scales, QuantizingKVCacheUpdate, attention
    scale slots; crates/llm/src/decoder.rs:405-470) and Options::quantize_activations
    (DynamicQuantizeLinear + QuantizedMatMul for every int8 linear; quantize_activations.rs) in the
    executor: a 16-token prefill chunk, then decode steps over the same caches, against the oracle
    with the same options."""
    cfg, w = llm_weights.synthetic_int8(SMALL if shape == "d32" else SMALL_D64, dt, seed=41)
    ref = orc.Model(cfg, w)
    ref.set_options(quant_kv_cache=kv8, quantize_activations=w8a8)
    ref.set_gemm_mode(2)
    dw = dev_weights(g, w, dt)
    dec = g.mynn.Decoder(cfg, dw, quant_kv_cache=kv8, quantize_activations=w8a8)
    # batch-1 decode: a linear with its norm (quantiser) and store is one launch (qkv, o, gate/up, down); the attention
    # block is one more (RoPE, append -- quantising for an int8 cache at head_dim 64 / 128 -- and attention) or, for an
    # int8 cache at head_dim 32, two; embedding, lm_head, greedy token
    nl = cfg["n_layers"]
    if not w8a8:  # (int8 cache, 16-bit activations: the layer's attention block is one launch as with a 16-bit cache)
        want_launches = 6 * nl + 3 if shape == "d32" else 3 * nl + 1
    else:
        want_launches = (6 if kv8 and shape == "d32" else 5) * nl + 3
    assert dec.stats()["launches_per_step"] == want_launches, dec.stats()
    pre = g.mynn.Decoder(cfg, dw, seq_q=16, kv=dec.kv, quant_kv_cache=kv8, quantize_activations=w8a8)
    rng = np.random.default_rng(3)
    ids = rng.integers(0, cfg["vocab"], 16)
    want = ref.forward(ids, np.arange(16), 0, 16, True)
    _, got = pre.step(ids, np.arange(16), 0, 16, want_logits=True)
    # (int8 activations at the wider heads: measured up to 2.7e-2 in the prefill chunk and 2.2e-2 in the decode steps,
    # the latter the same to the last bit whether a linear is one launch or four -- an activation's code that lands on
    # the other side of a rounding moves every output of the row)
    tol = 3e-2 if w8a8 and shape == "d64" else 2e-2
    assert max_err_rel_to_max(g.f32(got, dt), g.f32(want, dt)) <= tol
    past = 16
    for t in [7, 500, 31, 999, 2, 640]:
        want = ref.forward([t], [past], past, past + 1, False)
        nxt, got = dec.step([t], [past], past, past + 1, want_logits=True)
        assert max_err_rel_to_max(g.f32(got, dt), g.f32(want, dt)) <= tol, past
        assert nxt[0] == orc.argmax_last(got[0], dt)
        past += 1
    if kv8:
        for l in range(cfg["n_layers"]):
            k_ref, v_ref = ref.kv_cache(l)
            ks_ref, vs_ref = ref.kv_scales(l)
            k_gpu, v_gpu, ks_gpu, vs_gpu = [g.to_host(t)[0] for t in dec.kv[l]]
            assert k_gpu.dtype == np.int8 and not k_gpu[:, past:].any() and not v_gpu[:, past:].any()
            # the projections differ in summation order by a spacing of T here and there; when that hits
            # the row's amax every code of the row moves by up to 127 * 2^-8 (bf16), plus its own rounding
            assert np.abs(k_gpu[:, :past].astype(int) - k_ref[:, :past].astype(int)).max() <= 2
            assert np.abs(v_gpu[:, :past].astype(int) - v_ref[:, :past].astype(int)).max() <= 2
            assert np.mean(k_gpu[:, :past] == k_ref[:, :past]) > 0.85
            # a scale is amax/127 rounded to T: amax one spacing of T apart, then one more rounding
            assert max_abs_rel(g.f32(ks_gpu[:, :past], dt), g.f32(ks_ref[:, :past], dt)) <= 2e-2
            assert max_abs_rel(g.f32(vs_gpu[:, :past], dt), g.f32(vs_ref[:, :past], dt)) <= 2e-2
    pre.close(), dec.close()


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
def test_w8a8_batch1_one_launch_per_linear_vs_one_op_per_launch(g, dt):
    """Options::quantize_activations at batch 1: the executor's default (a linear with its norm, quantiser and store in
    one launch) against unfused_decode (RMSNorm, DynamicQuantizeLinear, QuantizedMatMul, Add / SwiGLU as launches of
    their own) and against the oracle.  The two forms sum the squares of a row in different orders, so a normalised
    value may differ by a spacing of T and with it an int8 code: they agree within the path's quantisation noise, not
    bit for bit."""
    cfg, w = llm_weights.synthetic_int8(SMALL, dt, seed=43)
    ref = orc.Model(cfg, w)
    ref.set_options(quant_kv_cache=False, quantize_activations=True)
    dw = dev_weights(g, w, dt)
    a = g.mynn.Decoder(cfg, dw, quantize_activations=True)
    b = g.mynn.Decoder(cfg, dw, quantize_activations=True, unfused_decode=True)
    assert a.stats()["launches_per_step"] == 5 * cfg["n_layers"] + 3
    assert b.stats()["launches_per_step"] > 3 * a.stats()["launches_per_step"] - 10
    for i, t in enumerate([11, 402, 77, 3, 950, 640, 12, 8]):
        want = ref.forward([t], [i], i, i + 1, False)
        na, la = a.step([t], [i], i, i + 1, want_logits=True)
        nb, lb = b.step([t], [i], i, i + 1, want_logits=True)
        assert max_err_rel_to_max(g.f32(la, dt), g.f32(want, dt)) <= 2e-2, i
        assert max_err_rel_to_max(g.f32(lb, dt), g.f32(want, dt)) <= 2e-2, i
        assert max_err_rel_to_max(g.f32(la, dt), g.f32(lb, dt)) <= 2e-2, i
        assert na[0] == orc.argmax_last(la[0], dt) and nb[0] == orc.argmax_last(lb[0], dt)
    a.close(), b.close()


W8A8_LARGE = dict(n_layers=1, hidden=2048, n_heads=16, n_kv_heads=4, head_dim=128, ffn=1024, vocab=2048, max_seq=1024,
                  eps=1e-5, rope_theta=10000.0)


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
def test_w8a8_prefill_large_int8_tiles_vs_oracle(g, dt):
    """Options::quantize_activations at a prefill size where every linear fills the 256-row int8 tiles
    (4 x 1024 rows; widths 2048..3072): RMSNorm + per-row quantisation in one launch, residual adds and
    SwiGLU on the product's store, gate/up as one interleaved product.  Logits of sampled rows and the
    first rows of the KV cache against the oracle with the same option."""
    cfg, w = llm_weights.synthetic_int8(W8A8_LARGE, dt, seed=5)
    B, S = 4, 1024
    dw = dev_weights(g, w, dt)
    pre = g.mynn.Decoder(cfg, dw, seq_q=S, batch=B, quantize_activations=True)
    rng = np.random.default_rng(17)
    ids = rng.integers(0, cfg["vocab"], B * S)
    _, got = pre.step(ids, np.arange(S), 0, S, want_logits=True)
    got = got.reshape(B, S, -1)
    ref = orc.Model(cfg, w)
    ref.set_options(quant_kv_cache=False, quantize_activations=True)
    ref.set_gemm_mode(2)
    n = 96  # causal: the first rows of a prompt do not depend on the rest
    for b in (0, 3):
        want = ref.forward(ids[b * S:b * S + n], np.arange(n), 0, n, True)
        gf, wf = g.f32(got[b, :n], dt), g.f32(want, dt)
        assert np.array_equal(got[b, 0], want[0])  # one key: attention returns V itself, the rest is exact
        # later rows: the attention kernels sum in another order, and where that moves an activation across a
        # rounding boundary of its row's int8 grid the value jumps by 1/127 of the row maximum (the whole W8A8
        # path differs from the 16-bit-activation one by 2.4e-2 on this model)
        assert max_err_rel_to_max(gf, wf) <= 4e-2, b
        assert float(np.mean(np.abs(gf - wf))) <= 1e-2 * float(np.max(np.abs(wf))), b
        k_ref, v_ref = ref.kv_cache(0)
        k_gpu, v_gpu = [g.to_host(t)[b] for t in pre.kv[0]]
        assert max_err_rel_to_max(g.f32(k_gpu[:, :n], dt), g.f32(k_ref[:, :n], dt)) <= 2e-2
        assert max_err_rel_to_max(g.f32(v_gpu[:, :n], dt), g.f32(v_ref[:, :n], dt)) <= 2e-2
    names = [k[0] for k in pre.profile(ids, np.arange(S), 0, S)]
    assert "qlinear_gateup_swiglu" in names and "rms_norm_quantize" in names and "add" not in names
    pre.close()


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
def test_w8a8_large_int8_tiles_rows_bit_exact(g, dt):
    """The same executor path on 4096 one-token sequences: attention over a single key returns V itself, so
    every operator of the layer is the oracle's arithmetic in the oracle's order (integer sums are exact,
    every float step is a single rounded operation) and whole rows of logits must match bit for bit --
    sampled from every part of the 256-row tiles."""
    cfg, w = llm_weights.synthetic_int8(dict(W8A8_LARGE, max_seq=4), dt, seed=6)
    B = 4096
    dw = dev_weights(g, w, dt)
    dec = g.mynn.Decoder(cfg, dw, seq_q=1, batch=B, quantize_activations=True)
    rng = np.random.default_rng(23)
    ids = rng.integers(0, cfg["vocab"], B)
    nxt, got = dec.step(ids, [0], 0, 1, want_logits=True)
    got = got.reshape(B, -1)
    assert "qlinear_down_residual" in [k[0] for k in dec.profile(ids, [0], 0, 1)]
    ref = orc.Model(cfg, w)
    ref.set_options(quant_kv_cache=False, quantize_activations=True)
    for r in [0, 1, 31, 32, 63, 127, 128, 255, 256, 1000, 2047, 2048, 4000, 4095]:
        want = ref.forward([ids[r]], [0], 0, 1, False)[0]
        assert np.array_equal(got[r], want), r
        assert nxt[r] == orc.argmax_last(want, dt)
    dec.close()


FEWROWS = dict(SMALL, ffn=768)  # every K a multiple of 128: 16..64 rows take the few-row int8 GEMM


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("rows", [16, 32, 48])
@pytest.mark.parametrize("hidden", [256, 1536])
def test_few_row_gemm_prefill_chunk_vs_oracle(g, dt, rows, hidden):
    """16 <= rows <= 64: linears stream the int8 weights once through the few-row matrix-core kernel
    (scale after the sum, K split over workgroups, residual / SwiGLU in the reducing launch).  With the
    longer rows (hidden 1536) the q|k|v projection's K range is split too, and the launch that sums it
    applies RoPE and appends to the caches."""
    shape = FEWROWS if hidden == 256 else dict(FEWROWS, hidden=1536, n_heads=48, n_kv_heads=12, n_layers=2)
    cfg, w = llm_weights.synthetic_int8(shape, dt, seed=51)
    ref = orc.Model(cfg, w)
    dec = g.mynn.Decoder(cfg, dev_weights(g, w, dt), seq_q=rows)
    names = [n for n, _, _, _ in dec.profile(np.zeros(rows, np.int64), np.arange(rows), 0, rows)]
    assert "linear_gateup_swiglu" in names and "swiglu" not in names
    assert ("rope_kv_append" in names) == (hidden == 256)
    # every RMSNorm but the first rides on the launch that finishes its input (o / down projection + residual)
    assert names.count("rms_norm") == 1
    rng = np.random.default_rng(rows)
    past = 0
    for chunk in range(2):
        ids = rng.integers(0, cfg["vocab"], rows)
        pos = np.arange(past, past + rows)
        want = ref.forward(ids, pos, past, past + rows, True)
        _, got = dec.step(ids, pos, past, past + rows, want_logits=True)
        assert max_err_rel_to_max(g.f32(got, dt), g.f32(want, dt)) <= 1e-2, chunk
        past += rows
    dec.close()


WIDE = dict(SMALL, n_layers=1, ffn=12288, vocab=24576)  # gate/up and lm_head wide enough to skip the K split


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("rows", [32, 48])
def test_few_row_gemm_unsplit_store_vs_oracle(g, dt, rows):
    """Few-row int8 GEMM on matrices of >= 24576 rows: one launch per linear that applies the scale (and
    SwiGLU) itself instead of writing partial sums for a second one."""
    cfg, w = llm_weights.synthetic_int8(WIDE, dt, seed=77)
    dw = dev_weights(g, w, dt)
    pre = g.mynn.Decoder(cfg, dw, seq_q=rows)
    ids = np.random.default_rng(rows).integers(0, cfg["vocab"], rows)
    names = [k[0] for k in pre.profile(ids, np.arange(rows), 0, rows)]
    assert "linear_gateup_swiglu" in names
    ref = orc.Model(cfg, w)
    want = ref.forward(ids, np.arange(rows), 0, rows, True)
    _, got = pre.step(ids, np.arange(rows), 0, rows, want_logits=True)
    assert max_err_rel_to_max(g.f32(got, dt), g.f32(want, dt)) <= 1e-2
    pre.close()


@pytest.mark.parametrize("dt", [orc.F16])
def test_batched_decode_equals_independent_sequences(g, dt):
    """Batch 16 decode (the shape of the batched-serving config, scaled down): every sequence must follow
    its own batch-1 oracle, sharing nothing but the weights."""
    B = 16
    cfg, w = llm_weights.synthetic_int8(FEWROWS, dt, seed=61)
    dec = g.mynn.Decoder(cfg, dev_weights(g, w, dt), batch=B)
    refs = [orc.Model(cfg, w) for _ in range(B)]
    rng = np.random.default_rng(4)
    for step in range(5):
        toks = rng.integers(0, cfg["vocab"], B)
        nxt, got = dec.step(toks, [step], step, step + 1, want_logits=True)
        for b in range(B):
            want = refs[b].forward([toks[b]], [step], step, step + 1, False)
            assert max_err_rel_to_max(g.f32(got[b:b + 1], dt), g.f32(want, dt)) <= 1e-2, (step, b)
            assert nxt[b] == orc.argmax_last(got[b], dt)
    dec.close()


def test_full_size_tinyllama_shape_greedy_tokens_match_oracle(g):
    """The benchmark's own model (TinyLlama-1.1B shape, int8, fp16 activations, seed 1234, GPU-generated
    weights): a 16-token prompt and 24 greedy tokens through the captured decode step, against the oracle
    on the same weights under three summation orders, teacher-forced with the GPU's tokens; a disagreement must
    be one the oracle's own orders disagree on."""
    import os
    import sys
    import torch

    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import bench

    dt = orc.F16
    cfg = dict(bench.TINYLLAMA, dtype=dt, max_seq=64)
    weights = bench.make_weights(cfg, dt, 1234)
    torch.cuda.synchronize()
    dec = g.mynn.Decoder(cfg, weights)
    assert dec.stats()["graph"] and dec.stats()["launches_per_step"] == 67
    prompt = np.random.default_rng(1234).integers(0, cfg["vocab"], 16).tolist()
    gpu_ids, ref_ids, undecided, different = g.greedy_compare(dict(cfg), bench.to_host_weights(weights), dec, prompt, 24, dt)
    assert not different, different
    assert sum(a == b for a, b in zip(gpu_ids, ref_ids)) >= 22
    dec.close()


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("kv8", [False, True], ids=["kv16", "kv_int8"])
def test_batched_decode_rope_and_append_in_the_reduce_launch_vs_separate_launches(g, dt, D, kv8):
    """16 sequences: the launch that sums the q|k|v projection's K ranges also rotates q and k and appends k and v (an
    int8 cache: quantises them) -- logits, cache rows and scales are those of the executor that keeps these as launches
    of their own (unfused_decode), bit for bit, and the logits follow the per-sequence oracles."""
    B = 16
    # (hidden 1536: the projection's K range is split, so there is a launch that sums the ranges)
    shape = dict(FEWROWS, n_layers=2, hidden=1536, n_heads=1536 // D, n_kv_heads=768 // D, head_dim=D)
    cfg, w = llm_weights.synthetic_int8(shape, dt, seed=77)
    dw = dev_weights(g, w, dt)
    a = g.mynn.Decoder(cfg, dw, batch=B, quant_kv_cache=kv8)
    b = g.mynn.Decoder(cfg, dw, batch=B, quant_kv_cache=kv8, unfused_decode=True)
    assert a.stats()["launches_per_step"] < b.stats()["launches_per_step"]
    refs = [orc.Model(cfg, w) for _ in range(3)]
    for r in refs:
        r.set_options(quant_kv_cache=kv8)
    rng = np.random.default_rng(8)
    for step in range(6):
        toks = rng.integers(0, cfg["vocab"], B)
        na, la = a.step(toks, [step], step, step + 1, want_logits=True)
        nb, lb = b.step(toks, [step], step, step + 1, want_logits=True)
        assert np.array_equal(la, lb) and na == nb, step
        for i, r in enumerate(refs):
            want = r.forward([toks[i]], [step], step, step + 1, False)
            assert max_err_rel_to_max(g.f32(la[i:i + 1], dt), g.f32(want, dt)) <= 2e-2 if kv8 else 1e-2, (step, i)
    for l in range(cfg["n_layers"]):
        for j in range(len(a.kv[l])):
            assert np.array_equal(g.to_host(a.kv[l][j]), g.to_host(b.kv[l][j])), (l, j)
    a.close(), b.close()
