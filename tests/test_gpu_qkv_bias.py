"""q / k / v projection bias (model_type "qwen2", crates/llm/src/decoder.rs:167-184, 542-600) through the executors,
against the oracle with the same biases.  The reference holds no fixture for this path; the oracle's bias handling is
pinned by tests/test_oracle_decoder.py against an independent float64 decoder."""
import json
import os
import struct

import numpy as np
import pytest

import oracle as orc
import llm_weights
from conftest import max_err_rel_to_max
from test_gpu_decoder import FEWROWS, SMALL, SMALL_D64, dev_weights

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def g():
    import gpu_util

    return gpu_util


def biased(cfg_shape, dt, seed):
    cfg, w = llm_weights.synthetic_int8(cfg_shape, dt, seed=seed)
    return cfg, llm_weights.add_qkv_bias(cfg, w, dt, seed=seed + 1, std=0.05)


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("shape", ["d32", "d64"])
@pytest.mark.parametrize("opts", [dict(), dict(unfused_decode=True), dict(quant_kv_cache=True), dict(quantize_activations=True)],
                         ids=["default", "unfused", "kv_int8", "w8a8"])
def test_biased_batch1_decode_vs_oracle(g, dt, shape, opts):
    cfg, w = biased(SMALL if shape == "d32" else SMALL_D64, dt, 41)
    ref = orc.Model(cfg, w)
    ref.set_options(quant_kv_cache=opts.get("quant_kv_cache", False), quantize_activations=opts.get("quantize_activations", False))
    plain = orc.Model(cfg, {k: v for k, v in w.items() if not k.endswith(".bias")})
    dec = g.mynn.Decoder(cfg, dev_weights(g, w, dt), **opts)
    assert dec.stats()["graph"]
    tol = 3e-2 if opts.get("quantize_activations") else 1e-2
    rng = np.random.default_rng(6)
    moved = 0.0
    for i, t in enumerate(rng.integers(0, cfg["vocab"], 10)):
        want = ref.forward([t], [i], i, i + 1, False)
        nxt, got = dec.step([t], [i], i, i + 1, want_logits=True)
        assert max_err_rel_to_max(g.f32(got, dt), g.f32(want, dt)) <= tol, i
        assert nxt[0] == orc.argmax_last(got[0], dt)
        if not opts:
            base = plain.forward([t], [i], i, i + 1, False)
            moved = max(moved, max_err_rel_to_max(g.f32(want, dt), g.f32(base, dt)))
    if not opts:  # the biases matter: without them the logits are far outside the bound
        assert moved > 0.1, moved
    out = dec.decode_loop(3, 10, 12)
    t, again = 3, []
    for i in range(12):
        nxt, _ = dec.step([t], [10 + i], 10 + i, 11 + i)
        again.append(nxt[0])
        t = nxt[0]
    assert out == again
    dec.close()


@pytest.mark.parametrize("dt", [orc.F16, orc.BF16])
@pytest.mark.parametrize("rows,batch", [(4, 1), (32, 1), (1, 16)], ids=["prefill4", "prefill32", "batch16"])
def test_biased_prefill_and_batched_decode_vs_oracle(g, dt, rows, batch):
    """Prefill chunks (the scale-after-sum kernels below 16 rows, the matrix cores from 16 on) and a batch of 16
    sequences (the few-row int8 GEMM), each followed by the bias Add."""
    cfg, w = biased(FEWROWS, dt, 43)
    dw = dev_weights(g, w, dt)
    if batch == 1:
        ref = orc.Model(cfg, w)
        ref.set_gemm_mode(2)
        dec = g.mynn.Decoder(cfg, dw, seq_q=rows)
        rng = np.random.default_rng(rows)
        past = 0
        for chunk in range(2):
            ids = rng.integers(0, cfg["vocab"], rows)
            pos = np.arange(past, past + rows)
            want = ref.forward(ids, pos, past, past + rows, True)
            _, got = dec.step(ids, pos, past, past + rows, want_logits=True)
            # (bf16, 32 rows, second chunk: 1.04e-2 measured = under three bf16 spacings of the largest logit; the biases move
            # the logits by more than ten times that, see the batch-1 test)
            assert max_err_rel_to_max(g.f32(got, dt), g.f32(want, dt)) <= (1.5e-2 if dt == orc.BF16 else 1e-2), chunk
            past += rows
        for l in range(cfg["n_layers"]):
            k_ref, v_ref = ref.kv_cache(l)
            k_gpu, v_gpu = g.to_host(dec.kv[l][0])[0], g.to_host(dec.kv[l][1])[0]
            assert max_err_rel_to_max(g.f32(k_gpu[:, :past], dt), g.f32(k_ref[:, :past], dt)) <= (1.5e-2 if dt == orc.BF16 else 1e-2)
            assert max_err_rel_to_max(g.f32(v_gpu[:, :past], dt), g.f32(v_ref[:, :past], dt)) <= (1.5e-2 if dt == orc.BF16 else 1e-2)
        dec.close()
        return
    dec = g.mynn.Decoder(cfg, dw, batch=batch)
    refs = [orc.Model(cfg, w) for _ in range(batch)]
    rng = np.random.default_rng(4)
    for step in range(4):
        toks = rng.integers(0, cfg["vocab"], batch)
        nxt, got = dec.step(toks, [step], step, step + 1, want_logits=True)
        for b in range(batch):
            want = refs[b].forward([toks[b]], [step], step, step + 1, False)
            assert max_err_rel_to_max(g.f32(got[b:b + 1], dt), g.f32(want, dt)) <= 1e-2, (step, b)
    dec.close()


def test_zero_bias_changes_no_bit(g):
    dt = orc.F16
    cfg, w = llm_weights.synthetic_int8(SMALL_D64, dt, seed=47)
    wz = dict(w)
    for k, v in llm_weights.add_qkv_bias(cfg, w, dt).items():
        if k.endswith(".bias"):
            wz[k] = np.zeros_like(v)
    a = g.mynn.Decoder(cfg, dev_weights(g, wz, dt))
    b = g.mynn.Decoder(cfg, dev_weights(g, w, dt), unfused_decode=True)
    assert a.cfg.qkv_bias == 1 and b.cfg.qkv_bias == 0
    for i, t in enumerate([5, 17, 900, 3]):
        _, la = a.step([t], [i], i, i + 1, want_logits=True)
        _, lb = b.step([t], [i], i, i + 1, want_logits=True)
        assert np.array_equal(la, lb), i
    a.close(), b.close()


def test_biased_checkpoint_upload_and_plain_weights(g, tmp_path):
    """A 16-bit checkpoint with `{q,k,v}_proj.bias` tensors read by the library's own loader (names of
    ModelSpec::from_hf) gives the logits of the same tensors handed over by hand, and both follow the oracle."""
    dt = orc.BF16
    cfg, w, golden = llm_weights.tiny_llama_random(dt)
    wb = llm_weights.add_qkv_bias(cfg, w, dt, seed=8, std=0.05)
    hdr, blob = {}, b""

    def put(name, arr):
        nonlocal blob
        raw = np.ascontiguousarray(arr).tobytes()
        hdr[name] = {"dtype": "BF16", "shape": list(arr.shape), "data_offsets": [len(blob), len(blob) + len(raw)]}
        blob += raw

    put("model.embed_tokens.weight", wb["embed"])
    put("lm_head.weight", wb["lm_head"])
    put("model.norm.weight", wb["final_norm"])
    for l in range(cfg["n_layers"]):
        p = "model.layers.%d." % l
        for k, nm in llm_weights.LIN.items():
            put(p + nm + ".weight", wb["layers.%d.%s" % (l, k)])
            if k in ("q", "k", "v"):
                put(p + nm + ".bias", wb["layers.%d.%s.bias" % (l, k)])
        put(p + "input_layernorm.weight", wb["layers.%d.norm1" % l])
        put(p + "post_attention_layernorm.weight", wb["layers.%d.norm2" % l])
    h = json.dumps(hdr).encode()
    (tmp_path / "model.safetensors").write_bytes(struct.pack("<Q", len(h)) + h + blob)
    from_file = g.mynn.Decoder(dict(cfg, qkv_bias=True), tmp_path)
    by_hand = g.mynn.Decoder(cfg, dev_weights(g, wb, dt))
    ref = orc.Model(cfg, wb)
    for i, t in enumerate(golden["prompt_ids"] + [7, 29871]):
        _, a = from_file.step([t], [i], i, i + 1, want_logits=True)
        _, b = by_hand.step([t], [i], i, i + 1, want_logits=True)
        assert np.array_equal(a, b), i
        want = ref.forward([t], [i], i, i + 1, False)
        assert max_err_rel_to_max(g.f32(a, dt), g.f32(want, dt)) <= 1e-2, i
    with pytest.raises(g.mynn.MynnError):  # the Llama checkpoint has no bias tensors
        g.mynn.Decoder(dict(cfg, qkv_bias=True), os.path.join(os.path.dirname(__file__), "golden", "tiny-llama-random"))
    from_file.close(), by_hand.close()
