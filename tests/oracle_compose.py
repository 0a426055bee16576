"""One run of the decoder graph composed in numpy from the operator-level functions of the oracle module (each of them
pinned on its own by the reference's fixtures and closed forms), op for op as crates/llm/src/decoder.rs:222-487 builds
it.  Pins the C decoder of the oracle (orc_model_forward and its options): which values are rounded where, which rows
are quantised where, which table row rotates which key."""
import numpy as np

import oracle as orc


def heads(x, S, H, D):
    """[S, H*D] -> [1, H, S, D] (reshape + Transpose[0,2,1,3], decoder.rs:253-275)"""
    return np.ascontiguousarray(x.reshape(S, H, D).transpose(1, 0, 2))[None]


def compose_step(cfg, w, caches, ids, positions, past, active, causal, dt, kv8=False, w8a8=False, ring=None, gemm_mode=-1):
    """caches: per layer [k, v] (+ [k_scale, v_scale] with kv8), updated in place.  ring = (sink, window, ring_start,
    kv_position) runs the streaming graph (decoder.rs:281-347, 472-487).  Returns logits [S, vocab]."""
    H, Hq, Hkv, D = cfg["hidden"], cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    S = len(ids)

    def lin(x, name):
        wq, sc = w[name]
        if w8a8 and wq.shape[1] % 32 == 0:
            # DynamicQuantizeLinear(axis 0, symmetric) + QuantizedMatMul (quantize_activations.rs:63-84, 121-183)
            a8, a_sc = orc.dynquant_i8(np.ascontiguousarray(x).reshape(S, -1), dt)
            return orc.quantized_matmul(a8, a_sc, wq, sc, dt)[0]
        mode = -1
        if gemm_mode == 2:
            mode = 2 if (S >= 16 and wq.shape[1] % 8 == 0 and dt != orc.F32) else 0
        return orc.dequant_matmul(np.ascontiguousarray(x).reshape(S, -1), wq, sc, dt, dt, mode)

    x = orc.gather_rows(orc.dequantize_linear(w["embed"][0], w["embed"][1], dt), ids)
    cos, sin = orc.rope_table(cfg["max_seq"], D, cfg["rope_theta"], dt)
    scale = np.float32(1.0) / np.sqrt(np.float32(D))
    for l in range(cfg["n_layers"]):
        n1 = orc.rms_norm(x, w["layers.%d.norm1" % l], cfg["eps"], dt)
        q = orc.rope(heads(lin(n1, "layers.%d.q" % l), S, Hq, D), cos, sin, positions, dt)
        k = heads(lin(n1, "layers.%d.k" % l), S, Hkv, D)
        v = heads(lin(n1, "layers.%d.v" % l), S, Hkv, D)
        c = caches[l]
        if ring is not None:
            sink, window, ring_start, kvp = ring
            if kv8:
                orc.quantizing_kv_cache_update_streaming(c[0], c[2], k, past, sink, window, ring_start, dt)
                orc.quantizing_kv_cache_update_streaming(c[1], c[3], v, past, sink, window, ring_start, dt)
                a = orc.attention_streaming(q, c[0], c[1], dt, scale, causal, active, sink, window, ring_start, c[2], c[3],
                                            (cos, sin, kvp))
            else:
                orc.kv_cache_update_streaming(c[0], k, past, sink, window, ring_start)
                orc.kv_cache_update_streaming(c[1], v, past, sink, window, ring_start)
                k_rot = orc.rope(c[0], cos, sin, kvp, dt)  # Rope over the whole cache: one table row per SLOT
                a = orc.attention_streaming(q, k_rot, c[1], dt, scale, causal, active, sink, window, ring_start)
        else:
            k = orc.rope(k, cos, sin, positions, dt)
            if kv8:
                orc.quantizing_kv_cache_update(c[0], c[2], k, past, dt)
                orc.quantizing_kv_cache_update(c[1], c[3], v, past, dt)
                a = orc.attention(q, c[0], c[1], dt, scale, causal, active, c[2], c[3])
            else:
                orc.kv_cache_update(c[0], k, past)
                orc.kv_cache_update(c[1], v, past)
                a = orc.attention(q, c[0], c[1], dt, scale, causal, active)
        a = np.ascontiguousarray(a[0].transpose(1, 0, 2)).reshape(S, Hq * D)
        x2 = orc.add(x, lin(a, "layers.%d.o" % l), dt)
        n2 = orc.rms_norm(x2, w["layers.%d.norm2" % l], cfg["eps"], dt)
        hm = orc.swiglu(lin(n2, "layers.%d.gate" % l), lin(n2, "layers.%d.up" % l), dt)
        x = orc.add(x2, lin(hm, "layers.%d.down" % l), dt)
    return lin(orc.rms_norm(x, w["final_norm"], cfg["eps"], dt), "lm_head")


def empty_caches(cfg, dt, kv8):
    Hkv, D, MS, L = cfg["n_kv_heads"], cfg["head_dim"], cfg["max_seq"], cfg["n_layers"]
    if kv8:
        return [[np.zeros((1, Hkv, MS, D), np.int8), np.zeros((1, Hkv, MS, D), np.int8),
                 np.zeros((1, Hkv, MS), orc.np_dtype(dt)), np.zeros((1, Hkv, MS), orc.np_dtype(dt))] for _ in range(L)]
    return [[np.zeros((1, Hkv, MS, D), orc.np_dtype(dt)), np.zeros((1, Hkv, MS, D), orc.np_dtype(dt))] for _ in range(L)]
