"""Weight sets for the decoder tests: the tiny random Llama checkpoint the reference's own
end-to-end test uses (crates/llm/tests/tinyllama_random.rs) and seeded synthetic int8 models
of any Llama shape (weights f32 ~ N(0, 0.02), quantised with the per-channel rule of
crates/llm/src/quantize.rs:124-169, norm weights 1)."""
import json
import os

import numpy as np

import oracle as orc
from conftest import GOLDEN

LIN = {"q": "self_attn.q_proj", "k": "self_attn.k_proj", "v": "self_attn.v_proj", "o": "self_attn.o_proj",
       "gate": "mlp.gate_proj", "up": "mlp.up_proj", "down": "mlp.down_proj"}

TINYLLAMA_CFG = dict(n_layers=22, hidden=2048, n_heads=32, n_kv_heads=4, head_dim=64, ffn=5632,
                     vocab=32000, max_seq=384, eps=1e-5, rope_theta=10000.0)


def tiny_llama_random(dt, max_seq=32):
    """Returns (cfg, weights, golden) for tests/golden/tiny-llama-random (f32 checkpoint narrowed
    to dt the way the reference narrows a checkpoint: RNE, crates/llm/src/quantize.rs:171-183)."""
    from safetensors.numpy import load_file

    d = os.path.join(GOLDEN, "tiny-llama-random")
    hf = json.load(open(os.path.join(d, "config.json")))
    st = load_file(os.path.join(d, "model.safetensors"))
    cfg = dict(n_layers=hf["num_hidden_layers"], hidden=hf["hidden_size"], n_heads=hf["num_attention_heads"],
               n_kv_heads=hf["num_key_value_heads"], head_dim=hf["head_dim"], ffn=hf["intermediate_size"],
               vocab=hf["vocab_size"], max_seq=max_seq, eps=hf["rms_norm_eps"], rope_theta=hf["rope_theta"],
               dtype=dt)
    w = {"embed": orc.to_storage(st["model.embed_tokens.weight"], dt),
         "lm_head": orc.to_storage(st["lm_head.weight"], dt),
         "final_norm": orc.to_storage(st["model.norm.weight"], dt)}
    for l in range(cfg["n_layers"]):
        p = "model.layers.%d." % l
        for k, nm in LIN.items():
            w["layers.%d.%s" % (l, k)] = orc.to_storage(st[p + nm + ".weight"], dt)
        w["layers.%d.norm1" % l] = orc.to_storage(st[p + "input_layernorm.weight"], dt)
        w["layers.%d.norm2" % l] = orc.to_storage(st[p + "post_attention_layernorm.weight"], dt)
    golden = json.load(open(os.path.join(d, "golden_ids.json")))
    return cfg, w, golden


def synthetic_int8(cfg, dt, seed=1234, std=0.02, quantize=None):
    """Seeded random-init int8 model.  `quantize(w_f32, scale_dt) -> (int8, scale)` defaults to
    the oracle's restatement of the reference quantiser."""
    quantize = quantize or orc.quantize_per_channel
    rng = np.random.default_rng(seed)
    H, F, V = cfg["hidden"], cfg["ffn"], cfg["vocab"]
    QD, KD = cfg["n_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"]

    def lin(n, k):
        return quantize((rng.standard_normal((n, k), dtype=np.float32) * np.float32(std)), dt)

    ones = orc.to_storage(np.ones(H, np.float32), dt)
    w = {"embed": lin(V, H), "lm_head": lin(V, H), "final_norm": ones}
    shapes = {"q": (QD, H), "k": (KD, H), "v": (KD, H), "o": (H, QD), "gate": (F, H), "up": (F, H), "down": (H, F)}
    for l in range(cfg["n_layers"]):
        for k, (n, kk) in shapes.items():
            w["layers.%d.%s" % (l, k)] = lin(n, kk)
        w["layers.%d.norm1" % l] = ones
        w["layers.%d.norm2" % l] = ones
    c = dict(cfg)
    c["dtype"] = dt
    return c, w


def add_qkv_bias(cfg, w, dt, seed=99, std=0.5):
    """q / k / v projection biases (model_type "qwen2", crates/llm/src/decoder.rs:542-600) for a weight dict: [N] in the
    model's type, seeded; large enough to move the logits."""
    rng = np.random.default_rng(seed)
    QD, KD = cfg["n_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"]
    out = dict(w)
    for l in range(cfg["n_layers"]):
        for nm, n in (("q", QD), ("k", KD), ("v", KD)):
            out["layers.%d.%s.bias" % (l, nm)] = orc.to_storage(rng.standard_normal(n).astype(np.float32) * np.float32(std), dt)
    return out
