#!/usr/bin/env python3
"""Headline benchmark: batch-1 greedy decode of a TinyLlama-1.1B-shape int8 model on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload decode|prefill]

`--workload prefill` times the matrix-core side of the same path instead: one step = one prefill
pass of 8 prompts x 1024 tokens through the decoder executor (roofline bound: MFMA).

One step = one decode step (one token) through the HIP decoder executor; the K timed steps are
replays of the captured hipGraph with inputs, weights and KV cache resident in HBM.  Prints ONE
JSON line: decode tok/s, the roofline of the dominant kernel (HIP-event timing of the same
launches), and a CPU baseline (the oracle, a port of the reference CPU backend) timed on the
host cores of the same box.
"""
import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
# HBM bytes per launch of the gate/up GEMV (TinyLlama shape, 16-bit activations) from rocprofv3
# --pmc FETCH_SIZE (x2.000, scaled by a 256 MiB copy) + WRITE_SIZE (x1.000): 11396.4 KiB * 2 + 35.0 KiB.
# Counters cannot be read from inside this process; the figure is carried here from that profile run.
GATEUP_GEMV_TRAFFIC_BYTES = 23375749
# the same for the dominant kernels of the other workloads (profiles/prefill_and_batched_decode_pmc_hbm_traffic.md):
# prefill gate/up GEMM + SwiGLU (f16, 8192 x 11264 x 2048): 287320.4 KiB * 2 + 90112.0 KiB;
# batched-decode gate/up few-row GEMM (Llama-3-8B shape, 32 rows): 61689.4 KiB * 2 + 896.3 KiB
PREFILL_GATEUP_GEMM_TRAFFIC_BYTES = 680706867
BATCHED_GATEUP_GEMM_TRAFFIC_BYTES = 127257702
# share of SIMD clocks in which the matrix pipe is busy during the prefill gate/up GEMM, from rocprofv3 --pmc
# SQ_VALU_MFMA_BUSY_CYCLES / (GRBM_GUI_ACTIVE / 8 XCDs * 1024 SIMDs); the shader clock under that load is 1.87 GHz
# (2.06 GHz with int8 activations), which is why it exceeds flop / time / peak-at-2.4-GHz
# (profiles/prefill_tinyllama_int8_8x1024_pmc_mfma_utilisation.md)
PREFILL_GATEUP_MFMA_BUSY_FRAC = {"f16": 0.513, "w8a8": 0.382}
MFMA_PEAK_TFLOPS = 2500.0  # MI355X published dense bf16/fp16 matrix rate
INT8_PEAK_TOPS = 5000.0    # MI355X published dense int8 matrix rate
PREFILL_BATCH, PREFILL_LEN = 8, 1024

TINYLLAMA = dict(n_layers=22, hidden=2048, n_heads=32, n_kv_heads=4, head_dim=64, ffn=5632, vocab=32000,
                 max_seq=384, eps=1e-5, rope_theta=10000.0)
PROMPT_LEN = 128


def make_weights(cfg, dt, seed):
    """Seeded random-init weights generated on the device: f32 ~ N(0, 0.02), quantised per output
    channel with the reference rule (crates/llm/src/quantize.rs:124-169: scale = amax/127,
    q = clamp(round_half_away(w/scale), -128, 127)); norm weights 1."""
    import torch

    tdt = {1: torch.bfloat16, 2: torch.float16}[dt]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    H, F, V = cfg["hidden"], cfg["ffn"], cfg["vocab"]
    QD, KD = cfg["n_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"]

    def lin(n, k):
        w = torch.randn((n, k), generator=gen, device="cuda", dtype=torch.float32) * 0.02
        amax = w.abs().amax(dim=1, keepdim=True)
        scale = torch.where(amax == 0, torch.ones_like(amax), amax / 127.0)
        r = w / scale
        q = (torch.sign(r) * torch.floor(r.abs() + 0.5)).clamp_(-128, 127).to(torch.int8)
        return q.contiguous(), scale.reshape(-1).to(tdt).contiguous()

    ones = torch.ones((H,), dtype=tdt, device="cuda")
    w = {"embed": lin(V, H), "lm_head": lin(V, H), "final_norm": ones}
    shapes = {"q": (QD, H), "k": (KD, H), "v": (KD, H), "o": (H, QD), "gate": (F, H), "up": (F, H), "down": (H, F)}
    for l in range(cfg["n_layers"]):
        for k, (n, kk) in shapes.items():
            w["layers.%d.%s" % (l, k)] = lin(n, kk)
        w["layers.%d.norm1" % l] = ones
        w["layers.%d.norm2" % l] = ones
    return w


def to_host_weights(w):
    import numpy as np
    import torch

    def h(t):
        if t.dtype in (torch.float16, torch.bfloat16):
            return t.view(torch.int16).cpu().numpy().view(np.uint16)
        return t.cpu().numpy()

    return {k: (h(v[0]), h(v[1])) if isinstance(v, tuple) else h(v) for k, v in w.items()}


def algorithmic_bytes_per_token(cfg, eb, context):
    """int8 weights + scales of every linear, embedding row, KV rows read at `context` and the
    row written."""
    H, F, V = cfg["hidden"], cfg["ffn"], cfg["vocab"]
    QD, KD = cfg["n_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"]
    per_layer_w = QD * H + 2 * KD * H + H * QD + 2 * F * H + H * F
    per_layer_s = (QD + 2 * KD + H + 2 * F + H) * eb
    w = cfg["n_layers"] * (per_layer_w + per_layer_s) + V * H + V * eb
    kv = cfg["n_layers"] * 2 * KD * eb * (context + 1)
    return w + kv + H + eb


def prefill_main(args, mynn, cfg):
    """8 x 1024 prompt tokens through the prefill executor: every linear on the matrix cores, causal
    flash attention, logits for every row (the reference computes [1, S, vocab])."""
    import numpy as np
    import torch

    B, S = PREFILL_BATCH, PREFILL_LEN
    K = 5 if args.steps is None else args.steps
    W = 2 if args.warmup is None else args.warmup
    cfg = dict(cfg, max_seq=S)
    weights = make_weights(cfg, cfg["dtype"], args.seed)
    torch.cuda.synchronize()
    dec = mynn.Decoder(cfg, weights, seq_q=S, batch=B, quantize_activations=args.w8a8)
    rng = np.random.default_rng(args.seed)
    ids = rng.integers(0, cfg["vocab"], B * S)
    pos = np.arange(S)
    for _ in range(W):
        dec.step(ids, pos, 0, S)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(K):
        dec.step(ids, pos, 0, S)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / K

    agg = {}
    for _ in range(2):
        for name, ms, nbytes, flops in dec.profile(ids, pos, 0, S):
            a = agg.setdefault(name, [0, 0.0, 0.0, 0.0])
            a[0] += 1
            a[1] += ms
            a[2] += nbytes
            a[3] += flops
    mm = {k: v for k, v in agg.items() if v[3] > 0}
    dom = max(mm, key=lambda k: mm[k][1])
    calls, ms_tot, _, fl_tot = mm[dom]
    achieved = fl_tot / (ms_tot * 1e-3) / 1e12
    step_flops = sum(v[3] for v in agg.values()) / 2
    lin = {k: v for k, v in mm.items() if k.startswith("linear_") or k.startswith("qlinear_")}
    # W8A8 (--w8a8): activations quantised per row, every linear an exact int8 x int8 -> int32 product
    peak = INT8_PEAK_TOPS if args.w8a8 else MFMA_PEAK_TFLOPS
    unit = "TOP/s" if args.w8a8 else "TFLOP/s"
    lin_tflops = sum(v[3] for v in lin.values()) / (sum(v[1] for v in lin.values()) * 1e-3) / 1e12
    out = {
        "metric": "prefill tok/s 8x1024 TinyLlama-shape int8; MFMA utilisation" + (" (W8A8: quantize_activations)" if args.w8a8 else ""),
        "value": round(B * S * K / elapsed, 1), "unit": "tok/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": ("int32 accumulate over int8 activations x int8 weights, %s elsewhere" % args.dtype) if args.w8a8 else
                 "f32 accumulate over %s (int8 weights dequantised to %s)" % (args.dtype, args.dtype),
        "data": "synthetic",
        "config": {"workload": "configs[3]: TinyLlama-1.1B-shape int8 decoder, prefill of 8 prompts x 1024 tokens, "
                               "KV cache filled, logits for every row" + (", activations quantised to int8 per row" if args.w8a8 else ""),
                   "batch": B, "seq": S, "launches_per_step": dec.stats()["launches_per_step"], "seed": args.seed,
                   "step_flops": step_flops,
                   "step_mfma_frac": round(step_flops / (ms_per_step * 1e-3) / 1e12 / peak, 4),
                   "per_kernel_ms": {k: round(v[1] / 2, 3) for k, v in sorted(agg.items(), key=lambda kv: -kv[1][1])}},
        "roofline": {"bound": "mfma", "kernel": dom, "achieved": round(achieved, 1), "peak": peak,
                     "unit": unit, "frac": round(achieved / peak, 4),
                     "traffic": PREFILL_GATEUP_GEMM_TRAFFIC_BYTES if dom == "linear_gateup_swiglu" and args.dtype == "f16" else None,
                     "mfma_busy_frac_pmc": (PREFILL_GATEUP_MFMA_BUSY_FRAC["w8a8" if args.w8a8 else "f16"]
                                            if dom == "linear_gateup_swiglu" and args.dtype == "f16" else None),
                     "flops_per_launch": fl_tot / calls, "avg_launch_us": round(ms_tot / calls * 1e3, 2),
                     "all_linear_TFLOPs": round(lin_tflops, 1)},
    }
    if not args.no_cpu_baseline:
        import oracle as orc

        ref = orc.Model(dict(cfg), to_host_weights(weights))
        n_cpu = 256  # bounded sample: the first rows of the first prompt
        t0 = time.perf_counter()
        ref.forward(ids[:n_cpu], pos[:n_cpu], 0, n_cpu, True)
        cpu_elapsed = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": round(n_cpu / cpu_elapsed, 2), "unit": "tok/s", "cores": orc.get_threads(),
                               "kind": "port",
                               "sample": "one causal prefill pass over the first %d tokens of the first prompt, C port "
                                         "of the reference CPU backend (dequantise + blocked f32 GEMM, OpenMP)" % n_cpu}
    dec.close()
    print(json.dumps(out))


def attention_main(args, mynn):
    """GQA decode attention op at the largest shape of configs[1]: 16 sequences x 4096 cached keys,
    32 query heads over 4 KV heads of 64 dims, fp16 cache, softmax scale 1/8.  One step = one
    attention call; the caches rotate over > 256 MB so no call finds its K/V in the Infinity Cache."""
    import torch

    B, L, Hq, Hkv, D = 16, 4096, 32, 4, 64
    K = 200 if args.steps is None else args.steps
    W = 10 if args.warmup is None else args.warmup
    tdt = {"f16": torch.float16, "bf16": torch.bfloat16}[args.dtype]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(args.seed)
    n = 6  # 6 x 67 MB of K/V
    ks = [torch.randn((B, Hkv, L, D), generator=gen, device="cuda", dtype=tdt) for _ in range(n)]
    vs = [torch.randn((B, Hkv, L, D), generator=gen, device="cuda", dtype=tdt) for _ in range(n)]
    q = torch.randn((B, Hq, 1, D), generator=gen, device="cuda", dtype=tdt)
    for i in range(W):
        mynn.attention(q, ks[i % n], vs[i % n], 0.125, active=L)
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for i in range(K):
        mynn.attention(q, ks[i % n], vs[i % n], 0.125, active=L)
    stop.record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    gpu_ms = start.elapsed_time(stop) / K  # launches are queued ahead of the GPU: this is device time per call
    nbytes = 2 * B * Hkv * L * D * 2 + 2 * B * Hq * D * 2
    achieved = nbytes / (gpu_ms * 1e-3) / 1e9
    out = {
        "metric": "GQA decode attention op: achieved HBM GB/s vs peak (configs[1], B=16, L=4096)",
        "value": round(achieved, 1), "unit": "GB/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(elapsed * 1e3 / K, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32 softmax and accumulate over %s K/V" % args.dtype, "data": "synthetic",
        "config": {"workload": "configs[1]: attention op, B=16, Hq=32, Hkv=4, D=64, L=4096, scale 0.125, seq_q=1",
                   "seed": args.seed, "rotating_kv_sets": n, "device_ms_per_call": round(gpu_ms, 4)},
        "roofline": {"bound": "hbm", "kernel": "attn_stream_kernel + attn_merge_kernel", "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                     "bytes_per_launch": nbytes, "avg_launch_us": round(gpu_ms * 1e3, 2)},
    }
    if not args.no_cpu_baseline:
        import numpy as np
        import oracle as orc

        dt = {"f16": orc.F16, "bf16": orc.BF16}[args.dtype]
        hq, hk, hv = [t.view(torch.int16).cpu().numpy().view(np.uint16) for t in (q, ks[0], vs[0])]
        t0 = time.perf_counter()
        orc.attention(hq, hk, hv, dt, 0.125)
        cpu = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": round(nbytes / cpu / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                               "sample": "one call at the same shape, C port of the reference CPU attention "
                                         "(single thread, as the reference)"}
    print(json.dumps(out))


LLAMA3_8B = dict(n_layers=32, hidden=4096, n_heads=32, n_kv_heads=8, head_dim=128, ffn=14336, vocab=128256,
                 max_seq=2304, eps=1e-5, rope_theta=500000.0)


def decode_batch_main(args, mynn):
    """configs[4]: Llama-3-8B-shape int8 decoder, 32 sequences decoded together at a context of 2048
    tokens.  The caches are filled with random K/V rows instead of running the 65,536-token prefill: the
    cost of a decode step does not depend on their values.  One step = one new token for each sequence."""
    import numpy as np
    import torch

    B, ctx = 32, 2048
    K = 32 if args.steps is None else args.steps
    W = 4 if args.warmup is None else args.warmup
    dt = {"f16": mynn.F16, "bf16": mynn.BF16}[args.dtype]
    tdt = {"f16": torch.float16, "bf16": torch.bfloat16}[args.dtype]
    cfg = dict(LLAMA3_8B, dtype=dt)
    assert ctx + W + K <= cfg["max_seq"]
    weights = make_weights(cfg, dt, args.seed)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(args.seed + 1)
    shape = (B, cfg["n_kv_heads"], cfg["max_seq"], cfg["head_dim"])
    kv = []
    for _ in range(cfg["n_layers"]):
        if args.kv_int8:
            bufs = []
            for _ in range(2):
                c = torch.zeros(shape, dtype=torch.int8, device="cuda")
                c[:, :, :ctx] = torch.randint(-127, 128, (B, shape[1], ctx, shape[3]), generator=gen, device="cuda",
                                              dtype=torch.int8)
                bufs.append(c)
            for _ in range(2):
                sc = torch.zeros(shape[:3], dtype=tdt, device="cuda")
                sc[:, :, :ctx] = (torch.rand((B, shape[1], ctx), generator=gen, device="cuda") * 0.02 + 0.01).to(tdt)
                bufs.append(sc)
            kv.append(tuple(bufs))
        else:
            k = torch.zeros(shape, dtype=tdt, device="cuda")
            v = torch.zeros(shape, dtype=tdt, device="cuda")
            k[:, :, :ctx] = torch.randn((B, shape[1], ctx, shape[3]), generator=gen, device="cuda", dtype=tdt)
            v[:, :, :ctx] = torch.randn((B, shape[1], ctx, shape[3]), generator=gen, device="cuda", dtype=tdt)
            kv.append((k, v))
    torch.cuda.synchronize()
    dec = mynn.Decoder(cfg, weights, batch=B, kv=kv, quant_kv_cache=args.kv_int8)
    stats = dec.stats()
    rng = np.random.default_rng(args.seed)
    toks = rng.integers(0, cfg["vocab"], B).tolist()
    past = ctx
    for _ in range(W):
        toks, _ = dec.step(toks, [past], past, past + 1)
        past += 1
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(K):
        toks, _ = dec.step(toks, [past], past, past + 1)
        past += 1
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / K

    agg = {}
    for _ in range(2):
        for name, ms, nbytes, flops in dec.profile(toks, [past], past, past + 1):
            a = agg.setdefault(name, [0, 0.0, 0.0])
            a[0] += 1
            a[1] += ms
            a[2] += nbytes
    eb = 2
    H, F, V = cfg["hidden"], cfg["ffn"], cfg["vocab"]
    QD, KD = cfg["n_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"]
    w_bytes = cfg["n_layers"] * (QD * H + 2 * KD * H + H * QD + 3 * F * H) + V * H
    kv_row = KD + cfg["n_kv_heads"] * eb if args.kv_int8 else KD * eb  # bytes of one token's k (or v) over all kv heads
    kv_bytes = cfg["n_layers"] * B * 2 * kv_row * (ctx + W + K // 2)
    step_bytes = w_bytes + kv_bytes
    lin = {k: v for k, v in agg.items() if k.startswith("linear_")}
    dom = max(lin, key=lambda k: lin[k][1])
    calls, ms_tot, bytes_tot = lin[dom]
    achieved = bytes_tot / (ms_tot * 1e-3) / 1e9
    out = {
        "metric": "decode tok/s, batch 32 at context 2048, Llama-3-8B-shape int8 (aggregate over the batch)",
        "value": round(B * K / elapsed, 1), "unit": "tok/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32 accumulate over int8 weights, %s activations, %s KV" % (args.dtype, "int8" if args.kv_int8 else args.dtype),
        "data": "synthetic",
        "config": {"workload": "configs[4]: Llama-3-8B-shape int8 decoder, batch 32, context 2048 (caches filled with "
                               "random rows%s), %d decode steps timed" % (", int8 KV cache" if args.kv_int8 else "", K),
                   "batch": B, "context": ctx, "launches_per_step": stats["launches_per_step"], "hipgraph": stats["graph"],
                   "seed": args.seed, "step_algorithmic_bytes": step_bytes,
                   "step_hbm_frac": round(step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                   "per_kernel_ms": {k: round(v[1] / 2, 3) for k, v in sorted(agg.items(), key=lambda kv: -kv[1][1])}},
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": BATCHED_GATEUP_GEMM_TRAFFIC_BYTES if dom == "linear_gateup_swiglu" and not args.kv_int8 else None,
                     "bytes_per_launch": bytes_tot / calls,
                     "avg_launch_us": round(ms_tot / calls * 1e3, 2)},
    }
    dec.close()
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--workload", choices=["decode", "prefill", "attention", "decode_batch"], default="decode")
    ap.add_argument("--steps", type=int, default=None, help="default 256 (decode) / 5 (prefill)")
    ap.add_argument("--warmup", type=int, default=None, help="default 16 (decode) / 2 (prefill)")
    ap.add_argument("--dtype", choices=["f16", "bf16"], default="f16")
    ap.add_argument("--seed", type=int, default=1234)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-steps", type=int, default=96)
    ap.add_argument("--traffic-calibration", action="store_true",
                    help="first run one 256 MiB device-to-device copy (a kernel of known traffic, for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--w8a8", action="store_true",
                    help="prefill: quantise activations per row and run every linear as int8 x int8 (Options::quantize_activations)")
    ap.add_argument("--kv-int8", action="store_true",
                    help="decode_batch: int8 KV cache with per-token scales (BuildOptions::quant_kv_cache)")
    ap.add_argument("--check-tokens", type=int, default=0,
                    help="also compare the first N greedy tokens with the oracle (slow: CPU decode)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU; --gpus %d is not supported (no collectives are built)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    mynn = importlib.import_module("my-nn-engine_amd")
    if args.traffic_calibration:
        src = torch.ones(256 << 20, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)  # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst
    dt = {"f16": mynn.F16, "bf16": mynn.BF16}[args.dtype]
    eb = 2
    cfg = dict(TINYLLAMA, dtype=dt)
    if args.workload == "prefill":
        return prefill_main(args, mynn, cfg)
    if args.workload == "attention":
        return attention_main(args, mynn)
    if args.workload == "decode_batch":
        return decode_batch_main(args, mynn)
    K = 256 if args.steps is None else args.steps
    W = 16 if args.warmup is None else args.warmup
    assert PROMPT_LEN + max(K, W) <= cfg["max_seq"], "steps/warmup do not fit max_seq %d" % cfg["max_seq"]

    weights = make_weights(cfg, dt, args.seed)
    torch.cuda.synchronize()
    dec = mynn.Decoder(cfg, weights)
    stats = dec.stats()
    rng = np.random.default_rng(args.seed)
    prompt = rng.integers(0, cfg["vocab"], PROMPT_LEN).tolist()

    # prompt through the decode path, token by token (the reference's path without a prefill session)
    # (each of these steps is a host round trip: inputs up, graph replay, token down -- timed for the record)
    first = None
    t_host = None
    for i, t in enumerate(prompt):
        if i == 16:
            torch.cuda.synchronize()
            t_host = time.perf_counter()
        first, _ = dec.step([t], [i], i, i + 1)
    host_tok_s = (PROMPT_LEN - 16) / (time.perf_counter() - t_host)
    first = first[0]

    if W > 0:
        dec.decode_loop(first, PROMPT_LEN, W)  # untimed; its KV rows are overwritten below
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    toks = dec.decode_loop(first, PROMPT_LEN, K)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    generated = [first] + toks[:-1]
    ms_per_step = elapsed * 1e3 / K
    tok_s = K / elapsed

    # ---- roofline of the dominant kernel: HIP events around every launch of eager steps at
    # contexts spread over the timed range, on the executor's own stream
    agg = {}
    n_prof = 8
    for j in range(n_prof):
        past = PROMPT_LEN + (j * (K - 1)) // max(n_prof - 1, 1)
        for name, ms, nbytes, _ in dec.profile_step(generated[min(past - PROMPT_LEN, K - 1)], past):
            a = agg.setdefault(name, [0, 0.0, 0.0])
            a[0] += 1
            a[1] += ms
            a[2] += nbytes
    gemv = {k: v for k, v in agg.items() if k.startswith("gemv_")}
    dom = max(gemv, key=lambda k: gemv[k][1])
    calls, ms_tot, bytes_tot = gemv[dom]
    achieved = bytes_tot / (ms_tot * 1e-3) / 1e9
    all_gemv_gbs = sum(v[2] for v in gemv.values()) / (sum(v[1] for v in gemv.values()) * 1e-3) / 1e9
    step_bytes = algorithmic_bytes_per_token(cfg, eb, PROMPT_LEN + K // 2)

    out = {
        "metric": "decode tok/s bs1 TinyLlama-shape int8; dequant-GEMV HBM GB/s vs peak",
        "value": round(tok_s, 2), "unit": "tok/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32 accumulate over int8 weights, %s activations/KV" % args.dtype, "data": "synthetic",
        "config": {"workload": "configs[2]: TinyLlama-1.1B-shape int8 decoder, batch 1 greedy decode, 128 prompt tokens "
                               "fed through the decode path then %d generated (timed: the generated tokens)" % K,
                   "prompt_len": PROMPT_LEN, "max_seq": cfg["max_seq"], "launches_per_step": stats["launches_per_step"],
                   "hipgraph": stats["graph"], "seed": args.seed,
                   "host_roundtrip_tok_s": round(host_tok_s, 1),
                   "step_algorithmic_bytes": step_bytes,
                   "step_hbm_frac": round(step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                   # average duration of every launch of the step (HIP events, eager steps): the fused
                   # q|k|v + attention + o launch is the longest, the gate/up GEMV moves the most bytes
                   "per_launch_us": {k: round(v[1] / v[0] * 1e3, 2) for k, v in sorted(agg.items(), key=lambda kv: -kv[1][1])}},
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": GATEUP_GEMV_TRAFFIC_BYTES if dom == "gemv_norm_gateup_swiglu" else None,
                     "bytes_per_launch": bytes_tot / calls, "avg_launch_us": round(ms_tot / calls * 1e3, 3),
                     "all_gemv_GBs": round(all_gemv_gbs, 1)},
    }

    if not args.no_cpu_baseline:
        import oracle as orc

        hw = to_host_weights(weights)
        ref = orc.Model(dict(cfg), hw)
        n_cpu = args.cpu_steps
        ref.past_len = 0
        stream = prompt + generated
        # bounded sample: the first n_cpu decode steps of the same token stream
        t0 = time.perf_counter()
        last = None
        for i in range(n_cpu):
            last = ref.decode_step(stream[i])
        cpu_elapsed = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": round(n_cpu / cpu_elapsed, 3), "unit": "tok/s", "cores": orc.get_threads(),
                               "kind": "port",
                               "sample": "first %d decode steps (contexts 0..%d) of the same model and token stream, "
                                         "C port of the reference CPU backend, OpenMP over N" % (n_cpu, n_cpu - 1)}
        if args.check_tokens:
            n = min(args.check_tokens, K)
            ref2 = orc.Model(dict(cfg), hw)
            want = ref2.generate(prompt, n)
            out["config"]["tokens_identical_to_oracle"] = (want == generated[:n])
            out["config"]["tokens_checked"] = n
    dec.close()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
