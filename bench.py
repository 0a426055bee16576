#!/usr/bin/env python3
"""Headline benchmark: batch-1 greedy decode of a TinyLlama-1.1B-shape int8 model on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload decode|prefill|attention|decode_batch|gemv]

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
# Figures that cannot be measured from inside this process (rocprofv3's own kernel durations, HBM traffic and
# matrix-pipe counters of a launch) are read from small JSON files under profiles/ that `--summarize-rocprof`
# writes from rocprofv3 output of this same script; each entry carries the kernel's mangled name, and is used
# only while the built library still contains that symbol.
PROFILE_JSON = {"decode": "decode_tinyllama_int8_bs1.json", "prefill": "prefill_tinyllama_int8_8x1024.json",
                "prefill_w8a8": "prefill_w8a8_tinyllama_8x1024.json", "decode_batch": "decode_llama3_8b_int8_bs32_ctx2048.json",
                "decode_batch_kv8": "decode_llama3_8b_int8_bs32_ctx2048_kv_int8.json",
                "attention": "attention_decode_b16_l4096.json", "gemv": "gemv_rotating_weight_sets.json"}
# launch role (the executor's name for a launch) -> pattern of the mangled kernel name
ROLE_PATTERNS = {
    "gemv_norm_gateup_swiglu": r"dequant_gemv1_kernelI\w+?Li\d+ELi\d+ELi2ELb1ELb0EE",
    "gemv_down_residual": r"dequant_gemv1_kernelI\w+?Li\d+ELi\d+ELi1ELb0ELb0EE",
    "gemv_norm_lm_head_argmax": r"dequant_gemv1_kernelI\w+?Li\d+ELi\d+ELi0ELb1ELb1EE",
    "qkv_attention_o": r"qkv_attention_kernelI\w+?Li\d+ELi\d+ELb0ELb0ELb0EE",   # <T, D, NC, EMBED = false, KV8 = false, PAGED = false>
    "embed_qkv_attention_o": r"qkv_attention_kernelI\w+?Li\d+ELi\d+ELb1ELb0ELb0EE",
    "linear_gateup_swiglu": r"(gemm_nt_dma_kernelI\w+?Li2ELb0EE|skinny_gemm_kernelI\w+?Li\d+ELb\dELi2ELi0EE)",  # (skinny: <T, MT, PACKED, FEPI = SwiGLU, ABL = 0>)
    "qlinear_gateup_swiglu": r"gemm_nt_dma_kernelI\w+?Li2ELb1EE",
    "attention": r"(attn_stream_kernel|attn_prefill_kernel)",
    # --workload gemv: the stand-alone GEMV launches and the read probe of the same geometry
    "gemv_configs0_f32": r"dequant_gemv_kernelIffLi\d+ELi1ELi0ELb0EE",
    "gemv_gate_up": r"dequant_gemv1_kernelI\w+?Li4ELi2ELi0ELb0ELb0EE",
    "gemv_down": r"dequant_gemv1_kernelI\w+?Li2ELi6ELi0ELb0ELb0EE",
    "read_probe_gate_up": r"gemv_read_probe_kernelILi4ELi2EE",
    "read_probe_down": r"gemv_read_probe_kernelILi2ELi6EE",
}
MFMA_PEAK_TFLOPS = 2500.0  # MI355X published dense bf16/fp16 matrix rate
INT8_PEAK_TOPS = 5000.0    # MI355X published dense int8 matrix rate
PREFILL_BATCH, PREFILL_LEN = 8, 1024



def source_digest():
    """sha256 over the kernel sources the library was built from (a profile taken from other sources is stale)."""
    import glob
    import hashlib

    h = hashlib.sha256()
    for f in sorted(glob.glob(os.path.join(ROOT, "my-nn-engine_amd", "csrc", "*"))):
        if f.endswith((".hip", ".h", "Makefile")):
            h.update(os.path.basename(f).encode())
            h.update(open(f, "rb").read())
    return h.hexdigest()[:16]


_lib_bytes = None


def library_has_symbol(mangled):
    global _lib_bytes
    if _lib_bytes is None:
        mynn = importlib.import_module("my-nn-engine_amd")
        _lib_bytes = open(mynn.LIB_PATH, "rb").read()
    return mangled.encode() in _lib_bytes


def load_profile(key):
    """The tracked rocprofv3 summary for a workload, or None.  Entries whose kernel the library no longer holds
    are dropped, so that a changed kernel never inherits an old figure."""
    path = os.path.join(ROOT, "profiles", PROFILE_JSON[key])
    if not os.path.exists(path):
        return None
    prof = json.load(open(path))
    prof["kernels"] = [k for k in prof.get("kernels", []) if library_has_symbol(k["mangled"])]
    prof["file"] = "profiles/" + PROFILE_JSON[key]
    prof["stale"] = prof.get("source_sha256") != source_digest()
    return prof


def profile_entry(prof, role):
    """The profile's entry for a launch role (matched on the mangled kernel name); None when absent."""
    import re

    if not prof or role not in ROLE_PATTERNS:
        return None
    hits = [k for k in prof["kernels"] if re.search(ROLE_PATTERNS[role], k["mangled"])]
    if not hits:
        return None
    return max(hits, key=lambda k: k["total_ms"])


def traffic_bytes(entry):
    """HBM bytes per launch from the two counter runs, scaled by what the same counters read for a 256 MiB copy."""
    if not entry or entry.get("fetch_kib") is None or entry.get("write_kib") is None:
        return None
    return int(round((entry["fetch_kib"] * entry["fetch_factor"] + entry["write_kib"] * entry["write_factor"]) * 1024))


def summarize_rocprof(args):
    """Reads rocprofv3 output of this script (kernel trace, and optionally the FETCH_SIZE and WRITE_SIZE counter
    runs, all as csv with mangled kernel names) and writes the JSON that later runs read back, plus the same
    figures as a markdown table."""
    import csv
    import glob

    def rows(d, suffix):
        files = glob.glob(os.path.join(d, "**", "*" + suffix), recursive=True)
        if not files:
            raise SystemExit("no *%s under %s" % (suffix, d))
        for f in files:
            with open(f, newline="") as fh:
                for r in csv.DictReader(fh):
                    yield r

    def kname(r):  # (mangled names come with the kernel descriptor's suffix)
        n = r["Kernel_Name"]
        return n[:-3] if n.endswith(".kd") else n

    kern = {}
    for r in rows(args.summarize_rocprof, "kernel_trace.csv"):
        name = kname(r)
        if "mynn" not in name:
            continue
        d = (int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3
        k = kern.setdefault(name, {"mangled": name, "calls": 0, "total_us": 0.0, "min_us": 1e30, "max_us": 0.0, "by_grid": {}})
        k["calls"] += 1
        k["total_us"] += d
        k["min_us"] = min(k["min_us"], d)
        k["max_us"] = max(k["max_us"], d)
        g = k["by_grid"].setdefault("%sx%sx%s" % (r.get("Grid_Size_X"), r.get("Grid_Size_Y"), r.get("Grid_Size_Z")), [0, 0.0])
        g[0] += 1
        g[1] += d
    copy = {}
    for which, d in (("fetch", args.pmc_fetch), ("write", args.pmc_write)):
        if not d:
            continue
        acc = {}
        per = 0.0  # counter reading of the one 256 MiB device-to-device copy (262144 KiB read, 262144 written): the largest copy
        for r in rows(d, "counter_collection.csv"):
            a = acc.setdefault(kname(r), [0, 0.0])
            a[0] += 1
            a[1] += float(r["Counter_Value"])
            if "copyBuffer" in r["Kernel_Name"]:
                per = max(per, float(r["Counter_Value"]))
        if per < 65536:
            raise SystemExit("%s: no 256 MiB __amd_rocclr_copyBuffer dispatch (run with --traffic-calibration)" % d)
        copy[which] = per
        for n, (cnt, tot) in acc.items():
            if n in kern:
                kern[n][which + "_kib"] = tot / cnt
                kern[n][which + "_factor"] = 262144.0 / per
    if args.pmc_mfma:
        # SQ_VALU_MFMA_BUSY_CYCLES (summed over the 1024 SIMDs) against GRBM_GUI_ACTIVE (summed over the 8 XCDs): the share
        # of SIMD clocks in which the matrix pipe is busy; and against the dispatch's own duration at the 2.4 GHz the
        # published peak is quoted at (the two differ by the clock the kernel actually ran at)
        acc = {}
        for r in rows(args.pmc_mfma, "counter_collection.csv"):
            a = acc.setdefault(kname(r), {"ns": 0.0})
            a[r["Counter_Name"]] = a.get(r["Counter_Name"], 0.0) + float(r["Counter_Value"])
            if r["Counter_Name"] == "SQ_VALU_MFMA_BUSY_CYCLES":
                a["ns"] += int(r["End_Timestamp"]) - int(r["Start_Timestamp"])
        for n, c in acc.items():
            if n in kern and c.get("GRBM_GUI_ACTIVE") and c["ns"] > 0:
                busy = c.get("SQ_VALU_MFMA_BUSY_CYCLES", 0.0)
                kern[n]["mfma_busy_frac"] = round(busy / (c["GRBM_GUI_ACTIVE"] / 8.0 * 1024.0), 4)
                kern[n]["mfma_busy_frac_at_2p4ghz"] = round(busy / 1024.0 / (c["ns"] * 2.4), 4)
                kern[n]["shader_clock_ghz"] = round(c["GRBM_GUI_ACTIVE"] / 8.0 / c["ns"], 3)
    out = {"workload": args.workload + ("_w8a8" if args.w8a8 else "") + ("_kv8" if args.kv_int8 else ""),
           "command": args.profile_command, "commit": args.profile_commit, "source_sha256": source_digest(),
           "calibration_copy_reading": copy, "kernels": []}
    for k in sorted(kern.values(), key=lambda k: -k["total_us"]):
        k["avg_us"] = round(k["total_us"] / k["calls"], 3)
        k["total_ms"] = round(k.pop("total_us") / 1e3, 3)
        k["min_us"], k["max_us"] = round(k["min_us"], 3), round(k["max_us"], 3)
        # one instantiation launched over several shapes (grids, in work-items): the average per grid beside the mixed one
        grids = k.pop("by_grid")
        if len(grids) > 1:
            k["by_grid"] = [{"grid": g, "calls": v[0], "avg_us": round(v[1] / v[0], 3)} for g, v in sorted(grids.items(), key=lambda kv: -kv[1][1])]
        for f in ("fetch_kib", "write_kib"):
            if f in k:
                k[f] = round(k[f], 1)
        out["kernels"].append(k)
    with open(args.out, "w") as fh:
        json.dump(out, fh, indent=1)
        fh.write("\n")
    lines = ["| kernel | calls | avg us | min us | max us | total ms | FETCH_SIZE KiB | WRITE_SIZE KiB | HBM bytes per launch |",
             "|---|---|---|---|---|---|---|---|---|"]
    for k in out["kernels"]:
        tb = traffic_bytes(k)
        lines.append("| `%s` | %d | %.2f | %.2f | %.2f | %.2f | %s | %s | %s |" % (
            k["mangled"], k["calls"], k["avg_us"], k["min_us"], k["max_us"], k["total_ms"], k.get("fetch_kib", "-"),
            k.get("write_kib", "-"), tb if tb is not None else "-"))
    for k in out["kernels"]:
        if k.get("by_grid"):
            lines.append("")
            lines.append("`%s` by grid (work-items): " % k["mangled"][:60] +
                         "; ".join("%s: %d launches, %.2f us" % (g["grid"], g["calls"], g["avg_us"]) for g in k["by_grid"]))
    print("\n".join(lines))


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
    prof = load_profile("prefill_w8a8" if args.w8a8 else "prefill") if args.dtype == "f16" else None
    entry = profile_entry(prof, dom)
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
                     "traffic": traffic_bytes(entry), "mfma_busy_frac_pmc": entry.get("mfma_busy_frac") if entry else None,
                     "avg_launch_us_rocprof": entry["avg_us"] if entry else None,
                     "profile": {"file": prof["file"], "commit": prof.get("commit"), "stale": prof["stale"]} if prof and entry else None,
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
    prof = load_profile("attention") if args.dtype == "f16" else None
    entry = profile_entry(prof, "attention")  # (the streaming launch; the merge launch is listed in the profile beside it)
    out = {
        "metric": "GQA decode attention op: achieved HBM GB/s vs peak (configs[1], B=16, L=4096)",
        "value": round(achieved, 1), "unit": "GB/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(elapsed * 1e3 / K, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32 softmax and accumulate over %s K/V" % args.dtype, "data": "synthetic",
        "config": {"workload": "configs[1]: attention op, B=16, Hq=32, Hkv=4, D=64, L=4096, scale 0.125, seq_q=1",
                   "seed": args.seed, "rotating_kv_sets": n, "device_ms_per_call": round(gpu_ms, 4)},
        "roofline": {"bound": "hbm", "kernel": "attn_stream_kernel + attn_merge_kernel", "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic_bytes(entry),
                     "avg_launch_us_rocprof": entry["avg_us"] if entry else None,
                     "profile": {"file": prof["file"], "commit": prof.get("commit"), "stale": prof["stale"]} if prof and entry else None,
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


def time_launches(fn, n_sets, steps, warmup):
    """Average device time of launches fn(i) that follow one another on one stream (each waits for the one before it,
    as the launches of a decode step do), rotating over n_sets operand sets.  fn allocates nothing and launches on the
    current stream; the launches are captured into a hipGraph in chunks of up to 200 and the graph is replayed, so the
    host's per-call cost is not in the figure.  Returns (us per launch, launches timed, wall seconds)."""
    import torch

    for i in range(max(warmup, 1)):  # eager first: function attributes are set outside the capture
        fn(i % n_sets)
    torch.cuda.synchronize()
    chunk = max(1, min(steps, 200))
    reps = max(1, steps // chunk)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for i in range(chunk):
            fn((i * 7) % n_sets)
    graph.replay()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(reps):
        graph.replay()
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return start.elapsed_time(stop) * 1e3 / (reps * chunk), reps * chunk, wall


def read_floor(mynn, shapes, steps=400, warmup=40, pool_bytes=1 << 30):
    """The pure-read floor of a dependent GEMV launch: mynn_gemv_read_probe (the decode GEMV's grid and loads, nothing
    else) over matrices rotating through a 1 GiB pool, so that no launch finds its bytes in the 256 MB Infinity Cache.
    shapes: {name: (N, K)}.  Returns {name: {bytes, us, GBs, frac}, "empty_launch_us": ..}."""
    import torch

    pool = torch.empty(pool_bytes, dtype=torch.uint8, device="cuda")
    pool.fill_(1)
    sink = torch.zeros(4, dtype=torch.uint8, device="cuda")
    lib = mynn.lib()
    cur = lambda: torch.cuda.current_stream().cuda_stream
    out = {}
    for name, (N, K) in shapes.items():
        nbytes = N * K
        stride = (nbytes + 255) // 256 * 256
        n_sets = pool_bytes // stride
        us, _, _ = time_launches(lambda i: mynn.check(lib.mynn_gemv_read_probe(pool.data_ptr() + i * stride, sink.data_ptr(), N, K, 0, cur())),
                                 n_sets, steps, warmup)
        out[name] = {"bytes": nbytes, "us": round(us, 3), "GBs": round(nbytes / us / 1e3, 1),
                     "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4), "rotating_sets": n_sets}
        if "empty_launch_us" not in out:
            e_us, _, _ = time_launches(lambda i: mynn.check(lib.mynn_gemv_read_probe(pool.data_ptr(), sink.data_ptr(), N, K, 1, cur())), 1, steps, warmup)
            out["empty_launch_us"] = round(e_us, 3)
    del pool
    torch.cuda.empty_cache()
    return out


def gemv_main(args, mynn):
    """The dequant GEMV on its own (configs[0] and the metric's second clause): one step = one launch of
    mynn_dequant_gemv, launched back to back on one stream over weight matrices that rotate through more than 256 MB
    (the Infinity Cache), so every launch streams its int8 weights from HBM.  The headline shape is configs[0] exactly
    (f32 x [1,2048], int8 W [5632,2048], f32 per-channel scales, f32 out); the 16-bit shapes of the TinyLlama decode
    step and a 537 MB matrix are timed beside it, each next to the pure-read floor of the same launch geometry."""
    import numpy as np
    import torch

    K_steps = 2000 if args.steps is None else args.steps
    W = 100 if args.warmup is None else args.warmup
    tdt = {"f16": torch.float16, "bf16": torch.bfloat16}[args.dtype]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(args.seed)
    shapes = [("configs[0] f32", 5632, 2048, torch.float32), ("gate_up %s" % args.dtype, 11264, 2048, tdt),
              ("down %s" % args.dtype, 2048, 5632, tdt), ("lm_head %s" % args.dtype, 32000, 2048, tdt),
              ("537 MB matrix %s" % args.dtype, 262144, 2048, tdt)]
    rows = {}
    head = None
    for name, N, Kd, t in shapes:
        nbytes = N * Kd
        n_sets = max(2, -(-(320 << 20) // nbytes))
        Ws = [torch.randint(-127, 128, (N, Kd), generator=gen, device="cuda", dtype=torch.int8) for _ in range(n_sets)]
        sc = (torch.rand((N,), generator=gen, device="cuda") * 9e-3 + 1e-3).to(t)
        x = torch.randn((Kd,), generator=gen, device="cuda", dtype=torch.float32).to(t)
        y = torch.empty((N,), dtype=t, device="cuda")
        code = {torch.float32: mynn.F32, torch.float16: mynn.F16, torch.bfloat16: mynn.BF16}[t]
        lib = mynn.lib()

        def launch(i):
            mynn.check(lib.mynn_dequant_gemv(y.data_ptr(), x.data_ptr(), Ws[i].data_ptr(), sc.data_ptr(), N, Kd, code, code,
                                             torch.cuda.current_stream().cuda_stream))

        us, timed, wall = time_launches(launch, n_sets, K_steps, W)
        eb = 4 if t == torch.float32 else 2
        alg = nbytes + N * eb + Kd * eb + N * eb  # int8 W + scales + activation + output
        row = {"N": N, "K": Kd, "bytes_per_launch": alg, "avg_launch_us": round(us, 3), "GBs": round(alg / us / 1e3, 1),
               "frac": round(alg / us / 1e3 / HBM_PEAK_GBS, 4), "rotating_sets": n_sets, "rotating_MB": round(n_sets * nbytes / 1e6)}
        if head is None:
            launch(0)
            torch.cuda.synchronize()
            head = (name, N, Kd, alg, us, wall, Ws[0], sc, x, y.clone(), timed)
        rows[name] = row
        del Ws
        torch.cuda.empty_cache()
    floor = read_floor(mynn, {n: (N, Kd) for n, N, Kd, _ in shapes[:4]})
    for n in list(rows)[:4]:
        rows[n]["read_floor_us"] = floor[n]["us"]
        rows[n]["read_floor_frac"] = floor[n]["frac"]
    name, N, Kd, alg, us, wall, W0, sc0, x0, y0, timed = head
    prof = load_profile("gemv") if args.dtype == "f16" else None
    entry = profile_entry(prof, "gemv_configs0_f32")
    achieved = alg / us / 1e3
    out = {
        "metric": "dequant-GEMV HBM GB/s vs peak (configs[0]: f32 [1,2048] x int8 [5632,2048], per-channel f32 scales)",
        "value": round(achieved, 1), "unit": "GB/s", "n_gpus": 1, "steps": timed, "warmup": W,
        "ms_per_step": round(wall * 1e3 / timed, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32 accumulate over int8 weights (f32 activation and scales for configs[0]; %s for the decode shapes)" % args.dtype,
        "data": "synthetic",
        "config": {"workload": "configs[0]: DequantizeLinear->MatMul as the fused DequantMatMul, M=1, K=2048, N=5632, f32; launched "
                               "back to back over %d weight matrices (%d MB) so each launch reads HBM" % (rows[name]["rotating_sets"], rows[name]["rotating_MB"]),
                   "seed": args.seed, "shapes": rows, "empty_launch_us": floor["empty_launch_us"],
                   "read_floor": "mynn_gemv_read_probe: the decode GEMV's grid and 16-byte loads with no arithmetic, same launch pattern"},
        "roofline": {"bound": "hbm", "kernel": "dequant_gemv_kernel<f32> (configs[0])", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic_bytes(entry),
                     "avg_launch_us_rocprof": entry["avg_us"] if entry else None,
                     "profile": {"file": prof["file"], "commit": prof.get("commit"), "stale": prof["stale"]} if prof and entry else None,
                     "bytes_per_launch": alg, "avg_launch_us": round(us, 3),
                     "floor": {"bytes": floor[name]["bytes"], "us": floor[name]["us"], "frac": floor[name]["frac"]},
                     "gate_up": rows["gate_up %s" % args.dtype], "largest_matrix": rows["537 MB matrix %s" % args.dtype]},
    }
    if not args.no_cpu_baseline:
        import oracle as orc

        hx, hs = x0.cpu().numpy(), sc0.cpu().numpy()
        hW = W0.cpu().numpy()
        want = orc.dequant_matmul(hx[None, :], hW, hs, orc.F32, orc.F32)[0]
        got = y0.cpu().numpy()
        exact = (hW.astype(np.float64) @ hx.astype(np.float64)) * hs.astype(np.float64)
        out["config"]["max_rel_err_vs_f64_closed_form"] = float(np.max(np.abs(got - exact)) / np.max(np.abs(exact)))
        out["config"]["max_rel_err_vs_oracle"] = float(np.max(np.abs(got - want)) / np.max(np.abs(want)))
        # the C port on the same shape, rotating over host copies of > 256 MB as well; about 10 s of CPU work
        copies = [hW] + [np.ascontiguousarray(np.roll(hW, i + 1, axis=0)) for i in range(31)]
        orc.dequant_matmul(hx[None, :], copies[1], hs, orc.F32, orc.F32)
        n, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < 10.0:
            orc.dequant_matmul(hx[None, :], copies[n % len(copies)], hs, orc.F32, orc.F32)
            n += 1
        cpu = (time.perf_counter() - t0) / n
        out["cpu_baseline"] = {"value": round(alg / cpu / 1e9, 2), "unit": "GB/s", "cores": orc.get_threads(), "kind": "port",
                               "sample": "%d calls of the same configs[0] GEMV (10 s), C port of the reference CPU backend "
                                         "(OpenMP over N, f32), rotating over 32 host copies of W" % n}
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
    if args.kv_pages is None:
        args.kv_pages = 256  # configs[4] names a paged cache
    if args.skinny_ablation:
        mynn.lib().mynn_skinny_set_ablation({"loads": 1, "nomfma": 2}[args.skinny_ablation])
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
    pages = pool = None
    if args.kv_pages:
        # paged cache: one pool for the batch, pages of every sequence interleaved (page = slot * B + sequence)
        assert cfg["max_seq"] % args.kv_pages == 0
        pool = mynn.KvPool(B * cfg["max_seq"] // args.kv_pages, args.kv_pages)
        pshape = (pool.n_pages, cfg["n_kv_heads"], args.kv_pages, cfg["head_dim"])
        for _ in range(cfg["n_layers"]):
            if args.kv_int8:
                kv.append(tuple([torch.randint(-127, 128, pshape, generator=gen, device="cuda", dtype=torch.int8) for _ in range(2)] +
                                [(torch.rand(pshape[:3], generator=gen, device="cuda") * 0.02 + 0.01).to(tdt) for _ in range(2)]))
            else:
                kv.append((torch.randn(pshape, generator=gen, device="cuda", dtype=tdt), torch.randn(pshape, generator=gen, device="cuda", dtype=tdt)))
        pages = mynn.KvPages(pool, B, cfg["max_seq"])
        pages.reserve(ctx)
    for _ in range(0 if args.kv_pages else cfg["n_layers"]):
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
    dec = mynn.Decoder(cfg, weights, batch=B, kv=kv, quant_kv_cache=args.kv_int8, kv_pages=pages)
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
    prof = load_profile("decode_batch_kv8" if args.kv_int8 else "decode_batch") if args.dtype == "f16" else None
    entry = profile_entry(prof, dom)
    out = {
        "metric": "decode tok/s, batch 32 at context 2048, Llama-3-8B-shape int8 (aggregate over the batch)",
        "value": round(B * K / elapsed, 1), "unit": "tok/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32 accumulate over int8 weights, %s activations, %s KV" % (args.dtype, "int8" if args.kv_int8 else args.dtype),
        "data": "synthetic",
        "config": {"workload": "configs[4]: Llama-3-8B-shape int8 decoder, batch 32, context 2048 (caches filled with "
                               "random rows%s), %d decode steps timed" % ((", int8 KV cache" if args.kv_int8 else "") + (", paged KV cache" if args.kv_pages else ""), K),
                   "batch": B, "context": ctx, "launches_per_step": stats["launches_per_step"], "hipgraph": stats["graph"],
                   "kv_page_rows": args.kv_pages or None, "skinny_ablation": args.skinny_ablation,
                   "kv_pages_mapped": (pool.n_pages - pool.free_pages) if pool else None,
                   "seed": args.seed, "step_algorithmic_bytes": step_bytes,
                   "step_hbm_frac": round(step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                   "per_kernel_ms": {k: round(v[1] / 2, 3) for k, v in sorted(agg.items(), key=lambda kv: -kv[1][1])}},
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": traffic_bytes(entry), "avg_launch_us_rocprof": entry["avg_us"] if entry else None,
                     "profile": {"file": prof["file"], "commit": prof.get("commit"), "stale": prof["stale"]} if prof and entry else None,
                     "bytes_per_launch": bytes_tot / calls,
                     "avg_launch_us": round(ms_tot / calls * 1e3, 2)},
    }
    if "attention" in agg:  # the launch with the most time in the step: K and V rows of every sequence at this context
        a_calls, a_ms, _ = agg["attention"]
        a_bytes = float(B) * 2 * kv_row * past
        a_entry = profile_entry(prof, "attention")
        out["roofline"]["attention"] = {"bytes_per_launch": a_bytes, "avg_launch_us": round(a_ms / a_calls * 1e3, 2),
                                        "frac": round(a_bytes / (a_ms / a_calls * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                                        "avg_launch_us_rocprof": a_entry["avg_us"] if a_entry else None,
                                        "traffic": traffic_bytes(a_entry)}
    dec.close()
    if pages:
        pages.close(), pool.close()
    print(json.dumps(out))


def short_prefill(mynn, cfg, weights, seed, weight_set=None):
    """Three timed passes (after three untimed ones) of the 8 x 1024 prefill (configs[3]) over the same weights (and, as in
    a session, the same weight set as the decode executor), outside any timed decode region: the matrix-core side of the
    path, for the same JSON line."""
    import numpy as np
    import torch

    B, S = PREFILL_BATCH, PREFILL_LEN
    pcfg = dict(cfg, max_seq=S)
    pre = mynn.Decoder(pcfg, weights, seq_q=S, batch=B, weight_set=weight_set)
    ids = np.random.default_rng(seed).integers(0, cfg["vocab"], B * S)
    pos = np.arange(S)
    for _ in range(3):  # (the matrix pipes' clock settles over the first passes)
        pre.step(ids, pos, 0, S)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(3):
        pre.step(ids, pos, 0, S)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / 3
    agg = {}
    for name, kms, _, flops in pre.profile(ids, pos, 0, S):
        a = agg.setdefault(name, [0.0, 0.0])
        a[0] += kms
        a[1] += flops
    step_flops = sum(v[1] for v in agg.values())
    gu = agg.get("linear_gateup_swiglu")
    out = {"workload": "configs[3]: %d x %d prefill, same weights, 3 warm-up + 3 timed passes" % (B, S), "ms_per_pass": round(ms, 3),
           "tok_s": round(B * S / (ms * 1e-3), 1), "launches_per_pass": pre.stats()["launches_per_step"],
           "step_mfma_frac": round(step_flops / (ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4),
           "gateup_TFLOPs": round(gu[1] / (gu[0] * 1e-3) / 1e12, 1) if gu and gu[0] > 0 else None}
    pre.close()
    torch.cuda.empty_cache()
    return out


def decode_variants(mynn, cfg, weights, wset, prompt, K, tdt):
    """The same batch-1 decode through the two other cache forms of the executor, on the same weights (and weight
    set), outside the timed region of the main figure: a paged KV cache (device-resident loop, as the main figure) and
    the streaming (sink + ring) cache, whose steps are host round trips because the ring inputs change per step."""
    import torch

    out = {}
    P = 128
    pool = mynn.KvPool(cfg["max_seq"] // P, P)
    pages = mynn.KvPages(pool, 1, cfg["max_seq"])
    kv = pool.buffers(cfg["n_layers"], cfg["n_kv_heads"], cfg["head_dim"], tdt)
    dec = mynn.Decoder(cfg, weights, kv=kv, kv_pages=pages, weight_set=wset)
    pages.reserve(cfg["max_seq"])
    first = None
    for i, t in enumerate(prompt):
        first, _ = dec.step([t], [i], i, i + 1)
    dec.decode_loop(first[0], len(prompt), 16)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    dec.decode_loop(first[0], len(prompt), K)
    torch.cuda.synchronize()
    el = time.perf_counter() - t0
    out["paged_kv_bs1"] = {"tok_s": round(K / el, 1), "ms_per_step": round(el * 1e3 / K, 4), "kv_page_rows": P,
                           "launches_per_step": dec.stats()["launches_per_step"]}
    dec.close(), pages.close(), pool.close()
    del kv

    # the session call a user of the reference makes (LlmSession::generate_ids): prompt token by token, then runs of the
    # device-resident loop
    gdec = mynn.Decoder(cfg, weights, weight_set=wset)
    llm = mynn.LlmSession(gdec, eos=-1)
    llm.generate_ids(prompt, 1)
    llm.reset()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    llm.generate_ids(prompt, 1)
    t1 = time.perf_counter()
    llm.reset()
    llm.generate_ids(prompt, 1 + K)
    t2 = time.perf_counter()
    gen_s = (t2 - t1) - (t1 - t0)
    out["llm_session_generate_ids"] = {"new_tokens": K, "tok_s_after_the_prompt": round(K / gen_s, 1) if gen_s > 0 else None,
                                       "prompt_tok_s": round(len(prompt) / (t1 - t0), 1)}
    llm.close(), gdec.close()

    sink, window = 4, 252
    sdec = mynn.Decoder(cfg, weights, streaming_kv=True, weight_set=wset)
    llm = mynn.LlmSession(sdec, eos=-1, streaming=(sink, window))
    n1 = sink + window - len(prompt) - 8  # stays inside the window
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ids = llm.generate_ids(prompt, n1)
    t1 = time.perf_counter()
    n2 = 256  # second turn: every step past the window
    llm.generate_ids(ids[-1:] + prompt[:7], 8)  # (walks over the edge)
    t2 = time.perf_counter()
    llm.generate_ids(prompt[:1], n2)
    t3 = time.perf_counter()
    out["streaming_kv_bs1"] = {"sink": sink, "window": window,
                               "tok_s_inside_window": round((len(prompt) + n1 - 1) / (t1 - t0), 1),
                               "tok_s_past_window": round(n2 / (t3 - t2), 1), "past_len": llm.past_len,
                               "launches_per_step": sdec.stats()["launches_per_step"],
                               "what": "LlmSession.generate_ids: one host round trip per token (ring inputs per step)"}
    llm.close(), sdec.close()
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--workload", choices=["decode", "prefill", "attention", "decode_batch", "gemv"], default="decode")
    ap.add_argument("--steps", type=int, default=None, help="default 256 (decode) / 5 (prefill)")
    ap.add_argument("--warmup", type=int, default=None, help="default 16 (decode) / 2 (prefill)")
    ap.add_argument("--dtype", choices=["f16", "bf16"], default="f16")
    ap.add_argument("--seed", type=int, default=1234)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-prefill", action="store_true", help="decode: leave the short prefill run (config.prefill) out")
    ap.add_argument("--cpu-steps", type=int, default=96, help="decode: generated positions the CPU port is timed (and tokens checked) on")
    ap.add_argument("--traffic-calibration", action="store_true",
                    help="first run one 256 MiB device-to-device copy (a kernel of known traffic, for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--w8a8", action="store_true",
                    help="prefill: quantise activations per row and run every linear as int8 x int8 (Options::quantize_activations)")
    ap.add_argument("--kv-int8", action="store_true",
                    help="decode / decode_batch: int8 KV cache with per-token scales (BuildOptions::quant_kv_cache)")
    ap.add_argument("--kv-pages", type=int, default=None, metavar="ROWS",
                    help="decode_batch: rows per page of the paged KV cache (kv_page_rows), one pool for the batch; default 256, "
                         "0 = contiguous caches")
    ap.add_argument("--skinny-ablation", choices=["loads", "nomfma"], default=None,
                    help="decode_batch: run the gate/up few-row GEMM as its loads alone / without its MFMAs (garbage results: "
                         "only the launch duration is meaningful)")
    ap.add_argument("--weight-arena", action="store_true", help="decode: all weights in one allocation in execution order (weight_arena)")
    ap.add_argument("--unfused", action="store_true", help="decode: every op a launch of its own (unfused_decode)")
    ap.add_argument("--check-tokens", type=int, default=0,
                    help="also compare the first N generated tokens with the oracle generating freely (slow: CPU decode)")
    ap.add_argument("--summarize-rocprof", metavar="DIR",
                    help="no GPU work: read rocprofv3 csv output of this script under DIR (kernel trace, mangled names) and "
                         "write the profile JSON given by --out")
    ap.add_argument("--pmc-fetch", metavar="DIR", help="with --summarize-rocprof: the --pmc FETCH_SIZE run")
    ap.add_argument("--pmc-write", metavar="DIR", help="with --summarize-rocprof: the --pmc WRITE_SIZE run")
    ap.add_argument("--pmc-mfma", metavar="DIR", help="with --summarize-rocprof: the --pmc SQ_VALU_MFMA_BUSY_CYCLES GRBM_GUI_ACTIVE run")
    ap.add_argument("--out", help="with --summarize-rocprof: the JSON file to write")
    ap.add_argument("--profile-command", default="", help="with --summarize-rocprof: the command line that was profiled")
    ap.add_argument("--profile-commit", default="", help="with --summarize-rocprof: the commit the library was built from")
    args = ap.parse_args()
    if args.summarize_rocprof:
        return summarize_rocprof(args)
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
    if args.workload == "gemv":
        return gemv_main(args, mynn)
    K = 256 if args.steps is None else args.steps
    W = 16 if args.warmup is None else args.warmup
    # the cache of configs[2] holds 128 + 256 rows; longer runs get a longer cache (whole 128-row pages, up to the 2048 rows
    # the single-launch layer covers at head_dim 64: the workload stays the same kernels)
    need = PROMPT_LEN + max(K, W)
    if need > cfg["max_seq"]:
        cfg["max_seq"] = (need + 127) // 128 * 128
    if cfg["max_seq"] > 2048:
        raise SystemExit("bench.py: --steps / --warmup of at most %d fit this workload (128 prompt rows + the generated ones <= 2048)"
                         % (2048 - PROMPT_LEN))

    weights = make_weights(cfg, dt, args.seed)
    torch.cuda.synchronize()
    wset = mynn.WeightSet(cfg, weights)  # one set of derived weight copies for the decode and the prefill executor
    dec = mynn.Decoder(cfg, weights, quant_kv_cache=args.kv_int8, quantize_activations=args.w8a8, unfused_decode=args.unfused,
                       weight_arena=args.weight_arena, weight_set=wset)
    stats = dec.stats()
    rng = np.random.default_rng(args.seed)
    prompt = rng.integers(0, cfg["vocab"], PROMPT_LEN).tolist()

    # prompt through the decode path, token by token (the reference's path without a prefill session)
    # (each of these steps is a host round trip: inputs up, graph replay, token down -- timed for the record)
    first = None
    t_host = None
    prompt_choice = []  # the greedy token after each prompt position (compared with the CPU baseline's below)
    for i, t in enumerate(prompt):
        if i == 16:
            torch.cuda.synchronize()
            t_host = time.perf_counter()
        first, _ = dec.step([t], [i], i, i + 1)
        prompt_choice.append(first[0])
    host_tok_s = (PROMPT_LEN - 16) / (time.perf_counter() - t_host)
    first = first[0]

    loop = dec.decode_loop
    if W > 0:
        loop(first, PROMPT_LEN, W)  # untimed; its KV rows are overwritten below
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    toks = loop(first, PROMPT_LEN, K)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    generated = [first] + toks[:-1]
    ms_per_step = elapsed * 1e3 / K
    tok_s = K / elapsed

    # ---- per-launch durations: HIP events tied to every launch of eager steps at contexts spread over the timed
    # range, on the executor's own stream.  The K / V rows an attention launch reads depend on the context, which the
    # executor's own byte count leaves out: added here.
    KD = cfg["n_kv_heads"] * cfg["head_dim"]
    agg = {}
    n_prof = 8
    for j in range(n_prof):
        past = PROMPT_LEN + (j * (K - 1)) // max(n_prof - 1, 1)
        for name, ms, nbytes, _ in dec.profile_step(generated[min(past - PROMPT_LEN, K - 1)], past):
            if "attention" in name:
                nbytes += 2.0 * ((KD + cfg["n_kv_heads"] * eb) if args.kv_int8 else KD * eb) * past
            a = agg.setdefault(name, [0, 0.0, 0.0])
            a[0] += 1
            a[1] += ms
            a[2] += nbytes
    prof = load_profile("decode") if (args.dtype == "f16" and not (args.kv_int8 or args.w8a8 or args.unfused)) else None

    def launch_roofline(role):
        """Algorithmic bytes per launch over the launch's average duration: by rocprofv3's kernel trace of this
        script where the tracked profile still matches the built kernel (`achieved`), and by the events of this
        run (`achieved_events`)."""
        calls, ms_tot, bytes_tot = agg[role]
        per_launch, ev_us = bytes_tot / calls, ms_tot / calls * 1e3
        entry = profile_entry(prof, role)
        ev_gbs = per_launch / (ev_us * 1e-6) / 1e9
        r = {"kernel": role, "mangled": entry["mangled"] if entry else None, "bytes_per_launch": round(per_launch),
             "avg_launch_us_events": round(ev_us, 3), "achieved_events": round(ev_gbs, 1),
             "frac_events": round(ev_gbs / HBM_PEAK_GBS, 4),
             "avg_launch_us_rocprof": entry["avg_us"] if entry else None, "traffic": traffic_bytes(entry)}
        if entry:
            gbs = per_launch / (entry["avg_us"] * 1e-6) / 1e9
            r.update({"achieved": round(gbs, 1), "frac": round(gbs / HBM_PEAK_GBS, 4), "duration_from": "rocprofv3 kernel trace"})
        else:
            r.update({"achieved": round(ev_gbs, 1), "frac": round(ev_gbs / HBM_PEAK_GBS, 4),
                      "duration_from": "hip events (no tracked profile matches the built kernel)"})
        return r

    dom = max(agg, key=lambda k: agg[k][1])  # the launch with the largest total time in the step
    gemv = {k: v for k, v in agg.items() if k.startswith("gemv_")}
    all_gemv_gbs = sum(v[2] for v in gemv.values()) / (sum(v[1] for v in gemv.values()) * 1e-3) / 1e9 if gemv else None
    step_bytes = algorithmic_bytes_per_token(cfg, eb, PROMPT_LEN + K // 2)
    roof = {"bound": "hbm", "peak": HBM_PEAK_GBS, "unit": "GB/s"}
    roof.update(launch_roofline(dom))
    roof["profile"] = {"file": prof["file"], "commit": prof.get("commit"), "stale": prof["stale"]} if prof else None
    if "gemv_norm_gateup_swiglu" in agg:  # the dequant GEMV that moves the most bytes, whichever launch dominates
        roof["gateup_gemv"] = launch_roofline("gemv_norm_gateup_swiglu")
    if "gemv_down_residual" in agg:
        roof["down_gemv"] = launch_roofline("gemv_down_residual")
    roof["all_gemv_GBs"] = round(all_gemv_gbs, 1) if all_gemv_gbs else None

    variant = (", int8 KV cache" if args.kv_int8 else "") + (", int8 activations (W8A8)" if args.w8a8 else "") + \
              (", one op per launch" if args.unfused else "")
    out = {
        "metric": "decode tok/s bs1 TinyLlama-shape int8; dequant-GEMV HBM GB/s vs peak",
        "value": round(tok_s, 2), "unit": "tok/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32 accumulate over int8 weights, %s activations/KV" % args.dtype, "data": "synthetic",
        "config": {"workload": "configs[2]: TinyLlama-1.1B-shape int8 decoder, batch 1 greedy decode, 128 prompt tokens "
                               "fed through the decode path then %d generated (timed: the generated tokens)%s" % (K, variant),
                   "prompt_len": PROMPT_LEN, "max_seq": cfg["max_seq"], "launches_per_step": stats["launches_per_step"],
                   "hipgraph": stats["graph"], "seed": args.seed,
                   "host_roundtrip_tok_s": round(host_tok_s, 1),
                   "step_algorithmic_bytes": step_bytes,
                   "step_hbm_frac": round(step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                   # average duration of every launch of the step (HIP events, eager steps)
                   "per_launch_us": {k: round(v[1] / v[0] * 1e3, 2) for k, v in sorted(agg.items(), key=lambda kv: -kv[1][1])}},
        "roofline": roof,
    }
    dec.close()
    # the pure-read floor of the two dequant-GEMV launches (same grid and loads, no arithmetic, dependent launches over
    # rotating matrices): what a launch of that geometry needs just to pull its weight bytes in
    H, F = cfg["hidden"], cfg["ffn"]
    fl = read_floor(mynn, {"gateup": (2 * F, H), "down": (H, F)})
    roof["floor"] = {"gateup": {k: fl["gateup"][k] for k in ("bytes", "us", "frac")},
                     "down": {k: fl["down"][k] for k in ("bytes", "us", "frac")}, "empty_launch_us": fl["empty_launch_us"],
                     "what": "mynn_gemv_read_probe: weight bytes of one launch / its average duration, 400 dependent launches "
                             "over matrices rotating through 1 GiB"}
    if not args.no_prefill and not (args.kv_int8 or args.w8a8 or args.unfused):
        out["config"]["prefill"] = short_prefill(mynn, cfg, weights, args.seed, wset)
        out["config"]["weight_set"] = wset.stats()
        out["config"]["variants"] = decode_variants(mynn, cfg, weights, wset, prompt, K, torch.float16 if args.dtype == "f16" else torch.bfloat16)

    if not args.no_cpu_baseline:
        import oracle as orc

        hw = to_host_weights(weights)
        # The oracle under three f32 summation orders (the reference leaves the order open), each with its own KV
        # cache, on the GPU's token stream: the prompt, then the first n_cpu generated positions -- the same contexts
        # the timed GPU steps start with.  The first order's forward calls at those contexts are the timed CPU sample.
        n_cpu = min(args.cpu_steps, K)
        ref = orc.SummationOrders(dict(cfg), hw, quant_kv_cache=args.kv_int8, quantize_activations=args.w8a8)
        stream = prompt + generated
        gpu_choice = prompt_choice + generated[1:]  # the GPU's greedy token after each position of the stream
        counts = {"identical": 0, "order_dependent": 0, "within_order_noise": 0, "different": 0}
        notes = []
        for i in range(PROMPT_LEN + n_cpu):
            if i == PROMPT_LEN:
                ref.seconds_first = 0.0
            rows = [l[0] for l in ref.forward([stream[i]], [i], i, i + 1, False)]
            if i >= len(gpu_choice):
                continue
            verdict, choices = ref.judge(rows, gpu_choice[i])
            if verdict != "identical":
                lf = orc.to_f32(rows[0], dt)
                gap, noise = float(lf[choices[0]] - lf[gpu_choice[i]]), ref.order_noise(rows)
                spacing = 2.0 ** (-11 if dt == orc.F16 else -8) * abs(float(lf[choices[0]]))
                notes.append({"step": i, "oracle_by_order": sorted(set(choices)), "orders_tried": len(choices), "gpu": gpu_choice[i],
                              "verdict": verdict, "oracle_gap_in_16bit_spacings": round(gap / spacing, 2),
                              "largest_logit_shift_between_orders_in_16bit_spacings": round(noise / spacing, 2)})
            counts[verdict] += 1
        cpu_elapsed = ref.seconds_first
        ref.close()
        out["cpu_baseline"] = {"value": round(n_cpu / cpu_elapsed, 3), "unit": "tok/s", "cores": orc.get_threads(),
                               "kind": "port",
                               "sample": "%d decode steps at contexts %d..%d (the contexts the timed GPU steps start with) of the same "
                                         "model and token stream, C port of the reference CPU backend, OpenMP over N"
                                         % (n_cpu, PROMPT_LEN, PROMPT_LEN + n_cpu - 1)}
        checked = sum(counts.values())
        out["config"]["tokens_identical_to_oracle"] = counts["identical"] == checked
        out["config"]["tokens_identical_or_order_dependent"] = counts["different"] + counts["within_order_noise"] == 0
        out["config"]["tokens_checked"] = {"steps": checked, "identical": counts["identical"], "order_dependent": counts["order_dependent"],
                                           "within_order_noise": counts["within_order_noise"], "different": counts["different"], "summation_orders": {"whole_stream": list(ref.lanes), "disputed_steps": list(ref.step_lanes)},
                                           "disagreements": notes,
                                           "what": "greedy choice after each of the first %d positions of the stream (prompt and generated), "
                                                   "oracle and GPU on the same context; the oracle follows the stream under four f32 summation "
                                                   "orders (16 / 8 / 32 / 64 partial sums, a KV cache each) and repeats a disputed step under "
                                                   "1 / 2 / 4; a GPU token that is not the first order's choice counts as order_dependent only "
                                                   "if it is the choice under another order or the orders disagree among themselves; of the rest, "
                                                   "within_order_noise where the oracle's own gap between the two tokens is below twice the "
                                                   "largest shift any logit of that step shows between the oracle's orders, different "
                                                   "otherwise" % checked}
        if args.check_tokens:
            n = min(args.check_tokens, K)
            ref2 = orc.Model(dict(cfg), hw)
            want = ref2.generate(prompt, n)
            out["config"]["generated_identical_to_free_running_oracle"] = {"tokens": n, "identical_prefix": next(
                (i for i in range(n) if want[i] != generated[i]), n)}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
