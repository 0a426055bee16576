"""Helpers shared by the GPU parity tests: load the product through its C ABI, move oracle
arrays (numpy, 16-bit floats as uint16 bit patterns) to the device and back."""
import importlib

import numpy as np

import oracle as orc

mynn = importlib.import_module("my-nn-engine_amd")

# max-abs-rel bound for float outputs (f32: two summation orders of a few thousand f32 terms; 16-bit: the reference's own bound)
TOL = {orc.F32: 5e-5, orc.BF16: 1e-2, orc.F16: 1e-2}


def torch_dtype(dt):
    import torch

    return {orc.F32: torch.float32, orc.BF16: torch.bfloat16, orc.F16: torch.float16}[dt]


def to_dev(a, dt=None):
    """numpy storage array -> cuda tensor (uint16 bit patterns become bf16/f16 per dt)."""
    import torch

    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        t = torch.from_numpy(a.view(np.int16)).cuda().view(torch_dtype(dt))
    else:
        t = torch.from_numpy(a).cuda()
    return t


def to_host(t):
    """cuda tensor -> numpy storage array (bf16/f16 come back as uint16 bit patterns)."""
    import torch

    t = t.detach().contiguous()
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16).cpu().numpy().view(np.uint16)
    return t.cpu().numpy()


def f32(a, dt):
    return orc.to_f32(a, dt)


def greedy_compare(cfg, weights, dec, prompt, n_new, dt, **oracle_options):
    """Runs the GPU decoder greedily (prompt fed token by token, as LlmSession does without a
    prefill session) and the oracle on the SAME token stream (teacher-forced with the GPU's
    choices, so both always see the same context), the oracle under three f32 summation orders
    (oracle.SummationOrders).  Returns (gpu_ids, oracle_ids, undecided, different):
    oracle_ids[i] is the first order's greedy choice at step i; the two lists hold the steps where
    the GPU's token is not that choice -- undecided where the oracle's own arithmetic does not
    separate the two tokens (the choice flips under another summation order, or the gap is inside
    the shifts the orders show among themselves: SummationOrders.judge), different otherwise (a
    failure)."""
    ref = orc.SummationOrders(cfg, weights, **oracle_options)
    gpu_ids, ref_ids, undecided, different = [], [], [], []
    stream = list(prompt)
    pos = 0
    while len(gpu_ids) < n_new:
        t = stream[pos]
        rows = [l[0] for l in ref.forward([t], [pos], pos, pos + 1, False)]
        nxt, _ = dec.step([t], [pos], pos, pos + 1)
        pos += 1
        if pos >= len(prompt):
            verdict, choices = ref.judge(rows, nxt[0])
            gpu_ids.append(nxt[0])
            ref_ids.append(choices[0])
            if verdict in ("order_dependent", "within_order_noise"):
                undecided.append((len(gpu_ids) - 1, verdict, sorted(set(choices)), nxt[0]))
            elif verdict == "different":
                different.append((len(gpu_ids) - 1, sorted(set(choices)), nxt[0]))
            stream.append(nxt[0])
    ref.close()
    return gpu_ids, ref_ids, undecided, different


def both_acceptable(cfg, weights, stream, candidates, dt, **oracle_options):
    """Two library paths part at the token after `stream`: every candidate must be a choice the oracle can make there
    -- its greedy token under one of the summation orders, or the orders disagree among themselves."""
    ref = orc.SummationOrders(cfg, weights, **oracle_options)
    rows = None
    for i, t in enumerate(stream):
        rows = [l[0] for l in ref.forward([t], [i], i, i + 1, False)]
    verdicts = [ref.judge(rows, c) for c in candidates]
    ref.close()
    return all(v != "different" for v, _ in verdicts), verdicts
