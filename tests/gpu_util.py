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


def greedy_compare(ref, dec, prompt, n_new, dt):
    """Runs the GPU decoder greedily (prompt fed token by token, as LlmSession does without a
    prefill session) and the oracle on the SAME token stream (teacher-forced with the GPU's
    choices, so both always see the same context).  Returns (gpu_ids, oracle_ids, near_ties):
    oracle_ids[i] is the oracle's greedy choice at step i; near_ties lists the steps where the two
    differ together with the oracle's logit gap between its choice and the GPU's, in units of the
    16-bit spacing at the top logit."""
    ulp = {orc.F32: 2.0 ** -23, orc.BF16: 2.0 ** -8, orc.F16: 2.0 ** -11}[dt]
    gpu_ids, ref_ids, near = [], [], []
    stream = list(prompt)
    pos = 0
    tok_gpu = None
    while len(gpu_ids) < n_new:
        t = stream[pos]
        logits = ref.forward([t], [pos], pos, pos + 1, False)[0]
        nxt, _ = dec.step([t], [pos], pos, pos + 1)
        pos += 1
        if pos >= len(prompt):
            lf = orc.to_f32(logits, dt)
            r = orc.argmax_last(logits, dt)
            gpu_ids.append(nxt[0])
            ref_ids.append(r)
            if r != nxt[0]:
                gap = float(lf[r] - lf[nxt[0]])
                near.append((len(gpu_ids) - 1, gap / (ulp * max(abs(float(lf[r])), 1e-30))))
            stream.append(nxt[0])
    return gpu_ids, ref_ids, near
