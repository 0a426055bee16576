"""CPU-side checks of the boundary: the library loads, exports every symbol include/mynn_hip.h
declares (and the ctypes table names each of them), and the host-side pieces of crates/llm that
need no GPU behave like the reference's tests say."""
import ctypes as C
import importlib
import json
import os
import re

import numpy as np
import pytest

import oracle as orc
from conftest import GOLDEN, ROOT

mynn = importlib.import_module("my-nn-engine_amd")


def header_symbols():
    text = open(os.path.join(ROOT, "include", "mynn_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = set(re.findall(r"\b((?:mynn_|model|alloc_pinned|free_pinned)\w*)\s*\(", text))
    names.discard("mynn_step_fn")
    return names


def test_library_exports_every_declared_symbol():
    names = header_symbols()
    assert len(names) >= 40
    assert mynn.missing_symbols() == []
    assert names == set(mynn.SIGNATURES), (names ^ set(mynn.SIGNATURES))
    lib = mynn.lib()
    for n in names:
        assert hasattr(lib, n), n
    assert lib.mynn_version() >= 1


def test_model_config_mirror_matches_the_header_field_for_field():
    text = open(os.path.join(ROOT, "include", "mynn_hip.h")).read()
    body = text[:text.index("} mynn_model_config;")]
    body = body[body.rindex("typedef struct {"):]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    fields = re.findall(r"\b(int|float)\s+([a-z_0-9, ]+);", body)
    names, kinds = [], []
    for kind, group in fields:
        for n in group.split(","):
            names.append(n.strip())
            kinds.append(kind)
    mirror = mynn.ModelConfig._fields_
    assert names == [n for n, _ in mirror]
    assert all((t is C.c_float) == (k == "float") for (_, t), k in zip(mirror, kinds))
    assert C.sizeof(mynn.ModelConfig) == 4 * len(names)


def test_rejected_arguments_return_status_not_exit():
    lib = mynn.lib()
    rc = lib.mynn_dequant_gemv(None, None, None, None, 8, 16, 2, 2, None)
    assert rc == -1 and b"bad operand" in lib.mynn_last_error()
    assert lib.model_init(None, None) is None  # not configured / null arrays


def test_kv_pool_is_host_side_bookkeeping():
    """The free list of a paged KV cache lives in host memory: it can be made, asked and destroyed without a GPU;
    bad sizes and the calls that would need the device with a null handle come back as errors."""
    lib = mynn.lib()
    for bad in ((0, 64), (4, 48), (4, 16), (-1, 256)):
        assert lib.mynn_kv_pool_create(*bad) is None and b"power of two" in lib.mynn_last_error()
    pool = mynn.KvPool(7, 128)
    assert pool.free_pages == 7
    assert lib.mynn_kv_pages_create(pool.handle, 0, 256) is None   # batch
    assert lib.mynn_kv_pages_create(pool.handle, 2, 200) is None   # not a multiple of the page
    assert lib.mynn_kv_pages_create(None, 2, 256) is None
    assert lib.mynn_kv_pages_reserve(None, 10) == -1 and lib.mynn_kv_pages_release(None) == -1
    assert lib.mynn_kv_pages_mapped_rows(None) == 0 and lib.mynn_kv_pages_table(None) is None
    assert lib.mynn_kv_pool_free_pages(None) == -1
    pool.close()
    assert pool.handle is None


def test_host_quantiser_known_answers_and_oracle_agreement():
    # crates/llm/tests/quantize.rs:106-159
    w = np.array([[127, -127, 0, 64], [2, -1, 0, 0.5], [0, 0, 0, 0]], np.float32)
    q, s = mynn.quantize_per_channel(w, mynn.BF16)
    assert q.tolist() == [[127, -127, 0, 64], [127, -64, 0, 32], [0, 0, 0, 0]]
    assert np.allclose(orc.to_f32(s, orc.BF16), [1.0, 2 / 127, 1.0], atol=1e-3)
    rng = np.random.default_rng(0)
    w = (rng.standard_normal((257, 640)) * 0.02).astype(np.float32)
    for dt in (orc.F32, orc.BF16, orc.F16):
        q1, s1 = mynn.quantize_per_channel(w, dt)
        q2, s2 = orc.quantize_per_channel(w, dt)
        assert np.array_equal(q1, q2) and np.array_equal(s1, s2)


@pytest.mark.parametrize("dt", [orc.F32, orc.BF16, orc.F16])
def test_host_rope_table_matches_oracle(dt):
    c1, s1 = mynn.rope_table(384, 64, 10000.0, dt)
    c2, s2 = orc.rope_table(384, 64, 10000.0, dt)
    assert np.array_equal(c1, c2) and np.array_equal(s1, s2)


def test_mock_step_session_follows_logit_table():
    """crates/llm/tests/mock_decode.rs: a 6-token logit table, prompt [0,1,2] -> [3,4,5,0,1];
    past_len counts every decode step; a stop rewinds it; an empty prompt yields nothing."""
    table = json.load(open(os.path.join(GOLDEN, "mock_decode", "expected_sequence.json")))
    vocab = table["vocab"]
    calls = []

    def step(user, token, past_len):
        calls.append((token, past_len))
        return (token + 1) % vocab

    lib = mynn.lib()
    cb = mynn.STEP_FN(step)
    h = lib.mynn_llm_create_with_step(cb, None, 16, 999)
    prompt = np.array([0, 1, 2], np.int64)
    out = np.empty(16, np.int64)
    n = lib.mynn_llm_generate_ids(h, prompt.ctypes.data_as(C.c_void_p), 3, 5, out.ctypes.data_as(C.c_void_p))
    assert n == 5 and out[:5].tolist() == [3, 4, 5, 0, 1] == table["sequence"][2:7]
    assert lib.mynn_llm_past_len(h) == 7 and [c[1] for c in calls] == list(range(7))
    lib.mynn_llm_set_past_len(h, 5)  # stop-string rewind (session.rs:411-424)
    assert lib.mynn_llm_past_len(h) == 5
    lib.mynn_llm_reset(h)
    assert lib.mynn_llm_generate_ids(h, prompt.ctypes.data_as(C.c_void_p), 0, 5, out.ctypes.data_as(C.c_void_p)) == 0
    # PromptTooLong: 17 tokens into max_seq 16
    long = np.arange(17, dtype=np.int64) % vocab
    assert lib.mynn_llm_generate_ids(h, long.ctypes.data_as(C.c_void_p), 17, 1, out.ctypes.data_as(C.c_void_p)) == -4
    # eos stops the loop: eos = 4 -> [3, 4]
    h2 = lib.mynn_llm_create_with_step(cb, None, 16, 4)
    n = lib.mynn_llm_generate_ids(h2, prompt.ctypes.data_as(C.c_void_p), 3, 5, out.ctypes.data_as(C.c_void_p))
    assert n == 2 and out[:2].tolist() == [3, 4]
    lib.mynn_llm_destroy(h), lib.mynn_llm_destroy(h2)


def test_bench_refuses_more_than_one_gpu():
    """bench.py --gpus N with N > 1 (or a multi-rank launch) exits with a message instead of measuring anything."""
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2 and "ONE GPU" in r.stderr and not r.stdout.strip()
    env = dict(os.environ, WORLD_SIZE="4")
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py")], capture_output=True, text=True, timeout=120, env=env)
    assert r.returncode == 2 and "ONE GPU" in r.stderr
