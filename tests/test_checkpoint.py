"""Checkpoint reader, offline int8 quantiser and upload (crates/llm/src/hf_weights.rs, quantize.rs)."""
import importlib
import json
import os
import struct

import numpy as np
import pytest

import oracle as orc
import llm_weights

mynn = importlib.import_module("my-nn-engine_amd")
TINY = os.path.join(os.path.dirname(__file__), "golden", "tiny-llama-random")


def read_safetensors_py(path):
    """Independent reader: 8-byte little-endian header length, JSON header, raw little-endian data."""
    with open(path, "rb") as f:
        n = struct.unpack("<Q", f.read(8))[0]
        hdr = json.loads(f.read(n))
        data = f.read()
    out = {}
    for name, info in hdr.items():
        if name == "__metadata__":
            continue
        a, b = info["data_offsets"]
        npdt = {"F32": np.float32, "BF16": np.uint16, "F16": np.uint16, "I8": np.int8}[info["dtype"]]
        out[name] = (info["dtype"], np.frombuffer(data[a:b], npdt).reshape(info["shape"]))
    return out


def test_reader_matches_an_independent_parse_of_the_reference_fixture():
    w = mynn.Weights(TINY)  # directory: falls through to model.safetensors (hf_weights.rs:75-91)
    want = read_safetensors_py(os.path.join(TINY, "model.safetensors"))
    assert sorted(w.names()) == sorted(want)
    for name, (dtype, arr) in want.items():
        code, shape, got = w.find(name)
        assert code == {"F32": mynn.F32, "BF16": mynn.BF16, "F16": mynn.F16, "I8": mynn.I8}[dtype]
        assert shape == arr.shape and np.array_equal(got, arr)
    with pytest.raises(mynn.MynnError):
        w.find("model.layers.99.mlp.up_proj.weight")
    w.close()
    with pytest.raises(mynn.MynnError):
        mynn.Weights(os.path.join(TINY, "config.json"))  # not a safetensors file
    with pytest.raises(mynn.MynnError):
        mynn.Weights(os.path.dirname(TINY))  # a directory without checkpoints


def test_quantize_safetensors_int8_follows_the_reference_file_rules(tmp_path):
    """quantize.rs:28-42, 313-337: the nine name patterns become int8 + '<name>.scale' (bf16), the
    rest is copied; values follow quantize_per_channel (pinned by the reference's known answers in
    test_oracle_closed_forms.py)."""
    dst = tmp_path / "model.int8.safetensors"
    nq, npass = mynn.quantize_safetensors_int8(TINY, dst)
    src = read_safetensors_py(os.path.join(TINY, "model.safetensors"))
    got = read_safetensors_py(dst)
    pats = ("q_proj.weight", "k_proj.weight", "v_proj.weight", "o_proj.weight", "gate_proj.weight", "up_proj.weight",
            "down_proj.weight", "lm_head.weight", "embed_tokens.weight")
    qnames = [n for n in src if n.endswith(pats)]
    assert nq == len(qnames) == 16 and npass == len(src) - nq
    assert set(got) == set(src) | {n + ".scale" for n in qnames}
    for n, (dtype, arr) in src.items():
        if n in qnames:
            q, s = orc.quantize_per_channel(arr, orc.BF16)
            assert got[n][0] == "I8" and np.array_equal(got[n][1], q)
            assert got[n + ".scale"][0] == "BF16" and np.array_equal(got[n + ".scale"][1], s)
        else:
            assert got[n][0] == dtype and np.array_equal(got[n][1], arr)
    # a directory holding model.int8.safetensors is opened through it (hf_weights.rs:77-80)
    w = mynn.Weights(tmp_path)
    assert w.find("lm_head.weight")[0] == mynn.I8 and "lm_head.weight.scale" in w.names()


def test_sharded_checkpoint_through_the_index_file(tmp_path):
    """model.safetensors.index.json -> distinct shard files (hf_weights.rs:99-118)."""
    src = read_safetensors_py(os.path.join(TINY, "model.safetensors"))
    names = sorted(src)
    parts = {"a.safetensors": names[: len(names) // 2], "b.safetensors": names[len(names) // 2:]}
    weight_map = {}
    for fn, ns in parts.items():
        hdr, blob = {}, b""
        for n in ns:
            raw = src[n][1].tobytes()
            hdr[n] = {"dtype": src[n][0], "shape": list(src[n][1].shape), "data_offsets": [len(blob), len(blob) + len(raw)]}
            blob += raw
            weight_map[n] = fn
        h = json.dumps(hdr).encode()
        (tmp_path / fn).write_bytes(struct.pack("<Q", len(h)) + h + blob)
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"metadata": {}, "weight_map": weight_map}))
    w = mynn.Weights(tmp_path)
    assert sorted(w.names()) == names
    for n in names:
        assert np.array_equal(w.find(n)[2], src[n][1])


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [orc.BF16, orc.F16])
def test_checkpoint_upload_reproduces_the_reference_ids(dt):
    """crates/llm/tests/tinyllama_random.rs:20-24 through the library's own loader: the f32 checkpoint is
    converted to the 16-bit type and uploaded in initializer order by mynn_weights_upload."""
    cfg, _, golden = llm_weights.tiny_llama_random(dt)
    dec = mynn.Decoder(cfg, TINY)
    llm = mynn.LlmSession(dec)
    ids = llm.generate_ids(golden["prompt_ids"], len(golden["expected_new_ids"]))
    assert ids == golden["expected_new_ids"]
    llm.close(), dec.close()


@pytest.mark.gpu
def test_int8_checkpoint_upload_matches_tensors_passed_by_hand(tmp_path):
    """The quantised file read back by the loader gives the same logits as the same int8 tensors handed
    over as device tensors."""
    import gpu_util as g

    dt = orc.BF16
    dst = tmp_path / "model.int8.safetensors"
    mynn.quantize_safetensors_int8(TINY, dst)
    cfg, wf, _ = llm_weights.tiny_llama_random(dt)
    from_file = mynn.Decoder(cfg, dst)
    st = read_safetensors_py(dst)

    def lin(name):
        return g.to_dev(st[name][1].copy()), g.to_dev(st[name + ".scale"][1].copy(), dt)

    w = {"embed": lin("model.embed_tokens.weight"), "lm_head": lin("lm_head.weight"), "final_norm": g.to_dev(wf["final_norm"], dt)}
    for l in range(cfg["n_layers"]):
        p = "model.layers.%d." % l
        for k, nm in llm_weights.LIN.items():
            w["layers.%d.%s" % (l, k)] = lin(p + nm + ".weight")
        w["layers.%d.norm1" % l] = g.to_dev(wf["layers.%d.norm1" % l], dt)
        w["layers.%d.norm2" % l] = g.to_dev(wf["layers.%d.norm2" % l], dt)
    by_hand = mynn.Decoder(cfg, w)
    for i, t in enumerate([15043, 7, 29871]):
        _, a = from_file.step([t], [i], i, i + 1, want_logits=True)
        _, b = by_hand.step([t], [i], i, i + 1, want_logits=True)
        assert np.array_equal(a, b)
    from_file.close(), by_hand.close()


def _write_raw(path, header_text, payload=b""):
    hdr = header_text.encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(hdr)))
        f.write(hdr)
        f.write(payload)


@pytest.mark.parametrize("header", [
    '{"t":{"dtype":"F32","shape":[2],"data_offsets":[0,16]}}',                       # length != count * element size
    '{"t":{"dtype":"F32","shape":[2],"data_offsets":[-8,0]}}',                       # negative offset
    '{"t":{"dtype":"F32","shape":[2],"data_offsets":[9223372036854775808,9223372036854775816]}}',  # offsets past 2^63
    '{"t":{"dtype":"I8","shape":[4294967296,4294967296],"data_offsets":[0,0]}}',     # extents whose product wraps
    '{"t":{"dtype":"F32","shape":[-2],"data_offsets":[0,8]}}',                       # negative extent
    '{"t":{"dtype":"F32","shape":[1.5],"data_offsets":[0,8]}}',                      # fractional extent
    '{"t":{"dtype":"F32","shape":[2],"data_offsets":[8,0]}}',                        # end before begin
    '{"t":{"dtype":"F32","shape":[4],"data_offsets":[0,16]}}',                       # data beyond the end of the file
    "[" * 100000,                                                                    # nesting without bound
    '{"t":{"dtype":"F32","shape":[2],"data_offsets":[0,8]}',                         # truncated
    '{"t":{"dtype":"F32","shape":"2","data_offsets":[0,8]}}',                        # wrong kinds
    '{"t":12345',                                                                    # a number that ends the file
])
def test_reader_rejects_hostile_headers_with_an_error(tmp_path, header):
    """A header the `safetensors` crate would refuse is refused here too -- with an error return, never a wild
    read, a wrapped size or an exception across the C boundary."""
    p = tmp_path / "bad.safetensors"
    _write_raw(p, header, b"\0" * 8)
    with pytest.raises(mynn.MynnError):
        mynn.Weights(p)


def test_reader_accepts_a_header_that_ends_the_file_and_refuses_path_tricks_in_the_index(tmp_path):
    p = tmp_path / "empty.safetensors"
    _write_raw(p, '{"t":{"dtype":"F32","shape":[0],"data_offsets":[0,0]}}')  # the header is the last byte of the mapping
    w = mynn.Weights(p)
    assert w.names() == ["t"] and w.find("t")[1] == (0,)
    w.close()
    d = tmp_path / "model"
    d.mkdir()
    (d / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"t": "../empty.safetensors"}}))
    with pytest.raises(mynn.MynnError, match="plain file name"):
        mynn.Weights(d)
