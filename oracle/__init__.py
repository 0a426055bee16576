"""ctypes binding of the CPU oracle (oracle/mynn_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg, as the checker or the timed CPU baseline.  The shipped package never
imports this module.

Arrays are numpy; 16-bit float tensors travel as uint16 bit patterns together with a dtype
code (F32 = 0, BF16 = 1, F16 = 2).
"""
import ctypes as C
import os
import subprocess

import numpy as np

F32, BF16, F16 = 0, 1, 2
_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libmynn_oracle.so")


def build(force=False):
    """Compiles the oracle with gcc (a few seconds)."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.check_call(["make", "-C", _HERE, "--no-print-directory"])
    return _SO


def _load():
    if not os.path.exists(_SO):
        build()
    return C.CDLL(_SO)


_lib = _load()
_vp, _sz, _i, _ll, _f, _d = C.c_void_p, C.c_size_t, C.c_int, C.c_longlong, C.c_float, C.c_double


def _sig(name, res, *args):
    fn = getattr(_lib, name)
    fn.restype = res
    fn.argtypes = list(args)
    return fn


_sig("orc_set_lanes", None, _i)
_sig("orc_get_lanes", _i)
_sig("orc_set_threads", None, _i)
_sig("orc_get_threads", _i)
_sig("orc_f32_to_bf16", C.c_uint16, _f)
_sig("orc_f32_to_f16", C.c_uint16, _f)
_sig("orc_f16_to_f32", _f, C.c_uint16)
_sig("orc_convert", None, _vp, _i, _vp, _i, _sz)
_sig("orc_dequantize_linear", None, _vp, _vp, _vp, _sz, _sz, _i)
_sig("orc_dequant_matmul", None, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _i, _i, _i)
_sig("orc_quantized_matmul", None, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _i)
_sig("orc_dynquant_i8", None, _vp, _vp, _vp, _sz, _sz, _i)
_sig("orc_dynquant_i8_per_tensor", None, _vp, _vp, _vp, _sz, _i)
_sig("orc_dynquant_u8_asym", None, _vp, _vp, _vp, _vp, _sz, _sz, _i)
_sig("orc_attention", None, _vp, _vp, _vp, _vp, _vp, _vp, _ll, _sz, _sz, _sz, _sz, _sz, _sz, _i, _f, _i, _i)
_sig("orc_attention_f64", None, _vp, _vp, _vp, _vp, _ll, _sz, _sz, _sz, _sz, _sz, _sz, _i, _d, _i)
_sig("orc_kv_cache_update", None, _vp, _vp, _ll, _sz, _sz, _sz, _sz, _sz)
_sig("orc_quantizing_kv_cache_update", None, _vp, _vp, _vp, _ll, _sz, _sz, _sz, _sz, _i)
_sig("orc_rms_norm", None, _vp, _vp, _vp, _sz, _sz, _d, _i)
_sig("orc_rope_table", None, _vp, _vp, _sz, _sz, _f, _i)
_sig("orc_rope", None, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _i)
_sig("orc_gather_rows", None, _vp, _vp, _vp, _sz, _sz, _sz)
_sig("orc_swish", None, _vp, _vp, _sz, _i)
_sig("orc_swiglu", None, _vp, _vp, _vp, _sz, _i)
_sig("orc_add", None, _vp, _vp, _vp, _sz, _i)
_sig("orc_argmax_last", C.c_int64, _vp, _sz, _i)
_sig("orc_quantize_per_channel", None, _vp, _vp, _vp, _sz, _sz, _i)
_sig("orc_ring_phys_index", _i, _i, _i, _i, _i)
_sig("orc_streaming_kv_position", None, _vp, _sz, _sz, _sz, _sz)


class ModelCfg(C.Structure):
    _fields_ = [("n_layers", _i), ("hidden", _i), ("n_heads", _i), ("n_kv_heads", _i),
                ("head_dim", _i), ("ffn", _i), ("vocab", _i), ("max_seq", _i),
                ("eps", _d), ("rope_theta", _f), ("dtype", _i)]


class Linear(C.Structure):
    _fields_ = [("q", _vp), ("scale", _vp), ("w", _vp)]


_sig("orc_model_create", _vp, C.POINTER(ModelCfg))
_sig("orc_model_destroy", None, _vp)
_sig("orc_model_set_embed", None, _vp, Linear)
_sig("orc_model_set_lm_head", None, _vp, Linear)
_sig("orc_model_set_final_norm", None, _vp, _vp)
_sig("orc_model_set_linear", None, _vp, _i, _i, Linear)
_sig("orc_model_set_norm", None, _vp, _i, _i, _vp)
_sig("orc_model_set_bias", None, _vp, _i, _i, _vp)
_sig("orc_model_reset", None, _vp)
_sig("orc_model_set_gemm_mode", None, _vp, _i)
_sig("orc_model_set_options", None, _vp, _i, _i)
_sig("orc_model_k_scale", _vp, _vp, _i)
_sig("orc_model_v_scale", _vp, _vp, _i)
_sig("orc_model_past_len", _ll, _vp)
_sig("orc_model_set_past_len", None, _vp, _ll)
_sig("orc_model_forward", None, _vp, _vp, _vp, _sz, _ll, _ll, _i, _vp)
_sig("orc_model_forward_streaming", None, _vp, _vp, _vp, _sz, _ll, _ll, _i, _i, _i, _i, _vp, _vp)
_sig("orc_model_set_streaming", None, _vp, _i, _i)
_sig("orc_kv_cache_update_ring", None, _vp, _vp, _ll, _sz, _sz, _sz, _sz, _sz, _i, _i, _i)
_sig("orc_quantizing_kv_cache_update_ring", None, _vp, _vp, _vp, _ll, _sz, _sz, _sz, _sz, _i, _i, _i, _i)
_sig("orc_attention_ring", None, _vp, _vp, _vp, _vp, _vp, _vp, _ll, _sz, _sz, _sz, _sz, _sz, _sz, _i, _f, _i, _i, _i, _i, _i,
     _vp, _vp, _vp)
_sig("orc_model_decode_step", C.c_int64, _vp, C.c_int64)
_sig("orc_model_prefill", C.c_int64, _vp, _vp, _sz, _sz)
_sig("orc_model_generate", _ll, _vp, _vp, _sz, _sz, _sz, C.c_int64, _vp)
_sig("orc_model_k_cache", _vp, _vp, _i)
_sig("orc_model_v_cache", _vp, _vp, _i)
_sig("orc_model_last_hidden", _vp, _vp)


# ------------------------------------------------------------------ helpers
def np_dtype(dt):
    return np.float32 if dt == F32 else np.uint16


def _p(a):
    return None if a is None else a.ctypes.data_as(_vp)


def _c(a, dt=None):
    a = np.ascontiguousarray(a)
    if dt is not None and a.dtype != np.dtype(dt):
        raise TypeError("expected %s, got %s" % (np.dtype(dt), a.dtype))
    return a


def set_lanes(n):
    _lib.orc_set_lanes(int(n))


def set_threads(n):
    _lib.orc_set_threads(int(n))


def get_threads():
    return _lib.orc_get_threads()


def to_storage(x, dt):
    """float32 array -> storage array of type dt (RNE)."""
    x = _c(np.asarray(x, dtype=np.float32))
    if dt == F32:
        return x.copy()
    out = np.empty(x.shape, np.uint16)
    _lib.orc_convert(_p(out), dt, _p(x), F32, x.size)
    return out


def to_f32(x, dt):
    """storage array -> float32 (exact)."""
    x = _c(x)
    if dt == F32:
        return x.astype(np.float32)
    out = np.empty(x.shape, np.float32)
    _lib.orc_convert(_p(out), F32, _p(x), dt, x.size)
    return out


def dequantize_linear(x_i8, scale, dt):
    x_i8 = _c(x_i8, np.int8)
    scale = _c(scale, np_dtype(dt))
    rows = x_i8.shape[0]
    cols = x_i8.size // rows
    out = np.empty(x_i8.shape, np_dtype(dt))
    _lib.orc_dequantize_linear(_p(out), _p(x_i8), _p(scale), rows, cols, dt)
    return out


def dequant_matmul(act, wq, scale, act_dt, out_dt, mode=-1):
    act, wq, scale = _c(act, np_dtype(act_dt)), _c(wq, np.int8), _c(scale, np_dtype(out_dt))
    N, K = wq.shape
    M = act.size // K
    out = np.empty(act.shape[:-1] + (N,), np_dtype(out_dt))
    _lib.orc_dequant_matmul(_p(out), _p(act), _p(wq), _p(scale), M, N, K, act_dt, out_dt, mode)
    return out


def quantized_matmul(lhs, lhs_scale, rhs, rhs_scale, dt):
    lhs, rhs = _c(lhs, np.int8), _c(rhs, np.int8)
    lhs_scale, rhs_scale = _c(lhs_scale, np_dtype(dt)), _c(rhs_scale, np_dtype(dt))
    M, K = lhs.shape
    N = rhs.shape[0]
    out = np.empty((M, N), np_dtype(dt))
    acc = np.empty((M, N), np.int32)
    _lib.orc_quantized_matmul(_p(out), _p(acc), _p(lhs), _p(lhs_scale), _p(rhs), _p(rhs_scale), M, N, K, dt)
    return out, acc


def dynquant_i8(x, dt):
    x = _c(x, np_dtype(dt))
    M, K = x.shape
    y = np.empty((M, K), np.int8)
    s = np.empty((M,), np_dtype(dt))
    _lib.orc_dynquant_i8(_p(y), _p(s), _p(x), M, K, dt)
    return y, s


def dynquant_i8_per_tensor(x, dt):
    x = _c(x, np_dtype(dt))
    y = np.empty(x.shape, np.int8)
    s = np.empty((1,), np_dtype(dt))
    _lib.orc_dynquant_i8_per_tensor(_p(y), _p(s), _p(x), x.size, dt)
    return y, s


def dynquant_u8_asym(x, dt):
    x = _c(x, np_dtype(dt))
    M, K = x.shape
    y = np.empty((M, K), np.uint8)
    s = np.empty((M,), np_dtype(dt))
    zp = np.empty((M,), np.uint8)
    _lib.orc_dynquant_u8_asym(_p(y), _p(s), _p(zp), _p(x), M, K, dt)
    return y, s, zp


def attention(q, k, v, dt, scale, is_causal=False, active=-1, k_scale=None, v_scale=None):
    kv_int8 = k.dtype == np.int8
    q = _c(q, np_dtype(dt))
    k = _c(k, np.int8 if kv_int8 else np_dtype(dt))
    v = _c(v, np.int8 if kv_int8 else np_dtype(dt))
    B, Hq, Sq, D = q.shape
    Hkv, Sk = k.shape[1], k.shape[2]
    out = np.empty(q.shape, np_dtype(dt))
    ks = _c(k_scale, np_dtype(dt)) if kv_int8 else None
    vs = _c(v_scale, np_dtype(dt)) if kv_int8 else None
    _lib.orc_attention(_p(out), _p(q), _p(k), _p(v), _p(ks), _p(vs), int(active), B, Hq, Hkv, Sq, Sk, D,
                       int(is_causal), float(scale), dt, int(kv_int8))
    return out


def attention_f64(q, k, v, dt, scale, is_causal=False, active=-1):
    q, k, v = _c(q, np_dtype(dt)), _c(k, np_dtype(dt)), _c(v, np_dtype(dt))
    B, Hq, Sq, D = q.shape
    Hkv, Sk = k.shape[1], k.shape[2]
    out = np.empty(q.shape, np.float64)
    _lib.orc_attention_f64(_p(out), _p(q), _p(k), _p(v), int(active), B, Hq, Hkv, Sq, Sk, D,
                           int(is_causal), float(scale), dt)
    return out


def kv_cache_update(cache, new_kv, offset):
    """cache [B,H,max_seq,D] is updated in place (and returned)."""
    assert cache.flags.c_contiguous
    new_kv = _c(new_kv, cache.dtype)
    B, H, max_seq, D = cache.shape
    _lib.orc_kv_cache_update(_p(cache), _p(new_kv), int(offset), B * H, new_kv.shape[2], max_seq, D,
                             cache.itemsize)
    return cache


def ring_phys_index(rank, ring_sink, ring_window, ring_start):
    """Cache row of the key with recency rank `rank` in the sink + ring layout
    (src/codegen/cuda/cpp/common.cuh:55-60): the first ring_sink rows are fixed, the following ring_window
    rows are a ring read from ring_start; ring_window == 0 switches the map off."""
    if ring_window == 0 or rank < ring_sink:
        return rank
    return ring_sink + (ring_start + (rank - ring_sink)) % ring_window


def kv_cache_update_streaming(cache, new_kv, offset, ring_sink, ring_window, ring_start):
    """KVCacheUpdate with the ring inputs (src/codegen/cuda/cpp/kvcache_update.cuh:12-26): row t of new_kv goes
    to row ring_phys_index(offset + t) of the cache, rows in increasing t (a later row wins a shared slot).
    cache [B,H,max_seq,D] is updated in place (and returned)."""
    assert cache.flags.c_contiguous
    new_kv = _c(new_kv, cache.dtype)
    for t in range(new_kv.shape[2]):
        cache[:, :, ring_phys_index(offset + t, ring_sink, ring_window, ring_start)] = new_kv[:, :, t]
    return cache


def quantizing_kv_cache_update_streaming(cache, scale, new_kv, offset, ring_sink, ring_window, ring_start, dt):
    """QuantizingKVCacheUpdate with the ring inputs (src/codegen/cuda/cpp/quantizing_kvcache_update.cuh:24-36):
    each row is quantised as quantizing_kv_cache_update does and, with its scale, goes to row
    ring_phys_index(offset + t), rows in increasing t."""
    assert cache.flags.c_contiguous and cache.dtype == np.int8 and scale.flags.c_contiguous
    B, H, _, D = cache.shape
    S_new = new_kv.shape[2]
    tmp_c = np.zeros((B, H, S_new, D), np.int8)
    tmp_s = np.zeros((B, H, S_new), scale.dtype)
    quantizing_kv_cache_update(tmp_c, tmp_s, new_kv, 0, dt)
    for t in range(S_new):
        row = ring_phys_index(offset + t, ring_sink, ring_window, ring_start)
        cache[:, :, row] = tmp_c[:, :, t]
        scale[:, :, row] = tmp_s[:, :, t]
    return cache, scale


def attention_streaming(q, k, v, dt, scale, is_causal, active, ring_sink, ring_window, ring_start, k_scale=None,
                        v_scale=None, rope=None):
    """Attention over the sink + ring layout (src/codegen/cuda/cpp/attention.cuh:386-404, 436-438, 548-550):
    keys are enumerated by recency rank 0..active-1, the key of rank r is cache row ring_phys_index(r), and
    the causal rule compares query positions with ranks.  Restated as the plain attention of this module over
    the rows gathered in rank order.

    rope = (cos_table, sin_table, kv_position) switches on the rotation of K inside the operator
    (attention.cuh:407-420, 559-570): the dequantised key of RANK r is rotated (half-split) by row
    kv_position[r] of the tables, all in f32, before the dot product; scores, softmax and P.V stay f32, so the
    restatement runs the f32 attention over the rotated / dequantised rows and rounds the result once."""
    rows = [ring_phys_index(r, ring_sink, ring_window, ring_start) for r in range(active)]
    if rope is None:
        kg, vg = np.ascontiguousarray(k[:, :, rows]), np.ascontiguousarray(v[:, :, rows])
        ks = np.ascontiguousarray(k_scale[:, :, rows]) if k_scale is not None else None
        vs = np.ascontiguousarray(v_scale[:, :, rows]) if v_scale is not None else None
        return attention(q, kg, vg, dt, scale, is_causal, active, ks, vs)
    cos_t, sin_t, kv_position = rope
    D = q.shape[-1]
    half = D // 2
    if k.dtype == np.int8:
        kf = k[:, :, rows].astype(np.float32) * to_f32(k_scale, dt)[:, :, rows, None]
        vf = v[:, :, rows].astype(np.float32) * to_f32(v_scale, dt)[:, :, rows, None]
    else:
        kf, vf = to_f32(k, dt)[:, :, rows], to_f32(v, dt)[:, :, rows]
    pos = np.asarray(kv_position, np.int64)[:active]
    c, sn = to_f32(cos_t, dt)[pos], to_f32(sin_t, dt)[pos]  # [active, D]
    pair = np.concatenate([kf[..., half:], kf[..., :half]], axis=-1)
    sign = np.concatenate([-np.ones(half, np.float32), np.ones(half, np.float32)])
    krot = (kf * c + (sign * pair) * sn).astype(np.float32)
    out = attention(to_f32(q, dt), np.ascontiguousarray(krot), np.ascontiguousarray(vf), F32, scale, is_causal, active)
    return to_storage(out, dt)


def attention_ring(q, k, v, dt, scale, is_causal, active, ring_sink, ring_window, ring_start, k_scale=None, v_scale=None,
                   rope=None):
    """The C restatement of the same operator (orc_attention_ring): one loop nest that follows the CUDA decode
    kernel key by key instead of gathering rows first; used by the streaming decoder of this module."""
    kv_int8 = k.dtype == np.int8
    q = _c(q, np_dtype(dt))
    k = _c(k, np.int8 if kv_int8 else np_dtype(dt))
    v = _c(v, np.int8 if kv_int8 else np_dtype(dt))
    B, Hq, Sq, D = q.shape
    Hkv, Sk = k.shape[1], k.shape[2]
    out = np.empty(q.shape, np_dtype(dt))
    ks = _c(k_scale, np_dtype(dt)) if kv_int8 else None
    vs = _c(v_scale, np_dtype(dt)) if kv_int8 else None
    cos_t = sin_t = kvp = None
    if rope is not None:
        cos_t, sin_t, kvp = _c(rope[0], np_dtype(dt)), _c(rope[1], np_dtype(dt)), _c(np.asarray(rope[2], np.int64))
    _lib.orc_attention_ring(_p(out), _p(q), _p(k), _p(v), _p(ks), _p(vs), int(active), B, Hq, Hkv, Sq, Sk, D, int(is_causal),
                            float(scale), dt, int(kv_int8), int(ring_sink), int(ring_window), int(ring_start), _p(cos_t),
                            _p(sin_t), _p(kvp))
    return out


def quantizing_kv_cache_update(cache, scale, new_kv, offset, dt):
    assert cache.flags.c_contiguous and cache.dtype == np.int8 and scale.flags.c_contiguous
    new_kv = _c(new_kv, np_dtype(dt))
    B, H, max_seq, D = cache.shape
    _lib.orc_quantizing_kv_cache_update(_p(cache), _p(scale), _p(new_kv), int(offset), B * H,
                                        new_kv.shape[2], max_seq, D, dt)
    return cache, scale


def rms_norm(x, w, eps, dt):
    x, w = _c(x, np_dtype(dt)), _c(w, np_dtype(dt))
    dim = x.shape[-1]
    out = np.empty(x.shape, np_dtype(dt))
    _lib.orc_rms_norm(_p(out), _p(x), _p(w), x.size // dim, dim, float(eps), dt)
    return out


def rope_table(max_seq, D, base, dt):
    cos = np.empty((max_seq, D), np_dtype(dt))
    sin = np.empty((max_seq, D), np_dtype(dt))
    _lib.orc_rope_table(_p(cos), _p(sin), max_seq, D, float(base), dt)
    return cos, sin


def rope(x, cos, sin, position, dt):
    """x [..., S, D]; position [S] int64."""
    x, cos, sin = _c(x, np_dtype(dt)), _c(cos, np_dtype(dt)), _c(sin, np_dtype(dt))
    position = _c(np.asarray(position, np.int64))
    S, D = x.shape[-2], x.shape[-1]
    out = np.empty(x.shape, np_dtype(dt))
    _lib.orc_rope(_p(out), _p(x), _p(cos), _p(sin), _p(position), x.size // (S * D), S, D, dt)
    return out


def gather_rows(data, idx):
    data = _c(data)
    idx = _c(np.asarray(idx, np.int64))
    rows = data.shape[0]
    row_bytes = data.nbytes // rows
    out = np.empty(idx.shape + data.shape[1:], data.dtype)
    _lib.orc_gather_rows(_p(out), _p(data), _p(idx), idx.size, rows, row_bytes)
    return out


def swish(x, dt):
    x = _c(x, np_dtype(dt))
    out = np.empty(x.shape, np_dtype(dt))
    _lib.orc_swish(_p(out), _p(x), x.size, dt)
    return out


def swiglu(gate, up, dt):
    gate, up = _c(gate, np_dtype(dt)), _c(up, np_dtype(dt))
    out = np.empty(gate.shape, np_dtype(dt))
    _lib.orc_swiglu(_p(out), _p(gate), _p(up), gate.size, dt)
    return out


def add(a, b, dt):
    a, b = _c(a, np_dtype(dt)), _c(b, np_dtype(dt))
    out = np.empty(a.shape, np_dtype(dt))
    _lib.orc_add(_p(out), _p(a), _p(b), a.size, dt)
    return out


def argmax_last(logits, dt):
    logits = _c(logits, np_dtype(dt))
    return int(_lib.orc_argmax_last(_p(logits), logits.size, dt))


def quantize_per_channel(w, scale_dt):
    w = _c(np.asarray(w, np.float32))
    rows = w.shape[0]
    q = np.empty(w.shape, np.int8)
    s = np.empty((rows,), np_dtype(scale_dt))
    _lib.orc_quantize_per_channel(_p(q), _p(s), _p(w), rows, w.size // rows, scale_dt)
    return q, s


def ring_phys_index(rank, sink, window, start):
    return _lib.orc_ring_phys_index(rank, sink, window, start)


def streaming_kv_position(sink, window, stream_pos, max_seq):
    out = np.empty((max_seq,), np.int64)
    _lib.orc_streaming_kv_position(_p(out), sink, window, stream_pos, max_seq)
    return out


LIN_NAMES = ("q", "k", "v", "o", "gate", "up", "down")


class Model:
    """The decoder of crates/llm (decoder.rs build_decoder) plus the LlmSession loop.

    weights: dict with
      "embed", "lm_head", "layers.{i}.{q,k,v,o,gate,up,down}" -> (int8 [N,K], scale [N]) tuples for
      quantised tensors or a single storage array [N,K] for plain ones;
      "final_norm", "layers.{i}.norm1", "layers.{i}.norm2" -> storage arrays;
      optional "layers.{i}.{q,k,v}.bias" -> storage arrays [N] (decoder.rs:167-184).
    """

    def __init__(self, cfg, weights):
        self.cfg = ModelCfg(**cfg)
        self.dt = cfg["dtype"]
        self._keep = []
        self._h = _lib.orc_model_create(C.byref(self.cfg))
        _lib.orc_model_set_embed(self._h, self._lin(weights["embed"]))
        _lib.orc_model_set_lm_head(self._h, self._lin(weights["lm_head"]))
        _lib.orc_model_set_final_norm(self._h, _p(self._hold(weights["final_norm"])))
        for l in range(cfg["n_layers"]):
            for wi, nm in enumerate(LIN_NAMES):
                _lib.orc_model_set_linear(self._h, l, wi, self._lin(weights["layers.%d.%s" % (l, nm)]))
            for bi, nm in enumerate(("q", "k", "v")):  # optional projection bias (qwen2)
                b = weights.get("layers.%d.%s.bias" % (l, nm))
                if b is not None:
                    _lib.orc_model_set_bias(self._h, l, bi, _p(self._hold(b)))
            _lib.orc_model_set_norm(self._h, l, 0, _p(self._hold(weights["layers.%d.norm1" % l])))
            _lib.orc_model_set_norm(self._h, l, 1, _p(self._hold(weights["layers.%d.norm2" % l])))

    def _hold(self, a):
        a = np.ascontiguousarray(a)
        self._keep.append(a)
        return a

    def _lin(self, w):
        if isinstance(w, tuple):
            q, s = self._hold(w[0]), self._hold(w[1])
            assert q.dtype == np.int8
            return Linear(q.ctypes.data, s.ctypes.data, None)
        a = self._hold(w)
        return Linear(None, None, a.ctypes.data)

    def close(self):
        if self._h:
            _lib.orc_model_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def reset(self):
        _lib.orc_model_reset(self._h)

    def set_gemm_mode(self, mode):
        """-1: CPU backend's kernel choice (default); 2: CUDA backend's."""
        _lib.orc_model_set_gemm_mode(self._h, int(mode))

    def set_options(self, quant_kv_cache=False, quantize_activations=False):
        """BuildOptions::quant_kv_cache / Options::quantize_activations; before the first forward."""
        self.quant_kv_cache = bool(quant_kv_cache)
        _lib.orc_model_set_options(self._h, int(quant_kv_cache), int(quantize_activations))

    @property
    def past_len(self):
        return _lib.orc_model_past_len(self._h)

    @past_len.setter
    def past_len(self, v):
        _lib.orc_model_set_past_len(self._h, int(v))

    def forward(self, ids, positions, past_len, active, is_causal):
        ids = _c(np.asarray(ids, np.int64))
        positions = _c(np.asarray(positions, np.int64))
        S = ids.size
        logits = np.empty((S, self.cfg.vocab), np_dtype(self.dt))
        _lib.orc_model_forward(self._h, _p(ids), _p(positions), S, int(past_len), int(active),
                               int(is_causal), _p(logits))
        return logits

    def set_streaming(self, sink, window):
        """DecodeKind::LlamaStreaming { sink, window } over the BuildOptions::streaming_kv graph: decode_step,
        prefill and generate then build the session's ring inputs themselves (session.rs:539-635)."""
        _lib.orc_model_set_streaming(self._h, int(sink), int(window))

    def forward_streaming(self, ids, positions, past_len, active, is_causal, sink, window, ring_start, kv_position):
        ids = _c(np.asarray(ids, np.int64))
        positions = _c(np.asarray(positions, np.int64))
        kv_position = _c(np.asarray(kv_position, np.int64))
        assert kv_position.size == self.cfg.max_seq
        S = ids.size
        logits = np.empty((S, self.cfg.vocab), np_dtype(self.dt))
        _lib.orc_model_forward_streaming(self._h, _p(ids), _p(positions), S, int(past_len), int(active), int(is_causal),
                                         int(sink), int(window), int(ring_start), _p(kv_position), _p(logits))
        return logits

    def decode_step(self, token):
        return int(_lib.orc_model_decode_step(self._h, int(token)))

    def prefill(self, ids, prefill_len):
        ids = _c(np.asarray(ids, np.int64))
        return int(_lib.orc_model_prefill(self._h, _p(ids), ids.size, prefill_len))

    def generate(self, prompt, max_new, prefill_len=0, eos=-1):
        prompt = _c(np.asarray(prompt, np.int64))
        out = np.empty((max(max_new, 1),), np.int64)
        n = _lib.orc_model_generate(self._h, _p(prompt), prompt.size, max_new, prefill_len, eos, _p(out))
        if n < 0:
            raise ValueError("PromptTooLong")
        return [int(t) for t in out[:n]]

    def kv_cache(self, layer):
        n = self.cfg.n_kv_heads * self.cfg.max_seq * self.cfg.head_dim
        shape = (self.cfg.n_kv_heads, self.cfg.max_seq, self.cfg.head_dim)
        kp = _lib.orc_model_k_cache(self._h, layer)
        vp = _lib.orc_model_v_cache(self._h, layer)
        typ = C.c_int8 if getattr(self, "quant_kv_cache", False) else (C.c_float if self.dt == F32 else C.c_uint16)
        k = np.ctypeslib.as_array(C.cast(kp, C.POINTER(typ)), (n,)).reshape(shape).copy()
        v = np.ctypeslib.as_array(C.cast(vp, C.POINTER(typ)), (n,)).reshape(shape).copy()
        return k, v

    def kv_scales(self, layer):
        """quant_kv_cache: the per-token scales [Hkv, max_seq] of layer's k and v caches."""
        n = self.cfg.n_kv_heads * self.cfg.max_seq
        typ = C.c_float if self.dt == F32 else C.c_uint16
        ks = np.ctypeslib.as_array(C.cast(_lib.orc_model_k_scale(self._h, layer), C.POINTER(typ)), (n,))
        vs = np.ctypeslib.as_array(C.cast(_lib.orc_model_v_scale(self._h, layer), C.POINTER(typ)), (n,))
        shape = (self.cfg.n_kv_heads, self.cfg.max_seq)
        return ks.reshape(shape).copy(), vs.reshape(shape).copy()


class SummationOrders:
    """The same decoder under several f32 summation orders (orc_set_lanes: n interleaved partial sums + a pairwise
    tree; 16 is the default, 1 = sequential), stepped together on one token stream.  The reference leaves the order of
    its f32 sums open (LLVM fast-math vectorisation, BLAS), so where two orders pick different greedy tokens the
    reference's own choice is not determined either; that is the only kind of disagreement a checked implementation
    may show.  `lanes`: orders that run the whole stream, one Model with its own KV cache each (the effect of an order
    on earlier cache rows is then part of the sample); `step_lanes`: further orders tried only at a disputed position,
    as a re-evaluation of that one step over each of those caches."""

    def __init__(self, cfg, weights, lanes=(16, 8, 32, 64), step_lanes=(1, 2, 4), quant_kv_cache=False,
                 quantize_activations=False, gemm_mode=None):
        self.lanes = tuple(lanes)
        self.step_lanes = tuple(step_lanes)
        self.models = []
        for _ in self.lanes:
            m = Model(dict(cfg), weights)
            if quant_kv_cache or quantize_activations:
                m.set_options(quant_kv_cache=quant_kv_cache, quantize_activations=quantize_activations)
            if gemm_mode is not None:
                m.set_gemm_mode(gemm_mode)
            self.models.append(m)
        self.dt = cfg["dtype"]
        self.seconds_first = 0.0  # wall time of the first order's forward calls (the CPU baseline times that one)
        self._last = None

    def forward(self, ids, positions, past_len, active, is_causal):
        """[logits of order 0, logits of order 1, ...] for the orders that follow the whole stream"""
        import time

        self._last = (ids, positions, past_len, active, is_causal)
        out = []
        try:
            for i, (n, m) in enumerate(zip(self.lanes, self.models)):
                set_lanes(n)
                t0 = time.perf_counter()
                out.append(m.forward(ids, positions, past_len, active, is_causal))
                if i == 0:
                    self.seconds_first += time.perf_counter() - t0
        finally:
            set_lanes(16)
        return out

    def judge(self, logits_rows, token):
        """logits_rows: the last row of each order's logits of the forward call just made.  Returns (verdict, choices):
        "identical" -- `token` is the first order's greedy choice;
        "order_dependent" -- it is the choice under another order, or the orders disagree among themselves (the
            oracle is undecided at this position), the step orders included;
        "within_order_noise" -- no order tried flips the choice, but the first order's own gap between its choice and
            `token` is below twice the largest shift any single logit of this step shows between the oracle's orders
            (order_noise): the oracle's arithmetic does not separate the two tokens;
        "different" otherwise.  choices: the greedy token of every order tried."""
        choices = [argmax_last(r, self.dt) for r in logits_rows]
        if token == choices[0]:
            return "identical", choices
        if token in choices or len(set(choices)) > 1:
            return "order_dependent", choices
        # undisputed so far: this one step again under the remaining orders, over each cache (the cache row the step
        # writes is put back by repeating the step under the cache's own order)
        try:
            for n_own, m in zip(self.lanes, self.models):
                for n in self.step_lanes:
                    set_lanes(n)
                    choices.append(argmax_last(m.forward(*self._last)[-1], self.dt))
                set_lanes(n_own)
                m.forward(*self._last)
        finally:
            set_lanes(16)
        if token in choices or len(set(choices)) > 1:
            return "order_dependent", choices
        lf = to_f32(logits_rows[0], self.dt)
        if float(lf[choices[0]] - lf[token]) <= 2.0 * self.order_noise(logits_rows):
            return "within_order_noise", choices
        return "different", choices

    def order_noise(self, logits_rows):
        """The largest shift any single logit shows between the first order and another whole-stream order at this
        step (f32): two logits closer than twice that are not separated by the oracle's own arithmetic."""
        base = to_f32(logits_rows[0], self.dt)
        return max(float(np.max(np.abs(to_f32(r, self.dt) - base))) for r in logits_rows[1:])

    def close(self):
        for m in self.models:
            m.close()
