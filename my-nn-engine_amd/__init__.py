"""MI355X-native quantized-LLM hot path of my-nn-engine: ctypes binding of lib/libmynn_hip.so.

The product is the C-ABI library (include/mynn_hip.h).  This module is plumbing for Python
callers: it loads the library, checks return codes, and passes torch tensors' device pointers
and the current HIP stream through.  There is no fallback: when the library is missing, or a
kernel rejects its arguments, the call raises.

The directory name carries a hyphen, so import it with
    importlib.import_module("my-nn-engine_amd")
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libmynn_hip.so")
CSRC = os.path.join(_HERE, "csrc")

F32, BF16, F16, I8 = 0, 1, 2, 3


class MynnError(RuntimeError):
    pass


def build(jobs=8):
    """Compiles every HIP source for gfx950 (hipcc cross-compiles without a GPU)."""
    import subprocess

    subprocess.check_call(["make", "-C", CSRC, "-j%d" % jobs, "--no-print-directory"])
    return LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise MynnError("HIP library not built: %s is missing (run __graft_entry__.build())" % LIB_PATH)
        # torch ships its own libamdhip64.so.7; it has to be in the process before this library
        # so that both share ONE HIP runtime (two runtimes in a process do not both see the GPU)
        import torch  # noqa: F401

        _lib = C.CDLL(LIB_PATH)
        _declare(_lib)
    return _lib


_vp, _i, _sz, _f, _i64 = C.c_void_p, C.c_int, C.c_size_t, C.c_float, C.c_int64


class ModelConfig(C.Structure):
    _fields_ = [("n_layers", _i), ("hidden", _i), ("n_heads", _i), ("n_kv_heads", _i), ("head_dim", _i),
                ("ffn", _i), ("vocab", _i), ("max_seq", _i), ("eps", _f), ("rope_theta", _f), ("dtype", _i),
                ("seq_q", _i), ("batch", _i), ("weights_int8", _i), ("quant_kv_cache", _i),
                ("quantize_activations", _i), ("streaming_kv", _i), ("gemm_tile", _i), ("unfused_decode", _i),
                ("handover_spin_limit", _i), ("weight_arena", _i), ("kv_page_rows", _i), ("qkv_bias", _i)]


class KernelTime(C.Structure):
    _fields_ = [("name", C.c_char_p), ("ms", _f), ("bytes", C.c_double), ("flops", C.c_double)]


STEP_FN = C.CFUNCTYPE(_i64, _vp, _i64, _i64)

# name -> (restype, argtypes): every symbol include/mynn_hip.h declares
SIGNATURES = {
    "mynn_last_error": (C.c_char_p, []),
    "mynn_version": (_i, []),
    "mynn_device_info": (_i, [C.POINTER(_i), C.POINTER(_i), C.POINTER(_i), C.c_char_p, _sz]),
    "mynn_dequantize_linear": (_i, [_vp, _vp, _vp, _sz, _sz, _i, _vp]),
    "mynn_dequant_gemv": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "mynn_gemv_read_probe": (_i, [_vp, _vp, _i, _i, _i, _vp]),
    "mynn_skinny_set_ablation": (None, [_i]),
    "mynn_dequant_matmul": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "mynn_dequant_matmul_workspace_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "mynn_dequant_matmul_ws": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _sz, _i, _vp]),
    "mynn_dequant_weight_bytes": (_sz, [_i, _i]),
    "mynn_dequant_weight_prepare": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "mynn_dequant_matmul_prepared": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "mynn_quantized_matmul": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "mynn_dynamic_quantize_linear": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "mynn_attention": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _f, _i, _i, _i, _i, _vp, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "mynn_attention_noalloc": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _f, _i, _i, _i, _i, _vp, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "mynn_attention_workspace_bytes": (_sz, [_i, _i, _i, _i, _i, _i, _i, _i]),
    "mynn_attention_ws": (_i, [_vp, _vp, _vp, _vp, _vp, C.c_long, C.c_long, _vp, _vp, _f, _i, _i, _i, _i, _vp, _i, _i, _i, _i, _i, _i,
                                _i, _vp, _sz, _vp]),
    "mynn_attention_paged_workspace_bytes": (_sz, [_i, _i, _i, _i, _i, _i, _i]),
    "mynn_attention_paged": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _f, _i, _i, _i, _i, _vp, _i, _i, _i, _i, _i, _i, _vp, _sz, _vp]),
    "mynn_kvcache_update_paged": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _i, _i, _vp]),
    "mynn_kv_pool_create": (_vp, [_i, _i]),
    "mynn_kv_pool_free_pages": (_i, [_vp]),
    "mynn_kv_pool_destroy": (_i, [_vp]),
    "mynn_kv_pages_create": (_vp, [_vp, _i, _i]),
    "mynn_kv_pages_reserve": (_i, [_vp, _i64]),
    "mynn_kv_pages_release": (_i, [_vp]),
    "mynn_kv_pages_mapped_rows": (_i, [_vp]),
    "mynn_kv_pages_per_seq": (_i, [_vp]),
    "mynn_kv_pages_table": (_vp, [_vp]),
    "mynn_kv_pages_table_host": (_i, [_vp, _vp]),
    "mynn_kv_pages_destroy": (_i, [_vp]),
    "mynn_kvcache_update": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _i, _vp]),
    "mynn_kvcache_update_streaming": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "mynn_quantizing_kvcache_update_streaming": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "mynn_attention_streaming": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _f, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "mynn_attention_streaming_workspace_bytes": (_sz, [_i, _i, _i, _i, _i, _i, _i, _i, _i]),
    "mynn_attention_streaming_ws": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _f, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp,
                                         _vp, _sz, _vp]),
    "mynn_quantizing_kvcache_update": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp]),
    "mynn_rms_norm": (_i, [_vp, _vp, _vp, _i, _i, _f, _i, _vp]),
    "mynn_rope": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "mynn_gather_rows": (_i, [_vp, _vp, _vp, _i, _i, _sz, _vp]),
    "mynn_swiglu": (_i, [_vp, _vp, _vp, _sz, _i, _vp]),
    "mynn_add": (_i, [_vp, _vp, _vp, _sz, _i, _vp]),
    "mynn_argmax_last": (_i, [_vp, _vp, _i, _i, _vp]),
    "mynn_model_configure": (_i, [C.POINTER(ModelConfig)]),
    "mynn_model_create": (_vp, [C.POINTER(ModelConfig), C.POINTER(_vp), C.POINTER(_vp)]),
    "mynn_weight_set_create": (_vp, [C.POINTER(ModelConfig), C.POINTER(_vp)]),
    "mynn_model_create_shared": (_vp, [C.POINTER(ModelConfig), _vp, C.POINTER(_vp)]),
    "mynn_weight_set_stats": (_i, [_vp, C.POINTER(_sz), C.POINTER(_i)]),
    "mynn_weight_set_destroy": (None, [_vp]),
    "model_init": (_vp, [C.POINTER(_vp), C.POINTER(_vp)]),
    "model": (None, [_vp, C.POINTER(_vp), C.POINTER(_vp)]),
    "model_destroy": (None, [_vp]),
    "model_device_sync": (None, []),
    "model_memcpy": (_i, [_vp, _vp, _sz, _i]),
    "alloc_pinned": (_vp, [_sz]),
    "free_pinned": (None, [_vp]),
    "mynn_model_step": (_i, [_vp, _vp, _vp, _i64, _i64, _vp, _vp]),
    "mynn_model_step_streaming": (_i, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp, _vp, _vp]),
    "mynn_model_handover_failures": (_i, [_vp]),
    "mynn_model_set_handover_rearm": (_i, [_vp, _i]),
    "mynn_model_release_kv_pages": (_i, [_vp]),
    "mynn_model_last_status": (_i, [_vp]),
    "mynn_model_argmax_row": (_i, [_vp, _i, C.POINTER(C.c_int32)]),
    "mynn_model_logits_device": (_vp, [_vp]),
    "mynn_model_stats": (_i, [_vp, C.POINTER(_sz), C.POINTER(_i), C.POINTER(_i)]),
    "mynn_model_decode_loop": (_i, [_vp, C.c_int32, _i64, _i, _vp]),
    "mynn_model_profile_step": (_i, [_vp, C.c_int32, _i64, C.POINTER(KernelTime), _i]),
    "mynn_model_profile": (_i, [_vp, _vp, _vp, _i64, _i64, C.POINTER(KernelTime), _i]),
    "mynn_weights_open": (_vp, [C.c_char_p]),
    "mynn_weights_close": (None, [_vp]),
    "mynn_weights_count": (_i, [_vp]),
    "mynn_weights_name": (C.c_char_p, [_vp, _i]),
    "mynn_weights_find": (_i, [_vp, C.c_char_p, C.POINTER(_i), C.POINTER(_i64), C.POINTER(_i), C.POINTER(_vp),
                               C.POINTER(_sz)]),
    "mynn_quantize_safetensors_int8": (_i, [C.c_char_p, C.c_char_p, C.POINTER(_i), C.POINTER(_i)]),
    "mynn_weights_upload": (_vp, [_vp, _vp]),
    "mynn_device_weights_initializer": (C.POINTER(_vp), [_vp]),
    "mynn_device_weights_int8": (_i, [_vp]),
    "mynn_device_weights_free": (None, [_vp]),
    "mynn_quantize_per_channel": (_i, [_vp, _vp, _vp, _sz, _sz, _i]),
    "mynn_rope_table": (_i, [_vp, _vp, _i, _i, _f, _i]),
    "mynn_llm_create": (_vp, [_vp, _vp, _i, _i, _i64]),
    "mynn_llm_destroy": (None, [_vp]),
    "mynn_llm_reset": (None, [_vp]),
    "mynn_llm_past_len": (_i64, [_vp]),
    "mynn_llm_set_past_len": (None, [_vp, _i64]),
    "mynn_llm_set_streaming": (_i, [_vp, _i, _i]),
    "mynn_llm_generate_ids": (_i, [_vp, _vp, _sz, _sz, _vp]),
    "mynn_llm_create_with_step": (_vp, [STEP_FN, _vp, _i, _i64]),
}


def missing_symbols():
    """Names declared in include/mynn_hip.h that the loaded library does not export."""
    l = lib()
    return [n for n in SIGNATURES if not hasattr(l, n)]


def _declare(l):
    for name, (res, args) in SIGNATURES.items():
        try:
            fn = getattr(l, name)
        except AttributeError:
            continue  # reported by missing_symbols(); calling it raises AttributeError
        fn.restype = res
        fn.argtypes = args


def check(rc):
    if rc != 0:
        raise MynnError("mynn error %d: %s" % (rc, lib().mynn_last_error().decode()))


# ------------------------------------------------------------------ torch plumbing
def _dt(t):
    import torch

    return {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}[t.dtype]


def _stream():
    import torch

    return torch.cuda.current_stream().cuda_stream


def _ptr(t):
    if t is None:
        return None
    assert t.is_cuda and t.is_contiguous(), "device-resident contiguous tensors only"
    return t.data_ptr()


def device_info():
    cu, wave, lds = _i(), _i(), _i()
    arch = C.create_string_buffer(64)
    check(lib().mynn_device_info(C.byref(cu), C.byref(wave), C.byref(lds), arch, 64))
    return {"cu_count": cu.value, "wave_size": wave.value, "lds_bytes": lds.value, "arch": arch.value.decode()}


def dequantize_linear(x_i8, scale):
    import torch

    out = torch.empty(x_i8.shape, dtype=scale.dtype, device=x_i8.device)
    rows = x_i8.shape[0]
    check(lib().mynn_dequantize_linear(_ptr(out), _ptr(x_i8), _ptr(scale), rows, x_i8.numel() // rows, _dt(scale),
                                       _stream()))
    return out


def dequant_gemv(act, wq, scale):
    import torch

    N, K = wq.shape
    out = torch.empty((N,), dtype=scale.dtype, device=wq.device)
    check(lib().mynn_dequant_gemv(_ptr(out), _ptr(act), _ptr(wq), _ptr(scale), N, K, _dt(act), _dt(scale), _stream()))
    return out


def dequant_matmul(act, wq, scale):
    import torch

    N, K = wq.shape
    M = act.numel() // K
    out = torch.empty(tuple(act.shape[:-1]) + (N,), dtype=scale.dtype, device=wq.device)
    check(lib().mynn_dequant_matmul(_ptr(out), _ptr(act), _ptr(wq), _ptr(scale), M, N, K, _dt(act), _dt(scale),
                                    _stream()))
    return out


def dequant_matmul_ws(act, wq, scale, gemm_tile=0):
    """mynn_dequant_matmul_ws: the caller's workspace (a torch tensor here), optional forced GEMM tile."""
    import torch

    N, K = wq.shape
    M = act.numel() // K
    out = torch.empty(tuple(act.shape[:-1]) + (N,), dtype=scale.dtype, device=wq.device)
    need = lib().mynn_dequant_matmul_workspace_bytes(M, N, K, _dt(act), _dt(scale))
    ws = torch.empty((max(need, 16),), dtype=torch.uint8, device=wq.device)
    check(lib().mynn_dequant_matmul_ws(_ptr(out), _ptr(act), _ptr(wq), _ptr(scale), M, N, K, _dt(act), _dt(scale), _ptr(ws), need,
                                       int(gemm_tile), _stream()))
    return out


def dequant_weight_prepare(wq, scale):
    """W dequantised once to the scale's type (mynn_dequant_weight_prepare); returns the opaque prepared buffer."""
    import torch

    N, K = wq.shape
    wt = torch.empty((lib().mynn_dequant_weight_bytes(N, K),), dtype=torch.uint8, device=wq.device)
    check(lib().mynn_dequant_weight_prepare(_ptr(wt), _ptr(wq), _ptr(scale), N, K, _dt(scale), _stream()))
    return wt


def dequant_matmul_prepared(act, wt, N, gemm_tile=0):
    import torch

    K = act.shape[-1]
    M = act.numel() // K
    out = torch.empty(tuple(act.shape[:-1]) + (N,), dtype=act.dtype, device=act.device)
    check(lib().mynn_dequant_matmul_prepared(_ptr(out), _ptr(act), _ptr(wt), M, N, K, _dt(act), int(gemm_tile), _stream()))
    return out


def quantized_matmul(lhs, lhs_scale, rhs, rhs_scale, want_acc=True):
    import torch

    M, K = lhs.shape
    N = rhs.shape[0]
    out = torch.empty((M, N), dtype=rhs_scale.dtype, device=lhs.device)
    acc = torch.empty((M, N), dtype=torch.int32, device=lhs.device) if want_acc else None
    check(lib().mynn_quantized_matmul(_ptr(out), _ptr(acc), _ptr(lhs), _ptr(lhs_scale), _ptr(rhs), _ptr(rhs_scale),
                                      M, N, K, _dt(rhs_scale), _stream()))
    return out, acc


def dynamic_quantize_linear(x, symmetric=True):
    import torch

    rows = x.shape[0]
    inner = x.numel() // rows
    y = torch.empty(x.shape, dtype=torch.int8 if symmetric else torch.uint8, device=x.device)
    s = torch.empty((rows,), dtype=x.dtype, device=x.device)
    zp = torch.empty((rows,), dtype=y.dtype, device=x.device)
    check(lib().mynn_dynamic_quantize_linear(_ptr(y), _ptr(s), _ptr(zp), _ptr(x), rows, inner, _dt(x),
                                             int(symmetric), _stream()))
    return y, s, zp


def attention(q, k, v, scale, is_causal=False, active=None, d_active=None, q_pos_offset=None, k_scale=None,
              v_scale=None):
    import torch

    B, Hq, Sq, D = q.shape
    Hkv, cache_len = k.shape[1], k.shape[2]
    if active is None:
        active = cache_len
    if q_pos_offset is None:
        q_pos_offset = 0 if Sq == cache_len else active - Sq
    out = torch.empty_like(q)
    check(lib().mynn_attention(_ptr(out), _ptr(q), _ptr(k), _ptr(v), _ptr(k_scale), _ptr(v_scale), float(scale),
                               int(is_causal), B, Sq, int(active), _ptr(d_active), cache_len, int(q_pos_offset),
                               Hq, Hkv, D, _dt(q), int(k.dtype == torch.int8), _stream()))
    return out


def attention_noalloc(q, k, v, scale, out, is_causal=False, active=None, d_active=None, q_pos_offset=None, k_scale=None,
                      v_scale=None):
    """mynn_attention_noalloc: the caller passes `out`; nothing is allocated on the way (not by this wrapper either)."""
    import torch

    B, Hq, Sq, D = q.shape
    Hkv, cache_len = k.shape[1], k.shape[2]
    if active is None:
        active = cache_len
    if q_pos_offset is None:
        q_pos_offset = 0 if Sq == cache_len else active - Sq
    check(lib().mynn_attention_noalloc(_ptr(out), _ptr(q), _ptr(k), _ptr(v), _ptr(k_scale), _ptr(v_scale), float(scale),
                                       int(is_causal), B, Sq, int(active), _ptr(d_active), cache_len, int(q_pos_offset),
                                       Hq, Hkv, D, _dt(q), int(k.dtype == torch.int8), _stream()))
    return out


def attention_ws(q, k, v, scale, is_causal=False, active=None, d_active=None, q_pos_offset=None, k_scale=None, v_scale=None,
                 mask=None):
    """mynn_attention_ws: caller-owned workspace, optional additive mask [..., Sq or 1, cache_len] broadcast over the
    leading (batch x head) dimensions when they multiply to 1 (operator slot 3)."""
    import torch

    B, Hq, Sq, D = q.shape
    Hkv, cache_len = k.shape[1], k.shape[2]
    if active is None:
        active = cache_len
    if q_pos_offset is None:
        q_pos_offset = 0 if Sq == cache_len else active - Sq
    out = torch.empty_like(q)
    kv8 = int(k.dtype == torch.int8)
    need = lib().mynn_attention_workspace_bytes(B, Sq, cache_len, Hq, Hkv, D, _dt(q), kv8)
    ws = torch.empty((max(need, 16),), dtype=torch.uint8, device=q.device)
    m_os = m_rs = 0
    if mask is not None:
        # the strides the reference derives from the mask's dims (src/codegen/cuda.rs:1297-1323)
        rows = mask.shape[-2] if mask.dim() >= 2 else 1
        cols = mask.shape[-1]
        assert cols == cache_len
        outer = mask.numel() // (rows * cols)
        m_rs = cols if rows > 1 else 0
        m_os = rows * cols if outer > 1 else 0
    check(lib().mynn_attention_ws(_ptr(out), _ptr(q), _ptr(k), _ptr(v), _ptr(mask), m_os, m_rs, _ptr(k_scale), _ptr(v_scale),
                                  float(scale), int(is_causal), B, Sq, int(active), _ptr(d_active), cache_len, int(q_pos_offset),
                                  Hq, Hkv, D, _dt(q), kv8, _ptr(ws), need, _stream()))
    return out


def kvcache_update(cache, new_kv, offset):
    B, H, max_seq, D = cache.shape
    check(lib().mynn_kvcache_update(_ptr(cache), _ptr(new_kv), int(offset), B * H, new_kv.shape[2], max_seq, D,
                                    _dt(cache), _stream()))
    return cache


class KvPool:
    """Free list of the page numbers of a paged KV cache (mynn_kv_pool); the pool buffers themselves are the
    caller's: `buffers(...)` makes one K and one V tensor [n_pages, Hkv, page_rows, D] per layer."""

    def __init__(self, n_pages, page_rows):
        self.n_pages, self.page_rows = int(n_pages), int(page_rows)
        self.handle = lib().mynn_kv_pool_create(self.n_pages, self.page_rows)
        if not self.handle:
            raise MynnError("kv_pool_create failed: %s" % lib().mynn_last_error().decode())

    @property
    def free_pages(self):
        return lib().mynn_kv_pool_free_pages(self.handle)

    def buffers(self, n_layers, n_kv_heads, head_dim, dtype, fill=None, kv_int8=False):
        """One (K pool, V pool) per layer, [n_pages, Hkv, page_rows, D] in `dtype`; kv_int8: (K codes, V codes, K scales,
        V scales) with int8 code pools and scale pools [n_pages, Hkv, page_rows] in `dtype`."""
        import torch

        shape = (self.n_pages, n_kv_heads, self.page_rows, head_dim)

        def make(sh, dt):
            return torch.zeros(sh, dtype=dt, device="cuda") if fill is None else torch.full(sh, fill, dtype=dt, device="cuda")

        if kv_int8:
            return [(torch.zeros(shape, dtype=torch.int8, device="cuda"), torch.zeros(shape, dtype=torch.int8, device="cuda"),
                     make(shape[:3], dtype), make(shape[:3], dtype)) for _ in range(n_layers)]
        return [(make(shape, dtype), make(shape, dtype)) for _ in range(n_layers)]

    def close(self):
        if getattr(self, "handle", None) and _lib is not None:
            check(_lib.mynn_kv_pool_destroy(self.handle))
            self.handle = None


class KvPages:
    """Page table of the `batch` sequences of one session over a KvPool (mynn_kv_pages)."""

    def __init__(self, pool, batch, max_seq):
        self.pool, self.batch, self.max_seq = pool, int(batch), int(max_seq)
        self.handle = lib().mynn_kv_pages_create(pool.handle, self.batch, self.max_seq)
        if not self.handle:
            raise MynnError("kv_pages_create failed: %s" % lib().mynn_last_error().decode())

    def reserve(self, rows):
        check(lib().mynn_kv_pages_reserve(self.handle, int(rows)))

    def release(self):
        check(lib().mynn_kv_pages_release(self.handle))

    @property
    def mapped_rows(self):
        return lib().mynn_kv_pages_mapped_rows(self.handle)

    @property
    def pages_per_seq(self):
        return lib().mynn_kv_pages_per_seq(self.handle)

    @property
    def table_ptr(self):
        return lib().mynn_kv_pages_table(self.handle)

    def table(self):
        """numpy int32 [batch, pages_per_seq]; -1 = not mapped"""
        import numpy as np

        out = np.empty((self.batch, self.pages_per_seq), np.int32)
        check(lib().mynn_kv_pages_table_host(self.handle, out.ctypes.data_as(_vp)))
        return out

    def close(self):
        if getattr(self, "handle", None) and _lib is not None:
            check(_lib.mynn_kv_pages_destroy(self.handle))
            self.handle = None


def attention_paged(q, k_pool, v_pool, table, page_rows, scale, is_causal, active, q_pos_offset=0, d_active=None,
                    k_scale_pool=None, v_scale_pool=None):
    """mynn_attention_paged: q [B,Hq,Sq,D]; pools [n_pages,Hkv,page_rows,D]; table: cuda int32 [B, pages_per_seq]."""
    import torch

    B, Hq, Sq, D = q.shape
    Hkv = k_pool.shape[1]
    pps = table.shape[1]
    assert table.dtype == torch.int32 and table.shape[0] == B and k_pool.shape[2] == page_rows
    out = torch.empty_like(q)
    need = lib().mynn_attention_paged_workspace_bytes(B, Sq, pps, int(page_rows), Hq, Hkv, D)
    ws = torch.empty((max(need, 16),), dtype=torch.uint8, device=q.device)
    check(lib().mynn_attention_paged(_ptr(out), _ptr(q), _ptr(k_pool), _ptr(v_pool), _ptr(k_scale_pool), _ptr(v_scale_pool),
                                     _ptr(table), pps, int(page_rows), float(scale), int(is_causal), B, Sq, int(active), _ptr(d_active),
                                     int(q_pos_offset), Hq, Hkv, D, _dt(q), int(k_pool.dtype == torch.int8), _ptr(ws), need, _stream()))
    return out


def kvcache_update_paged(pool, new_kv, offset, table, page_rows):
    """mynn_kvcache_update_paged: new_kv [B,Hkv,S_new,D] into pool [n_pages,Hkv,page_rows,D] through table [B,pages_per_seq]."""
    B, Hkv, S_new, D = new_kv.shape
    check(lib().mynn_kvcache_update_paged(_ptr(pool), _ptr(new_kv), int(offset), B, Hkv, S_new, D, _dt(new_kv), _ptr(table),
                                          table.shape[1], int(page_rows), _stream()))
    return pool


def kvcache_update_streaming(cache, new_kv, offset, ring_sink, ring_window, ring_start):
    """KVCacheUpdate through the sink + ring slot map (the reference's streaming-KV graph)."""
    import torch

    B, H, max_seq, D = cache.shape
    check(lib().mynn_kvcache_update_streaming(_ptr(cache), _ptr(new_kv), int(offset), B * H, new_kv.shape[2], max_seq, D,
                                              int(ring_sink), int(ring_window), int(ring_start),
                                              I8 if cache.dtype == torch.int8 else _dt(cache), _stream()))
    return cache


def quantizing_kvcache_update_streaming(cache, scale, new_kv, offset, ring_sink, ring_window, ring_start):
    B, H, max_seq, D = cache.shape
    check(lib().mynn_quantizing_kvcache_update_streaming(_ptr(cache), _ptr(scale), _ptr(new_kv), int(offset), B * H,
                                                         new_kv.shape[2], max_seq, D, int(ring_sink), int(ring_window),
                                                         int(ring_start), _dt(new_kv), _stream()))
    return cache, scale


def attention_streaming(q, k, v, scale, is_causal, active, ring_sink, ring_window, ring_start, q_pos_offset=None,
                        k_scale=None, v_scale=None, rope=None, workspace=None):
    """Attention over the sink + ring layout: keys by recency rank, rank -> cache row by the ring map.
    rope = (cos_table, sin_table, kv_position int64): rotate K inside the operator.
    workspace (uint8 tensor of mynn_attention_streaming_workspace_bytes): the caller's scratch memory."""
    import torch

    B, Hq, Sq, D = q.shape
    Hkv, cache_len = k.shape[1], k.shape[2]
    if q_pos_offset is None:
        q_pos_offset = active - Sq
    out = torch.empty_like(q)
    if workspace is not None:
        check(lib().mynn_attention_streaming_ws(_ptr(out), _ptr(q), _ptr(k), _ptr(v), _ptr(k_scale), _ptr(v_scale), float(scale),
                                                int(is_causal), B, Sq, int(active), cache_len, int(q_pos_offset), Hq, Hkv, D,
                                                _dt(q), int(k.dtype == torch.int8), int(ring_sink), int(ring_window),
                                                int(ring_start), _ptr(rope[0]) if rope else None, _ptr(rope[1]) if rope else None,
                                                _ptr(rope[2]) if rope else None, _ptr(workspace), workspace.numel(), _stream()))
        return out
    check(lib().mynn_attention_streaming(_ptr(out), _ptr(q), _ptr(k), _ptr(v), _ptr(k_scale), _ptr(v_scale), float(scale),
                                         int(is_causal), B, Sq, int(active), cache_len, int(q_pos_offset), Hq, Hkv, D,
                                         _dt(q), int(k.dtype == torch.int8), int(ring_sink), int(ring_window),
                                         int(ring_start), _ptr(rope[0]) if rope else None, _ptr(rope[1]) if rope else None,
                                         _ptr(rope[2]) if rope else None, _stream()))
    return out


def quantizing_kvcache_update(cache, scale, new_kv, offset):
    B, H, max_seq, D = cache.shape
    check(lib().mynn_quantizing_kvcache_update(_ptr(cache), _ptr(scale), _ptr(new_kv), int(offset), B * H,
                                               new_kv.shape[2], max_seq, D, _dt(new_kv), _stream()))
    return cache, scale


def rms_norm(x, w, eps):
    import torch

    out = torch.empty_like(x)
    dim = x.shape[-1]
    check(lib().mynn_rms_norm(_ptr(out), _ptr(x), _ptr(w), x.numel() // dim, dim, float(eps), _dt(x), _stream()))
    return out


def rope(x, cos_t, sin_t, position):
    import torch

    out = torch.empty_like(x)
    S, D = x.shape[-2], x.shape[-1]
    check(lib().mynn_rope(_ptr(out), _ptr(x), _ptr(cos_t), _ptr(sin_t), _ptr(position), x.numel() // (S * D), S, D,
                          _dt(x), _stream()))
    return out


def gather_rows(data, idx):
    import torch

    rows = data.shape[0]
    row_bytes = data.numel() // rows * data.element_size()
    out = torch.empty(tuple(idx.shape) + tuple(data.shape[1:]), dtype=data.dtype, device=data.device)
    check(lib().mynn_gather_rows(_ptr(out), _ptr(data), _ptr(idx), idx.numel(), rows, row_bytes, _stream()))
    return out


def swiglu(gate, up):
    import torch

    out = torch.empty_like(gate)
    check(lib().mynn_swiglu(_ptr(out), _ptr(gate), _ptr(up), gate.numel(), _dt(gate), _stream()))
    return out


def add(a, b):
    import torch

    out = torch.empty_like(a)
    check(lib().mynn_add(_ptr(out), _ptr(a), _ptr(b), a.numel(), _dt(a), _stream()))
    return out


def argmax_last(logits):
    import torch

    out = torch.empty((1,), dtype=torch.int32, device=logits.device)
    check(lib().mynn_argmax_last(_ptr(out), _ptr(logits), logits.numel(), _dt(logits), _stream()))
    return out


# ------------------------------------------------------------------ decoder executor (seam 1)
LIN_NAMES = ("q", "k", "v", "o", "gate", "up", "down")


class Weights:
    """HfWeights: a .safetensors file or model directory, memory-mapped (crates/llm/src/hf_weights.rs)."""

    def __init__(self, path):
        self.handle = lib().mynn_weights_open(str(path).encode())
        if not self.handle:
            raise MynnError(lib().mynn_last_error().decode())

    def names(self):
        return [lib().mynn_weights_name(self.handle, i).decode() for i in range(lib().mynn_weights_count(self.handle))]

    def find(self, name):
        """(dtype code, shape, numpy view of the mapped bytes)."""
        import numpy as np

        dt, nd, ptr, nb = _i(), _i(), _vp(), _sz()
        shape = (_i64 * 8)()
        check(lib().mynn_weights_find(self.handle, name.encode(), C.byref(dt), shape, C.byref(nd), C.byref(ptr), C.byref(nb)))
        npdt = {F32: np.float32, BF16: np.uint16, F16: np.uint16, I8: np.int8}[dt.value]
        buf = (C.c_char * nb.value).from_address(ptr.value) if nb.value else b""
        arr = np.frombuffer(buf, dtype=npdt).reshape([shape[i] for i in range(nd.value)])
        return dt.value, tuple(arr.shape), arr

    def close(self):
        if getattr(self, "handle", None) and _lib is not None:
            _lib.mynn_weights_close(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def quantize_safetensors_int8(src, dst):
    """crates/llm/src/quantize.rs quantize_safetensors_int8(_dir): returns (quantized, passthrough)."""
    q, p = _i(), _i()
    check(lib().mynn_quantize_safetensors_int8(str(src).encode(), str(dst).encode(), C.byref(q), C.byref(p)))
    return q.value, p.value


class DeviceWeights:
    """A checkpoint uploaded in `initializer` order (mynn_weights_upload); owns the device memory."""

    def __init__(self, weights, cfg_struct):
        self.handle = lib().mynn_weights_upload(weights.handle, C.byref(cfg_struct))
        if not self.handle:
            raise MynnError(lib().mynn_last_error().decode())
        self.int8 = bool(lib().mynn_device_weights_int8(self.handle))
        self.initializer = lib().mynn_device_weights_initializer(self.handle)

    def close(self):
        if getattr(self, "handle", None) and _lib is not None:
            _lib.mynn_device_weights_free(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def _initializer_array(cfg, weights, quant):
    """The `initializer` array of model_init for a weight dict (order of the reference's graph initializers)."""
    init = []

    def lin(w):
        if quant:
            init.extend([_ptr(w[0]), _ptr(w[1])])
        else:
            init.extend([_ptr(w), None])

    lin(weights["embed"])
    for l in range(cfg.n_layers):
        init.append(_ptr(weights["layers.%d.norm1" % l]))
        for nm in ("q", "k", "v", "o"):
            lin(weights["layers.%d.%s" % (l, nm)])
            if cfg.qkv_bias and nm != "o":
                init.append(_ptr(weights["layers.%d.%s.bias" % (l, nm)]))
        init.append(_ptr(weights["layers.%d.norm2" % l]))
        for nm in ("gate", "up", "down"):
            lin(weights["layers.%d.%s" % (l, nm)])
    init.append(_ptr(weights["final_norm"]))
    lin(weights["lm_head"])
    return (_vp * len(init))(*init)


class WeightSet:
    """mynn_weight_set: the library's derived copies of one checkpoint's weights (decode repacks, 16-bit resident copy,
    tiled int8 copy, W8A8 interleave), each made once and shared by every Decoder built with weight_set=this."""

    def __init__(self, cfg, weights):
        import torch

        quant = isinstance(weights["embed"], tuple)
        qkv_bias = bool(cfg.get("qkv_bias")) or "layers.0.q.bias" in weights
        self.cfg = ModelConfig(cfg["n_layers"], cfg["hidden"], cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"], cfg["ffn"],
                               cfg["vocab"], cfg["max_seq"], float(cfg["eps"]), float(cfg["rope_theta"]), cfg["dtype"], 1, 1,
                               int(quant), 0, 0, 0, 0, 0, 0, 0, 0, int(qkv_bias))
        self.weights = weights
        self._init = _initializer_array(self.cfg, weights, quant)
        torch.cuda.synchronize()
        self.handle = lib().mynn_weight_set_create(C.byref(self.cfg), self._init)
        if not self.handle:
            raise MynnError("weight_set_create failed: %s" % lib().mynn_last_error().decode())

    def stats(self):
        b = (_sz * 4)()
        n = _i(0)
        check(lib().mynn_weight_set_stats(self.handle, b, C.byref(n)))
        return {"repack_bytes": b[0], "resident16_bytes": b[1], "tiled_int8_bytes": b[2], "w8a8_interleave_bytes": b[3],
                "holders": n.value}

    def close(self):
        if getattr(self, "handle", None) and _lib is not None:
            _lib.mynn_weight_set_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Decoder:
    """Thin holder around model_init / model_step / model_destroy.

    weights: dict of cuda tensors keyed like the oracle's Model:
      "embed", "lm_head", "layers.{i}.{q,k,v,o,gate,up,down}" -> (int8 [N,K], scale [N]) or a
      single float tensor [N,K]; "final_norm", "layers.{i}.norm1|norm2"; optional "layers.{i}.{q,k,v}.bias" [N].
    kv: optional list of (k_cache, v_cache) cuda tensors [batch,Hkv,max_seq,D] per layer, so a
      prefill and a decode model can share them (PersistentBuffers in the reference).
    """

    def __init__(self, cfg, weights, seq_q=1, batch=1, kv=None, quant_kv_cache=False, quantize_activations=False,
                 streaming_kv=False, gemm_tile=0, unfused_decode=False, handover_spin_limit=0, weight_arena=False,
                 reference_abi=False, kv_pages=None, weight_set=None):
        """weight_set: a WeightSet made from the same cfg shapes and weights -- the executor then shares the library's
        derived weight copies with the other executors built on it (mynn_model_create_shared)."""
        import torch

        tdt = {F16: torch.float16, BF16: torch.bfloat16}[cfg["dtype"]]
        from_file = isinstance(weights, (str, os.PathLike, Weights))
        quant = True if from_file else isinstance(weights["embed"], tuple)
        # q / k / v projection biases (qwen2): cfg["qkv_bias"], or "layers.{i}.{q,k,v}.bias" entries in a weight dict
        qkv_bias = bool(cfg.get("qkv_bias")) or (not from_file and "layers.0.q.bias" in weights)
        self.cfg = ModelConfig(cfg["n_layers"], cfg["hidden"], cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"],
                               cfg["ffn"], cfg["vocab"], cfg["max_seq"], float(cfg["eps"]), float(cfg["rope_theta"]),
                               cfg["dtype"], seq_q, batch, int(quant), int(quant_kv_cache), int(quantize_activations),
                               int(streaming_kv), int(gemm_tile), int(unfused_decode), int(handover_spin_limit), int(weight_arena),
                               kv_pages.pool.page_rows if kv_pages is not None else 0, int(qkv_bias))
        self.weights = weights  # keep the tensors alive
        self.kv_pages = kv_pages
        self.weight_set = weight_set
        if kv_pages is not None:
            # paged cache: kv = the pool buffers (KvPool.buffers), one (K pool, V pool) per layer, shared by every session of the pool
            assert kv is not None, "a paged decoder takes the pool's buffers as kv"
        if kv is None:
            shape = (batch, cfg["n_kv_heads"], cfg["max_seq"], cfg["head_dim"])
            if quant_kv_cache:  # (k i8, v i8, k_scale, v_scale) per layer
                kv = [(torch.zeros(shape, dtype=torch.int8, device="cuda"), torch.zeros(shape, dtype=torch.int8, device="cuda"),
                       torch.zeros(shape[:3], dtype=tdt, device="cuda"), torch.zeros(shape[:3], dtype=tdt, device="cuda"))
                      for _ in range(cfg["n_layers"])]
            else:
                kv = [(torch.zeros(shape, dtype=tdt, device="cuda"), torch.zeros(shape, dtype=tdt, device="cuda"))
                      for _ in range(cfg["n_layers"])]
        self.kv = kv
        state = []
        for bufs in kv:
            state.extend([_ptr(t) for t in bufs])
        if kv_pages is not None:
            state.append(kv_pages.handle)
        self._state = (_vp * len(state))(*state)
        if from_file:
            # a checkpoint: read, convert and upload by the library (names as the reference's ModelSpec)
            src = weights if isinstance(weights, Weights) else Weights(weights)
            self.weights = DeviceWeights(src, self.cfg)
            self.cfg.weights_int8 = int(self.weights.int8)
            self.handle = self._create(self.weights.initializer, reference_abi)
            return
        if weight_set is not None:
            handle = lib().mynn_model_create_shared(C.byref(self.cfg), weight_set.handle, self._state)
            if not handle:
                raise MynnError("model_create_shared failed: %s" % lib().mynn_last_error().decode())
            self.handle = handle
            return
        self._init = _initializer_array(self.cfg, weights, quant)
        torch.cuda.synchronize()
        self.handle = self._create(self._init, reference_abi)

    def _create(self, init, reference_abi):
        """reference_abi: mynn_model_configure + model_init (the symbols SessionCUDA binds) instead of the one call
        that touches nothing process-wide."""
        if reference_abi:
            check(lib().mynn_model_configure(C.byref(self.cfg)))
            handle = lib().model_init(init, self._state)
        else:
            handle = lib().mynn_model_create(C.byref(self.cfg), init, self._state)
        if not handle:
            raise MynnError("model_init failed: %s" % lib().mynn_last_error().decode())
        return handle

    def close(self):
        if getattr(self, "handle", None) and _lib is not None:
            _lib.model_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:  # interpreter shutdown
            pass

    def step(self, ids, positions, past_len, active, want_logits=False):
        """One graph run; returns (next tokens per sequence, logits numpy or None)."""
        import numpy as np

        ids = np.ascontiguousarray(np.asarray(ids, np.int64).ravel())
        positions = np.ascontiguousarray(np.asarray(positions, np.int64).ravel())
        assert ids.size == self.cfg.batch * self.cfg.seq_q and positions.size == self.cfg.seq_q
        nxt = (C.c_int32 * self.cfg.batch)()
        logits = None
        lp = None
        if want_logits:
            npdt = np.uint16
            logits = np.empty((self.cfg.batch * self.cfg.seq_q, self.cfg.vocab), npdt)
            lp = logits.ctypes.data_as(_vp)
        check(lib().mynn_model_step(self.handle, ids.ctypes.data_as(_vp), positions.ctypes.data_as(_vp),
                                    int(past_len), int(active), nxt, lp))
        return list(nxt), logits

    def step_streaming(self, ids, positions, past_len, active, sink, window, start, kv_position, want_logits=False):
        """One run of a streaming_kv model: the four ring inputs of the reference's streaming session."""
        import numpy as np

        ids = np.ascontiguousarray(np.asarray(ids, np.int64).ravel())
        positions = np.ascontiguousarray(np.asarray(positions, np.int64).ravel())
        kvp = np.ascontiguousarray(np.asarray(kv_position, np.int64).ravel())
        assert ids.size == self.cfg.batch * self.cfg.seq_q and positions.size == self.cfg.seq_q and kvp.size == self.cfg.max_seq
        nxt = (C.c_int32 * self.cfg.batch)()
        logits, lp = None, None
        if want_logits:
            logits = np.empty((self.cfg.batch * self.cfg.seq_q, self.cfg.vocab), np.uint16)
            lp = logits.ctypes.data_as(_vp)
        check(lib().mynn_model_step_streaming(self.handle, ids.ctypes.data_as(_vp), positions.ctypes.data_as(_vp), int(past_len),
                                              int(active), int(sink), int(window), int(start), kvp.ctypes.data_as(_vp), nxt, lp))
        return list(nxt), logits

    def model(self, ids, positions, past_len, active, ring=None):
        """The reference ABI call `model(state, output, input)` with host pointers; ring = (sink, window, start,
        kv_position) for a streaming_kv model.  Raises when the state's status after the void call is not 0."""
        import numpy as np

        ids = np.ascontiguousarray(np.asarray(ids, np.int64).ravel())
        positions = np.ascontiguousarray(np.asarray(positions, np.int64).ravel())
        pl = np.array([past_len], np.int64)
        ac = np.array([active], np.int64)
        logits = np.empty((self.cfg.batch * self.cfg.seq_q, self.cfg.vocab), np.uint16)
        ptrs = [ids.ctypes.data, positions.ctypes.data, pl.ctypes.data, ac.ctypes.data]
        keep = []
        if ring is not None:
            keep = [np.array([ring[0]], np.int64), np.array([ring[1]], np.int64), np.array([ring[2]], np.int64),
                    np.ascontiguousarray(np.asarray(ring[3], np.int64))]
            ptrs += [a.ctypes.data for a in keep]
        inp = (_vp * len(ptrs))(*ptrs)
        out = (_vp * 1)(logits.ctypes.data)
        lib().model(self.handle, out, inp)
        check(lib().mynn_model_last_status(self.handle))
        return logits

    @property
    def handover_failures(self):
        return lib().mynn_model_handover_failures(self.handle)

    def set_handover_rearm(self, clean_steps):
        """Steps without a give-up after which a model that fell back to one op per launch tries the shared launches
        again (0: never)."""
        check(lib().mynn_model_set_handover_rearm(self.handle, int(clean_steps)))

    def decode_loop(self, token, past_len, n_steps):
        out = (C.c_int32 * n_steps)()
        check(lib().mynn_model_decode_loop(self.handle, int(token), int(past_len), n_steps, out))
        return list(out)

    def profile_step(self, token, past_len, cap=1024):
        """[(name, ms, algorithmic bytes, flops)] of one eager batch-1 decode step."""
        arr = (KernelTime * cap)()
        n = lib().mynn_model_profile_step(self.handle, int(token), int(past_len), arr, cap)
        if n < 0:
            check(n)
        return [(arr[i].name.decode(), arr[i].ms, arr[i].bytes, arr[i].flops) for i in range(n)]

    def profile(self, ids, positions, past_len, active, cap=2048):
        """Same for any model shape; operands as in step()."""
        import numpy as np

        ids = np.ascontiguousarray(np.asarray(ids, np.int64).ravel())
        positions = np.ascontiguousarray(np.asarray(positions, np.int64).ravel())
        assert ids.size == self.cfg.batch * self.cfg.seq_q and positions.size == self.cfg.seq_q
        arr = (KernelTime * cap)()
        n = lib().mynn_model_profile(self.handle, ids.ctypes.data_as(_vp), positions.ctypes.data_as(_vp),
                                     int(past_len), int(active), arr, cap)
        if n < 0:
            check(n)
        return [(arr[i].name.decode(), arr[i].ms, arr[i].bytes, arr[i].flops) for i in range(n)]

    def stats(self):
        a, n, g = _sz(), _i(), _i()
        check(lib().mynn_model_stats(self.handle, C.byref(a), C.byref(n), C.byref(g)))
        return {"arena_bytes": a.value, "launches_per_step": n.value, "graph": bool(g.value)}


class LlmSession:
    """crates/llm LlmSession: decode model + optional prefill model over shared weights and KV."""

    def __init__(self, decoder, prefill=None, eos=-1, streaming=None):
        """streaming = (sink, window): DecodeKind::LlamaStreaming; the models must have been built with streaming_kv."""
        self.decoder, self.prefill = decoder, prefill
        pl = prefill.cfg.seq_q if prefill is not None else 0
        self.handle = lib().mynn_llm_create(decoder.handle, prefill.handle if prefill is not None else None, pl,
                                            decoder.cfg.max_seq, int(eos))
        if not self.handle:
            raise MynnError(lib().mynn_last_error().decode())
        if streaming is not None:
            check(lib().mynn_llm_set_streaming(self.handle, int(streaming[0]), int(streaming[1])))

    def close(self):
        if getattr(self, "handle", None) and _lib is not None:
            _lib.mynn_llm_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:  # interpreter shutdown
            pass

    def reset(self):
        lib().mynn_llm_reset(self.handle)

    @property
    def past_len(self):
        return lib().mynn_llm_past_len(self.handle)

    @past_len.setter
    def past_len(self, v):
        lib().mynn_llm_set_past_len(self.handle, int(v))

    def generate_ids(self, prompt_ids, max_new_tokens):
        import numpy as np

        p = np.ascontiguousarray(np.asarray(prompt_ids, np.int64))
        out = np.empty((max(max_new_tokens, 1),), np.int64)
        n = lib().mynn_llm_generate_ids(self.handle, p.ctypes.data_as(_vp), p.size, max_new_tokens,
                                        out.ctypes.data_as(_vp))
        if n < 0:
            raise MynnError("generate_ids error %d: %s" % (n, lib().mynn_last_error().decode()))
        return [int(t) for t in out[:n]]


def quantize_per_channel(w_f32, scale_dt):
    """Host quantiser of the library (numpy in, numpy out)."""
    import numpy as np

    w = np.ascontiguousarray(np.asarray(w_f32, np.float32))
    rows = w.shape[0]
    q = np.empty(w.shape, np.int8)
    s = np.empty((rows,), np.float32 if scale_dt == F32 else np.uint16)
    check(lib().mynn_quantize_per_channel(q.ctypes.data_as(_vp), s.ctypes.data_as(_vp), w.ctypes.data_as(_vp), rows,
                                          w.size // rows, scale_dt))
    return q, s


def rope_table(max_seq, head_dim, base, dt):
    import numpy as np

    npdt = np.float32 if dt == F32 else np.uint16
    cos = np.empty((max_seq, head_dim), npdt)
    sin = np.empty((max_seq, head_dim), npdt)
    check(lib().mynn_rope_table(cos.ctypes.data_as(_vp), sin.ctypes.data_as(_vp), max_seq, head_dim, float(base), dt))
    return cos, sin
