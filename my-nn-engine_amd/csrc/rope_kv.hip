// RoPE(q), RoPE(k), KVCacheUpdate(k), KVCacheUpdate(v) in one launch.
//
// The reference runs these as ~16 kernels per layer: the decomposed RoPE graph of
// crates/llm/src/builder.rs:402-438 (Slice, Slice, Neg, Concat, Mul, Mul, Add for q and again for
// k), the [S,H,D]->[H,S,D] transposes and two kvcache_update launches (kvcache_update.cuh:6-26).
// Arithmetic is unchanged: lo' = lo*cos[p,j] - hi*sin[p,j], hi' = hi*cos[p,j+D/2] + lo*sin[p,j+D/2]
// with separate products and one rounding; v is copied.
#include "kernels.h"
#include "mfma.h"

namespace mynn {

template <typename T>
__global__ void rope_kv_append_kernel(T *q_out, T *k_cache, T *v_cache, const T *qkv, const T *cos_t, const T *sin_t,
                                      const int64_t *position, const int32_t *d_past, int past_host, int S, int Hq,
                                      int Hkv, int D, int max_seq, KvPaging pg) {
    const int s = blockIdx.x, head = blockIdx.y, b = blockIdx.z;
    const int half = D / 2;
    const int past = d_past ? *d_past : past_host;
    const size_t row = (size_t)b * S + s;
    const int width = (Hq + 2 * Hkv) * D;
    const T *src = qkv + row * width + (size_t)head * D;
    if (head < Hq && !q_out) return;
    if (head < Hq + Hkv) {
        T *dst = head < Hq ? q_out + row * (size_t)Hq * D + (size_t)head * D
                           : k_cache + kv_cache_row(pg, b, head - Hq, past + s, Hkv, max_seq) * D;
        const size_t tab = (size_t)position[s] * D;
        for (int j = threadIdx.x; j < half; j += blockDim.x) {
            float xl = Elem<T>::ld(src, j), xh = Elem<T>::ld(src, j + half);
            float cl = Elem<T>::ld(cos_t, tab + j), ch = Elem<T>::ld(cos_t, tab + j + half);
            float sl = Elem<T>::ld(sin_t, tab + j), sh = Elem<T>::ld(sin_t, tab + j + half);
            Elem<T>::st(dst, j, xl * cl - xh * sl);
            Elem<T>::st(dst, j + half, xh * ch + xl * sh);
        }
    } else {
        T *dst = v_cache + kv_cache_row(pg, b, head - Hq - Hkv, past + s, Hkv, max_seq) * D;
        for (int j = threadIdx.x; j < D; j += blockDim.x) dst[j] = src[j];
    }
}

// Same work for head_dim % 16 == 0, 128 bits per access: one workgroup per token row, one thread per
// (head, 8 rotation pairs) -- it loads the 8 low and the 8 high elements and the matching table
// entries, and writes both halves; v heads copy two chunks.
template <typename T>
__global__ __launch_bounds__(256) void rope_kv_append_vec_kernel(T *q_out, T *k_cache, T *v_cache, const T *qkv,
                                                                 const T *cos_t, const T *sin_t, const int64_t *position,
                                                                 const int32_t *d_past, int past_host, int S, int Hq,
                                                                 int Hkv, int D, int max_seq, KvPaging pg) {
    const int s = blockIdx.x, b = blockIdx.y;
    const int half = D / 2, upc = half / 8;  // units per head
    const int past = d_past ? *d_past : past_host;
    const size_t row = (size_t)b * S + s;
    const int heads = Hq + 2 * Hkv;
    const T *src_row = qkv + row * (size_t)heads * D;
    const size_t tab = (size_t)position[s] * D;
    // (q_out == nullptr: the queries are rotated by their consumer; only k and v are done here)
    for (int u = threadIdx.x + (q_out ? 0 : Hq * upc); u < heads * upc; u += blockDim.x) {
        const int head = u / upc, j = (u % upc) * 8;
        const T *src = src_row + (size_t)head * D;
        const U4 lo = *(const U4 *)(src + j), hi = *(const U4 *)(src + j + half);
        if (head >= Hq + Hkv) {
            T *dst = v_cache + kv_cache_row(pg, b, head - Hq - Hkv, past + s, Hkv, max_seq) * D;
            *(U4 *)(dst + j) = lo;
            *(U4 *)(dst + j + half) = hi;
            continue;
        }
        T *dst = head < Hq ? q_out + row * (size_t)Hq * D + (size_t)head * D
                           : k_cache + kv_cache_row(pg, b, head - Hq, past + s, Hkv, max_seq) * D;
        float xl[8], xh[8], cl[8], ch[8], sl[8], sh[8], ol[8], oh[8];
        widen8<T>(lo, xl);
        widen8<T>(hi, xh);
        widen8<T>(*(const U4 *)(cos_t + tab + j), cl);
        widen8<T>(*(const U4 *)(cos_t + tab + j + half), ch);
        widen8<T>(*(const U4 *)(sin_t + tab + j), sl);
        widen8<T>(*(const U4 *)(sin_t + tab + j + half), sh);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            ol[i] = xl[i] * cl[i] - xh[i] * sl[i];
            oh[i] = xh[i] * ch[i] + xl[i] * sh[i];
        }
        *(U4 *)(dst + j) = U4{pack2<T>(ol[0], ol[1]), pack2<T>(ol[2], ol[3]), pack2<T>(ol[4], ol[5]), pack2<T>(ol[6], ol[7])};
        *(U4 *)(dst + j + half) = U4{pack2<T>(oh[0], oh[1]), pack2<T>(oh[2], oh[3]), pack2<T>(oh[4], oh[5]), pack2<T>(oh[6], oh[7])};
    }
}

// int8 KV cache (BuildOptions::quant_kv_cache): RoPE(q) -> q_out; RoPE(k) rounded to T and v are quantised
// per token row with the rule of quantizing_kvcache_update (CPU backend rounding: s = amax/127,
// q = trunc(x * 127/amax +- 0.5) clamped to [-128,127]) into the int8 caches and their scale rows
// [B,Hkv,max_seq].  One wave per (token, head); needs D <= 128.
template <typename T>
__global__ __launch_bounds__(64) void rope_quant_kv_append_kernel(T *q_out, int8_t *k_cache, int8_t *v_cache, T *k_scale,
                                                                 T *v_scale, const T *qkv, const T *cos_t, const T *sin_t,
                                                                 const int64_t *position, const int32_t *d_past, int S,
                                                                 int Hq, int Hkv, int D, int max_seq, KvPaging pg) {
    const int s = blockIdx.x, head = blockIdx.y, b = blockIdx.z, lane = threadIdx.x;
    const int half = D / 2;
    const int past = *d_past;
    const size_t row = (size_t)b * S + s;
    const T *src = qkv + row * (size_t)(Hq + 2 * Hkv) * D + (size_t)head * D;
    // lane j < D/2 owns elements j and j + D/2
    float lo = 0.f, hi = 0.f;
    const bool on = lane < half;
    if (on) {
        lo = Elem<T>::ld(src, lane);
        hi = Elem<T>::ld(src, lane + half);
        if (head < Hq + Hkv) {
            const size_t tab = (size_t)position[s] * D;
            const float cl = Elem<T>::ld(cos_t, tab + lane), ch = Elem<T>::ld(cos_t, tab + lane + half);
            const float sl = Elem<T>::ld(sin_t, tab + lane), sh = Elem<T>::ld(sin_t, tab + lane + half);
            const float rl = Elem<T>::rnd(lo * cl - hi * sl), rh = Elem<T>::rnd(hi * ch + lo * sh);
            lo = rl;
            hi = rh;
        }
    }
    if (head < Hq) {
        if (on) {
            T *dst = q_out + row * (size_t)Hq * D + (size_t)head * D;
            Elem<T>::st(dst, lane, lo);
            Elem<T>::st(dst, lane + half, hi);
        }
        return;
    }
    const bool is_k = head < Hq + Hkv;
    const int hk = is_k ? head - Hq : head - Hq - Hkv;
    const size_t tok = kv_cache_row(pg, b, hk, past + s, Hkv, max_seq);  // (paged: the scale pools share the table)
    const float amax = wave_max(fmaxf(fabsf(lo), fabsf(hi)));
    const float inv = amax == 0.f ? 0.f : 127.0f / amax;
    if (lane == 0) Elem<T>::st(is_k ? k_scale : v_scale, tok, amax * (1.0f / 127.0f));
    if (on) {
        int8_t *dst = (is_k ? k_cache : v_cache) + tok * D;
        const float a = lo * inv, c = hi * inv;
        int qa = (int)(a + (a >= 0.f ? 0.5f : -0.5f)), qc = (int)(c + (c >= 0.f ? 0.5f : -0.5f));
        qa = qa < -128 ? -128 : (qa > 127 ? 127 : qa);
        qc = qc < -128 ? -128 : (qc > 127 ? 127 : qc);
        dst[lane] = (int8_t)qa;
        dst[lane + half] = (int8_t)qc;
    }
}

template <typename T>
int rope_quant_kv_append(void *q_out, int8_t *k_cache, int8_t *v_cache, void *k_scale, void *v_scale, const void *qkv,
                         const void *cos_t, const void *sin_t, const int64_t *position, const int32_t *d_past, int B,
                         int S, int Hq, int Hkv, int D, int max_seq, hipStream_t s, KvPaging paging) {
    MYNN_REQUIRE(D % 2 == 0 && D <= 128, MYNN_ERR_UNSUPPORTED, "int8 KV append: head_dim %d", D);
    MYNN_REQUIRE(!paging.table || (paging.shift > 0 && paging.shift < 31 && max_seq == paging.pages_per_seq << paging.shift),
                 MYNN_ERR_INVALID, "int8 KV append: %d rows per sequence are not %d pages of %d rows", max_seq,
                 paging.pages_per_seq, 1 << paging.shift);
    MYNN_REQUIRE(S <= 65535 * 32 && Hq + 2 * Hkv <= 65535 && B <= 65535, MYNN_ERR_UNSUPPORTED, "int8 KV append: grid");
    MYNN_REQUIRE(d_past, MYNN_ERR_INVALID, "int8 KV append: null past_len");
    MYNN_LAUNCH(rope_quant_kv_append_kernel<T>, dim3(S, Hq + 2 * Hkv, B), dim3(64), 0, s, (T *)q_out, k_cache, v_cache,
                (T *)k_scale, (T *)v_scale, (const T *)qkv, (const T *)cos_t, (const T *)sin_t, position, d_past, S, Hq,
                Hkv, D, max_seq, paging);
    return launch_status("rope_quant_kv_append_kernel");
}
template int rope_quant_kv_append<bf16_t>(void *, int8_t *, int8_t *, void *, void *, const void *, const void *, const void *,
                                          const int64_t *, const int32_t *, int, int, int, int, int, int, hipStream_t, KvPaging);
template int rope_quant_kv_append<f16_t>(void *, int8_t *, int8_t *, void *, void *, const void *, const void *, const void *,
                                         const int64_t *, const int32_t *, int, int, int, int, int, int, hipStream_t, KvPaging);

template <typename T>
int rope_kv_append(void *q_out, void *k_cache, void *v_cache, const void *qkv, const void *cos_t, const void *sin_t,
                   const int64_t *position, const int32_t *d_past, int past_host, int B, int S, int Hq, int Hkv, int D,
                   int max_seq, hipStream_t s, KvPaging paging) {
    MYNN_REQUIRE(S <= 65535 * 32 && Hq + 2 * Hkv <= 65535 && B <= 65535, MYNN_ERR_UNSUPPORTED, "rope_kv_append: grid");
    MYNN_REQUIRE(!paging.table || (paging.shift > 0 && paging.shift < 31 && max_seq == paging.pages_per_seq << paging.shift),
                 MYNN_ERR_INVALID, "rope_kv_append: %d rows per sequence are not %d pages of %d rows", max_seq,
                 paging.pages_per_seq, 1 << paging.shift);
    if (D % 16 == 0 && S <= 65535 * 32 && (!q_out || aligned16(q_out)) && aligned16(k_cache) && aligned16(v_cache) && aligned16(qkv) &&
        aligned16(cos_t) && aligned16(sin_t)) {
        const int units = (q_out ? Hq + 2 * Hkv : 2 * Hkv) * (D / 16);
        const int threads = units >= 256 ? 256 : (units + 63) / 64 * 64;
        MYNN_LAUNCH(rope_kv_append_vec_kernel<T>, dim3(S, B), dim3(threads), 0, s, (T *)q_out, (T *)k_cache,
                           (T *)v_cache, (const T *)qkv, (const T *)cos_t, (const T *)sin_t, position, d_past, past_host,
                           S, Hq, Hkv, D, max_seq, paging);
        return launch_status("rope_kv_append_vec_kernel");
    }
    int threads = D / 2 >= 64 ? 64 : 32;
    MYNN_LAUNCH(rope_kv_append_kernel<T>, dim3(S, Hq + 2 * Hkv, B), dim3(threads), 0, s, (T *)q_out,
                       (T *)k_cache, (T *)v_cache, (const T *)qkv, (const T *)cos_t, (const T *)sin_t, position, d_past,
                       past_host, S, Hq, Hkv, D, max_seq, paging);
    return launch_status("rope_kv_append_kernel");
}
template int rope_kv_append<bf16_t>(void *, void *, void *, const void *, const void *, const void *, const int64_t *,
                                    const int32_t *, int, int, int, int, int, int, int, hipStream_t, KvPaging);
template int rope_kv_append<f16_t>(void *, void *, void *, const void *, const void *, const void *, const int64_t *,
                                   const int32_t *, int, int, int, int, int, int, int, hipStream_t, KvPaging);

// KVCacheUpdate into a pool: pool row of (b, hk, offset + t) <- new[b, hk, t, :]; rows of `units` 4-byte units
__global__ void kvcache_update_paged_kernel(uint32_t *pool, const uint32_t *src, int offset, int Hkv, int S_new, int units,
                                            KvPaging pg, size_t total) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int u = (int)(i % units);
    const size_t row = i / units;
    const int t = (int)(row % S_new), hk = (int)((row / S_new) % Hkv), b = (int)(row / ((size_t)S_new * Hkv));
    pool[kv_cache_row(pg, b, hk, offset + t, Hkv, 0) * units + u] = src[i];
}

}  // namespace mynn

using namespace mynn;

extern "C" int mynn_kvcache_update_paged(void *pool, const void *new_kv, int offset, int B, int Hkv, int S_new, int D, int dtype,
                                         const int32_t *page_table, int pages_per_seq, int page_rows, mynn_stream s) {
    MYNN_REQUIRE(pool && new_kv && page_table, MYNN_ERR_INVALID, "kvcache_update_paged: null operand");
    MYNN_REQUIRE(page_rows >= 32 && page_rows <= (1 << 20) && (page_rows & (page_rows - 1)) == 0 && pages_per_seq > 0, MYNN_ERR_INVALID,
                 "kvcache_update_paged: %d pages of %d rows (rows per page: a power of two, 32 or more)", pages_per_seq, page_rows);
    MYNN_REQUIRE(B > 0 && Hkv > 0 && S_new > 0 && D > 0 && offset >= 0 && (long)offset + S_new <= (long)pages_per_seq * page_rows,
                 MYNN_ERR_INVALID, "kvcache_update_paged: offset %d + %d rows exceeds %d pages of %d rows", offset, S_new, pages_per_seq,
                 page_rows);
    MYNN_REQUIRE(dtype_ok(dtype), MYNN_ERR_INVALID, "kvcache_update_paged: dtype %d", dtype);
    const size_t row_bytes = (size_t)D * dtype_size(dtype);
    MYNN_REQUIRE(row_bytes % 4 == 0, MYNN_ERR_UNSUPPORTED, "kvcache_update_paged: rows of %zu bytes", row_bytes);
    KvPaging pg;
    pg.table = page_table;
    pg.pages_per_seq = pages_per_seq;
    while ((1 << pg.shift) < page_rows) pg.shift++;
    const int units = (int)(row_bytes / 4);
    const size_t total = (size_t)B * Hkv * S_new * units;
    MYNN_LAUNCH(kvcache_update_paged_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, as_stream(s), (uint32_t *)pool,
                (const uint32_t *)new_kv, offset, Hkv, S_new, units, pg, total);
    return launch_status("kvcache_update_paged_kernel");
}
