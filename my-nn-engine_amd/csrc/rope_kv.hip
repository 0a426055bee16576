// RoPE(q), RoPE(k), KVCacheUpdate(k), KVCacheUpdate(v) in one launch.
//
// The reference runs these as ~16 kernels per layer: the decomposed RoPE graph of
// crates/llm/src/builder.rs:402-438 (Slice, Slice, Neg, Concat, Mul, Mul, Add for q and again for
// k), the [S,H,D]->[H,S,D] transposes and two kvcache_update launches (kvcache_update.cuh:6-26).
// Arithmetic is unchanged: lo' = lo*cos[p,j] - hi*sin[p,j], hi' = hi*cos[p,j+D/2] + lo*sin[p,j+D/2]
// with separate products and one rounding; v is copied.
#include "kernels.h"

namespace mynn {

template <typename T>
__global__ void rope_kv_append_kernel(T *q_out, T *k_cache, T *v_cache, const T *qkv, const T *cos_t, const T *sin_t,
                                      const int64_t *position, const int32_t *d_past, int past_host, int S, int Hq,
                                      int Hkv, int D, int max_seq) {
    const int s = blockIdx.x, head = blockIdx.y, b = blockIdx.z;
    const int half = D / 2;
    const int past = d_past ? *d_past : past_host;
    const size_t row = (size_t)b * S + s;
    const int width = (Hq + 2 * Hkv) * D;
    const T *src = qkv + row * width + (size_t)head * D;
    if (head < Hq + Hkv) {
        T *dst = head < Hq ? q_out + row * (size_t)Hq * D + (size_t)head * D
                           : k_cache + (((size_t)b * Hkv + (head - Hq)) * max_seq + past + s) * D;
        const size_t tab = (size_t)position[s] * D;
        for (int j = threadIdx.x; j < half; j += blockDim.x) {
            float xl = Elem<T>::ld(src, j), xh = Elem<T>::ld(src, j + half);
            float cl = Elem<T>::ld(cos_t, tab + j), ch = Elem<T>::ld(cos_t, tab + j + half);
            float sl = Elem<T>::ld(sin_t, tab + j), sh = Elem<T>::ld(sin_t, tab + j + half);
            Elem<T>::st(dst, j, xl * cl - xh * sl);
            Elem<T>::st(dst, j + half, xh * ch + xl * sh);
        }
    } else {
        T *dst = v_cache + (((size_t)b * Hkv + (head - Hq - Hkv)) * max_seq + past + s) * D;
        for (int j = threadIdx.x; j < D; j += blockDim.x) dst[j] = src[j];
    }
}

template <typename T>
int rope_kv_append(void *q_out, void *k_cache, void *v_cache, const void *qkv, const void *cos_t, const void *sin_t,
                   const int64_t *position, const int32_t *d_past, int past_host, int B, int S, int Hq, int Hkv, int D,
                   int max_seq, hipStream_t s) {
    MYNN_REQUIRE(S <= 65535 * 32 && Hq + 2 * Hkv <= 65535 && B <= 65535, MYNN_ERR_UNSUPPORTED, "rope_kv_append: grid");
    int threads = D / 2 >= 64 ? 64 : 32;
    hipLaunchKernelGGL(rope_kv_append_kernel<T>, dim3(S, Hq + 2 * Hkv, B), dim3(threads), 0, s, (T *)q_out,
                       (T *)k_cache, (T *)v_cache, (const T *)qkv, (const T *)cos_t, (const T *)sin_t, position, d_past,
                       past_host, S, Hq, Hkv, D, max_seq);
    return launch_status("rope_kv_append_kernel");
}
template int rope_kv_append<bf16_t>(void *, void *, void *, const void *, const void *, const void *, const int64_t *,
                                    const int32_t *, int, int, int, int, int, int, int, hipStream_t);
template int rope_kv_append<f16_t>(void *, void *, void *, const void *, const void *, const void *, const int64_t *,
                                   const int32_t *, int, int, int, int, int, int, int, hipStream_t);

}  // namespace mynn
