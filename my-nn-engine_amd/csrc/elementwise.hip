// The small memory-bound operators of the decoder: RMSNorm, RoPE, KV-cache updates (plain and
// quantizing), DequantizeLinear, row gather, SwiGLU / Add groups, dynamic activation
// quantisation and the greedy argmax.  All compute in f32 and round once at the store.
#include "kernels.h"
#include "mfma.h"

namespace mynn {

constexpr int kEwThreads = 256;

// block-wide reductions over kEwThreads threads (4 waves)
__device__ inline float block_sum(float v, float *red) {
    v = wave_sum(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int w = 0; w < (int)(blockDim.x >> 6); w++) t += red[w];
    return t;
}
__device__ inline float block_max(float v, float *red) {
    v = wave_max(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = red[0];
    for (int w = 1; w < (int)(blockDim.x >> 6); w++) t = fmaxf(t, red[w]);
    return t;
}
__device__ inline float block_min(float v, float *red) { return -block_max(-v, red); }

// ---- RMSNormalization (reference rms_norm.cuh:9-59) ------------------------------------------
template <typename T>
__global__ __launch_bounds__(kEwThreads) void rms_norm_kernel(T *out, const T *x, const T *w, int dim, float eps) {
    __shared__ float red[4];
    const size_t base = (size_t)blockIdx.x * dim;
    float ss = 0.f;
    for (int i = threadIdx.x; i < dim; i += kEwThreads) {
        float v = Elem<T>::ld(x, base + i);
        ss += v * v;
    }
    float tot = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(tot / (float)dim + eps);
    for (int i = threadIdx.x; i < dim; i += kEwThreads)
        Elem<T>::st(out, base + i, (Elem<T>::ld(x, base + i) * inv) * Elem<T>::ld(w, i));
}

// Rows of 16-bit values whose length is a multiple of 8 and at most 8 * 4 * kEwThreads: 128-bit
// loads, the row read once and kept in registers between the two passes.
template <typename T>
__global__ __launch_bounds__(kEwThreads) void rms_norm_vec_kernel(T *out, const T *x, const T *w, int dim, float eps) {
    __shared__ float red[4];
    const size_t base = (size_t)blockIdx.x * dim;
    const int chunks = dim >> 3;
    U4 v[4];
    float ss = 0.f;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int c = threadIdx.x + q * kEwThreads;
        if (c < chunks) {
            v[q] = *(const U4 *)(x + base + (size_t)c * 8);
            float f[8];
            widen8<T>(v[q], f);
#pragma unroll
            for (int i = 0; i < 8; i++) ss += f[i] * f[i];
        }
    }
    const float tot = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(tot / (float)dim + eps);
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int c = threadIdx.x + q * kEwThreads;
        if (c < chunks) {
            float f[8], g[8];
            widen8<T>(v[q], f);
            widen8<T>(*(const U4 *)(w + (size_t)c * 8), g);
            U4 o;
            o.x = pack2<T>((f[0] * inv) * g[0], (f[1] * inv) * g[1]);
            o.y = pack2<T>((f[2] * inv) * g[2], (f[3] * inv) * g[3]);
            o.z = pack2<T>((f[4] * inv) * g[4], (f[5] * inv) * g[5]);
            o.w = pack2<T>((f[6] * inv) * g[6], (f[7] * inv) * g[7]);
            *(U4 *)(out + base + (size_t)c * 8) = o;
        }
    }
}

// ---- Rope (reference rope.cuh:18-46): one thread per (row, j < D/2) --------------------------
template <typename T>
__global__ void rope_kernel(T *out, const T *x, const T *cos_t, const T *sin_t, const int64_t *position,
                            int S, int D, size_t total_pairs) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total_pairs) return;
    const int half = D / 2;
    size_t row = idx / half;
    int j = (int)(idx % half);
    int s = (int)(row % S);
    size_t tab = (size_t)position[s] * D, xo = row * D;
    float xl = Elem<T>::ld(x, xo + j), xh = Elem<T>::ld(x, xo + j + half);
    float cl = Elem<T>::ld(cos_t, tab + j), ch = Elem<T>::ld(cos_t, tab + j + half);
    float sl = Elem<T>::ld(sin_t, tab + j), sh = Elem<T>::ld(sin_t, tab + j + half);
    // separate multiplies and one add/sub, no contraction: the reference's Mul, Mul, Add group
    float lo = __fsub_rn(__fmul_rn(xl, cl), __fmul_rn(xh, sl));
    float hi = __fadd_rn(__fmul_rn(xh, ch), __fmul_rn(xl, sh));
    Elem<T>::st(out, xo + j, lo);
    Elem<T>::st(out, xo + j + half, hi);
}

// ---- KVCacheUpdate (reference kvcache_update.cuh:6-26) ---------------------------------------
template <typename W>
__global__ void kvcache_update_kernel(W *cache, const W *new_kv, int offset, int S_new, int max_seq, int D_words,
                                      size_t total) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    int d = (int)(idx % D_words);
    size_t rest = idx / D_words;
    int t = (int)(rest % S_new);
    size_t bh = rest / S_new;
    cache[(bh * max_seq + offset + t) * D_words + d] = new_kv[idx];
}

// ---- QuantizingKVCacheUpdate (reference quantizing_kvcache_update.cuh:16-70, CPU rounding) ----
// one wave per token row
template <typename T>
__global__ __launch_bounds__(64) void quantizing_kvcache_update_kernel(int8_t *cache, T *scale, const T *new_kv,
                                                                       int offset, int S_new, int max_seq, int D, int ring_sink,
                                                                       int ring_window, int ring_start) {
    const size_t rowi = blockIdx.x;  // bh * S_new + t
    const int t = (int)(rowi % S_new);
    const size_t bh = rowi / S_new;
    // streaming KV: the row goes to its ring slot; of rows a whole window apart the later one keeps the slot
    if (ring_window > 0 && offset + t >= ring_sink && t + ring_window < S_new) return;
    const size_t tok = bh * max_seq + ring_phys_index(offset + t, ring_sink, ring_window, ring_start);
    const int lane = threadIdx.x;
    float amax = 0.f;
    for (int d = lane; d < D; d += 64) amax = fmaxf(amax, fabsf(Elem<T>::ld(new_kv, rowi * D + d)));
    amax = wave_max(amax);
    const float s = amax * (1.0f / 127.0f);
    const float inv = amax == 0.f ? 0.f : 127.0f / amax;
    if (lane == 0) Elem<T>::st(scale, tok, s);
    for (int d = lane; d < D; d += 64) {
        float sc = Elem<T>::ld(new_kv, rowi * D + d) * inv;
        float biased = sc + (sc >= 0.f ? 0.5f : -0.5f);
        int q = (int)biased;  // truncation toward zero
        q = q < -128 ? -128 : (q > 127 ? 127 : q);
        cache[tok * D + d] = (int8_t)q;
    }
}

// ---- DequantizeLinear axis 0 (reference dequantize.cuh:5-19) ---------------------------------
template <typename T>
__global__ void dequantize_linear_kernel(T *out, const int8_t *x, const T *scale, size_t cols, size_t total) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    Elem<T>::st(out, idx, (float)x[idx] * Elem<T>::ld(scale, idx / cols));
}

// ---- Gather axis 0 (reference gather.cuh:5-21) -------------------------------------------------
__global__ void gather_rows_kernel(uint8_t *out, const uint8_t *data, const int64_t *idx, int rows, size_t row_bytes) {
    int64_t r = idx[blockIdx.x];
    if (r < 0) r += rows;
    const uint8_t *src = data + (size_t)r * row_bytes;
    uint8_t *dst = out + (size_t)blockIdx.x * row_bytes;
    if (((row_bytes | (uintptr_t)src | (uintptr_t)dst) & 15) == 0) {
        for (size_t i = threadIdx.x; i < row_bytes / 16; i += blockDim.x) ((U4 *)dst)[i] = ((const U4 *)src)[i];
    } else {
        for (size_t i = threadIdx.x; i < row_bytes; i += blockDim.x) dst[i] = src[i];
    }
}

// embedding lookup fused with the table's DequantizeLinear: out[i,:] = T(q[id,:] * scale[id])
template <typename T>
__global__ void embed_dequant_kernel(T *out, const int8_t *table, const T *scale, const int64_t *ids, int vocab,
                                     int hidden) {
    int64_t r = ids[blockIdx.x];
    if (r < 0) r += vocab;
    const float s = Elem<T>::ld(scale, (size_t)r);
    for (int i = threadIdx.x; i < hidden; i += blockDim.x)
        Elem<T>::st(out, (size_t)blockIdx.x * hidden + i, (float)table[(size_t)r * hidden + i] * s);
}

// ---- elementwise groups ------------------------------------------------------------------------
template <typename T>
__global__ void swiglu_kernel(T *out, const T *gate, const T *up, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float g = Elem<T>::ld(gate, i);
    float sig = 1.0f / (1.0f + expf(-g));
    Elem<T>::st(out, i, (g * sig) * Elem<T>::ld(up, i));
}
template <typename T>
__global__ void add_kernel(T *out, const T *a, const T *b, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    Elem<T>::st(out, i, Elem<T>::ld(a, i) + Elem<T>::ld(b, i));
}

// ---- DynamicQuantizeLinear (reference dynamic_quantize_linear.cuh:39-153) ----------------------
template <typename T, bool SYM>
__global__ __launch_bounds__(kEwThreads) void dynquant_kernel(void *y_, T *y_scale, void *y_zp_, const T *x, int inner) {
    __shared__ float red[4];
    const size_t base = (size_t)blockIdx.x * inner;
    if constexpr (SYM) {
        int8_t *y = (int8_t *)y_;
        float amax = 0.f;
        for (int i = threadIdx.x; i < inner; i += kEwThreads) amax = fmaxf(amax, fabsf(Elem<T>::ld(x, base + i)));
        amax = block_max(amax, red);
        const float sc = amax > 0.f ? amax / 127.0f : 1.0f;
        const float inv = 1.0f / sc;
        for (int i = threadIdx.x; i < inner; i += kEwThreads) {
            float q = roundf(Elem<T>::ld(x, base + i) * inv);  // half away from zero
            q = fminf(fmaxf(q, -127.f), 127.f);
            y[base + i] = (int8_t)q;
        }
        if (threadIdx.x == 0) {
            Elem<T>::st(y_scale, blockIdx.x, sc);
            if (y_zp_) ((int8_t *)y_zp_)[blockIdx.x] = 0;
        }
    } else {
        uint8_t *y = (uint8_t *)y_;
        float mn = INFINITY, mx = -INFINITY;
        for (int i = threadIdx.x; i < inner; i += kEwThreads) {
            float v = Elem<T>::ld(x, base + i);
            mn = fminf(mn, v);
            mx = fmaxf(mx, v);
        }
        mx = block_max(mx, red);
        mn = block_min(mn, red);
        mn = fminf(mn, 0.f);
        mx = fmaxf(mx, 0.f);
        float sc = (mx - mn) / 255.0f;
        if (sc == 0.f) sc = 1.f;
        int zp = (int)nearbyintf(-mn / sc);
        zp = zp < 0 ? 0 : (zp > 255 ? 255 : zp);
        for (int i = threadIdx.x; i < inner; i += kEwThreads) {
            int q = (int)nearbyintf(Elem<T>::ld(x, base + i) / sc) + zp;
            y[base + i] = (uint8_t)(q < 0 ? 0 : (q > 255 ? 255 : q));
        }
        if (threadIdx.x == 0) {
            Elem<T>::st(y_scale, blockIdx.x, sc);
            if (y_zp_) ((uint8_t *)y_zp_)[blockIdx.x] = (uint8_t)zp;
        }
    }
}

// Symmetric per-row quantisation of 16-bit rows of at most 8 * 64 * NCH values (a multiple of 8): one wave
// per row, the row read once with 128-bit loads and kept in registers, reductions inside the wave (no
// workgroup barrier); same arithmetic as dynquant_kernel<T, true>.
// NORM: the row is first RMS-normalised exactly as rms_norm_vec_kernel does (rounded to the storage type)
// and only the quantised form is written -- the normalised activations of a W8A8 layer have no other reader.
template <typename T, bool NORM, int NCH>
__global__ __launch_bounds__(kEwThreads) void dynquant_rows_vec_kernel(int8_t *y, T *y_scale, int8_t *y_zp, const T *x, const T *w,
                                                                       int rows, int dim, float eps) {
    const int lane = threadIdx.x & 63, row = blockIdx.x * (kEwThreads / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;  // whole wave
    const size_t base = (size_t)row * dim;
    const int chunks = dim >> 3;
    U4 v[NCH];
    float ss = 0.f;
#pragma unroll
    for (int q = 0; q < NCH; q++) {
        const int c = lane + q * 64;
        v[q] = U4{0u, 0u, 0u, 0u};
        if (c < chunks) {
            v[q] = *(const U4 *)(x + base + (size_t)c * 8);
            if (NORM) {
                float f[8];
                widen8<T>(v[q], f);
#pragma unroll
                for (int i = 0; i < 8; i++) ss += f[i] * f[i];
            }
        }
    }
    if (NORM) {
        const float tot = wave_sum(ss);
        const float inv = 1.0f / sqrtf(tot / (float)dim + eps);
#pragma unroll
        for (int q = 0; q < NCH; q++) {
            const int c = lane + q * 64;
            if (c < chunks) {
                float f[8], g[8];
                widen8<T>(v[q], f);
                widen8<T>(*(const U4 *)(w + (size_t)c * 8), g);
                v[q].x = pack2<T>((f[0] * inv) * g[0], (f[1] * inv) * g[1]);
                v[q].y = pack2<T>((f[2] * inv) * g[2], (f[3] * inv) * g[3]);
                v[q].z = pack2<T>((f[4] * inv) * g[4], (f[5] * inv) * g[5]);
                v[q].w = pack2<T>((f[6] * inv) * g[6], (f[7] * inv) * g[7]);
            }
        }
    }
    float amax = 0.f;
#pragma unroll
    for (int q = 0; q < NCH; q++) {
        float f[8];
        widen8<T>(v[q], f);
#pragma unroll
        for (int i = 0; i < 8; i++) amax = fmaxf(amax, fabsf(f[i]));
    }
    amax = wave_max(amax);
    const float sc = amax > 0.f ? amax / 127.0f : 1.0f;
    const float inv = 1.0f / sc;
#pragma unroll
    for (int q = 0; q < NCH; q++) {
        const int c = lane + q * 64;
        if (c < chunks) {
            float f[8];
            widen8<T>(v[q], f);
            uint32_t b[2] = {0u, 0u};
#pragma unroll
            for (int i = 0; i < 8; i++) {
                float r = roundf(f[i] * inv);  // half away from zero
                r = fminf(fmaxf(r, -127.f), 127.f);
                b[i >> 2] |= ((uint32_t)(int)r & 0xFFu) << (8 * (i & 3));
            }
            *(uint2 *)(y + base + (size_t)c * 8) = uint2{b[0], b[1]};
        }
    }
    if (lane == 0) {
        Elem<T>::st(y_scale, row, sc);
        if (y_zp) y_zp[row] = 0;
    }
}

template <typename T, bool NORM>
static int dynquant_rows_vec(int8_t *y, void *y_scale, int8_t *y_zp, const void *x, const void *w, int rows, int dim, float eps, hipStream_t s) {
    const dim3 grid((rows + kEwThreads / 64 - 1) / (kEwThreads / 64)), block(kEwThreads);
    const int nch = (dim / 8 + 63) / 64;
    if (nch <= 4)
        MYNN_LAUNCH((dynquant_rows_vec_kernel<T, NORM, 4>), grid, block, 0, s, y, (T *)y_scale, y_zp, (const T *)x, (const T *)w, rows, dim, eps);
    else if (nch <= 8)
        MYNN_LAUNCH((dynquant_rows_vec_kernel<T, NORM, 8>), grid, block, 0, s, y, (T *)y_scale, y_zp, (const T *)x, (const T *)w, rows, dim, eps);
    else if (nch <= 12)
        MYNN_LAUNCH((dynquant_rows_vec_kernel<T, NORM, 12>), grid, block, 0, s, y, (T *)y_scale, y_zp, (const T *)x, (const T *)w, rows, dim, eps);
    else
        MYNN_LAUNCH((dynquant_rows_vec_kernel<T, NORM, 16>), grid, block, 0, s, y, (T *)y_scale, y_zp, (const T *)x, (const T *)w, rows, dim, eps);
    return launch_status("dynquant_rows_vec_kernel");
}

static bool dynquant_vec_ok(const void *y, const void *x, int dim) {
    return dim % 8 == 0 && dim <= 8 * 64 * 16 && aligned16(x) && ((uintptr_t)y & 7) == 0;
}

// RMSNorm followed by symmetric per-row quantisation (the pair RMSNormalization -> DynamicQuantizeLinear of a
// W8A8 layer), one launch; falls back to the two operators for rows the vector kernel does not take.
int rms_norm_dynquant(int8_t *y, void *y_scale, void *scratch_norm, const void *x, const void *w, int rows, int dim, float eps,
                      int dtype, hipStream_t s) {
    if (dtype != MYNN_F32 && dynquant_vec_ok(y, x, dim) && aligned16(w)) {
        return dispatch_dtype16(dtype, [&](auto *t) {
            using T = std::remove_pointer_t<decltype(t)>;
            return dynquant_rows_vec<T, true>(y, y_scale, nullptr, x, w, rows, dim, eps, s);
        });
    }
    int rc = mynn_rms_norm(scratch_norm, x, w, rows, dim, eps, dtype, s);
    if (rc) return rc;
    return mynn_dynamic_quantize_linear(y, y_scale, nullptr, scratch_norm, rows, dim, dtype, 1, s);
}

// dst rows [(r / group) * 2 * group + which * group + r % group] <- src rows r, row_bytes each (a multiple of 2):
// the gate (which = 0) and up (1) halves of a fused gate/up weight whose SwiGLU store pairs column tiles
__global__ void interleave_rows_kernel(uint16_t *dst, const uint16_t *src, size_t row_halfwords, size_t total, int group, int which) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const size_t r = i / row_halfwords, c = i % row_halfwords;
    const size_t d = (r / group) * 2 * group + (size_t)which * group + r % group;
    dst[d * row_halfwords + c] = src[i];
}
int interleave_row_groups(void *dst, const void *src, size_t rows, size_t row_bytes, int group, int which, hipStream_t s) {
    MYNN_REQUIRE(dst && src && row_bytes % 2 == 0 && group > 0 && rows % group == 0, MYNN_ERR_INVALID, "interleave_row_groups: bad operand");
    const size_t total = rows * (row_bytes / 2);
    MYNN_LAUNCH(interleave_rows_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, (uint16_t *)dst, (const uint16_t *)src,
                row_bytes / 2, total, group, which);
    return launch_status("interleave_rows_kernel");
}

// ---- greedy argmax, last maximum wins (reference crates/llm/src/session.rs:683-690) -----------
// one workgroup of 1024 threads per row, 16-byte loads; (value, index) ordered by value, then index
template <typename T>
__global__ __launch_bounds__(1024) void argmax_last_kernel(int32_t *out, const T *logits, int n, AdvanceState adv) {
    __shared__ float sv[16];
    __shared__ int si[16];
    const T *row = logits + (size_t)blockIdx.x * n;
    // the loop state this launch moves on: read now, so that the tail is stores only
    int st_step = 0, st_past = 0, st_active = 0;
    int64_t st_pos = 0;
    if (adv.ids && threadIdx.x == 0) {
        st_step = *adv.step;
        st_pos = adv.pos[0];
        st_past = *adv.past;
        st_active = *adv.active;
    }
    float bv = -INFINITY;
    int bi = -1;
    if constexpr (sizeof(T) == 2) {
        const int nvec = (((uintptr_t)row & 15) == 0) ? n / 8 : 0;
        // eight loads in flight per thread (one at a time, a 128256-entry row was sixteen dependent round trips: 17 us)
        constexpr int kAhead = 8;
        for (int c0 = threadIdx.x; c0 < nvec; c0 += 1024 * kAhead) {
            U4 v[kAhead];
#pragma unroll
            for (int j = 0; j < kAhead; j++) v[j] = ((const U4 *)row)[min(c0 + j * 1024, nvec - 1)];
#pragma unroll
            for (int j = 0; j < kAhead; j++) {
                const int c = c0 + j * 1024;
                if (c >= nvec) break;
                float f[8];
                widen8<T>(v[j], f);
#pragma unroll
                for (int e = 0; e < 8; e++) argmax_take(bv, bi, f[e], c * 8 + e);
            }
        }
        for (int i = nvec * 8 + threadIdx.x; i < n; i += 1024) argmax_take(bv, bi, Elem<T>::ld(row, i), i);
    } else {
        for (int i = threadIdx.x; i < n; i += 1024) argmax_take(bv, bi, Elem<T>::ld(row, i), i);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        float ov = __shfl_xor(bv, off, 64);
        int oi = __shfl_xor(bi, off, 64);
        if (oi >= 0) argmax_take(bv, bi, ov, oi);
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) { sv[wave] = bv; si[wave] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; w++)
            if (si[w] >= 0) argmax_take(bv, bi, sv[w], si[w]);
        out[blockIdx.x] = bi;
        if (adv.ids) {
            if (st_step < adv.cap) adv.tokens[st_step] = bi;
            *adv.step = st_step + 1;
            adv.ids[0] = bi;
            adv.pos[0] = st_pos + 1;
            *adv.past = st_past + 1;
            *adv.active = st_active + 1;
        }
    }
}

template <typename T>
int argmax_rows(int32_t *out, const void *logits, int rows, int n, AdvanceState adv, hipStream_t s) {
    MYNN_LAUNCH(argmax_last_kernel<T>, dim3(rows), dim3(1024), 0, s, out, (const T *)logits, n, adv);
    return launch_status("argmax_last_kernel");
}
template int argmax_rows<bf16_t>(int32_t *, const void *, int, int, AdvanceState, hipStream_t);
template int argmax_rows<f16_t>(int32_t *, const void *, int, int, AdvanceState, hipStream_t);
template int argmax_rows<float>(int32_t *, const void *, int, int, AdvanceState, hipStream_t);

template <typename T>
int embed_dequant(void *out, const int8_t *table, const void *scale, const int64_t *ids, int n_ids, int vocab,
                  int hidden, hipStream_t s) {
    MYNN_LAUNCH(embed_dequant_kernel<T>, dim3(n_ids), dim3(256), 0, s, (T *)out, table, (const T *)scale, ids,
                       vocab, hidden);
    return launch_status("embed_dequant_kernel");
}
template int embed_dequant<bf16_t>(void *, const int8_t *, const void *, const int64_t *, int, int, int, hipStream_t);
template int embed_dequant<f16_t>(void *, const int8_t *, const void *, const int64_t *, int, int, int, hipStream_t);

static inline unsigned nblocks(size_t n, int t) { return (unsigned)((n + t - 1) / t); }

}  // namespace mynn

using namespace mynn;

extern "C" int mynn_rms_norm(void *out, const void *x, const void *w, int rows, int dim, float eps, int dtype,
                             mynn_stream s) {
    MYNN_REQUIRE(out && x && w && rows > 0 && dim > 0, MYNN_ERR_INVALID, "rms_norm: bad operand");
    return dispatch_dtype(dtype, [&](auto *t) {
        using T = std::remove_pointer_t<decltype(t)>;
        if constexpr (sizeof(T) == 2) {
            if (dim % 8 == 0 && dim <= 8 * 4 * kEwThreads && aligned16(out) && aligned16(x) && aligned16(w)) {
                MYNN_LAUNCH(rms_norm_vec_kernel<T>, dim3(rows), dim3(kEwThreads), 0, as_stream(s), (T *)out,
                                   (const T *)x, (const T *)w, dim, eps);
                return launch_status("rms_norm_vec_kernel");
            }
        }
        MYNN_LAUNCH(rms_norm_kernel<T>, dim3(rows), dim3(kEwThreads), 0, as_stream(s), (T *)out, (const T *)x,
                           (const T *)w, dim, eps);
        return launch_status("rms_norm_kernel");
    });
}

extern "C" int mynn_rope(void *out, const void *x, const void *cos_t, const void *sin_t, const int64_t *position,
                         int outer, int S, int D, int dtype, mynn_stream s) {
    MYNN_REQUIRE(out && x && cos_t && sin_t && position, MYNN_ERR_INVALID, "rope: null operand");
    MYNN_REQUIRE(outer > 0 && S > 0 && D > 0 && D % 2 == 0, MYNN_ERR_INVALID, "rope: outer=%d S=%d D=%d", outer, S, D);
    size_t pairs = (size_t)outer * S * (D / 2);
    return dispatch_dtype(dtype, [&](auto *t) {
        using T = std::remove_pointer_t<decltype(t)>;
        MYNN_LAUNCH(rope_kernel<T>, dim3(nblocks(pairs, 256)), dim3(256), 0, as_stream(s), (T *)out,
                           (const T *)x, (const T *)cos_t, (const T *)sin_t, position, S, D, pairs);
        return launch_status("rope_kernel");
    });
}

extern "C" int mynn_kvcache_update(void *cache, const void *new_kv, int offset, int BH, int S_new, int max_seq, int D,
                                   int dtype, mynn_stream s) {
    MYNN_REQUIRE(cache && new_kv, MYNN_ERR_INVALID, "kvcache_update: null operand");
    MYNN_REQUIRE(BH > 0 && S_new > 0 && D > 0 && offset >= 0 && offset + S_new <= max_seq, MYNN_ERR_INVALID,
                 "kvcache_update: offset %d + %d rows exceeds max_seq %d", offset, S_new, max_seq);
    MYNN_REQUIRE(dtype_ok(dtype), MYNN_ERR_INVALID, "kvcache_update: dtype %d", dtype);
    size_t eb = dtype_size(dtype);
    size_t row_bytes = (size_t)D * eb;
    if (row_bytes % 4 == 0) {
        int dw = (int)(row_bytes / 4);
        size_t total = (size_t)BH * S_new * dw;
        MYNN_LAUNCH(kvcache_update_kernel<uint32_t>, dim3(nblocks(total, 256)), dim3(256), 0, as_stream(s),
                           (uint32_t *)cache, (const uint32_t *)new_kv, offset, S_new, max_seq, dw, total);
    } else {
        size_t total = (size_t)BH * S_new * D;
        MYNN_LAUNCH(kvcache_update_kernel<uint16_t>, dim3(nblocks(total, 256)), dim3(256), 0, as_stream(s),
                           (uint16_t *)cache, (const uint16_t *)new_kv, offset, S_new, max_seq, D, total);
    }
    return launch_status("kvcache_update_kernel");
}

extern "C" int mynn_quantizing_kvcache_update_streaming(int8_t *cache, void *scale, const void *new_kv, int offset, int BH,
                                                        int S_new, int max_seq, int D, int ring_sink, int ring_window,
                                                        int ring_start, int dtype, mynn_stream s) {
    MYNN_REQUIRE(cache && scale && new_kv, MYNN_ERR_INVALID, "quantizing_kvcache_update: null operand");
    MYNN_REQUIRE(BH > 0 && S_new > 0 && D > 0 && offset >= 0, MYNN_ERR_INVALID, "quantizing_kvcache_update: BH=%d S_new=%d D=%d offset=%d",
                 BH, S_new, D, offset);
    MYNN_REQUIRE(ring_sink >= 0 && ring_window >= 0 && ring_start >= 0 && (ring_window == 0 || ring_start < ring_window),
                 MYNN_ERR_INVALID, "quantizing_kvcache_update: ring sink=%d window=%d start=%d", ring_sink, ring_window, ring_start);
    if (ring_window == 0)
        MYNN_REQUIRE(offset + S_new <= max_seq, MYNN_ERR_INVALID, "quantizing_kvcache_update: offset %d + %d rows exceeds max_seq %d",
                     offset, S_new, max_seq);
    else
        MYNN_REQUIRE(ring_sink + ring_window <= max_seq, MYNN_ERR_INVALID,
                     "quantizing_kvcache_update: sink %d + window %d exceeds max_seq %d", ring_sink, ring_window, max_seq);
    return dispatch_dtype(dtype, [&](auto *t) {
        using T = std::remove_pointer_t<decltype(t)>;
        MYNN_LAUNCH(quantizing_kvcache_update_kernel<T>, dim3(BH * S_new), dim3(64), 0, as_stream(s), cache,
                           (T *)scale, (const T *)new_kv, offset, S_new, max_seq, D, ring_sink, ring_window, ring_start);
        return launch_status("quantizing_kvcache_update_kernel");
    });
}

extern "C" int mynn_quantizing_kvcache_update(int8_t *cache, void *scale, const void *new_kv, int offset, int BH,
                                              int S_new, int max_seq, int D, int dtype, mynn_stream s) {
    return mynn_quantizing_kvcache_update_streaming(cache, scale, new_kv, offset, BH, S_new, max_seq, D, 0, 0, 0, dtype, s);
}

extern "C" int mynn_dequantize_linear(void *out, const int8_t *x, const void *scale, size_t rows, size_t cols,
                                      int dtype, mynn_stream s) {
    MYNN_REQUIRE(out && x && scale && rows > 0 && cols > 0, MYNN_ERR_INVALID, "dequantize_linear: bad operand");
    size_t total = rows * cols;
    return dispatch_dtype(dtype, [&](auto *t) {
        using T = std::remove_pointer_t<decltype(t)>;
        MYNN_LAUNCH(dequantize_linear_kernel<T>, dim3(nblocks(total, 256)), dim3(256), 0, as_stream(s),
                           (T *)out, x, (const T *)scale, cols, total);
        return launch_status("dequantize_linear_kernel");
    });
}

extern "C" int mynn_gather_rows(void *out, const void *data, const int64_t *idx, int n_idx, int rows, size_t row_bytes,
                                mynn_stream s) {
    MYNN_REQUIRE(out && data && idx && n_idx > 0 && rows > 0 && row_bytes > 0, MYNN_ERR_INVALID,
                 "gather_rows: bad operand");
    MYNN_LAUNCH(gather_rows_kernel, dim3(n_idx), dim3(256), 0, as_stream(s), (uint8_t *)out,
                       (const uint8_t *)data, idx, rows, row_bytes);
    return launch_status("gather_rows_kernel");
}

extern "C" int mynn_swiglu(void *out, const void *gate, const void *up, size_t n, int dtype, mynn_stream s) {
    MYNN_REQUIRE(out && gate && up && n > 0, MYNN_ERR_INVALID, "swiglu: bad operand");
    return dispatch_dtype(dtype, [&](auto *t) {
        using T = std::remove_pointer_t<decltype(t)>;
        MYNN_LAUNCH(swiglu_kernel<T>, dim3(nblocks(n, 256)), dim3(256), 0, as_stream(s), (T *)out,
                           (const T *)gate, (const T *)up, n);
        return launch_status("swiglu_kernel");
    });
}

extern "C" int mynn_add(void *out, const void *a, const void *b, size_t n, int dtype, mynn_stream s) {
    MYNN_REQUIRE(out && a && b && n > 0, MYNN_ERR_INVALID, "add: bad operand");
    return dispatch_dtype(dtype, [&](auto *t) {
        using T = std::remove_pointer_t<decltype(t)>;
        MYNN_LAUNCH(add_kernel<T>, dim3(nblocks(n, 256)), dim3(256), 0, as_stream(s), (T *)out, (const T *)a,
                           (const T *)b, n);
        return launch_status("add_kernel");
    });
}

// x[r, n] = T(x[r, n] + bias[n]) in place: the broadcast Add behind a projection with a bias (crates/llm/src/decoder.rs:167-184)
namespace mynn {
template <typename T>
__global__ void add_bias_rows_kernel(T *x, const T *bias, int N, size_t total) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    Elem<T>::st(x, i, Elem<T>::ld(x, i) + Elem<T>::ld(bias, i % N));
}
int add_bias_rows(void *x, const void *bias, int rows, int N, int dtype, hipStream_t s) {
    MYNN_REQUIRE(x && bias && rows > 0 && N > 0, MYNN_ERR_INVALID, "add_bias_rows: bad operand");
    const size_t total = (size_t)rows * N;
    return dispatch_dtype(dtype, [&](auto *t) {
        using T = std::remove_pointer_t<decltype(t)>;
        MYNN_LAUNCH(add_bias_rows_kernel<T>, dim3(nblocks(total, 256)), dim3(256), 0, s, (T *)x, (const T *)bias, N, total);
        return launch_status("add_bias_rows_kernel");
    });
}
}  // namespace mynn

extern "C" int mynn_dynamic_quantize_linear(void *y, void *y_scale, void *y_zero_point, const void *x, int axis_dim,
                                            int inner_size, int dtype, int symmetric, mynn_stream s) {
    MYNN_REQUIRE(y && y_scale && x && axis_dim > 0 && inner_size > 0, MYNN_ERR_INVALID,
                 "dynamic_quantize_linear: bad operand");
    MYNN_REQUIRE(symmetric || y_zero_point, MYNN_ERR_INVALID, "dynamic_quantize_linear: asymmetric needs y_zero_point");
    return dispatch_dtype(dtype, [&](auto *t) {
        using T = std::remove_pointer_t<decltype(t)>;
        if constexpr (sizeof(T) == 2) {
            if (symmetric && dynquant_vec_ok(y, x, inner_size)) {
                return dynquant_rows_vec<T, false>((int8_t *)y, y_scale, (int8_t *)y_zero_point, x, nullptr, axis_dim, inner_size, 0.f,
                                                   as_stream(s));
            }
        }
        if (symmetric)
            MYNN_LAUNCH((dynquant_kernel<T, true>), dim3(axis_dim), dim3(kEwThreads), 0, as_stream(s), y,
                               (T *)y_scale, y_zero_point, (const T *)x, inner_size);
        else
            MYNN_LAUNCH((dynquant_kernel<T, false>), dim3(axis_dim), dim3(kEwThreads), 0, as_stream(s), y,
                               (T *)y_scale, y_zero_point, (const T *)x, inner_size);
        return launch_status("dynquant_kernel");
    });
}

extern "C" int mynn_argmax_last(int32_t *out_index, const void *logits, int n, int dtype, mynn_stream s) {
    MYNN_REQUIRE(out_index && logits && n > 0, MYNN_ERR_INVALID, "argmax_last: bad operand");
    return dispatch_dtype(dtype, [&](auto *t) {
        using T = std::remove_pointer_t<decltype(t)>;
        return argmax_rows<T>(out_index, logits, 1, n, AdvanceState{}, as_stream(s));
    });
}
