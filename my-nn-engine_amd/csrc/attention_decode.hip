// Grouped-query attention over the KV cache, one query row at a time ("flash-decode").
//
// Replaces the reference's attention_decode (attention.cuh:495-606), which walks the cache rows
// serially with two block barriers per key and re-reads K/V once per query head.  Here one
// workgroup serves ALL query heads of a KV head (so K/V are read once per group), the cache
// length is split over gridDim.y workgroups, every lane streams 16-byte pieces of K and V rows,
// and the online-softmax states (m, l, o) are merged lane-group -> wave -> workgroup -> split.
// The last workgroup of a (batch, kv head, row) to finish merges the splits (a counter in
// device memory; nobody spins).
//
// The same kernel with gridDim.z = Sq is the correct-but-plain path for Sq > 1 (causal rows get
// their own key bound); the matrix-core prefill kernel lives in attention_prefill.hip.
#include "attention.h"

namespace mynn {


constexpr int kAttnThreads = 256;
constexpr int kAttnWaves = 4;

__device__ inline void merge_state(float &m, float &l, float *o, int n, float m2, float l2, const float *o2) {
    float mn = fmaxf(m, m2);
    float c1 = (m == -INFINITY) ? 0.f : fast_exp(m - mn);
    float c2 = (m2 == -INFINITY) ? 0.f : fast_exp(m2 - mn);
    l = l * c1 + l2 * c2;
    for (int i = 0; i < n; i++) o[i] = o[i] * c1 + o2[i] * c2;
    m = mn;
}

template <typename T, int D, int G, bool KVI8>
__global__ __launch_bounds__(kAttnThreads) void attn_decode_kernel(AttnParams p) {
    constexpr int EPL = D >= 8 ? 8 : D;  // elements of a key row per lane
    constexpr int LPK = D / EPL;         // lanes per key row
    constexpr int KPW = 64 / LPK;        // keys per wave pass
    static_assert(D % EPL == 0 && LPK <= 64 && (LPK & (LPK - 1)) == 0, "head_dim must be a power of two");
    __shared__ float sm_o[kAttnWaves][G][D];
    __shared__ float sm_ml[kAttnWaves][G][2];
    __shared__ int sm_last;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int ks = lane / LPK, dc = lane % LPK;
    const int bhkv = blockIdx.x, split = blockIdx.y, sq = blockIdx.z;
    const int b = bhkv / p.Hkv, hkv = bhkv % p.Hkv;
    const int Sq = p.Sq;

    int active = p.d_active ? *p.d_active : p.active;
    int qoff = p.d_active ? active - Sq : p.q_pos_offset;
    int bound = active;
    if (p.is_causal) bound = min(bound, qoff + sq + 1);
    bound = min(bound, p.cache_len);
    // key range of this split: equal chunks, rounded up to whole workgroup passes
    constexpr int PASS = kAttnWaves * KPW;
    int chunk = (bound + p.nsplit - 1) / p.nsplit;
    chunk = (chunk + PASS - 1) / PASS * PASS;
    const int k0 = split * chunk;
    const int k1 = min(bound, k0 + chunk);

    const T *Q = (const T *)p.q;
    float q[G][EPL];
#pragma unroll
    for (int g = 0; g < G; g++) {
        const size_t qo = (size_t)b * p.q_bs + (size_t)(hkv * G + g) * p.q_hs + (size_t)sq * p.q_rs + dc * EPL;
#pragma unroll
        for (int i = 0; i < EPL; i++) q[g][i] = Elem<T>::ld(Q, qo + i);
    }
    float m[G], l[G], o[G][EPL];
#pragma unroll
    for (int g = 0; g < G; g++) {
        m[g] = -INFINITY;
        l[g] = 0.f;
#pragma unroll
        for (int i = 0; i < EPL; i++) o[g][i] = 0.f;
    }

    const size_t kv_base = (size_t)bhkv * p.cache_len;
    for (int kk = k0 + wave * KPW + ks; kk < k1; kk += PASS) {
        float kf[EPL], vf[EPL];
        float ksc = 1.f, vsc = 1.f;
        const size_t ro = (kv_base + kk) * D + dc * EPL;
        if constexpr (KVI8) {
            if constexpr (EPL == 8) {
                const uint2 kr = *(const uint2 *)((const int8_t *)p.k + ro);
                const uint2 vr = *(const uint2 *)((const int8_t *)p.v + ro);
                const uint32_t kw[2] = {kr.x, kr.y}, vw[2] = {vr.x, vr.y};
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    kf[i] = (float)(int8_t)((kw[i >> 2] >> (8 * (i & 3))) & 0xFF);
                    vf[i] = (float)(int8_t)((vw[i >> 2] >> (8 * (i & 3))) & 0xFF);
                }
            } else {
#pragma unroll
                for (int i = 0; i < EPL; i++) {
                    kf[i] = (float)((const int8_t *)p.k)[ro + i];
                    vf[i] = (float)((const int8_t *)p.v)[ro + i];
                }
            }
            ksc = Elem<T>::ld((const T *)p.k_scale, kv_base + kk);
            vsc = Elem<T>::ld((const T *)p.v_scale, kv_base + kk);
        } else {
            if constexpr (sizeof(T) == 2 && EPL == 8) {
                const U4 kr = *(const U4 *)((const T *)p.k + ro);
                const U4 vr = *(const U4 *)((const T *)p.v + ro);
                widen8<T>(kr, kf);
                widen8<T>(vr, vf);
            } else {
#pragma unroll
                for (int i = 0; i < EPL; i++) {
                    kf[i] = Elem<T>::ld((const T *)p.k, ro + i);
                    vf[i] = Elem<T>::ld((const T *)p.v, ro + i);
                }
            }
        }
#pragma unroll
        for (int g = 0; g < G; g++) {
            float part = 0.f;
#pragma unroll
            for (int i = 0; i < EPL; i++) part = fmaf(q[g][i], kf[i], part);
            part = group_sum<LPK>(part);
            if constexpr (KVI8) part *= ksc;
            const float s = part * p.scale;
            const float mn = fmaxf(m[g], s);
            const float corr = fast_exp(m[g] - mn);  // exp(-inf) = 0 on the first key
            const float e = fast_exp(s - mn);
            l[g] = fmaf(l[g], corr, e);
            const float ev = KVI8 ? e * vsc : e;
#pragma unroll
            for (int i = 0; i < EPL; i++) o[g][i] = fmaf(ev, vf[i], o[g][i] * corr);
            m[g] = mn;
        }
    }

    // ---- merge the KPW key slots of the wave (lanes that share dc)
#pragma unroll
    for (int off = LPK; off < 64; off <<= 1) {
#pragma unroll
        for (int g = 0; g < G; g++) {
            float m2 = __shfl_xor(m[g], off, 64), l2 = __shfl_xor(l[g], off, 64);
            float o2[EPL];
#pragma unroll
            for (int i = 0; i < EPL; i++) o2[i] = __shfl_xor(o[g][i], off, 64);
            merge_state(m[g], l[g], o[g], EPL, m2, l2, o2);
        }
    }
    if (ks == 0) {
#pragma unroll
        for (int g = 0; g < G; g++) {
#pragma unroll
            for (int i = 0; i < EPL; i++) sm_o[wave][g][dc * EPL + i] = o[g][i];
            if (dc == 0) { sm_ml[wave][g][0] = m[g]; sm_ml[wave][g][1] = l[g]; }
        }
    }
    __syncthreads();

    // ---- merge the waves; thread handles (g, d) pairs
    T *out = (T *)p.out;
    const size_t row_base = (size_t)(b * p.Hq + hkv * G) * Sq + sq;  // + g*Sq
    for (int idx = threadIdx.x; idx < G * D; idx += kAttnThreads) {
        const int g = idx / D, d = idx % D;
        float mt = -INFINITY;
#pragma unroll
        for (int w = 0; w < kAttnWaves; w++) mt = fmaxf(mt, sm_ml[w][g][0]);
        float lt = 0.f, ot = 0.f;
#pragma unroll
        for (int w = 0; w < kAttnWaves; w++) {
            float mw = sm_ml[w][g][0];
            float c = (mw == -INFINITY) ? 0.f : fast_exp(mw - mt);
            lt += sm_ml[w][g][1] * c;
            ot += sm_o[w][g][d] * c;
        }
        const size_t row = row_base + (size_t)g * Sq;
        const size_t oo = (size_t)b * p.o_bs + (size_t)(hkv * G + g) * p.o_hs + (size_t)sq * p.o_rs + d;
        if (p.nsplit == 1) {
            Elem<T>::st(out, oo, ot / lt);
        } else {
            p.part_o[(row * p.nsplit + split) * D + d] = ot;
            if (d == 0) {
                p.part_ml[(row * p.nsplit + split) * 2] = mt;
                p.part_ml[(row * p.nsplit + split) * 2 + 1] = lt;
            }
        }
    }
    if (p.nsplit == 1) return;

    // ---- last workgroup of this (batch, kv head, row) merges the splits
    __threadfence();
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned prev = atomicAdd(&p.counters[(size_t)bhkv * Sq + sq], 1u);
        sm_last = (prev == (unsigned)p.nsplit - 1);
    }
    __syncthreads();
    if (!sm_last) return;
    __threadfence();
    for (int idx = threadIdx.x; idx < G * D; idx += kAttnThreads) {
        const int g = idx / D, d = idx % D;
        const size_t row = row_base + (size_t)g * Sq;
        const float *ml = p.part_ml + row * p.nsplit * 2;
        const float *po = p.part_o + row * p.nsplit * D;
        float mt = -INFINITY;
        for (int s = 0; s < p.nsplit; s++) mt = fmaxf(mt, __builtin_nontemporal_load(&ml[2 * s]));
        float lt = 0.f, ot = 0.f;
        for (int s = 0; s < p.nsplit; s++) {
            float ms = __builtin_nontemporal_load(&ml[2 * s]);
            float c = (ms == -INFINITY) ? 0.f : fast_exp(ms - mt);
            lt += __builtin_nontemporal_load(&ml[2 * s + 1]) * c;
            ot += __builtin_nontemporal_load(&po[s * D + d]) * c;
        }
        const size_t oo = (size_t)b * p.o_bs + (size_t)(hkv * G + g) * p.o_hs + (size_t)sq * p.o_rs + d;
        Elem<T>::st(out, oo, ot / lt);
    }
    if (threadIdx.x == 0) p.counters[(size_t)bhkv * Sq + sq] = 0;  // ready for the next launch
}

template <typename T, int D, bool KVI8>
static int launch_g(const AttnParams &p, hipStream_t s) {
    dim3 grid(p.B * p.Hkv, p.nsplit, p.Sq), block(kAttnThreads);
    const int G = p.Hq / p.Hkv;
    switch (G) {
    case 1: hipLaunchKernelGGL((attn_decode_kernel<T, D, 1, KVI8>), grid, block, 0, s, p); break;
    case 2: hipLaunchKernelGGL((attn_decode_kernel<T, D, 2, KVI8>), grid, block, 0, s, p); break;
    case 4: hipLaunchKernelGGL((attn_decode_kernel<T, D, 4, KVI8>), grid, block, 0, s, p); break;
    case 8: hipLaunchKernelGGL((attn_decode_kernel<T, D, 8, KVI8>), grid, block, 0, s, p); break;
    default: return fail(MYNN_ERR_UNSUPPORTED, "attention: %d query heads per kv head (supported: 1,2,4,8)", G);
    }
    return launch_status("attn_decode_kernel");
}

template <typename T, bool KVI8>
static int launch_d(const AttnParams &p, int D, hipStream_t s) {
    switch (D) {
    case 4: return launch_g<T, 4, KVI8>(p, s);
    case 8: return launch_g<T, 8, KVI8>(p, s);
    case 16: return launch_g<T, 16, KVI8>(p, s);
    case 32: return launch_g<T, 32, KVI8>(p, s);
    case 64: return launch_g<T, 64, KVI8>(p, s);
    case 128: return launch_g<T, 128, KVI8>(p, s);
    default: return fail(MYNN_ERR_UNSUPPORTED, "attention: head_dim %d (supported: 4,8,16,32,64,128)", D);
    }
}

// number of key-range splits for a launch: enough workgroups to cover the chip, at least 64
// keys each, at most 64 splits
int attn_pick_nsplit(int B, int Hkv, int Sq, int kv_len) {
    int groups = B * Hkv * Sq;
    int want = (512 + groups - 1) / groups;
    int by_len = (kv_len + 63) / 64;
    int n = want < by_len ? want : by_len;
    if (n < 1) n = 1;
    if (n > 64) n = 64;
    return n;
}
size_t attn_scratch_bytes(int B, int Hq, int Sq, int D, int nsplit) {
    size_t rows = (size_t)B * Hq * Sq;
    size_t bytes = rows * nsplit * (D + 2) * sizeof(float);
    return (bytes + 255) / 256 * 256;
}
size_t attn_counter_bytes(int B, int Hkv, int Sq) {
    return ((size_t)B * Hkv * Sq * sizeof(unsigned) + 255) / 256 * 256;
}

// scratch = [part_o | part_ml] (contents need not survive); counters = one unsigned per
// (batch, kv head, row), zero on entry and zero again when the kernel has finished
int attention_decode_launch(AttnParams p, int D, int dtype, int kv_int8, void *scratch, void *counters,
                            hipStream_t s) {
    if (p.nsplit > 1) {
        size_t rows = (size_t)p.B * p.Hq * p.Sq;
        p.part_o = (float *)scratch;
        p.part_ml = p.part_o + rows * p.nsplit * D;
        p.counters = (unsigned *)counters;
    }
    return dispatch_dtype(dtype, [&](auto *t) {
        using T = std::remove_pointer_t<decltype(t)>;
        return kv_int8 ? launch_d<T, true>(p, D, s) : launch_d<T, false>(p, D, s);
    });
}

// ---- library-owned scratch for the op-level entry point: grown on demand.  The counters live
// in their own allocation so that partial results of an earlier, differently shaped call can
// never be mistaken for a count.
struct Grown {
    void *ptr = nullptr;
    size_t bytes = 0;
};
static Grown g_scratch, g_counters;
static int ensure(Grown &g, size_t bytes, bool zero, hipStream_t s) {
    if (bytes <= g.bytes) return 0;
    MYNN_HIP(hipStreamSynchronize(s));
    if (g.ptr) MYNN_HIP(hipFree(g.ptr));
    g.ptr = nullptr;
    g.bytes = 0;
    MYNN_HIP(hipMalloc(&g.ptr, bytes));
    if (zero) MYNN_HIP(hipMemset(g.ptr, 0, bytes));
    g.bytes = bytes;
    return 0;
}


}  // namespace mynn

using namespace mynn;

extern "C" int mynn_attention(void *out, const void *Q, const void *K, const void *V, const void *k_scale,
                              const void *v_scale, float scale, int is_causal, int B, int Sq, int active_seq_kv,
                              const int32_t *d_active, int cache_seq_len, int q_pos_offset, int num_q_heads,
                              int num_kv_heads, int head_dim, int dtype, int kv_int8, mynn_stream s) {
    MYNN_REQUIRE(out && Q && K && V, MYNN_ERR_INVALID, "attention: null operand");
    MYNN_REQUIRE(B > 0 && Sq > 0 && cache_seq_len > 0 && num_q_heads > 0 && num_kv_heads > 0, MYNN_ERR_INVALID,
                 "attention: B=%d Sq=%d cache=%d Hq=%d Hkv=%d", B, Sq, cache_seq_len, num_q_heads, num_kv_heads);
    MYNN_REQUIRE(num_q_heads % num_kv_heads == 0, MYNN_ERR_INVALID,
                 "attention: %d query heads is not a multiple of %d kv heads", num_q_heads, num_kv_heads);
    MYNN_REQUIRE(!kv_int8 || (k_scale && v_scale), MYNN_ERR_INVALID, "attention: int8 KV needs k_scale and v_scale");
    MYNN_REQUIRE(d_active || (active_seq_kv >= 1), MYNN_ERR_INVALID, "attention: active_seq_kv=%d", active_seq_kv);
    MYNN_REQUIRE(aligned16(K) && aligned16(V), MYNN_ERR_INVALID, "attention: K and V must be 16-byte aligned");
    AttnParams p{};
    p.out = out; p.q = Q; p.k = K; p.v = V; p.k_scale = k_scale; p.v_scale = v_scale; p.scale = scale;
    p.is_causal = is_causal; p.B = B; p.Sq = Sq; p.Hq = num_q_heads; p.Hkv = num_kv_heads;
    p.cache_len = cache_seq_len; p.active = active_seq_kv; p.d_active = d_active; p.q_pos_offset = q_pos_offset;
    attn_reference_layout(p, head_dim);
    hipStream_t st = as_stream(s);
    if (Sq > 1 && attention_prefill_supported(p, head_dim, dtype, kv_int8))
        return attention_prefill_launch(p, head_dim, dtype, st);
    int kv_len = d_active ? cache_seq_len : (active_seq_kv < cache_seq_len ? active_seq_kv : cache_seq_len);
    p.nsplit = attn_pick_nsplit(B, num_kv_heads, Sq, kv_len);
    if (p.nsplit > 1) {
        int rc = ensure(g_scratch, attn_scratch_bytes(B, num_q_heads, Sq, head_dim, p.nsplit), false, st);
        if (rc) return rc;
        rc = ensure(g_counters, attn_counter_bytes(B, num_kv_heads, Sq), true, st);
        if (rc) return rc;
    }
    return attention_decode_launch(p, head_dim, dtype, kv_int8, g_scratch.ptr, g_counters.ptr, st);
}
