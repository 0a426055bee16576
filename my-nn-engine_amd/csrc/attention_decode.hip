// Grouped-query attention over the KV cache, one query row at a time ("flash-decode").
//
// Replaces the reference's attention_decode (attention.cuh:495-606), which walks the cache rows
// serially with two block barriers per key and re-reads K/V once per query head.  Here one
// workgroup of 512 threads serves ALL query heads of a KV head over one slice of the cache:
//   1. every lane issues all of its 16-byte K and V loads for the slice at once (one HBM latency),
//   2. K stays in registers: a group of D/8 lanes owns a key, dots its piece with all G query
//      heads and reduces inside the group; scores go to LDS,
//   3. V is parked in LDS; one wave per query head does max / exp / sum over the slice,
//   4. thread (head, d) accumulates sum_k p[head,k] * V[k,d] from LDS -- no cross-lane merging.
// Longer caches are cut into slices over gridDim.y; a small second launch (attn_merge_kernel) merges
// the slices' partial results.
//
// FUSE form (decoder executor, one new token): the kernel also applies RoPE to q and to the new
// k row, appends k/v to the cache and attends to the new row from registers -- the reference's
// ~16 launches for Slice/Neg/Concat/Mul/Add RoPE (crates/llm/src/builder.rs:402-438), the
// transposes and the two kvcache_update launches (kvcache_update.cuh:6-26) disappear.
//
// The same kernel with gridDim.z = Sq is the plain path for Sq > 1 (each causal row gets its own
// key bound); the matrix-core prefill kernel lives in attention_prefill.hip.
#include <type_traits>

#include <map>
#include <mutex>

#include "attention.h"
#include "mfma.h"
#include "attention_short.h"

namespace mynn {

constexpr int kAttnThreads = 512;
constexpr int kAttnWaves = kAttnThreads / 64;
constexpr int kAttnNI = 8;  // key rows per lane group and slice, at most

template <typename TKV, int EPL> struct ChunkOf { using type = uint32_t; static constexpr bool vec = false; };
template <> struct ChunkOf<bf16_t, 8> { using type = U4; static constexpr bool vec = true; };
template <> struct ChunkOf<f16_t, 8> { using type = U4; static constexpr bool vec = true; };
template <> struct ChunkOf<int8_t, 8> { using type = uint2; static constexpr bool vec = true; };

// G = query heads served by one workgroup: all heads of the kv head, or a part of them when there
// are too few (batch, kv head) pairs to fill the chip (K/V are then read once per part, from L2).
template <typename T, int D, int G, bool KVI8, bool FUSE>
__global__ __launch_bounds__(kAttnThreads) void attn_decode_kernel(AttnParams p) {
    constexpr int EPL = D >= 8 ? 8 : D;      // elements of a key row per lane
    constexpr int LPK = D / EPL;             // lanes per key row
    constexpr int GPB = kAttnThreads / LPK;  // key rows per pass of the workgroup
    static_assert(D % EPL == 0 && (LPK & (LPK - 1)) == 0 && LPK <= 64, "head_dim must be a power of two");
    using TKV = typename std::conditional<KVI8, int8_t, T>::type;
    using Chunk = typename ChunkOf<TKV, EPL>::type;
    constexpr bool kVec = ChunkOf<TKV, EPL>::vec;

    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float q_s[G][D];
    __shared__ float new_s[2][D];  // FUSE: rotated k row and v row of the new token (values rounded to T)
    __shared__ float ml_s[G][2];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int grp = tid / LPK, dc = tid % LPK;
    const int Gt = p.Hq / p.Hkv, nparts = Gt / G;  // heads per kv head, parts per kv head
    const int bhkv = blockIdx.x / nparts, part = blockIdx.x % nparts;
    const int split = blockIdx.y, sq = blockIdx.z;
    const int b = bhkv / p.Hkv, hkv = bhkv % p.Hkv;
    const int head0 = hkv * Gt + part * G;  // first query head of this workgroup
    const int Sq = p.Sq;

    const int active = p.d_active ? *p.d_active : p.active;
    const int qoff = p.d_active ? active - Sq : p.q_pos_offset;
    int bound = active;
    if (p.is_causal) bound = min(bound, qoff + sq + 1);
    bound = min(bound, p.cache_len);
    const int nmax = p.slice;  // key rows per slice (multiple of GPB, <= GPB * kAttnNI)
    const int k0 = split * nmax;
    const int k1 = min(bound, k0 + nmax);
    const int n = max(k1 - k0, 0);
    const int new_row = FUSE ? *p.d_past : -1;  // cache row of the token being decoded (KVCacheUpdate's offset = past_len)

    TKV *v_s = (TKV *)smem;                                        // [nmax][D]
    float *sc = (float *)(smem + (size_t)nmax * D * sizeof(TKV));  // [G][nmax]
    float *vsc_s = sc + (size_t)G * nmax;                          // [nmax] (int8 KV: per-token v scale)

    // ---- 1. all K / V loads of the slice
    const size_t kv_base = (size_t)bhkv * p.cache_len;
    Chunk kreg[kAttnNI], vreg[kAttnNI];
    float kfl[kVec ? 1 : kAttnNI][kVec ? 1 : EPL], vfl[kVec ? 1 : kAttnNI][kVec ? 1 : EPL];
#pragma unroll
    for (int i = 0; i < kAttnNI; i++) {
        const int key = k0 + grp + i * GPB;
        if (key < k1 && key != new_row) {
            const size_t ro = (kv_base + key) * D + dc * EPL;
            if constexpr (kVec) {
                kreg[i] = *(const Chunk *)((const TKV *)p.k + ro);
                vreg[i] = *(const Chunk *)((const TKV *)p.v + ro);
            } else {
#pragma unroll
                for (int e = 0; e < EPL; e++) {
                    if constexpr (KVI8) {
                        kfl[i][e] = (float)((const int8_t *)p.k)[ro + e];
                        vfl[i][e] = (float)((const int8_t *)p.v)[ro + e];
                    } else {
                        kfl[i][e] = Elem<T>::ld((const T *)p.k, ro + e);
                        vfl[i][e] = Elem<T>::ld((const T *)p.v, ro + e);
                    }
                }
            }
        }
    }

    // ---- 0. query rows (and, FUSE, the new k/v rows) into LDS while the loads fly
    if constexpr (FUSE) {
        const int half = D / 2;
        const int width = (p.Hq + 2 * p.Hkv) * D;
        const T *row = (const T *)p.qkv + (size_t)b * width;
        const size_t tab = (size_t)(*p.d_pos) * D;
        const T *cos_t = (const T *)p.cos_t, *sin_t = (const T *)p.sin_t;
        // G query heads + 1 key head to rotate: (G+1) * D/2 pairs; then D values of v to copy
        for (int idx = tid; idx < (G + 1) * half; idx += kAttnThreads) {
            const int h = idx / half, j = idx % half;
            const T *src = h < G ? row + (size_t)(head0 + h) * D : row + (size_t)(p.Hq + hkv) * D;
            const float xl = Elem<T>::ld(src, j), xh = Elem<T>::ld(src, j + half);
            const float cl = Elem<T>::ld(cos_t, tab + j), ch = Elem<T>::ld(cos_t, tab + j + half);
            const float sl = Elem<T>::ld(sin_t, tab + j), sh = Elem<T>::ld(sin_t, tab + j + half);
            const float lo = Elem<T>::rnd(xl * cl - xh * sl), hi = Elem<T>::rnd(xh * ch + xl * sh);
            if (h < G) {
                q_s[h][j] = lo;
                q_s[h][j + half] = hi;
            } else {
                new_s[0][j] = lo;
                new_s[0][j + half] = hi;
                if (split == 0 && part == 0) {  // one workgroup appends the row
                    T *kc = (T *)p.k + (kv_base + new_row) * D;
                    Elem<T>::st(kc, j, lo);
                    Elem<T>::st(kc, j + half, hi);
                }
            }
        }
        for (int d = tid; d < D; d += kAttnThreads) {
            const T *src = row + (size_t)(p.Hq + p.Hkv + hkv) * D;
            new_s[1][d] = Elem<T>::ld(src, d);
            if (split == 0 && part == 0) ((T *)p.v)[(kv_base + new_row) * D + d] = src[d];
        }
    } else {
        for (int idx = tid; idx < G * D; idx += kAttnThreads) {
            const int g = idx / D, d = idx % D;
            const size_t qo = (size_t)b * p.q_bs + (size_t)(head0 + g) * p.q_hs + (size_t)sq * p.q_rs + d;
            q_s[g][d] = Elem<T>::ld((const T *)p.q, qo);
        }
    }
    __syncthreads();

    // ---- 2. scores: group of LPK lanes per key, all G heads
    float q[G][EPL];
#pragma unroll
    for (int g = 0; g < G; g++)
#pragma unroll
        for (int e = 0; e < EPL; e++) q[g][e] = q_s[g][dc * EPL + e];
#pragma unroll
    for (int i = 0; i < kAttnNI; i++) {
        const int key = k0 + grp + i * GPB;
        if (key < k1) {
            float kf[EPL], vf[EPL];
            if (FUSE && key == new_row) {
#pragma unroll
                for (int e = 0; e < EPL; e++) {
                    kf[e] = new_s[0][dc * EPL + e];
                    vf[e] = new_s[1][dc * EPL + e];
                }
            } else if constexpr (kVec && !KVI8) {
                widen8<T>(kreg[i], kf);
                widen8<T>(vreg[i], vf);
            } else if constexpr (kVec && KVI8) {
                const uint32_t kw[2] = {kreg[i].x, kreg[i].y}, vw[2] = {vreg[i].x, vreg[i].y};
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    kf[e] = (float)(int8_t)((kw[e >> 2] >> (8 * (e & 3))) & 0xFF);
                    vf[e] = (float)(int8_t)((vw[e >> 2] >> (8 * (e & 3))) & 0xFF);
                }
            } else {
#pragma unroll
                for (int e = 0; e < EPL; e++) {
                    kf[e] = kfl[kVec ? 0 : i][kVec ? 0 : e];
                    vf[e] = vfl[kVec ? 0 : i][kVec ? 0 : e];
                }
            }
            // park V (storage type) for phase 4: the loaded chunk as it is when there is one
            TKV *vrow = v_s + (size_t)(key - k0) * D + dc * EPL;
            if (kVec && !(FUSE && key == new_row)) {
                *(Chunk *)vrow = vreg[i];
            } else {
#pragma unroll
                for (int e = 0; e < EPL; e++) {
                    if constexpr (KVI8) vrow[e] = (int8_t)vf[e];
                    else Elem<T>::st((T *)vrow, e, vf[e]);
                }
            }
            float ksc = 1.f;
            if constexpr (KVI8) {
                ksc = Elem<T>::ld((const T *)p.k_scale, kv_base + key);
                if (dc == 0) vsc_s[key - k0] = Elem<T>::ld((const T *)p.v_scale, kv_base + key);
            }
#pragma unroll
            for (int g = 0; g < G; g++) {
                float part = 0.f;
#pragma unroll
                for (int e = 0; e < EPL; e++) part = fmaf(q[g][e], kf[e], part);
                part = group_sum<LPK>(part);
                if constexpr (KVI8) part *= ksc;
                if (dc == g % LPK) {
                    float val = part * p.scale;
                    if (!FUSE && p.mask)
                        val += Elem<T>::ld((const T *)p.mask, (size_t)(b * p.Hq + head0 + g) * p.mask_os + (size_t)sq * p.mask_rs + key);
                    sc[(size_t)g * nmax + (key - k0)] = val;
                }
            }
        }
    }
    __syncthreads();

    // ---- 3. softmax statistics: one wave per head
    for (int g = wave; g < G; g += kAttnWaves) {
        float *row = sc + (size_t)g * nmax;
        float m = -INFINITY;
        for (int k = lane; k < n; k += 64) m = fmaxf(m, row[k]);
        m = wave_max(m);
        const float mm = m == -INFINITY ? 0.f : m;  // (every key masked out: all weights 0, not exp(-inf + inf))
        float l = 0.f;
        for (int k = lane; k < n; k += 64) {
            const float e = fast_exp(row[k] - mm);
            l += e;
            row[k] = KVI8 ? e * vsc_s[k] : e;
        }
        l = wave_sum(l);
        if (lane == 0) {
            ml_s[g][0] = m;
            ml_s[g][1] = l;
        }
    }
    __syncthreads();

    // ---- 4. o[g,d] = sum_k p[g,k] * V[k,d]; thread owns (g, d) and one of KP interleaved key
    // subsets; the KP partial sums meet in LDS
    constexpr int KP = (G * D >= kAttnThreads) ? 1 : kAttnThreads / (G * D);
    T *out = (T *)p.out;
    const size_t row_base = (size_t)(b * p.Hq + head0) * Sq + sq;  // + g*Sq
    float *part_s = vsc_s + nmax;  // [KP][G*D] (KP > 1 only)
    for (int idx0 = 0; idx0 < G * D * KP; idx0 += kAttnThreads) {
        const int idx = idx0 + tid;
        const int kp = idx / (G * D), gd = idx % (G * D);
        const int g = gd / D, d = gd % D;
        const float *pr = sc + (size_t)g * nmax;
        auto vld = [&](int k) -> float {
            if constexpr (KVI8) return (float)((const int8_t *)v_s)[(size_t)k * D + d];
            else return Elem<T>::ld((const T *)v_s, (size_t)k * D + d);
        };
        float acc0 = 0.f, acc1 = 0.f, acc2 = 0.f, acc3 = 0.f;
        int k = kp;
        for (; k + 3 * KP < n; k += 4 * KP) {
            acc0 = fmaf(pr[k], vld(k), acc0);
            acc1 = fmaf(pr[k + KP], vld(k + KP), acc1);
            acc2 = fmaf(pr[k + 2 * KP], vld(k + 2 * KP), acc2);
            acc3 = fmaf(pr[k + 3 * KP], vld(k + 3 * KP), acc3);
        }
        for (; k < n; k += KP) acc0 = fmaf(pr[k], vld(k), acc0);
        float ot = (acc0 + acc1) + (acc2 + acc3);
        if constexpr (KP > 1) {
            part_s[kp * (G * D) + gd] = ot;
            __syncthreads();
            if (kp != 0) continue;
#pragma unroll
            for (int q = 1; q < KP; q++) ot += part_s[q * (G * D) + gd];
        }
        const float mt = ml_s[g][0], lt = ml_s[g][1];
        const size_t row = row_base + (size_t)g * Sq;
        if (p.nsplit == 1) {
            const size_t oo = (size_t)b * p.o_bs + (size_t)(head0 + g) * p.o_hs + (size_t)sq * p.o_rs + d;
            Elem<T>::st(out, oo, ot / lt);
        } else {
            p.part_o[(row * p.nsplit + split) * D + d] = ot;
            if (d == 0) {
                p.part_ml[(row * p.nsplit + split) * 2] = mt;
                p.part_ml[(row * p.nsplit + split) * 2 + 1] = lt;
            }
        }
    }
}

// ---- FUSE form for a cache that one workgroup covers in registers: one workgroup per query head, the
// body is attn_short_body (attention_short.h)
template <typename T, int D, bool KV8>
__global__ __launch_bounds__(kAttnThreads) void attn_decode_short_kernel(AttnParams p) {
    static_assert(kAttnWaves == kShortWaves, "the short form is written for 8 waves");
    __shared__ float part_s[kShortWaves][D + 2];
    const int tid = threadIdx.x;
    const int b = blockIdx.x / p.Hq, h = blockIdx.x % p.Hq;
    const int Gt = p.Hq / p.Hkv, hkv = h / Gt;
    const int active = p.d_active ? *p.d_active : p.active;
    const int bound = min(active, p.cache_len);
    const size_t kv_base = (size_t)(b * p.Hkv + hkv) * p.cache_len;
    const T *row = (const T *)p.qkv + (size_t)b * (p.Hq + 2 * p.Hkv) * D;
    const size_t tab = (size_t)(*p.d_pos) * D;
    float r;
    using TKV = typename std::conditional<KV8, int8_t, T>::type;
    if (attn_short_body<T, D, KV8>(row + (size_t)h * D, row + (size_t)(p.Hq + hkv) * D, row + (size_t)(p.Hq + p.Hkv + hkv) * D,
                                   (TKV *)p.k + kv_base * D, (TKV *)p.v + kv_base * D, KV8 ? (T *)p.k_scale + kv_base : nullptr,
                                   KV8 ? (T *)p.v_scale + kv_base : nullptr, bound, *p.d_past, h % Gt == 0,
                                   (const T *)p.cos_t + tab, (const T *)p.sin_t + tab, p.scale, part_s, tid, r, [] {}))
        Elem<T>::st((T *)p.out, (size_t)b * p.o_bs + (size_t)h * p.o_hs + tid, r);
}

bool attention_short_supported(const AttnParams &p, int D, int dtype) {
    if (dtype == MYNN_F32 || (D != 64 && D != 128) || p.Sq != 1 || !p.qkv) return false;
    const int kpp = kAttnWaves * (64 / (D / 8));
    return p.cache_len <= kShortRounds * kShortPasses * kpp && (long)p.B * p.Hq <= 65535;
}

// LDS the kernel may use per workgroup for the V slice, the scores and the v scales
constexpr size_t kAttnLdsBudget = 96 * 1024;

static int slice_rows(int D, int G, size_t kv_elem) {
    const int EPL = D >= 8 ? 8 : D, LPK = D / EPL, GPB = kAttnThreads / LPK;
    size_t per_row = (size_t)D * kv_elem + (size_t)G * 4 + 4;
    int rows = (int)(kAttnLdsBudget / per_row);
    rows = rows / GPB * GPB;
    if (rows > GPB * kAttnNI) rows = GPB * kAttnNI;
    if (rows < GPB) rows = GPB;
    return rows;
}
static size_t slice_lds_bytes(int rows, int D, int G, size_t kv_elem) {
    // V slice | scores | v scales | key-subset partials (at most one value per thread)
    return (size_t)rows * D * kv_elem + (size_t)G * rows * 4 + (size_t)rows * 4 + (size_t)kAttnThreads * 4;
}

template <typename T, int D, int G, bool KVI8, bool FUSE>
static int launch_one(const AttnParams &p, hipStream_t s) {
    const size_t kv_elem = KVI8 ? 1 : sizeof(T);
    const size_t lds = slice_lds_bytes(p.slice, D, G, kv_elem);
    static bool attr_set = false;
    if (!attr_set) {
        MYNN_HIP(hipFuncSetAttribute((const void *)attn_decode_kernel<T, D, G, KVI8, FUSE>,
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)(kAttnLdsBudget + 16384)));
        attr_set = true;
    }
    dim3 grid(p.B * p.Hkv * ((p.Hq / p.Hkv) / G), p.nsplit, p.Sq), block(kAttnThreads);
    MYNN_LAUNCH((attn_decode_kernel<T, D, G, KVI8, FUSE>), grid, block, lds, s, p);
    return launch_status("attn_decode_kernel");
}

template <typename T, int D, bool KVI8, bool FUSE>
static int launch_g(const AttnParams &p, hipStream_t s) {
    switch (p.heads_per_wg) {
    case 1: return launch_one<T, D, 1, KVI8, FUSE>(p, s);
    case 2: return launch_one<T, D, 2, KVI8, FUSE>(p, s);
    case 4: return launch_one<T, D, 4, KVI8, FUSE>(p, s);
    case 8: return launch_one<T, D, 8, KVI8, FUSE>(p, s);
    default:
        return fail(MYNN_ERR_UNSUPPORTED, "attention: %d query heads per kv head (supported: 1,2,4,8)", p.Hq / p.Hkv);
    }
}

template <typename T, bool KVI8, bool FUSE>
static int launch_d(const AttnParams &p, int D, hipStream_t s) {
    if constexpr (!FUSE) {
        switch (D) {
        case 4: return launch_g<T, 4, KVI8, FUSE>(p, s);
        case 8: return launch_g<T, 8, KVI8, FUSE>(p, s);
        case 16: return launch_g<T, 16, KVI8, FUSE>(p, s);
        default: break;
        }
    }
    switch (D) {
    case 32: return launch_g<T, 32, KVI8, FUSE>(p, s);
    case 64: return launch_g<T, 64, KVI8, FUSE>(p, s);
    case 128: return launch_g<T, 128, KVI8, FUSE>(p, s);
    default: break;
    }
    return fail(MYNN_ERR_UNSUPPORTED, "attention: head_dim %d (supported: 4,8,16,32,64,128; fused decode: 32,64,128)", D);
}

bool attention_fused_supported(int D, int G) {
    return (D == 32 || D == 64 || D == 128) && (G == 1 || G == 2 || G == 4 || G == 8);
}

// the fused form over an int8 cache exists for caches one workgroup covers (attention_short.h)
bool attention_fused_kv8_supported(int D, int cache_len) {
    if (D != 64 && D != 128) return false;
    const int kpp = kAttnWaves * (64 / (D / 8));
    return cache_len <= kShortRounds * kShortPasses * kpp;
}

// Slice length, number of slices and query heads per workgroup for a launch.  kv_len = longest key
// range any row can have.  All heads of a kv head share one workgroup (one K/V read) unless that
// leaves fewer than ~64 workgroups; then the heads are divided, halving until there are enough.
void attn_plan(int B, int Sq, int Hq, int Hkv, int D, int dtype, int kv_int8, int kv_len, int cache_len, bool fused,
               int *slice, int *nsplit, int *heads_per_wg) {
    const int Gt = Hq / Hkv;
    if (!fused && attn_stream_eligible(B, Sq, Hq, Hkv, D, dtype, kv_int8, kv_len, cache_len)) {
        attn_stream_plan(B, Hkv, kv_len, slice, nsplit);
        *heads_per_wg = Gt;
        return;
    }
    const size_t kv_elem = kv_int8 ? 1 : dtype_size(dtype);
    const int rows = slice_rows(D, Gt, kv_elem);
    int n = (kv_len + rows - 1) / rows;
    if (n < 1) n = 1;
    int hb = Gt;
    while (hb > 1 && hb % 2 == 0 && (long)B * Hkv * Sq * n * (Gt / hb) < 64) hb /= 2;
    *slice = rows;
    *nsplit = n;
    *heads_per_wg = hb;
}
size_t attn_scratch_bytes(int B, int Hq, int Sq, int D, int nsplit) {
    size_t rows = (size_t)B * Hq * Sq;
    size_t bytes = rows * nsplit * (D + 2) * sizeof(float);
    return (bytes + 255) / 256 * 256;
}
// The plan of a call depends on its active length and the number of key ranges is not monotonic in it, so a
// caller-owned workspace is sized for the most ranges any length up to cache_len can get: the per-slice kernel's
// count grows with the length, the streaming kernel's is bounded by the CUs per (sequence, kv head).
size_t attn_max_scratch_bytes(int B, int Sq, int Hq, int Hkv, int D, int dtype, int kv_int8, int cache_len) {
    const int Gt = Hq / Hkv;
    const size_t kv_elem = kv_int8 ? 1 : dtype_size(dtype);
    const int rows = slice_rows(D, Gt, kv_elem);
    int n = (cache_len + rows - 1) / rows;
    if (attn_stream_possible(B, Sq, Hq, Hkv, D, dtype, cache_len)) {
        const int ns = attn_stream_max_ranges(B, Hkv, cache_len);
        if (ns > n) n = ns;
    }
    return n > 1 ? attn_scratch_bytes(B, Hq, Sq, D, n) : 0;
}
// scratch = [part_o | part_ml] of attn_scratch_bytes (contents need not survive the call)
int attention_decode_launch(AttnParams p, int D, int dtype, int kv_int8, void *scratch, hipStream_t s) {
    if (p.nsplit > 1) {
        size_t rows = (size_t)p.B * p.Hq * p.Sq;
        p.part_o = (float *)scratch;
        p.part_ml = p.part_o + rows * p.nsplit * D;
    }
    const bool fuse = p.qkv != nullptr;
    MYNN_REQUIRE(!fuse || (p.d_past && p.d_pos && p.d_active && p.cos_t && p.sin_t), MYNN_ERR_INVALID,
                 "fused decode attention: position, past_len and active length must be device scalars");
    // the plan (attn_plan, with the same kv_len) was made for the streaming kernel when it is eligible
    const int kv_len = p.d_active ? p.cache_len : (p.active < p.cache_len ? p.active : p.cache_len);
    if (!fuse && !p.mask && attn_stream_eligible(p.B, p.Sq, p.Hq, p.Hkv, D, dtype, kv_int8, kv_len, p.cache_len))
        return attention_stream_launch(p, D, dtype, kv_int8, s);
    if (p.page_table) {  // (the plan is the streaming kernel's: that kernel has the paged form)
        MYNN_REQUIRE(!fuse && !p.mask, MYNN_ERR_UNSUPPORTED, "paged attention: neither the fused decode form nor a mask");
        return attention_stream_launch(p, D, dtype, kv_int8, s);
    }
    bool whole = false;  // the launch wrote the finished output: nothing to merge whatever the plan's split count
    int rc = dispatch_dtype(dtype, [&](auto *t) {
        using T = std::remove_pointer_t<decltype(t)>;
        if constexpr (sizeof(T) == 2) {
            if (fuse) {
                if (attention_short_supported(p, D, dtype)) {
                    whole = true;
                    MYNN_REQUIRE(!kv_int8 || (p.k_scale && p.v_scale), MYNN_ERR_INVALID, "fused decode attention: int8 KV without scales");
                    const dim3 grid(p.B * p.Hq), block(kAttnThreads);
                    if (D == 64 && kv_int8) MYNN_LAUNCH((attn_decode_short_kernel<T, 64, true>), grid, block, 0, s, p);
                    else if (D == 64) MYNN_LAUNCH((attn_decode_short_kernel<T, 64, false>), grid, block, 0, s, p);
                    else if (kv_int8) MYNN_LAUNCH((attn_decode_short_kernel<T, 128, true>), grid, block, 0, s, p);
                    else MYNN_LAUNCH((attn_decode_short_kernel<T, 128, false>), grid, block, 0, s, p);
                    return launch_status("attn_decode_short_kernel");
                }
                if (kv_int8) return fail(MYNN_ERR_UNSUPPORTED, "fused decode attention: int8 KV beyond the short form");
                return launch_d<T, false, true>(p, D, s);
            }
        } else {
            if (fuse) return fail(MYNN_ERR_UNSUPPORTED, "fused decode attention needs a 16-bit type");
        }
        return kv_int8 ? launch_d<T, true, false>(p, D, s) : launch_d<T, false, false>(p, D, s);
    });
    if (rc || p.nsplit == 1 || whole) return rc;
    return attention_merge_launch(p, D, dtype, s);
}

// ---- library-owned scratch, grown on demand (the streaming-KV operators below; one set for all streams)
struct Grown {
    void *ptr = nullptr;
    size_t bytes = 0;
};
static int ensure(Grown &g, size_t bytes, bool zero, hipStream_t s) {
    if (bytes <= g.bytes) return 0;
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &cs) == hipSuccess && cs != hipStreamCaptureStatusNone)
        return fail(MYNN_ERR_STATE, "the library's scratch memory cannot grow while the stream is being captured");
    MYNN_HIP(hipStreamSynchronize(s));
    if (g.ptr) MYNN_HIP(hipFree(g.ptr));
    g.ptr = nullptr;
    g.bytes = 0;
    MYNN_HIP(hipMalloc(&g.ptr, bytes));
    if (zero) MYNN_HIP(hipMemset(g.ptr, 0, bytes));
    g.bytes = bytes;
    return 0;
}
// mynn_attention: the partial results of a cache split over workgroups, one block per stream
static std::mutex g_scratch_mu;
static std::map<hipStream_t, Grown> g_scratch;

// mynn_attention_noalloc: the same partial results in a device array of the library (one copy per GPU, held until the
// process ends).  The array's name is only a handle on the host: the address kernels get is asked for once per device.
constexpr size_t kStaticScratchBytes = 8u << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
static void *g_static_ptr[kMaxDevices] = {};
static std::mutex g_static_mu;
static int static_scratch(void **out) {
    int dev = 0;
    MYNN_HIP(hipGetDevice(&dev));
    MYNN_REQUIRE(dev >= 0 && dev < kMaxDevices, MYNN_ERR_UNSUPPORTED, "attention_noalloc: device %d", dev);
    std::lock_guard<std::mutex> lk(g_static_mu);
    if (!g_static_ptr[dev]) {
        void *ptr = nullptr;
        MYNN_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        MYNN_REQUIRE(ptr, MYNN_ERR_STATE, "attention_noalloc: the scratch array has no device address");
        g_static_ptr[dev] = ptr;
    }
    *out = g_static_ptr[dev];
    return 0;
}

enum { WS_LIBRARY = 0, WS_CALLER = 1, WS_STATIC = 2 };

static int attention_entry(void *out, const void *Q, const void *K, const void *V, const void *mask, long mask_os, long mask_rs,
                           const void *k_scale, const void *v_scale, float scale, int is_causal, int B, int Sq, int active_seq_kv,
                           const int32_t *d_active, int cache_seq_len, int q_pos_offset, int num_q_heads, int num_kv_heads,
                           int head_dim, int dtype, int kv_int8, int ws_mode, void *workspace, size_t workspace_bytes, hipStream_t st) {
    MYNN_REQUIRE(out && Q && K && V, MYNN_ERR_INVALID, "attention: null operand");
    MYNN_REQUIRE(B > 0 && Sq > 0 && cache_seq_len > 0 && num_q_heads > 0 && num_kv_heads > 0, MYNN_ERR_INVALID,
                 "attention: B=%d Sq=%d cache=%d Hq=%d Hkv=%d", B, Sq, cache_seq_len, num_q_heads, num_kv_heads);
    MYNN_REQUIRE(num_q_heads % num_kv_heads == 0, MYNN_ERR_INVALID,
                 "attention: %d query heads is not a multiple of %d kv heads", num_q_heads, num_kv_heads);
    MYNN_REQUIRE(!kv_int8 || (k_scale && v_scale), MYNN_ERR_INVALID, "attention: int8 KV needs k_scale and v_scale");
    MYNN_REQUIRE(d_active || (active_seq_kv >= 1), MYNN_ERR_INVALID, "attention: active_seq_kv=%d", active_seq_kv);
    MYNN_REQUIRE(aligned16(K) && aligned16(V), MYNN_ERR_INVALID, "attention: K and V must be 16-byte aligned");
    MYNN_REQUIRE(dtype_ok(dtype), MYNN_ERR_INVALID, "attention: dtype %d", dtype);
    MYNN_REQUIRE(Sq <= 65535, MYNN_ERR_UNSUPPORTED, "attention: Sq=%d too large for the per-row kernel", Sq);
    MYNN_REQUIRE(!mask || (mask_os >= 0 && mask_rs >= 0), MYNN_ERR_INVALID, "attention: negative mask stride");
    AttnParams p{};
    p.out = out; p.q = Q; p.k = K; p.v = V; p.k_scale = k_scale; p.v_scale = v_scale; p.scale = scale;
    p.is_causal = is_causal; p.B = B; p.Sq = Sq; p.Hq = num_q_heads; p.Hkv = num_kv_heads;
    p.cache_len = cache_seq_len; p.active = active_seq_kv; p.d_active = d_active; p.q_pos_offset = q_pos_offset;
    p.mask = mask; p.mask_os = mask_os; p.mask_rs = mask_rs;
    attn_reference_layout(p, head_dim);
    if (!mask && Sq > 1 && attention_prefill_supported(p, head_dim, dtype, kv_int8))
        return attention_prefill_launch(p, head_dim, dtype, st);
    int kv_len = d_active ? cache_seq_len : (active_seq_kv < cache_seq_len ? active_seq_kv : cache_seq_len);
    attn_plan(B, Sq, num_q_heads, num_kv_heads, head_dim, dtype, kv_int8, kv_len, cache_seq_len, mask != nullptr, &p.slice, &p.nsplit,
              &p.heads_per_wg);
    MYNN_REQUIRE(p.nsplit <= 65535, MYNN_ERR_UNSUPPORTED, "attention: cache of %d rows needs too many slices", kv_len);
    void *scr = nullptr;
    if (p.nsplit > 1) {
        const size_t need = attn_scratch_bytes(B, num_q_heads, Sq, head_dim, p.nsplit);
        if (ws_mode == WS_CALLER) {
            MYNN_REQUIRE(workspace && aligned16(workspace) && workspace_bytes >= need, MYNN_ERR_INVALID,
                         "attention: the workspace must hold %zu bytes (mynn_attention_workspace_bytes), 16-byte aligned", need);
            scr = workspace;
        } else if (ws_mode == WS_STATIC) {
            MYNN_REQUIRE(need <= kStaticScratchBytes, MYNN_ERR_UNSUPPORTED,
                         "attention_noalloc: this shape needs %zu bytes of partial results, the library's fixed array holds %zu", need,
                         kStaticScratchBytes);
            int rc = static_scratch(&scr);
            if (rc) return rc;
        } else {
            std::lock_guard<std::mutex> lk(g_scratch_mu);
            Grown &g = g_scratch[st];
            int rc = ensure(g, need, false, st);
            if (rc) return rc;
            scr = g.ptr;
        }
    }
    return attention_decode_launch(p, head_dim, dtype, kv_int8, scr, st);
}

}  // namespace mynn

using namespace mynn;

extern "C" int mynn_attention(void *out, const void *Q, const void *K, const void *V, const void *k_scale,
                              const void *v_scale, float scale, int is_causal, int B, int Sq, int active_seq_kv,
                              const int32_t *d_active, int cache_seq_len, int q_pos_offset, int num_q_heads,
                              int num_kv_heads, int head_dim, int dtype, int kv_int8, mynn_stream s) {
    return attention_entry(out, Q, K, V, nullptr, 0, 0, k_scale, v_scale, scale, is_causal, B, Sq, active_seq_kv, d_active,
                           cache_seq_len, q_pos_offset, num_q_heads, num_kv_heads, head_dim, dtype, kv_int8, WS_LIBRARY, nullptr, 0,
                           as_stream(s));
}

extern "C" size_t mynn_attention_workspace_bytes(int B, int Sq, int cache_seq_len, int num_q_heads, int num_kv_heads, int head_dim,
                                                 int dtype, int kv_int8) {
    if (B <= 0 || Sq <= 0 || cache_seq_len <= 0 || num_q_heads <= 0 || num_kv_heads <= 0 || num_q_heads % num_kv_heads) return 0;
    // enough for every active length up to the cache length, with and without a mask
    return attn_max_scratch_bytes(B, Sq, num_q_heads, num_kv_heads, head_dim, dtype, kv_int8, cache_seq_len);
}

extern "C" int mynn_attention_ws(void *out, const void *Q, const void *K, const void *V, const void *mask, long mask_outer_stride,
                                 long mask_row_stride, const void *k_scale, const void *v_scale, float scale, int is_causal, int B,
                                 int Sq, int active_seq_kv, const int32_t *d_active, int cache_seq_len, int q_pos_offset,
                                 int num_q_heads, int num_kv_heads, int head_dim, int dtype, int kv_int8, void *workspace,
                                 size_t workspace_bytes, mynn_stream s) {
    return attention_entry(out, Q, K, V, mask, mask_outer_stride, mask_row_stride, k_scale, v_scale, scale, is_causal, B, Sq,
                           active_seq_kv, d_active, cache_seq_len, q_pos_offset, num_q_heads, num_kv_heads, head_dim, dtype, kv_int8,
                           WS_CALLER, workspace, workspace_bytes, as_stream(s));
}

extern "C" int mynn_attention_noalloc(void *out, const void *Q, const void *K, const void *V, const void *k_scale,
                                      const void *v_scale, float scale, int is_causal, int B, int Sq, int active_seq_kv,
                                      const int32_t *d_active, int cache_seq_len, int q_pos_offset, int num_q_heads,
                                      int num_kv_heads, int head_dim, int dtype, int kv_int8, mynn_stream s) {
    return attention_entry(out, Q, K, V, nullptr, 0, 0, k_scale, v_scale, scale, is_causal, B, Sq, active_seq_kv, d_active,
                           cache_seq_len, q_pos_offset, num_q_heads, num_kv_heads, head_dim, dtype, kv_int8, WS_STATIC, nullptr, 0,
                           as_stream(s));
}

// ---- paged K/V: the same operator over pools and a page table
static void paged_plan(int B, int Sq, int Hkv, int kv_len, int page_shift, int *slice, int *nsplit) {
    *slice = 0;
    *nsplit = 1;
    if (Sq == 1) attn_stream_plan_paged(B, Hkv, kv_len, page_shift, slice, nsplit);
}

extern "C" size_t mynn_attention_paged_workspace_bytes(int B, int Sq, int pages_per_seq, int page_rows, int num_q_heads,
                                                       int num_kv_heads, int head_dim) {
    if (B <= 0 || Sq <= 0 || pages_per_seq <= 0 || page_rows <= 0 || num_q_heads <= 0 || num_kv_heads <= 0) return 0;
    if (Sq != 1) return 0;
    int shift = 0;
    while ((1 << shift) < page_rows) shift++;
    const int nsplit = attn_stream_max_ranges_paged(B, num_kv_heads, pages_per_seq * page_rows, shift);
    return nsplit > 1 ? attn_scratch_bytes(B, num_q_heads, Sq, head_dim, nsplit) : 0;
}

extern "C" int mynn_attention_paged(void *out, const void *Q, const void *K_pool, const void *V_pool, const void *k_scale_pool,
                                    const void *v_scale_pool, const int32_t *page_table, int pages_per_seq, int page_rows,
                                    float scale, int is_causal, int B, int Sq, int active_seq_kv, const int32_t *d_active,
                                    int q_pos_offset, int num_q_heads, int num_kv_heads, int head_dim, int dtype, int kv_int8,
                                    void *workspace, size_t workspace_bytes, mynn_stream s) {
    MYNN_REQUIRE(out && Q && K_pool && V_pool && page_table, MYNN_ERR_INVALID, "attention_paged: null operand");
    MYNN_REQUIRE(B > 0 && Sq > 0 && pages_per_seq > 0 && num_q_heads > 0 && num_kv_heads > 0 && num_q_heads % num_kv_heads == 0,
                 MYNN_ERR_INVALID, "attention_paged: B=%d Sq=%d pages=%d Hq=%d Hkv=%d", B, Sq, pages_per_seq, num_q_heads, num_kv_heads);
    MYNN_REQUIRE(page_rows >= 32 && page_rows <= (1 << 20) && (page_rows & (page_rows - 1)) == 0, MYNN_ERR_INVALID,
                 "attention_paged: %d rows per page (a power of two, 32 or more)", page_rows);
    MYNN_REQUIRE((long)pages_per_seq * page_rows <= INT32_MAX, MYNN_ERR_INVALID, "attention_paged: %d pages of %d rows", pages_per_seq, page_rows);
    MYNN_REQUIRE(!kv_int8 || (k_scale_pool && v_scale_pool), MYNN_ERR_INVALID, "attention_paged: int8 KV needs the scale pools");
    MYNN_REQUIRE(d_active || (active_seq_kv >= 1), MYNN_ERR_INVALID, "attention_paged: active_seq_kv=%d", active_seq_kv);
    MYNN_REQUIRE(dtype == MYNN_F16 || dtype == MYNN_BF16, MYNN_ERR_UNSUPPORTED, "attention_paged: dtype %d (fp16 or bf16)", dtype);
    AttnParams p{};
    p.out = out; p.q = Q; p.k = K_pool; p.v = V_pool; p.k_scale = k_scale_pool; p.v_scale = v_scale_pool; p.scale = scale;
    p.is_causal = is_causal; p.B = B; p.Sq = Sq; p.Hq = num_q_heads; p.Hkv = num_kv_heads;
    p.cache_len = pages_per_seq * page_rows; p.active = active_seq_kv; p.d_active = d_active; p.q_pos_offset = q_pos_offset;
    p.page_table = page_table; p.pages_per_seq = pages_per_seq;
    while ((1 << p.page_shift) < page_rows) p.page_shift++;
    attn_reference_layout(p, head_dim);
    if (Sq > 1) {
        MYNN_REQUIRE(!kv_int8 && (head_dim == 64 || head_dim == 128) && scale > 0.f && aligned16(Q) && aligned16(out) && aligned16(K_pool) &&
                         aligned16(V_pool),
                     MYNN_ERR_UNSUPPORTED, "attention_paged: several query rows need a 16-bit cache, head_dim 64 or 128, a positive scale and 16-byte aligned operands");
        return attention_prefill_launch(p, head_dim, dtype, as_stream(s));
    }
    const int kv_len = d_active ? p.cache_len : (active_seq_kv < p.cache_len ? active_seq_kv : p.cache_len);
    paged_plan(B, Sq, num_kv_heads, kv_len, p.page_shift, &p.slice, &p.nsplit);
    p.heads_per_wg = num_q_heads / num_kv_heads;
    if (p.nsplit > 1) {
        const size_t need = attn_scratch_bytes(B, num_q_heads, Sq, head_dim, p.nsplit);
        MYNN_REQUIRE(workspace && aligned16(workspace) && workspace_bytes >= need, MYNN_ERR_INVALID,
                     "attention_paged: the workspace must hold %zu bytes (mynn_attention_paged_workspace_bytes), 16-byte aligned", need);
        const size_t rows = (size_t)B * num_q_heads * Sq;
        p.part_o = (float *)workspace;
        p.part_ml = p.part_o + rows * p.nsplit * head_dim;
    }
    return attention_stream_launch(p, head_dim, dtype, kv_int8, as_stream(s));
}

// ---- streaming KV (sink + ring cache): the slot map of the reference's kernels and the two operators that
// take it.  Attention is order-free over its keys apart from the causal rule, which is stated in ranks, so
// the rows are gathered into rank order (library-owned scratch) and handed to the kernels above.
namespace mynn {

// dst[bh][r][:] = src[bh][ring_phys_index(r)][:] for r < rows (gather), or, SCATTER,
// dst[bh][ring_phys_index(offset + r)][:] = src[bh][r][:]; rows of `units` 2-byte units
template <bool SCATTER>
__global__ void ring_rows_kernel(uint16_t *dst, const uint16_t *src, size_t units, int rows, int cache_len, int offset, int sink,
                                 int window, int start, size_t total) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const size_t u = i % units, r = (i / units) % rows, bh = i / (units * rows);
    if (SCATTER) {
        // rows that share a slot: the last one in t order wins, as in the reference's sequential loop
        // (two ranks share a ring slot exactly when both are past the sink and a multiple of the window apart)
        const int slot = ring_phys_index(offset + (int)r, sink, window, start);
        if (window > 0 && offset + (int)r >= sink && (int)r + window < rows) return;  // a later row takes the slot
        dst[(bh * cache_len + slot) * units + u] = src[i];
    } else {
        dst[i] = src[(bh * cache_len + ring_phys_index((int)r, sink, window, start)) * units + u];
    }
}


// K rotated inside the operator (reference attention.cuh:407-420, 559-570): the key of rank r, dequantised,
// is rotated by table row kv_position[r], everything in f32; V is dequantised.  Both land in rank order as f32.
template <typename T, bool KVI8>
__global__ void ring_rope_rows_kernel(float *kf, float *vf, const void *K, const void *V, const T *k_scale, const T *v_scale,
                                      const T *cos_t, const T *sin_t, const int64_t *kv_position, int D, int rows, int cache_len,
                                      int sink, int window, int start, size_t total) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int d = (int)(i % D), r = (int)((i / D) % rows);
    const size_t bh = i / ((size_t)D * rows);
    const size_t tok = bh * cache_len + ring_phys_index(r, sink, window, start);
    const int half = D / 2, dp = d < half ? d + half : d - half;
    const float sign = d < half ? -1.0f : 1.0f;
    float k, kp, v;
    if constexpr (KVI8) {
        const float ks = Elem<T>::ld(k_scale, tok), vs = Elem<T>::ld(v_scale, tok);
        k = (float)((const int8_t *)K)[tok * D + d] * ks;
        kp = (float)((const int8_t *)K)[tok * D + dp] * ks;
        v = (float)((const int8_t *)V)[tok * D + d] * vs;
    } else {
        k = Elem<T>::ld((const T *)K, tok * D + d);
        kp = Elem<T>::ld((const T *)K, tok * D + dp);
        v = Elem<T>::ld((const T *)V, tok * D + d);
    }
    const size_t tab = (size_t)kv_position[r] * D + d;
    kf[i] = k * Elem<T>::ld(cos_t, tab) + (sign * kp) * Elem<T>::ld(sin_t, tab);
    vf[i] = v;
}
template <typename T>
__global__ void widen_rows_kernel(float *dst, const T *src, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = Elem<T>::ld(src, i);
}
template <typename T>
__global__ void narrow_rows_kernel(T *dst, const float *src, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) Elem<T>::st(dst, i, src[i]);
}

}  // namespace mynn

extern "C" int mynn_kvcache_update_streaming(void *cache, const void *new_kv, int offset, int BH, int S_new, int max_seq, int D,
                                             int ring_sink, int ring_window, int ring_start, int dtype, mynn_stream s) {
    using namespace mynn;
    MYNN_REQUIRE(cache && new_kv, MYNN_ERR_INVALID, "kvcache_update: null operand");
    MYNN_REQUIRE(BH > 0 && S_new > 0 && D > 0 && offset >= 0, MYNN_ERR_INVALID, "kvcache_update: BH=%d S_new=%d D=%d offset=%d", BH,
                 S_new, D, offset);
    MYNN_REQUIRE(dtype_ok(dtype) || dtype == MYNN_I8, MYNN_ERR_INVALID, "kvcache_update: dtype %d", dtype);
    MYNN_REQUIRE(ring_sink >= 0 && ring_window >= 0 && ring_start >= 0 && (ring_window == 0 || ring_start < ring_window),
                 MYNN_ERR_INVALID, "kvcache_update: ring sink=%d window=%d start=%d", ring_sink, ring_window, ring_start);
    if (ring_window == 0) {
        MYNN_REQUIRE(offset + S_new <= max_seq, MYNN_ERR_INVALID, "kvcache_update: offset %d + %d rows exceeds max_seq %d", offset,
                     S_new, max_seq);
    } else {
        MYNN_REQUIRE(ring_sink + ring_window <= max_seq, MYNN_ERR_INVALID, "kvcache_update: sink %d + window %d exceeds max_seq %d",
                     ring_sink, ring_window, max_seq);
    }
    const size_t row_bytes = (size_t)D * (dtype == MYNN_I8 ? 1 : dtype_size(dtype));
    MYNN_REQUIRE(row_bytes % 2 == 0, MYNN_ERR_UNSUPPORTED, "kvcache_update: rows of %zu bytes", row_bytes);
    const size_t units = row_bytes / 2, total = (size_t)BH * S_new * units;
    MYNN_LAUNCH((ring_rows_kernel<true>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, as_stream(s), (uint16_t *)cache,
                (const uint16_t *)new_kv, units, S_new, max_seq, offset, ring_sink, ring_window, ring_start, total);
    return launch_status("ring_rows_kernel");
}

// ---- mynn_attention_streaming: one workspace, carved into the rank-ordered K / V rows (and scales), the widened
// queries and f32 output of the rotating form, and the partial results of the attention kernels behind it
namespace mynn {
struct RingCarve {
    size_t k, v, ks, vs, q, o, attn, attn_bytes, total;
};
static RingCarve ring_carve(int B, int Sq, int Hq, int Hkv, int D, int dtype, int kv_int8, bool rope_on, int rows_max) {
    RingCarve c{};
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t o = off; off = (off + bytes + 255) / 256 * 256; return o; };
    const size_t BH = (size_t)B * Hkv, eb = dtype_size(dtype), q_n = (size_t)B * Hq * Sq * D;
    if (rope_on) {
        c.k = take(BH * rows_max * D * 4);
        c.v = take(BH * rows_max * D * 4);
        c.q = take(dtype != MYNN_F32 ? q_n * 4 : 0);
        c.o = take(dtype != MYNN_F32 ? q_n * 4 : 0);
        c.attn_bytes = attn_max_scratch_bytes(B, Sq, Hq, Hkv, D, MYNN_F32, 0, rows_max);
    } else {
        const size_t rb = (size_t)D * (kv_int8 ? 1 : eb);
        c.k = take(BH * rows_max * rb);
        c.v = take(BH * rows_max * rb);
        c.ks = take(kv_int8 ? BH * rows_max * eb : 0);
        c.vs = take(kv_int8 ? BH * rows_max * eb : 0);
        c.attn_bytes = attn_max_scratch_bytes(B, Sq, Hq, Hkv, D, dtype, kv_int8, rows_max);
    }
    c.attn = take(c.attn_bytes);
    c.total = off;
    return c;
}
static std::mutex g_ring_mu;
static std::map<hipStream_t, Grown> g_ring;  // mynn_attention_streaming: one block per stream
}  // namespace mynn

extern "C" size_t mynn_attention_streaming_workspace_bytes(int B, int Sq, int cache_seq_len, int num_q_heads, int num_kv_heads,
                                                           int head_dim, int dtype, int kv_int8, int rope_on) {
    if (B <= 0 || Sq <= 0 || cache_seq_len <= 0 || num_q_heads <= 0 || num_kv_heads <= 0 || num_q_heads % num_kv_heads ||
        head_dim <= 0 || !mynn::dtype_ok(dtype))
        return 0;
    return mynn::ring_carve(B, Sq, num_q_heads, num_kv_heads, head_dim, dtype, kv_int8, rope_on != 0, cache_seq_len).total;
}

extern "C" int mynn_attention_streaming_ws(void *out, const void *Q, const void *K, const void *V, const void *k_scale,
                                           const void *v_scale, float scale, int is_causal, int B, int Sq, int active_seq_kv,
                                           int cache_seq_len, int q_pos_offset, int num_q_heads, int num_kv_heads, int head_dim,
                                           int dtype, int kv_int8, int ring_sink, int ring_window, int ring_start,
                                           const void *cos_t, const void *sin_t, const int64_t *kv_position, void *workspace,
                                           size_t workspace_bytes, mynn_stream s) {
    using namespace mynn;
    MYNN_REQUIRE(ring_sink >= 0 && ring_window >= 0 && ring_start >= 0 && (ring_window == 0 || ring_start < ring_window),
                 MYNN_ERR_INVALID, "attention: ring sink=%d window=%d start=%d", ring_sink, ring_window, ring_start);
    const bool rope_on = cos_t || sin_t || kv_position;
    MYNN_REQUIRE(!rope_on || (cos_t && sin_t && kv_position), MYNN_ERR_INVALID,
                 "attention: the K rotation needs cos, sin and kv_position together");
    MYNN_REQUIRE(out && Q && K && V, MYNN_ERR_INVALID, "attention: null operand");
    MYNN_REQUIRE(B > 0 && Sq > 0 && cache_seq_len > 0 && num_q_heads > 0 && num_kv_heads > 0 && head_dim > 0 &&
                     num_q_heads % num_kv_heads == 0,
                 MYNN_ERR_INVALID, "attention: B=%d Sq=%d cache=%d Hq=%d Hkv=%d D=%d", B, Sq, cache_seq_len, num_q_heads, num_kv_heads,
                 head_dim);
    MYNN_REQUIRE(active_seq_kv >= 1, MYNN_ERR_INVALID, "attention: active_seq_kv=%d", active_seq_kv);
    MYNN_REQUIRE(ring_sink + ring_window <= cache_seq_len, MYNN_ERR_INVALID, "attention: sink %d + window %d exceeds the cache of %d rows",
                 ring_sink, ring_window, cache_seq_len);
    MYNN_REQUIRE(!kv_int8 || (k_scale && v_scale), MYNN_ERR_INVALID, "attention: int8 KV needs k_scale and v_scale");
    MYNN_REQUIRE(dtype_ok(dtype), MYNN_ERR_INVALID, "attention: dtype %d", dtype);
    // ranks past sink + window would read ring rows a second time (the reference's kernels do); the session
    // never asks for them, and the plain kernels clamp the same way
    int rows = active_seq_kv < ring_sink + ring_window ? active_seq_kv : ring_sink + ring_window;
    if (ring_window == 0) rows = active_seq_kv < cache_seq_len ? active_seq_kv : cache_seq_len;
    const RingCarve c = ring_carve(B, Sq, num_q_heads, num_kv_heads, head_dim, dtype, kv_int8, rope_on, rows);
    MYNN_REQUIRE(workspace && ((uintptr_t)workspace & 255) == 0 && workspace_bytes >= c.total, MYNN_ERR_INVALID,
                 "attention: the workspace must hold %zu bytes (mynn_attention_streaming_workspace_bytes), 256-byte aligned", c.total);
    char *ws = (char *)workspace;
    const int BH = B * num_kv_heads;
    hipStream_t st = as_stream(s);
    if (rope_on) {
        // f32 throughout, as the reference's kernel computes it: rotated / dequantised K and V in rank order, the
        // queries widened, the f32 attention over them, one rounding of the result
        MYNN_REQUIRE(head_dim % 2 == 0, MYNN_ERR_INVALID, "attention: head_dim %d", head_dim);
        const size_t kv_n = (size_t)BH * rows * head_dim, q_n = (size_t)B * num_q_heads * Sq * head_dim;
        float *kf = (float *)(ws + c.k), *vf = (float *)(ws + c.v);
        const void *qf = Q;
        void *of = out;
        if (dtype != MYNN_F32) {
            qf = ws + c.q;
            of = ws + c.o;
        }
        int rc = dispatch_dtype(dtype, [&](auto *t) {
            using T = std::remove_pointer_t<decltype(t)>;
            const dim3 grid((unsigned)((kv_n + 255) / 256));
            if (kv_int8)
                MYNN_LAUNCH((ring_rope_rows_kernel<T, true>), grid, dim3(256), 0, st, kf, vf, K, V, (const T *)k_scale, (const T *)v_scale,
                            (const T *)cos_t, (const T *)sin_t, kv_position, head_dim, rows, cache_seq_len, ring_sink, ring_window,
                            ring_start, kv_n);
            else
                MYNN_LAUNCH((ring_rope_rows_kernel<T, false>), grid, dim3(256), 0, st, kf, vf, K, V, (const T *)nullptr, (const T *)nullptr,
                            (const T *)cos_t, (const T *)sin_t, kv_position, head_dim, rows, cache_seq_len, ring_sink, ring_window,
                            ring_start, kv_n);
            if (dtype != MYNN_F32)
                MYNN_LAUNCH(widen_rows_kernel<T>, dim3((unsigned)((q_n + 255) / 256)), dim3(256), 0, st, (float *)(ws + c.q), (const T *)Q, q_n);
            return launch_status("ring_rope_rows_kernel");
        });
        if (rc) return rc;
        rc = attention_entry(of, qf, kf, vf, nullptr, 0, 0, nullptr, nullptr, scale, is_causal, B, Sq, rows, nullptr, rows, q_pos_offset,
                             num_q_heads, num_kv_heads, head_dim, MYNN_F32, 0, WS_CALLER, ws + c.attn, c.attn_bytes, st);
        if (rc || dtype == MYNN_F32) return rc;
        return dispatch_dtype16(dtype, [&](auto *t) {
            using T = std::remove_pointer_t<decltype(t)>;
            MYNN_LAUNCH(narrow_rows_kernel<T>, dim3((unsigned)((q_n + 255) / 256)), dim3(256), 0, st, (T *)out, (const float *)(ws + c.o), q_n);
            return launch_status("narrow_rows_kernel");
        });
    }
    const size_t eb = dtype_size(dtype), row_bytes = (size_t)head_dim * (kv_int8 ? 1 : eb);
    MYNN_REQUIRE(row_bytes % 2 == 0 && eb % 2 == 0, MYNN_ERR_UNSUPPORTED, "attention: rows of %zu bytes", row_bytes);
    auto gather = [&](void *dst, const void *src, size_t rb) -> int {
        const size_t units = rb / 2, total = (size_t)BH * rows * units;
        MYNN_LAUNCH((ring_rows_kernel<false>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, (uint16_t *)dst,
                    (const uint16_t *)src, units, rows, cache_seq_len, 0, ring_sink, ring_window, ring_start, total);
        return launch_status("ring_rows_kernel");
    };
    int rc = gather(ws + c.k, K, row_bytes);
    if (!rc) rc = gather(ws + c.v, V, row_bytes);
    if (!rc && kv_int8) rc = gather(ws + c.ks, k_scale, eb);
    if (!rc && kv_int8) rc = gather(ws + c.vs, v_scale, eb);
    if (rc) return rc;
    return attention_entry(out, Q, ws + c.k, ws + c.v, nullptr, 0, 0, kv_int8 ? ws + c.ks : nullptr, kv_int8 ? ws + c.vs : nullptr, scale,
                           is_causal, B, Sq, rows, nullptr, rows, q_pos_offset, num_q_heads, num_kv_heads, head_dim, dtype, kv_int8,
                           WS_CALLER, ws + c.attn, c.attn_bytes, st);
}

extern "C" int mynn_attention_streaming(void *out, const void *Q, const void *K, const void *V, const void *k_scale,
                                        const void *v_scale, float scale, int is_causal, int B, int Sq, int active_seq_kv,
                                        int cache_seq_len, int q_pos_offset, int num_q_heads, int num_kv_heads, int head_dim,
                                        int dtype, int kv_int8, int ring_sink, int ring_window, int ring_start,
                                        const void *cos_t, const void *sin_t, const int64_t *kv_position, mynn_stream s) {
    using namespace mynn;
    const bool rope_on = cos_t || sin_t || kv_position;
    if (ring_window == 0 && !rope_on && ring_sink >= 0 && ring_start >= 0)
        return mynn_attention(out, Q, K, V, k_scale, v_scale, scale, is_causal, B, Sq, active_seq_kv, nullptr, cache_seq_len,
                              q_pos_offset, num_q_heads, num_kv_heads, head_dim, dtype, kv_int8, s);
    MYNN_REQUIRE(B > 0 && Sq > 0 && cache_seq_len > 0 && num_q_heads > 0 && num_kv_heads > 0 && head_dim > 0 &&
                     num_q_heads % num_kv_heads == 0 && dtype_ok(dtype),
                 MYNN_ERR_INVALID, "attention: B=%d Sq=%d cache=%d Hq=%d Hkv=%d D=%d dtype=%d", B, Sq, cache_seq_len, num_q_heads,
                 num_kv_heads, head_dim, dtype);
    // the library's block of this stream, sized once for the whole cache (it then never grows for this shape)
    const size_t need = ring_carve(B, Sq, num_q_heads, num_kv_heads, head_dim, dtype, kv_int8, rope_on, cache_seq_len).total;
    hipStream_t st = as_stream(s);
    void *ws = nullptr;
    {
        std::lock_guard<std::mutex> lk(g_ring_mu);
        Grown &g = g_ring[st];
        int rc = ensure(g, need, false, st);
        if (rc) return rc;
        ws = g.ptr;
    }
    return mynn_attention_streaming_ws(out, Q, K, V, k_scale, v_scale, scale, is_causal, B, Sq, active_seq_kv, cache_seq_len, q_pos_offset,
                                       num_q_heads, num_kv_heads, head_dim, dtype, kv_int8, ring_sink, ring_window, ring_start, cos_t,
                                       sin_t, kv_position, ws, need, s);
}
