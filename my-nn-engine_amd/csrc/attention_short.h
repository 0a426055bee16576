// Decode attention for a cache that one workgroup covers in a few rounds of registers (a round is 8 passes of
// 64 / (D/8) keys per wave and 8 waves; cache_len <= kShortRounds rounds): one workgroup of 512 threads per query head, and everything
// between the loads and the final merge stays inside a wave -- a group of D/8 lanes owns a key per
// pass, keeps an online softmax (m, l) and the 8 output dims of its lane over its keys, groups meet by
// shuffles, waves through one LDS exchange.  No V parking, one barrier.  RoPE of the query and of the new
// key, and both cache appends, are part of it.  Shared by the stand-alone kernel and the single-launch
// decode step.
#pragma once
#include "mynn_common.h"
#include "mfma.h"
#include <type_traits>

namespace mynn {

typedef _Float16 h2_t __attribute__((ext_vector_type(2)));

constexpr int kShortPasses = 8;  // keys per lane group held in registers at a time
constexpr int kShortRounds = 4;  // rounds of kShortPasses passes: the cache may be 4 x 512 rows at D = 64, 4 x 256 at D = 128
constexpr int kShortWaves = 8;

// qsrc / ksrc / vsrc: the D raw projection values of this query head, of its kv head's new key and new value
// (any address space).  Kc / Vc: cache rows of this (batch, kv head), row stride D.  cs / sn: the RoPE table
// rows of the token's position.  append: this workgroup writes the new row into the caches.
// part_s: kShortWaves x (D + 2) floats of LDS.  Every thread of the 512 calls it; threads tid < D get the
// output dim tid in `result` and return true.  `ready()` runs once the cache loads are on their way and before
// qsrc / ksrc / vsrc are read: a caller whose projection values arrive late waits for them there.
// KV8 (BuildOptions::quant_kv_cache): Kcache / Vcache hold int8 rows and Kscale / Vscale one scale of type T per row
// (QuantizingKVCacheUpdate, kvcache.cuh): the new key and value are quantised as that operator does it (scale = amax /
// 127 stored as T, codes rounded half away from zero), appended as codes, and met by the query as the codes times the
// stored scale -- exactly what a later step reads back; a score is (q . codes) * k_scale * scale and a weight
// exp(..) * v_scale, as the int8-KV attention operator computes them (attention.cuh:495-513 with its scale slots).
// PAGED: Kcache / Vcache (and the scales) are page pools [n_pages, Hkv, 1 << shift rows, ..] and cache row r of this
// kv head is row ((page(r >> shift) * Hkv + hkv) << shift) + r % (1 << shift) of them; `pages` holds the sequence's
// page table with entry j in lane j (at most 64 pages; a wave-wide shuffle picks a key's entry, so the table costs
// one load per wave before the cache loads and nothing per key).  Same keys, same order: the same bits as the
// contiguous form.
struct ShortPaging {
    int pages = 0;  // lane j: page number of the sequence's j-th page
    int shift = 0, Hkv = 1, hkv = 0;
};
template <typename T, int D, bool KV8 = false, bool PAGED = false, typename Ready>
__device__ __forceinline__ bool attn_short_body(const T *qsrc, const T *ksrc, const T *vsrc, void *Kcache_v, void *Vcache_v, T *Kscale,
                                                T *Vscale, int bound, int new_row, bool append, const T *cs, const T *snp, float scale,
                                                float (*part_s)[D + 2], int tid, float &result, Ready ready, const ShortPaging pg = ShortPaging{}) {
    constexpr int LPK = D / 8, GPW = 64 / LPK, KPP = kShortWaves * GPW;  // lanes per key, keys per wave / workgroup and pass
    const int lane = tid & 63, wave = tid >> 6;
    const int dc = lane % LPK, grp = lane / LPK;
    using TKV = typename std::conditional<KV8, int8_t, T>::type;
    using Chunk = typename std::conditional<KV8, uint2, U4>::type;  // this lane's 8 dims of a row
    TKV *Kcache = (TKV *)Kcache_v, *Vcache = (TKV *)Vcache_v;
    const TKV *Kc = Kcache + dc * 8, *Vc = Vcache + dc * 8;

    // row of the cache buffers that holds cache row `key` (every lane of the wave calls it: the page entry comes
    // from another lane)
    auto row_of = [&](int key) -> size_t {
        if constexpr (PAGED) {
            const int page = __shfl(pg.pages, min(max(key, 0), max(bound - 1, 0)) >> pg.shift, 64);
            return (((size_t)page * pg.Hkv + pg.hkv) << pg.shift) + (size_t)(key & ((1 << pg.shift) - 1));
        } else {
            return (size_t)key;
        }
    };
    // ---- all K / V loads of this lane for a round of kShortPasses passes (the first round before anything else)
    Chunk kreg[kShortPasses], vreg[kShortPasses];
    T ksc[KV8 ? kShortPasses : 1], vsc[KV8 ? kShortPasses : 1];  // as loaded
    auto load_round = [&](int base) {
#pragma unroll
        for (int i = 0; i < kShortPasses; i++) {
            const int key = base + i * KPP + wave * GPW + grp;
            const size_t row = row_of(key);
            kreg[i] = vreg[i] = Chunk{};
            if constexpr (KV8) ksc[i] = vsc[i] = T{};
            if (key < bound && key != new_row) {
                kreg[i] = *(const Chunk *)(Kc + row * D);
                vreg[i] = *(const Chunk *)(Vc + row * D);
                if constexpr (KV8) {
                    ksc[i] = Kscale[row];
                    vsc[i] = Vscale[row];
                }
            }
        }
    };
    load_round(0);
    // (the RoPE table rows too: they depend on the position only, not on the projection)
    constexpr int half = D / 2;
    const int d0 = dc * 8, dp = d0 < half ? d0 + half : d0 - half;
    const U4 c_raw = *(const U4 *)(cs + d0), s_raw = *(const U4 *)(snp + d0);

    ready();
    // ---- this lane's 8 dims of the rotated query, of the rotated new key and of the new value
    float c[8], sn[8], q[8], kn[8], vn[8];
    widen8<T>(c_raw, c);
    widen8<T>(s_raw, sn);
    const U4 v_new = *(const U4 *)(vsrc + d0);
    widen8<T>(v_new, vn);
    {
        float own[8], oth[8];
        widen8<T>(*(const U4 *)(qsrc + d0), own);
        widen8<T>(*(const U4 *)(qsrc + dp), oth);
        // the first half of the dims subtracts the partner's product, the second adds it: the sign goes into the sine once
#pragma unroll
        for (int e = 0; e < 8; e++) sn[e] = d0 < half ? -sn[e] : sn[e];
#pragma unroll
        for (int e = 0; e < 8; e++) q[e] = Elem<T>::rnd(own[e] * c[e] + oth[e] * sn[e]);
        // the rotated new key is needed where its row is met (one wave) and where it is appended
        if (wave == (new_row % KPP) / GPW || (append && wave == 0)) {
            widen8<T>(*(const U4 *)(ksrc + d0), own);
            widen8<T>(*(const U4 *)(ksrc + dp), oth);
#pragma unroll
            for (int e = 0; e < 8; e++) kn[e] = Elem<T>::rnd(own[e] * c[e] + oth[e] * sn[e]);
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++) kn[e] = 0.f;
        }
    }
    const U4 kn_packed = U4{pack2<T>(kn[0], kn[1]), pack2<T>(kn[2], kn[3]), pack2<T>(kn[4], kn[5]), pack2<T>(kn[6], kn[7])};
    const U4 q_packed = U4{pack2<T>(q[0], q[1]), pack2<T>(q[2], q[3]), pack2<T>(q[4], q[5]), pack2<T>(q[6], q[7])};
    Chunk kn_q{}, vn_q{};       // KV8: the new row's codes (this lane's 8 dims)
    float kn_sc = 0.f, vn_sc = 0.f;  // ... and its scales as stored
    if constexpr (KV8) {
        // per-row symmetric quantisation over the D values of the row (the lanes of this group)
        auto quantise = [&](const float *x, Chunk &codes, float &stored_scale) {
            float amax = 0.f;
#pragma unroll
            for (int e = 0; e < 8; e++) amax = fmaxf(amax, fabsf(x[e]));
            amax = group_max<LPK>(amax);
            const float inv = amax == 0.f ? 0.f : 127.0f / amax;
            stored_scale = Elem<T>::rnd(amax * (1.0f / 127.0f));
            uint32_t b[2] = {0u, 0u};
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float a = x[e] * inv;
                int c = (int)(a + (a >= 0.f ? 0.5f : -0.5f));
                c = c < -128 ? -128 : (c > 127 ? 127 : c);
                b[e >> 2] |= ((uint32_t)c & 0xFFu) << (8 * (e & 3));
            }
            codes = Chunk{b[0], b[1]};
        };
        quantise(kn, kn_q, kn_sc);
        quantise(vn, vn_q, vn_sc);
        const size_t new_at = row_of(new_row);
        if (append && wave == 0 && grp == 0) {
            *(Chunk *)(Kcache + new_at * D + d0) = kn_q;
            *(Chunk *)(Vcache + new_at * D + d0) = vn_q;
            if (dc == 0) {
                Elem<T>::st(Kscale, new_at, kn_sc);
                Elem<T>::st(Vscale, new_at, vn_sc);
            }
        }
    } else {
        const size_t new_at = row_of(new_row);
        if (append && wave == 0 && grp == 0) {  // one lane group appends the new row
            *(U4 *)(Kcache + new_at * D + d0) = kn_packed;
            *(U4 *)(Vcache + new_at * D + d0) = v_new;
        }
    }

    // ---- softmax over this lane group's keys: the scores of a round are independent of each other (all dot
    //      products, then one maximum, then one exponential per key); only rounds are chained through (m, l, o)
    float m = -INFINITY, l = 0.f, o[8];
#pragma unroll
    for (int e = 0; e < 8; e++) o[e] = 0.f;
    for (int base = 0; base < bound; base += kShortPasses * KPP) {
        if (base > 0) load_round(base);  // (a cache beyond one round: its loads are not overlapped with the round before)
        float sc[kShortPasses];
        float mr = -INFINITY;
        const int i_new = new_row >= base ? (new_row - base) / KPP : -1;  // the pass of this round that meets the new row
#pragma unroll
        for (int i = 0; i < kShortPasses; i++) {
            sc[i] = -INFINITY;
            if (base + i * KPP >= bound) continue;  // no wave has keys in this pass
            const int key = base + i * KPP + wave * GPW + grp;
            float d = 0.f;
            float k_scale_i = 1.f;
            if constexpr (KV8) {
                Chunk kk = kreg[i];
                k_scale_i = Elem<T>::ld(&ksc[i], 0);
                if (i == i_new && key == new_row) {
                    kk = kn_q;
                    k_scale_i = kn_sc;
                }
                const uint32_t kw[2] = {kk.x, kk.y};
#pragma unroll
                for (int e = 0; e < 8; e++) d = fmaf(q[e], (float)(int8_t)((kw[e >> 2] >> (8 * (e & 3))) & 0xFF), d);
            } else if constexpr (std::is_same_v<T, f16_t>) {
                // fp16: query and key stay packed, two products per instruction with f32 accumulation
                U4 kk = kreg[i];
                if (i == i_new && key == new_row) kk = kn_packed;  // (i == i_new is uniform: only this pass can hold the new row)
                const uint32_t kw[4] = {kk.x, kk.y, kk.z, kk.w}, qw[4] = {q_packed.x, q_packed.y, q_packed.z, q_packed.w};
#pragma unroll
                for (int e = 0; e < 4; e++)
                    d = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, qw[e]), __builtin_bit_cast(h2_t, kw[e]), d, false);
            } else {
                float kf[8];
                widen8<T>(kreg[i], kf);
                if (i == i_new) {
#pragma unroll
                    for (int e = 0; e < 8; e++) kf[e] = key == new_row ? kn[e] : kf[e];
                }
#pragma unroll
                for (int e = 0; e < 8; e++) d = fmaf(q[e], kf[e], d);
            }
            d = group_sum<LPK>(d);
            if constexpr (KV8) d *= k_scale_i;
            d *= scale;
            if (key < bound) sc[i] = d;
            mr = fmaxf(mr, sc[i]);
        }
        if (mr == -INFINITY) continue;  // this lane group has no key in the round
        const float mn = fmaxf(m, mr);
        const float corr = fast_exp(m - mn);  // (m = -inf: 0)
        l *= corr;
#pragma unroll
        for (int e = 0; e < 8; e++) o[e] *= corr;
#pragma unroll
        for (int i = 0; i < kShortPasses; i++) {
            if (base + i * KPP >= bound) continue;
            const int key = base + i * KPP + wave * GPW + grp;
            const float pe = fast_exp(sc[i] - mn);  // (no key: exp(-inf) = 0)
            l += pe;
            if constexpr (KV8) {
                Chunk vv = vreg[i];
                float v_scale_i = Elem<T>::ld(&vsc[i], 0);
                if (i == i_new && key == new_row) {
                    vv = vn_q;
                    v_scale_i = vn_sc;
                }
                const float pv = pe * v_scale_i;
                const uint32_t vw[2] = {vv.x, vv.y};
#pragma unroll
                for (int e = 0; e < 8; e++) o[e] = fmaf(pv, (float)(int8_t)((vw[e >> 2] >> (8 * (e & 3))) & 0xFF), o[e]);
                continue;
            }
            U4 vv;
            if constexpr (!KV8) vv = vreg[i];
            if (i == i_new && key == new_row) vv = v_new;
            if constexpr (std::is_same_v<T, f16_t>) {
                // (the widening of a half operand rides on the multiply-add: v_fma_mix_f32)
                const uint32_t vw[4] = {vv.x, vv.y, vv.z, vv.w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const h2_t hv = __builtin_bit_cast(h2_t, vw[e]);
                    o[2 * e] = fmaf(pe, (float)hv[0], o[2 * e]);
                    o[2 * e + 1] = fmaf(pe, (float)hv[1], o[2 * e + 1]);
                }
            } else {
                float vf[8];
                widen8<T>(vv, vf);
#pragma unroll
                for (int e = 0; e < 8; e++) o[e] = fmaf(pe, vf[e], o[e]);
            }
        }
        m = mn;
    }
    // ---- lane groups of the wave meet (lanes of equal dc), then the waves through LDS.  First the wave's maximum,
    //      then every group rescales its (l, o) to it once, and the groups' values are plain sums.
    // (lane ^ 8 is in the same row of 16: DPP; lane ^ 16 and lane ^ 32 through the row swaps; the same pairs either way)
    auto meet_sum = [&](float v, int off) { return off == 8 ? v + dpp_get<kDppRor8>(v) : off == 16 ? xor16_sum(v) : xor32_sum(v); };
    auto meet_max = [&](float v, int off) { return off == 8 ? fmaxf(v, dpp_get<kDppRor8>(v)) : off == 16 ? xor16_max(v) : xor32_max(v); };
    float mw = m;
#pragma unroll
    for (int off = LPK; off < 64; off <<= 1) mw = meet_max(mw, off);
    {
        const float a = m == -INFINITY ? 0.f : fast_exp(m - mw);  // (a wave without keys: everything stays 0, mw = -inf)
        l *= a;
#pragma unroll
        for (int e = 0; e < 8; e++) o[e] *= a;
        m = mw;
    }
#pragma unroll
    for (int off = LPK; off < 64; off <<= 1) {
        l = meet_sum(l, off);
#pragma unroll
        for (int e = 0; e < 8; e++) o[e] = meet_sum(o[e], off);
    }
    if (grp == 0) {
#pragma unroll
        for (int e = 0; e < 8; e++) part_s[wave][d0 + e] = o[e];
        if (dc == 0) {
            part_s[wave][D] = m;
            part_s[wave][D + 1] = l;
        }
    }
    __syncthreads();
    if (tid >= D) return false;
    float mt = -INFINITY;
#pragma unroll
    for (int w = 0; w < kShortWaves; w++) mt = fmaxf(mt, part_s[w][D]);
    float lt = 0.f, ot = 0.f;
#pragma unroll
    for (int w = 0; w < kShortWaves; w++) {
        const float mw = part_s[w][D];
        const float a = mw == -INFINITY ? 0.f : fast_exp(mw - mt);
        lt += part_s[w][D + 1] * a;
        ot += part_s[w][tid] * a;
    }
    result = ot / lt;
    return true;
}

}  // namespace mynn
