// Batch-1 decode: RMSNorm + q|k|v projection, RoPE + KV append + attention, and o projection + residual in ONE launch.
//
// As separate launches each of them starts 3.5-4 us after its producer's last store (the cost of a dependent
// dispatch on this part) with nothing of its own in flight.  Here one grid holds all three as ROLES in block order:
// the first workgroups are the q|k|v projection (the row-pair GEMV of gemv.hip, operation for operation), the next Hq
// workgroups are the attention of one query head each (attn_short_body), the last ones the o projection.  A consumer
// requests at once everything that does not depend on its input (K / V cache rows; weight rows, scales, residual)
// and then waits for the input, which arrives through memory with the data as its own flag: producers write 16-bit
// elements with agent-scope atomic stores into a vector that holds 0xFFFF ("empty": a NaN no conversion here
// produces) and consumers poll their words until no element is empty (the attention: q of its head, k and v of its
// kv head; the o projection: the whole attention output).  Workgroups are dispatched in block order, so a producer
// is resident or finished before any of its consumers is placed, and the first role never waits; every wait is
// bounded by a spin limit that raises an error word -- the launch always drains.  The vectors are emptied again by
// the launch that follows (the gate/up GEMV).  This pays because the weight streams in flight while the consumers
// poll are small (5 MB and 4 MB): the same construction behind the 23 MB gate/up stream made the layer slower.
//
// Reference ops: rms_norm.cuh:9-59, dequant_gemv.cuh:12-59, rope.cuh, kvcache.cuh, attention.cuh:495-513.
#include "kernels.h"
#include "gemv_dot.h"
#include "attention_short.h"

namespace mynn {

constexpr int kQaThreads = 512, kQaWaves = kQaThreads / 64;
constexpr int kQaStageThreads = 256;  // the activation is staged, and its RMSNorm summed, as the 256-thread GEMV does

__device__ inline void qa_put16(void *vec, int idx, uint32_t bits) {
    if (bits == 0xFFFFu) bits = 0xFFFEu;  // (an all-ones NaN stays a NaN and stops meaning "empty")
    __hip_atomic_store((uint16_t *)vec + idx, (uint16_t)bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// true when one of the four 16-bit elements of w is still empty
__device__ inline bool qa_some_empty(uint64_t w) {
    const uint64_t t = ~w;  // an empty element is a zero element of t
    return ((t - 0x0001000100010001ull) & ~t & 0x8000800080008000ull) != 0;
}
__device__ inline uint64_t qa_wait(const uint64_t *p, int limit, int *err) {
    uint64_t v = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    for (int spins = 0; qa_some_empty(v); spins++) {
        if (spins > limit) {
            __hip_atomic_store(err, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
        }
        __builtin_amdgcn_s_sleep(1);
        v = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return v;
}
template <typename T> __device__ inline uint32_t qa_bits(float v);
template <> __device__ inline uint32_t qa_bits<f16_t>(float v) { return __builtin_bit_cast(uint16_t, f32_to_f16(v)); }
template <> __device__ inline uint32_t qa_bits<bf16_t>(float v) { return f32_to_bf16_bits(v); }

// One GEMV role of the launch: row pairs of wq [N, K] against an activation vector, as dequant_gemv1_kernel
// does it (same staging partition for the RMSNorm sums, same row sums).  Wave w of role block `blk` takes the
// row pairs blk * 8 + w, + total waves, ..; its first pair is requested before the activation is staged.
//   NORM: the activation is read from memory and RMS-normalised (256 staging threads, as the 256-thread kernel)
//   POLL: the activation arrives through a hand-over vector and is waited for
//   RESID: out = T(T(sum * scale) + residual), stored plainly; else out is a hand-over vector, written element-wise
struct QaGemv {
    const void *act;       // NORM: [K] values; POLL: hand-over words
    const void *norm_w;
    float eps;
    const int8_t *wq;
    const void *scale, *residual;
    void *out;
    int N, K;
    // EMBED: the activation (NORM role) / the residual (RESID role) is row `erow` of the int8 embedding table times
    // its scale, rounded to T -- what embed_dequant_kernel would have written
    const int8_t *erow;
    float escale;
};

template <typename T, int NC, bool NORM, bool POLL, bool RESID, bool EMBED>
__device__ __forceinline__ void qa_gemv(const QaGemv &a, float *act_lds, float *red, int blk, int nblk, int limit, int *err) {
    constexpr int R = 2;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int K = a.K, N = a.N, nchunks = K >> 4, groups = (N + R - 1) / R;
    const int total_waves = nblk * kQaWaves;
    int g = blk * kQaWaves + wave;
    struct Group {
        U4 w[R][NC];
        T sc, res;        // as loaded: widening them here would make the wave wait for every load above
        int8_t eres;      // EMBED: the residual's table entry
    };
    const T *scale = (const T *)a.scale;
    auto load_group = [&](int gg, Group &G) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int row = gg * R + r < N ? gg * R + r : N - 1;
            const U4 *wrow = (const U4 *)(a.wq + (size_t)row * K);
#pragma unroll
            for (int j = 0; j < NC; j++)  // (unconditional, so that waits on earlier loads can be counted; chunks past K are not used)
                G.w[r][j] = __builtin_nontemporal_load(&wrow[min(lane + j * kWave, nchunks - 1)]);
        }
        const int row = min(gg * R + min(lane, R - 1), N - 1);
        G.sc = scale[row];
        if constexpr (RESID) {
            if constexpr (EMBED) G.eres = a.erow[row];
            else G.res = ((const T *)a.residual)[row];
        }
    };
    // An activation that is read from memory (and its norm weights) is requested BEFORE the weights: loads return in
    // order, so a wave that asked for its weights first would sit out the whole weight fetch before it could stage.
    const int npieces = K >> 3;
    constexpr int NT = NORM ? kQaStageThreads : kQaThreads;  // thread t < NT owns the 8-element pieces t, t + NT, ..
    constexpr int PMAX = (NC * 1024 / 8 + NT - 1) / NT;
    U4 apv[PMAX], nwv[NORM ? PMAX : 1];
    if constexpr (!POLL) {
        if (tid < NT) {
#pragma unroll
            for (int q = 0; q < PMAX; q++) {
                const int pc = tid + q * NT;
                if (pc < npieces) {
                    if constexpr (EMBED) {
                        const uint2 w = *(const uint2 *)(a.erow + (size_t)pc * 8);
                        apv[q] = U4{w.x, w.y, 0u, 0u};
                    } else {
                        apv[q] = ((const U4 *)a.act)[pc];
                    }
                    if constexpr (NORM) nwv[q] = ((const U4 *)a.norm_w)[pc];
                }
            }
        }
    }
    Group ga;
    load_group(min(g, groups - 1), ga);  // in flight while the activation is staged

    {
        float f[PMAX][8];
        float ss = 0.f;
        if (tid < NT) {
#pragma unroll
            for (int q = 0; q < PMAX; q++) {
                const int pc = tid + q * NT;
                if (pc < npieces) {
                    U4 raw;
                    if constexpr (POLL) {
                        const uint64_t *wp = (const uint64_t *)a.act + 2 * pc;
                        uint64_t w0 = __hip_atomic_load(wp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        uint64_t w1 = __hip_atomic_load(wp + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        if (qa_some_empty(w0)) w0 = qa_wait(wp, limit, err);
                        if (qa_some_empty(w1)) w1 = qa_wait(wp + 1, limit, err);
                        raw = U4{(uint32_t)w0, (uint32_t)(w0 >> 32), (uint32_t)w1, (uint32_t)(w1 >> 32)};
                    } else {
                        if constexpr (EMBED) {
                            const uint32_t ww[2] = {apv[q].x, apv[q].y};
                            uint32_t b[8];
#pragma unroll
                            for (int i = 0; i < 8; i++) b[i] = qa_bits<T>((float)(int8_t)((ww[i >> 2] >> (8 * (i & 3))) & 0xFF) * a.escale);
                            raw = U4{b[0] | (b[1] << 16), b[2] | (b[3] << 16), b[4] | (b[5] << 16), b[6] | (b[7] << 16)};
                        } else {
                            raw = apv[q];
                        }
                    }
                    widen8<T>(raw, f[q]);
                    if constexpr (NORM) {
#pragma unroll
                        for (int i = 0; i < 8; i++) ss = fmaf(f[q][i], f[q][i], ss);
                    }
                }
            }
            if constexpr (NORM) {
                ss = wave_sum(ss);
                if (lane == 0) red[wave] = ss;
            }
        }
        float inv = 1.f;
        if constexpr (NORM) {
            __syncthreads();
            float tot = 0.f;
#pragma unroll
            for (int i = 0; i < kQaStageThreads / 64; i++) tot += red[i];
            inv = 1.0f / sqrtf(tot / (float)K + a.eps);
        }
        if (tid < NT) {
#pragma unroll
            for (int q = 0; q < PMAX; q++) {
                const int pc = tid + q * NT;
                if (pc < npieces) {
                    if constexpr (NORM) {
                        float nw[8];
                        widen8<T>(nwv[q], nw);
#pragma unroll
                        for (int i = 0; i < 8; i++) f[q][i] = Elem<T>::rnd((f[q][i] * inv) * nw[i]);
                    }
                    gemv_stage_piece<T>(act_lds, K, pc, f[q]);
                }
            }
        }
    }
    __syncthreads();

    bool loaded = true;
    for (; g < groups; g += total_waves) {
        if (!loaded) load_group(g, ga);
        loaded = false;
        float acc[R];
        gemv_rows_dot<T, R, NC>(act_lds, K, lane, ga.w, acc);
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] = wave_sum(acc[r]);
        const int row = g * R + lane;
        if (lane < R && row < N) {
            float y = (lane == 0 ? acc[0] : acc[1]) * Elem<T>::ld(&ga.sc, 0);
            if constexpr (RESID) {
                const float res = EMBED ? Elem<T>::rnd((float)ga.eres * a.escale) : Elem<T>::ld(&ga.res, 0);
                Elem<T>::st((T *)a.out, row, Elem<T>::rnd(y) + res);
            }
            else qa_put16(a.out, row, qa_bits<T>(y));
        }
    }
}

// EMBED: the layer's input row is the embedding row of token *p.d_ids (first layer of a step)
// What a workgroup's first loads need are leading scalar arguments (copies of the fields of p): they arrive
// preloaded in SGPRs with the wave instead of through a scalar load from the kernarg segment.
template <typename T, int D, int NC, bool EMBED, bool KV8, bool PAGED>
__global__ __launch_bounds__(kQaThreads, 2) void qkv_attention_kernel(const void *x, const void *norm_w, const int8_t *wq,
                                                                          const int32_t *d_active, const int64_t *d_pos,
                                                                          int gemv_blocks, int N, int K, int Hq, QkvAttnParams p) {
    extern __shared__ float act_lds[];  // [K], GEMV workgroups
    __shared__ float red[kQaStageThreads / 64];
    __shared__ float part_s[kShortWaves][D + 2];
    __shared__ __align__(16) T qkv_l[3 * D];
    const int tid = threadIdx.x;
    const int QD = Hq * D;

    const int8_t *erow = nullptr;
    float escale = 0.f;
    if constexpr (EMBED) {
        if ((int)blockIdx.x < gemv_blocks || (int)blockIdx.x >= gemv_blocks + Hq) {
            int64_t tok = p.d_ids[0];
            if (tok < 0) tok += p.vocab;
            erow = p.embed_w + (size_t)tok * K;
            escale = Elem<T>::ld((const T *)p.embed_s, (size_t)tok);
        }
    }
    if ((int)blockIdx.x < gemv_blocks) {
        // ---- RMSNorm + q|k|v projection into the hand-over vector
        const QaGemv a{x, norm_w, p.eps, wq, p.scale, nullptr, p.qkv, N, K, erow, escale};
        qa_gemv<T, NC, true, false, false, EMBED>(a, act_lds, red, blockIdx.x, gemv_blocks, p.spin_limit, p.err);
        return;
    }
    if ((int)blockIdx.x >= gemv_blocks + Hq) {
        // ---- o projection + residual: waits for the attention's output vector
        const QaGemv a{p.attn_words, nullptr, 0.f, p.o_wq, p.o_scale, x, p.o_out, K, QD, erow, escale};
        qa_gemv<T, NC, false, true, true, EMBED>(a, act_lds, red, blockIdx.x - gemv_blocks - Hq, p.o_blocks, p.spin_limit, p.err);
        return;
    }

    // ---- attention: one workgroup per query head
    const int h = blockIdx.x - gemv_blocks, Gt = Hq / p.Hkv, hkv = h / Gt;
    const int active = *d_active;
    const int64_t pos = *d_pos;
    // contiguous caches [Hkv, max_seq, D]; PAGED: pools, rows found through the sequence's page table (one entry per lane)
    const size_t kv_rows = PAGED ? 0 : (size_t)hkv * p.max_seq;
    const size_t kv_base = kv_rows * D;  // in elements of the cache's type
    ShortPaging sp{};
    if constexpr (PAGED) {
        const int lane = tid & 63;
        sp.pages = lane < p.paging.pages_per_seq ? p.paging.table[lane] : 0;
        sp.shift = p.paging.shift; sp.Hkv = p.Hkv; sp.hkv = hkv;
    }
    using TKV = typename std::conditional<KV8, int8_t, T>::type;
    constexpr int WPH = D / 4;  // 8-byte words per head slice
    auto ready = [&] {
        if (tid < 3 * WPH) {
            const int part = tid / WPH, w = tid % WPH;
            const int head = part == 0 ? h : part == 1 ? Hq + hkv : Hq + p.Hkv + hkv;
            ((uint64_t *)qkv_l)[tid] = qa_wait(p.qkv + head * WPH + w, p.spin_limit, p.err);
        }
        __syncthreads();
    };
    float r = 0.f;
    if (attn_short_body<T, D, KV8, PAGED>(qkv_l, qkv_l + D, qkv_l + 2 * D, (TKV *)p.k_cache + kv_base, (TKV *)p.v_cache + kv_base,
                                          KV8 ? (T *)p.k_scale + kv_rows : nullptr, KV8 ? (T *)p.v_scale + kv_rows : nullptr,
                                          min(active, p.max_seq), *p.d_past, h % Gt == 0, (const T *)p.cos_t + pos * D,
                                          (const T *)p.sin_t + pos * D, p.softmax_scale, part_s, tid, r, ready, sp)) {
        if (p.o_blocks) qa_put16(p.attn_words, h * D + tid, qa_bits<T>(r));
        else Elem<T>::st((T *)p.out, (size_t)h * D + tid, r);
    }
}

bool qkv_attention_supported(int H, int Hq, int Hkv, int D, int max_seq, int dtype) {
    if (dtype != MYNN_F16 && dtype != MYNN_BF16) return false;
    if (D != 64 && D != 128) return false;
    const int kpp = kShortWaves * (64 / (D / 8));
    if (max_seq > kShortRounds * kShortPasses * kpp) return false;
    const int N = (Hq + 2 * Hkv) * D;
    if (H % 16 || H > 4096 || N % 4 || Hq % Hkv || Hq > 1024) return false;
    return (size_t)H * sizeof(float) <= 48 * 1024;
}

int qkv_attention_launch(QkvAttnParams p, int D, int dtype, hipStream_t s) {
    MYNN_REQUIRE((p.embed_w || aligned16(p.x)) && aligned16(p.norm_w) && aligned16(p.wq) && aligned16(p.qkv) && aligned16(p.k_cache) &&
                     aligned16(p.v_cache) && aligned16(p.cos_t) && aligned16(p.sin_t),
                 MYNN_ERR_INVALID, "qkv + attention: operands must be 16-byte aligned");
    p.groups = p.N / 2;
    const int max_waves = 256 * 16;
    const int passes = (p.groups + max_waves - 1) / max_waves;
    const int waves = (p.groups + passes - 1) / passes;
    p.gemv_blocks = (waves + kQaWaves - 1) / kQaWaves;
    p.o_blocks = 0;
    if (p.o_wq) {
        // the o projection rides along: K rows of [K, Hq * D] (hidden == heads x head_dim in this decoder)
        MYNN_REQUIRE(p.o_scale && p.o_out && p.attn_words && aligned16(p.o_wq) && aligned16(p.attn_words), MYNN_ERR_INVALID,
                     "qkv + attention + o: bad operand");
        const int ogroups = (p.K + 1) / 2;
        p.o_blocks = (ogroups < max_waves ? ogroups : max_waves) / kQaWaves + ((ogroups < max_waves ? ogroups : max_waves) % kQaWaves != 0);
    }
    const int nc = (p.K + 1023) / 1024;
    const size_t lds = (size_t)p.K * sizeof(float);
    const dim3 grid(p.gemv_blocks + p.Hq + p.o_blocks), block(kQaThreads);
    const bool embed = p.embed_w != nullptr, kv8 = p.k_scale != nullptr, paged = p.paging.table != nullptr;
    MYNN_REQUIRE(!paged || (p.paging.pages_per_seq <= 64 && (p.paging.pages_per_seq << p.paging.shift) == p.max_seq), MYNN_ERR_UNSUPPORTED,
                 "qkv + attention: a paged cache of %d pages of %d rows (at most 64 pages, covering max_seq %d)", p.paging.pages_per_seq,
                 1 << p.paging.shift, p.max_seq);
    MYNN_REQUIRE(!kv8 || p.v_scale, MYNN_ERR_INVALID, "qkv + attention: int8 KV needs both scale buffers");
    MYNN_REQUIRE(!embed || (p.embed_s && p.d_ids && p.vocab > 0 && p.o_wq && ((uintptr_t)p.embed_w & 7) == 0 && p.K % 8 == 0),
                 MYNN_ERR_INVALID, "qkv + attention + o: bad embedding operand");
    return dispatch_dtype16(dtype, [&](auto *t) {
        using T = std::remove_pointer_t<decltype(t)>;
#define MYNN_QA_LAUNCH(...) MYNN_LAUNCH((qkv_attention_kernel<T, __VA_ARGS__>), grid, block, lds, s, p.x, p.norm_w, p.wq, p.d_active, p.d_pos, p.gemv_blocks, p.N, p.K, p.Hq, p)
#define MYNN_QA(D_, NC_)                                                                          \
    do {                                                                                          \
        if (paged) {                                                                              \
            if (embed && kv8) MYNN_QA_LAUNCH(D_, NC_, true, true, true);                          \
            else if (embed) MYNN_QA_LAUNCH(D_, NC_, true, false, true);                           \
            else if (kv8) MYNN_QA_LAUNCH(D_, NC_, false, true, true);                             \
            else MYNN_QA_LAUNCH(D_, NC_, false, false, true);                                     \
        } else if (embed && kv8) MYNN_QA_LAUNCH(D_, NC_, true, true, false);                      \
        else if (embed) MYNN_QA_LAUNCH(D_, NC_, true, false, false);                              \
        else if (kv8) MYNN_QA_LAUNCH(D_, NC_, false, true, false);                                \
        else MYNN_QA_LAUNCH(D_, NC_, false, false, false);                                        \
        return launch_status("qkv_attention_kernel");                                             \
    } while (0)
        if (D == 64) {
            if (nc <= 1) MYNN_QA(64, 1);
            if (nc <= 2) MYNN_QA(64, 2);
            MYNN_QA(64, 4);
        }
        if (nc <= 1) MYNN_QA(128, 1);
        if (nc <= 2) MYNN_QA(128, 2);
        MYNN_QA(128, 4);
#undef MYNN_QA
#undef MYNN_QA_LAUNCH
    });
}

}  // namespace mynn
