// One decode step (batch 1, int8 weights, 16-bit activations and KV cache) as ONE launch.
//
// The per-op decode step is a chain of 5 dependent launches per layer, and on this part each launch
// boundary costs 3.5-4 us before the next kernel's first byte arrives -- more than the transfer of the
// weights themselves.  Here one workgroup per CU stays resident for the whole step and the ops hand
// their (few KB) output vectors to each other through memory, with the data as its own flag: a vector
// is written in 8-byte words by agent-scope atomic stores into a buffer that holds an "empty" pattern,
// and consumers poll the words they need with agent-scope loads until none is empty (measured 1.6 us for
// a 4 KB vector across 256 workgroups).  While a wave waits for its input it already holds the weights of
// its first rows in registers, so the weight stream does not stop at op boundaries.
//
// Arithmetic is that of the per-op kernels, operation for operation (same row sums, same roundings,
// same attention body), so both executors give bit-identical logits:
//   embed row -> per layer { RMSNorm + qkv GEMV | RoPE + KV append + attention | o GEMV + residual |
//   RMSNorm + gate/up GEMV + SwiGLU | down GEMV + residual } -> RMSNorm + lm_head GEMV -> argmax, loop state
// (reference ops: dequant_gemv.cuh:12-59, rms_norm.cuh:9-59, rope.cuh, kvcache.cuh, attention.cuh:495-513).
//
// Hand-over buffers come in two sets used by alternate steps; a step clears the other set for the next
// one (everything that read it finished with the previous launch).  Every wait is bounded: a thread that
// polls longer than the spin limit raises the error word and stops waiting, so the launch always drains.
#include "kernels.h"
#include "attention_short.h"
#include "decode_persistent.h"

namespace mynn {

constexpr uint64_t kPdEmpty = ~0ull;

// (value, index) ordered by value, then index: the later of equal maxima wins (session.rs:683-690)
__device__ inline void argmax_take(float &bv, int &bi, float v, int i) {
    if (bi < 0 || v > bv || (v == bv && i > bi)) { bv = v; bi = i; }
}

template <typename T> __device__ inline uint32_t pd_bits(float v);
template <> __device__ inline uint32_t pd_bits<f16_t>(float v) { return __builtin_bit_cast(uint16_t, f32_to_f16(v)); }
template <> __device__ inline uint32_t pd_bits<bf16_t>(float v) { return f32_to_bf16_bits(v); }

// threadIdx.x behind an opaque move: address arithmetic built on it stays where it is used instead of being
// computed for every op ahead of the layer loop and kept (spilled) across it
__device__ __forceinline__ int pd_tid() {
    int t = threadIdx.x;
    asm volatile("" : "+v"(t));
    return t;
}

// op boundary for the compiler: the relaxed atomics order nothing, and without this the weight loads of
// later ops are hoisted over earlier ones and spilled
__device__ __forceinline__ void pd_boundary() { asm volatile("" ::: "memory"); }

__device__ inline void pd_put(uint64_t *dst, uint64_t word) {
    if (word == kPdEmpty) word = kPdEmpty - 1;  // four all-ones NaNs: still four NaNs, no longer "empty"
    __hip_atomic_store(dst, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

struct PdWait {
    int limit;
    int *err;
    bool dead = false;
    __device__ inline uint64_t get(const uint64_t *p) {
        uint64_t v = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        int spins = 0;
        while (v == kPdEmpty && !dead) {
            if (++spins > limit) {
                dead = true;
                __hip_atomic_store(err, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                break;
            }
            __builtin_amdgcn_s_sleep(1);
            v = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        return v;
    }
    // the two words of a 16-byte piece, both loads in flight together
    __device__ inline U4 get_piece(const uint64_t *p) {
        uint64_t a = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        uint64_t b = __hip_atomic_load(p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (a == kPdEmpty) a = get(p);
        if (b == kPdEmpty) b = get(p + 1);
        return U4{(uint32_t)a, (uint32_t)(a >> 32), (uint32_t)b, (uint32_t)(b >> 32)};
    }
};

// ---- the activation vector of a GEMV: polled from `src` (or, EMBED, made from the int8 embedding row),
// optionally kept raw in `xres` for a later residual, optionally RMS-normalised, left in `act` as f32.
// The statistics are summed exactly as the per-op kernel does (256 threads, thread t owns pieces t, t+256, ..).
constexpr int kPdPieces = 4;  // 16-byte pieces per staging thread

template <typename T, bool NORM, bool KEEP>
__device__ __forceinline__ void pd_stage(float *act, T *xres, float *red, const uint64_t *src, const int8_t *erow, float escale,
                                         int K, const T *norm_w, float eps, PdWait &wt) {
    const int tid = pd_tid(), lane = tid & 63, wave = tid >> 6;
    constexpr int NT = NORM ? 256 : kPdThreads;
    const int npieces = K >> 3;
    U4 raw[kPdPieces], nwv[kPdPieces];
    float ss = 0.f;
    if (tid < NT) {
#pragma unroll
        for (int q = 0; q < kPdPieces; q++) {
            const int pc = tid + q * NT;
            if (pc < npieces) {
                if constexpr (NORM) nwv[q] = ((const U4 *)norm_w)[pc];
                if (erow) {
                    const uint2 w = *(const uint2 *)(erow + (size_t)pc * 8);
                    const uint32_t ww[2] = {w.x, w.y};
                    uint32_t b[8];
#pragma unroll
                    for (int i = 0; i < 8; i++) b[i] = pd_bits<T>((float)(int8_t)((ww[i >> 2] >> (8 * (i & 3))) & 0xFF) * escale);
                    raw[q] = U4{b[0] | (b[1] << 16), b[2] | (b[3] << 16), b[4] | (b[5] << 16), b[6] | (b[7] << 16)};
                } else {
                    raw[q] = wt.get_piece(src + 2 * pc);
                }
                if constexpr (NORM) {
                    float f[8];
                    widen8<T>(raw[q], f);
#pragma unroll
                    for (int i = 0; i < 8; i++) ss = fmaf(f[i], f[i], ss);
                }
            }
        }
    }
    __syncthreads();  // every wave is done with the previous contents of act / xres / red
    float inv = 1.f;
    if constexpr (NORM) {
        ss = wave_sum(ss);
        if (lane == 0 && wave < 4) red[wave] = ss;
        __syncthreads();
        float tot = 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) tot += red[i];
        inv = 1.0f / sqrtf(tot / (float)K + eps);
    }
    if (tid < NT) {
#pragma unroll
        for (int q = 0; q < kPdPieces; q++) {
            const int pc = tid + q * NT;
            if (pc < npieces) {
                if constexpr (KEEP) *(U4 *)(xres + (size_t)pc * 8) = raw[q];
                float f[8];
                widen8<T>(raw[q], f);
                if constexpr (NORM) {
                    float nw[8];
                    widen8<T>(nwv[q], nw);
#pragma unroll
                    for (int i = 0; i < 8; i++) f[i] = Elem<T>::rnd((f[i] * inv) * nw[i]);
                }
                float4 *dst = (float4 *)(act + (size_t)pc * 8);
                dst[0] = float4{f[0], f[1], f[2], f[3]};
                dst[1] = float4{f[4], f[5], f[6], f[7]};
            }
        }
    }
    __syncthreads();
}

// ---- RW rows of an int8 matrix against the staged vector: lane l holds chunks l, l + 64, .. of each row
template <int RW, int NC>
struct PdUnit {
    U4 w[RW][NC];
    float sc;  // lane r < RW: the scale of row r
};

template <typename T, int RW, int NC>
__device__ __forceinline__ void pd_load(PdUnit<RW, NC> &G, const int8_t *wq, const T *scale, int unit, int N, int K) {
    const int lane = pd_tid() & 63, nchunks = K >> 4;
#pragma unroll
    for (int r = 0; r < RW; r++) {
        const int row = min(unit * RW + r, N - 1);
        const U4 *wrow = (const U4 *)(wq + (size_t)row * K);
#pragma unroll
        for (int j = 0; j < NC; j++) {
            const int c = lane + j * kWave;
            if (c < nchunks) G.w[r][j] = __builtin_nontemporal_load(&wrow[c]);
            else G.w[r][j] = U4{0u, 0u, 0u, 0u};
        }
    }
    G.sc = Elem<T>::ld(scale, min(unit * RW + min(lane, RW - 1), N - 1));
}

// the row sums (every lane ends with all of them); returns the one of row `lane` (lanes >= RW: of the last row)
template <int RW, int NC>
__device__ __forceinline__ float pd_dot(PdUnit<RW, NC> &G, const float *act, int K) {
    const int lane = pd_tid() & 63, nchunks = K >> 4;
    float acc[RW];
#pragma unroll
    for (int r = 0; r < RW; r++) acc[r] = 0.f;
#pragma unroll
    for (int j = 0; j < NC; j++) {
        const int c = lane + j * kWave;
        if (c < nchunks) {
            float a[16];
            const float4 *ap = (const float4 *)(act + c * 16);
#pragma unroll
            for (int q = 0; q < 4; q++) {
                float4 t = ap[q];
                a[4 * q] = t.x; a[4 * q + 1] = t.y; a[4 * q + 2] = t.z; a[4 * q + 3] = t.w;
            }
#pragma unroll
            for (int r = 0; r < RW; r++) {
                float wf[16];
                pin(G.w[r][j]);
                widen16_i8(G.w[r][j], wf);
#pragma unroll
                for (int i = 0; i < 16; i++) acc[r] = fmaf(a[i], wf[i], acc[r]);
            }
        }
        __builtin_amdgcn_sched_barrier(0);  // keeps the LDS reads of later chunks from being hoisted (NC x 16 registers)
    }
    float mine = 0.f;
#pragma unroll
    for (int r = 0; r < RW; r++) {
        acc[r] = wave_sum(acc[r]);
        if (lane >= r) mine = acc[r];
    }
    return mine;
}

// four 16-bit values held by lanes 0, STEP, 2*STEP, 3*STEP -> one word in lane 0
template <int STEP> __device__ __forceinline__ uint64_t pd_word(uint32_t bits) {
    const uint64_t b0 = __shfl(bits, 0, kWave), b1 = __shfl(bits, STEP, kWave), b2 = __shfl(bits, 2 * STEP, kWave),
                   b3 = __shfl(bits, 3 * STEP, kWave);
    return b0 | (b1 << 16) | (b2 << 32) | (b3 << 48);
}

enum { PD_PLAIN = 0, PD_RESIDUAL = 1, PD_SWIGLU = 2 };

// one GEMV op: N rows of `wq` against the staged vector, output words to `dst`.  The first unit of a wave
// must already be loaded in G when `loaded` is set (it was fetched before the input was waited for).
template <typename T, int EPI, int NC>
__device__ __forceinline__ void pd_gemv(PdUnit<EPI == PD_SWIGLU ? 8 : 4, NC> &G, const int8_t *wq, const T *scale, int N, int K,
                                        const float *act, const T *xres, uint64_t *dst, int gw, int total_waves) {
    constexpr int RW = EPI == PD_SWIGLU ? 8 : 4;
    const int lane = pd_tid() & 63, nunits = N / RW;
    bool loaded = true;
    for (int u = gw; u < nunits; u += total_waves) {
        if (!loaded) pd_load<T, RW, NC>(G, wq, scale, u, N, K);
        loaded = false;
        const float sum = pd_dot<RW, NC>(G, act, K);
        uint64_t word;
        if constexpr (EPI == PD_SWIGLU) {
            const float t = Elem<T>::rnd(sum * G.sc);  // lanes 0..7: gate, up, gate, up, ..
            const float up = __shfl_down(t, 1, kWave);
            const float sig = 1.0f / (1.0f + expf(-t));
            word = pd_word<2>(pd_bits<T>((t * sig) * up));
        } else {
            float y = sum * G.sc;
            if constexpr (EPI == PD_RESIDUAL) y = Elem<T>::rnd(y) + Elem<T>::ld(xres, u * RW + min(lane, RW - 1));
            word = pd_word<1>(pd_bits<T>(y));
        }
        if (lane == 0) pd_put(dst + u, word);
    }
}

template <typename T, int D, int NCH, int NCF>
__global__ __launch_bounds__(kPdThreads) void decode_persistent_kernel(PdParams p) {
    extern __shared__ __align__(16) char pd_lds[];
    __shared__ float part_s[kShortWaves][D + 2];
    __shared__ __align__(16) T qkv_l[3 * D];
    __shared__ float red[4];
    __shared__ float sv[kPdWaves];
    __shared__ int si[kPdWaves];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int NB = gridDim.x, total_waves = NB * kPdWaves, gw = wave * NB + blockIdx.x;
    const int H = p.H, QD = p.Hq * D, KD = p.Hkv * D, NQKV = QD + 2 * KD, F = p.F, V = p.V;
    float *act = (float *)pd_lds;                    // the staged vector, f32
    T *xres = (T *)(pd_lds + (size_t)p.act_floats * 4);  // the residual stream row, raw
    PdWait wt{p.spin_limit, p.err};

    // ---- loop state, buffer sets
    const unsigned epoch = *p.epoch;
    uint64_t *set = p.hand + (size_t)(epoch & 1) * p.set_words;
    {
        uint64_t *other = p.hand + (size_t)((epoch & 1) ^ 1) * p.set_words;
        for (int i = blockIdx.x * kPdThreads + tid; i < p.set_words; i += NB * kPdThreads)
            __hip_atomic_store(other + i, kPdEmpty, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    int st_step = 0, st_past = 0;
    if (blockIdx.x == 0 && tid == 0) {
        st_step = *p.adv.step;
        st_past = *p.adv.past;
    }
    const int active = *p.adv.active;
    const int64_t pos = p.adv.pos[0];
    int64_t tok = p.adv.ids[0];
    if (tok < 0) tok += V;
    const int8_t *erow = p.embed_w + (size_t)tok * H;
    const float escale = Elem<T>::ld((const T *)p.embed_s, (size_t)tok);

    const int layer_words = (NQKV + QD + H + F + H) / 4;
    const uint64_t *x_in = nullptr;
    for (int li = 0; li < p.n_layers; li++) {
        const PdLayer L = p.layers[li];
        uint64_t *b_qkv = set + (size_t)li * layer_words, *b_attn = b_qkv + NQKV / 4, *b_x1 = b_attn + QD / 4, *b_h = b_x1 + H / 4,
                 *b_x2 = b_h + F / 4;
        // ---- RMSNorm + q|k|v projection
        {
            pd_boundary();
            PdUnit<4, NCH> G;
            if (gw < NQKV / 4) pd_load<T, 4, NCH>(G, L.qkv_w, (const T *)L.qkv_s, gw, NQKV, H);
            pd_stage<T, true, true>(act, xres, red, x_in, li == 0 ? erow : nullptr, escale, H, (const T *)L.norm1, p.eps, wt);
            pd_gemv<T, PD_PLAIN, NCH>(G, L.qkv_w, (const T *)L.qkv_s, NQKV, H, act, xres, b_qkv, gw, total_waves);
        }
        // ---- o projection weights first (in flight during the attention), then RoPE + append + attention
        pd_boundary();
        PdUnit<4, NCH> Go;
        if (gw < H / 4) pd_load<T, 4, NCH>(Go, L.o_w, (const T *)L.o_s, gw, H, QD);
        if ((int)blockIdx.x < p.Hq) {
            const int h = blockIdx.x, Gt = p.Hq / p.Hkv, hkv = h / Gt;
            constexpr int WPH = D / 4;  // words per head
            if (tid < 3 * WPH) {
                const int part = tid / WPH, w = tid % WPH;
                const int head = part == 0 ? h : part == 1 ? p.Hq + hkv : p.Hq + p.Hkv + hkv;
                ((uint64_t *)qkv_l)[tid] = wt.get(b_qkv + head * WPH + w);
            }
            __syncthreads();
            const size_t kv_base = (size_t)hkv * p.max_seq * D;
            float r = 0.f;
            const bool has = attn_short_body<T, D>(qkv_l, qkv_l + D, qkv_l + 2 * D, (T *)L.k_cache + kv_base, (T *)L.v_cache + kv_base,
                                                   min(active, p.max_seq), active - 1, h % Gt == 0, (const T *)p.cos_t + pos * D,
                                                   (const T *)p.sin_t + pos * D, p.softmax_scale, part_s, tid, r);
            // lanes 4i .. 4i+3 of the first D threads -> word i of the head
            const uint32_t bits = pd_bits<T>(r);
            const uint64_t b1 = __shfl_down(bits, 1, kWave), b2 = __shfl_down(bits, 2, kWave), b3 = __shfl_down(bits, 3, kWave);
            if (has && (tid & 3) == 0) pd_put(b_attn + (h * D + tid) / 4, (uint64_t)bits | (b1 << 16) | (b2 << 32) | (b3 << 48));
        }
        // ---- o projection + residual
        {
            pd_boundary();
            pd_stage<T, false, false>(act, xres, red, b_attn, nullptr, 0.f, QD, (const T *)nullptr, 0.f, wt);
            pd_gemv<T, PD_RESIDUAL, NCH>(Go, L.o_w, (const T *)L.o_s, H, QD, act, xres, b_x1, gw, total_waves);
        }
        // ---- RMSNorm + gate/up projection + SwiGLU
        {
            pd_boundary();
            PdUnit<8, NCH> G;
            if (gw < 2 * F / 8) pd_load<T, 8, NCH>(G, L.gu_w, (const T *)L.gu_s, gw, 2 * F, H);
            pd_stage<T, true, true>(act, xres, red, b_x1, nullptr, 0.f, H, (const T *)L.norm2, p.eps, wt);
            pd_gemv<T, PD_SWIGLU, NCH>(G, L.gu_w, (const T *)L.gu_s, 2 * F, H, act, xres, b_h, gw, total_waves);
        }
        // ---- down projection + residual
        {
            pd_boundary();
            PdUnit<4, NCF> G;
            if (gw < H / 4) pd_load<T, 4, NCF>(G, L.down_w, (const T *)L.down_s, gw, H, F);
            pd_stage<T, false, false>(act, xres, red, b_h, nullptr, 0.f, F, (const T *)nullptr, 0.f, wt);
            pd_gemv<T, PD_RESIDUAL, NCF>(G, L.down_w, (const T *)L.down_s, H, F, act, xres, b_x2, gw, total_waves);
        }
        x_in = b_x2;
    }

    // ---- final RMSNorm + lm_head + argmax.  8 logits per unit, the next unit's weights in flight while one is summed.
    float bv = -INFINITY;
    int bi = -1;
    {
        pd_boundary();
        constexpr int RW = 8;
        const int nunits = (V + RW - 1) / RW;
        const T *scale = (const T *)p.lm_s;
        PdUnit<RW, NCH> Ga, Gb;
        if (gw < nunits) pd_load<T, RW, NCH>(Ga, p.lm_w, scale, gw, V, H);
        pd_stage<T, true, false>(act, xres, red, x_in, nullptr, 0.f, H, (const T *)p.final_norm, p.eps, wt);
        T *logits = (T *)p.logits;
        auto finish = [&](PdUnit<RW, NCH> &G, int u) {
            const float y = Elem<T>::rnd(pd_dot<RW, NCH>(G, act, H) * G.sc);
            const int row = u * RW + lane;
            if (lane < RW && row < V) {
                Elem<T>::st(logits, row, y);
                argmax_take(bv, bi, y, row);
            }
        };
        for (int u = gw; u < nunits; u += 2 * total_waves) {
            const int u2 = u + total_waves;
            if (u2 < nunits) pd_load<T, RW, NCH>(Gb, p.lm_w, scale, u2, V, H);
            finish(Ga, u);
            if (u2 + total_waves < nunits) pd_load<T, RW, NCH>(Ga, p.lm_w, scale, u2 + total_waves, V, H);
            if (u2 < nunits) finish(Gb, u2);
        }
    }
    auto wave_argmax = [&]() {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float ov = __shfl_xor(bv, off, kWave);
            const int oi = __shfl_xor(bi, off, kWave);
            if (oi >= 0) argmax_take(bv, bi, ov, oi);
        }
    };
    wave_argmax();
    if (lane == 0) { sv[wave] = bv; si[wave] = bi; }
    __syncthreads();
    uint64_t *b_arg = set + (size_t)p.n_layers * layer_words;
    if (tid == 0) {
        for (int w = 1; w < kPdWaves; w++)
            if (si[w] >= 0) argmax_take(bv, bi, sv[w], si[w]);
        pd_put(b_arg + blockIdx.x, (uint64_t)(uint32_t)bi | ((uint64_t)__builtin_bit_cast(uint32_t, bv) << 32));
    }
    if (blockIdx.x != 0) return;
    // ---- workgroup 0: the token over all workgroups (value, then the later index), and the loop state moves on
    __syncthreads();
    bv = -INFINITY;
    bi = -1;
    for (int i = tid; i < NB; i += kPdThreads) {
        const uint64_t w = wt.get(b_arg + i);
        const int oi = (int)(uint32_t)w;
        if (oi >= 0 && !wt.dead) argmax_take(bv, bi, __builtin_bit_cast(float, (uint32_t)(w >> 32)), oi);
    }
    wave_argmax();
    if (lane == 0) { sv[wave] = bv; si[wave] = bi; }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < kPdWaves; w++)
            if (si[w] >= 0) argmax_take(bv, bi, sv[w], si[w]);
        p.next[0] = bi;
        if (st_step < p.adv.cap) p.adv.tokens[st_step] = bi;
        *p.adv.step = st_step + 1;
        p.adv.ids[0] = bi;
        p.adv.pos[0] = pos + 1;
        *p.adv.past = st_past + 1;
        *p.adv.active = active + 1;
        *p.epoch = epoch + 1;
    }
}

// ---- host side
bool decode_persistent_supported(const PdShape &s, int dtype, int cus) {
    if (dtype != MYNN_F16 && dtype != MYNN_BF16) return false;
    if (s.D != 64 && s.D != 128) return false;
    const int kpp = kShortWaves * (64 / (s.D / 8));
    if (s.max_seq > kShortPasses * kpp) return false;
    const int QD = s.Hq * s.D, NQKV = QD + 2 * s.Hkv * s.D;
    if (s.H % 16 || QD % 16 || s.F % 16 || NQKV % 4) return false;
    if (s.H > 4096 || QD > 4096 || s.F > 6144) return false;  // weight registers of a unit; staging pieces per thread
    if (s.H > 256 * 8 * kPdPieces || s.F > kPdThreads * 8 * kPdPieces) return false;
    if (s.Hq % s.Hkv || cus < s.Hq || cus < 1 || cus > kPdThreads) return false;
    return true;
}

size_t decode_persistent_set_words(const PdShape &s, int nb) {
    const int QD = s.Hq * s.D, NQKV = QD + 2 * s.Hkv * s.D;
    return (size_t)s.n_layers * ((NQKV + QD + s.H + s.F + s.H) / 4) + nb;
}

int decode_persistent_launch(PdParams p, const PdShape &s, int dtype, int nb, hipStream_t st) {
    const int QD = s.Hq * s.D;
    const int kmax = s.F > s.H ? (s.F > QD ? s.F : QD) : (s.H > QD ? s.H : QD);
    p.act_floats = kmax;
    const size_t lds = (size_t)kmax * 4 + (size_t)s.H * 2;
    MYNN_REQUIRE(lds <= 56 * 1024, MYNN_ERR_UNSUPPORTED, "decode step (single launch): %zu bytes of LDS", lds);
    const bool wide = s.H > 2048 || QD > 2048;
    return dispatch_dtype16(dtype, [&](auto *t) {
        using T = std::remove_pointer_t<decltype(t)>;
#define MYNN_PD(D_, NCH_)                                                                                          \
    do {                                                                                                           \
        MYNN_LAUNCH((decode_persistent_kernel<T, D_, NCH_, 6>), dim3(nb), dim3(kPdThreads), lds, st, p);           \
        return launch_status("decode_persistent_kernel");                                                          \
    } while (0)
        if (s.D == 64) {
            if (wide) MYNN_PD(64, 4);
            MYNN_PD(64, 2);
        }
        if (wide) MYNN_PD(128, 4);
        MYNN_PD(128, 2);
#undef MYNN_PD
    });
}

}  // namespace mynn
