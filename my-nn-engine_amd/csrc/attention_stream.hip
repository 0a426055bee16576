// Streaming GQA decode attention for large (batch x context) products: one query row per sequence,
// 16-bit K/V, head_dim 64 or 128, up to 8 query heads per kv head.
//
// attention_decode.hip is built for latency (one pass, everything in flight at once, one workgroup
// per CU); with tens of megabytes of K/V per launch the job is bandwidth instead, and this kernel
// keeps the loads streaming: a workgroup of 4 waves walks its key range in tiles of 16 keys per wave,
// the next tile's K and V already in registers while the current one is used.
//   scores   S^T[16 keys x 16 heads] = K_tile . Q^T with v_mfma_f32_16x16x32 (K rows are the A operand
//            straight from global memory: lane l holds key l%16, dims 8*(l/16)..+7 of each 32-dim block;
//            heads beyond G are zero columns),
//   softmax  online, per head, f32; the tile's p values and the rescale factors cross to the layout of
//            the next step through a 1 KB LDS patch per wave,
//   P.V      on the vector ALUs: a lane owns one key of the pass and 8 dims, and accumulates
//            o[g][8 dims] for all G heads from one 16-byte V load (8 FMAs per head per key),
// then lanes and waves are combined, and key ranges by a small second launch (attn_merge_kernel).
// Replaces the reference's attention_decode (attention.cuh:495-606) for these shapes.
#include "attention.h"
#include "mfma.h"

namespace mynn {

typedef float f4_t __attribute__((ext_vector_type(4)));
template <typename T> struct Mfma16;
template <> struct Mfma16<f16_t> {
    __device__ static f4_t run(const U4 &a, const U4 &b, f4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8_t, a), __builtin_bit_cast(h8_t, b), c, 0, 0, 0);
    }
};
template <> struct Mfma16<bf16_t> {
    __device__ static f4_t run(const U4 &a, const U4 &b, f4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(b8_t, a), __builtin_bit_cast(b8_t, b), c, 0, 0, 0);
    }
};

constexpr int kStreamWaves = 4, kStreamThreads = kStreamWaves * 64, kStreamTile = 16;

template <typename T, int D, int G>
__global__ __launch_bounds__(kStreamThreads) void attn_stream_kernel(AttnParams p) {
    constexpr int KB = D / 32;        // 32-dim blocks of a key row (MFMA K steps)
    constexpr int LPK = D / 8;        // lanes per key in the P.V layout
    constexpr int KPP = 64 / LPK;     // keys per P.V pass of a wave
    constexpr int NP = kStreamTile / KPP;  // passes per tile
    __shared__ float p_s[kStreamWaves][kStreamTile][16];  // p[key][head] of the wave's tile
    __shared__ float a_s[kStreamWaves][16];               // rescale factor per head
    __shared__ float m_s[kStreamWaves][G], l_s[kStreamWaves][G];
    __shared__ float o_s[kStreamWaves][G][D];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bhkv = blockIdx.x, split = blockIdx.y;
    const int b = bhkv / p.Hkv, hkv = bhkv % p.Hkv;
    const int head0 = hkv * G;
    const int active = p.d_active ? *p.d_active : p.active;
    const int bound = min(active, p.cache_len);
    const int k0 = split * p.slice, k1 = min(bound, k0 + p.slice);
    const size_t kv_base = (size_t)bhkv * p.cache_len;
    const T *Kp = (const T *)p.k + kv_base * D, *Vp = (const T *)p.v + kv_base * D;

    // Q^T as the MFMA B operand: lane l = head l%16 (zero beyond G), dims 8*(l/16)..+7 of each block
    U4 qf[KB];
    {
        const int h = lane & 15;
        const T *qrow = (const T *)p.q + (size_t)b * p.q_bs + (size_t)(head0 + (h < G ? h : 0)) * p.q_hs;
#pragma unroll
        for (int j = 0; j < KB; j++) {
            qf[j] = *(const U4 *)(qrow + j * 32 + (lane >> 4) * 8);
            if (h >= G) qf[j] = U4{0u, 0u, 0u, 0u};
        }
    }

    // running state.  Scores layout (after the MFMA): lane l = head l%16, keys 4*(l/16)+e of the tile.
    float m_run = -INFINITY, l_run = 0.f;  // of head l%16 (the 4 lanes sharing a head hold partial l)
    float o[G][8];
#pragma unroll
    for (int g = 0; g < G; g++)
#pragma unroll
        for (int e = 0; e < 8; e++) o[g][e] = 0.f;

    const int kk_m = lane & 15, kd_m = (lane >> 4) * 8;   // K load: key within tile, dim offset within a block
    const int kk_v = lane / LPK, vd = (lane % LPK) * 8;   // V load: key within pass, dim offset
    auto load_tile = [&](int t0, U4 *kr, U4 *vr) {
        // rows past the range re-read the last valid row; their scores are masked below
        const int krow = min(t0 + kk_m, k1 - 1);
#pragma unroll
        for (int j = 0; j < KB; j++) kr[j] = *(const U4 *)(Kp + (size_t)krow * D + j * 32 + kd_m);
#pragma unroll
        for (int q = 0; q < NP; q++) {
            const int vrow = min(t0 + q * KPP + kk_v, k1 - 1);
            vr[q] = *(const U4 *)(Vp + (size_t)vrow * D + vd);
        }
    };

    auto process = [&](int t, const U4 *kr, const U4 *vr) {
        // ---- scores of this tile
        f4_t s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < KB; j++) s4 = Mfma16<T>::run(kr[j], qf[j], s4);
        float sv[4], tmax = -INFINITY;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int key = t + (lane >> 4) * 4 + e;
            sv[e] = key < k1 ? s4[e] * p.scale : -INFINITY;
            tmax = fmaxf(tmax, sv[e]);
        }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const float m_new = fmaxf(m_run, tmax);  // finite: the tile has at least one key in range
        const float alpha = fast_exp(m_run - m_new);
        m_run = m_new;
        float psum = 0.f;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float pe = fast_exp(sv[e] - m_new);
            psum += pe;
            p_s[wave][(lane >> 4) * 4 + e][lane & 15] = pe;
        }
        l_run = l_run * alpha + psum;
        if (lane < 16) a_s[wave][lane] = alpha;
        __builtin_amdgcn_wave_barrier();
        // ---- P.V: rescale the accumulators when some head's maximum moved, then add this tile
        float al[G];
        bool moved = false;
#pragma unroll
        for (int g = 0; g < G; g++) {
            al[g] = a_s[wave][g];
            moved |= al[g] != 1.f;
        }
        if (moved) {
#pragma unroll
            for (int g = 0; g < G; g++)
#pragma unroll
                for (int e = 0; e < 8; e++) o[g][e] *= al[g];
        }
#pragma unroll
        for (int q = 0; q < NP; q++) {
            float vf[8];
            widen8<T>(vr[q], vf);
            const float *pk = p_s[wave][q * KPP + kk_v];  // 0 for keys past the range
#pragma unroll
            for (int g = 0; g < G; g++) {
                const float pg = pk[g];
#pragma unroll
                for (int e = 0; e < 8; e++) o[g][e] = fmaf(pg, vf[e], o[g][e]);
            }
        }
        __builtin_amdgcn_wave_barrier();
    };

    // two register sets, named so that the wait for one never covers the other; the load of the tile
    // after next is issued unconditionally (rows clamp to the last valid one) to keep the loop free of
    // branches around loads
    U4 kA[KB], vA[NP], kB[KB], vB[NP];
    const int tstep = kStreamWaves * kStreamTile;
    int t = k0 + wave * kStreamTile;
    if (t < k1) {
        load_tile(t, kA, vA);
        while (true) {
            load_tile(t + tstep, kB, vB);
            process(t, kA, vA);
            t += tstep;
            if (t >= k1) break;
            load_tile(t + tstep, kA, vA);
            process(t, kB, vB);
            t += tstep;
            if (t >= k1) break;
        }
    }

    // ---- combine inside the wave: l over the 4 lanes of a head, o over the KPP key slots
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
#pragma unroll
    for (int g = 0; g < G; g++)
#pragma unroll
        for (int e = 0; e < 8; e++) {
            float v = o[g][e];
#pragma unroll
            for (int off = LPK; off < 64; off <<= 1) v += __shfl_xor(v, off, 64);
            o[g][e] = v;
        }
    if (lane < G) {
        m_s[wave][lane] = m_run;
        l_s[wave][lane] = l_run;
    }
    if (lane < LPK) {
#pragma unroll
        for (int g = 0; g < G; g++)
#pragma unroll
            for (int e = 0; e < 8; e++) o_s[wave][g][lane * 8 + e] = o[g][e];
    }
    __syncthreads();

    // ---- combine the waves (a wave with no tile has m = -inf, l = 0, o = 0)
    T *out = (T *)p.out;
    for (int idx = tid; idx < G * D; idx += kStreamThreads) {
        const int g = idx / D, d = idx % D;
        float mt = -INFINITY;
#pragma unroll
        for (int w = 0; w < kStreamWaves; w++) mt = fmaxf(mt, m_s[w][g]);
        float lt = 0.f, ot = 0.f;
#pragma unroll
        for (int w = 0; w < kStreamWaves; w++) {
            const float c = m_s[w][g] == -INFINITY ? 0.f : fast_exp(m_s[w][g] - mt);
            lt = fmaf(l_s[w][g], c, lt);
            ot = fmaf(o_s[w][g][d], c, ot);
        }
        const size_t row = (size_t)(b * p.Hq + head0 + g);
        if (p.nsplit == 1) {
            Elem<T>::st(out, (size_t)b * p.o_bs + (size_t)(head0 + g) * p.o_hs + d, ot / lt);
        } else {
            // merged by attn_merge_kernel in the next launch
            p.part_o[(row * p.nsplit + split) * D + d] = ot;
            if (d == 0) {
                p.part_ml[(row * p.nsplit + split) * 2] = mt;
                p.part_ml[(row * p.nsplit + split) * 2 + 1] = lt;
            }
        }
    }
}

// ---- merge of key ranges: out[row, d] = sum_s o_s * exp(m_s - m) / sum_s l_s * exp(m_s - m).
// A launch of its own: a kernel boundary is the cheap way to make the partial results of workgroups on
// other XCDs visible (in-kernel hand-over needs either cache-wide fences, which slowed the whole
// launch down 2-3x, or loads past the L2 at 1-2 us each).
template <typename T>
__global__ __launch_bounds__(256) void attn_merge_kernel(AttnParams p, int D) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;  // (b, head, sq, d)
    const size_t rows = (size_t)p.B * p.Hq * p.Sq;
    if (idx >= rows * D) return;
    const size_t row = idx / D;
    const int d = (int)(idx % D);
    const float *ml = p.part_ml + row * p.nsplit * 2;
    const float *po = p.part_o + row * p.nsplit * D;
    float mt = -INFINITY;
#pragma unroll 8
    for (int s = 0; s < p.nsplit; s++) mt = fmaxf(mt, ml[2 * s]);
    float lt = 0.f, ot = 0.f;
#pragma unroll 8
    for (int s = 0; s < p.nsplit; s++) {
        const float ms = ml[2 * s];
        const float c = (ms == -INFINITY) ? 0.f : fast_exp(ms - mt);
        lt = fmaf(ml[2 * s + 1], c, lt);
        ot = fmaf(po[s * D + d], c, ot);
    }
    const size_t sq = row % p.Sq, bh = row / p.Sq, h = bh % p.Hq, b = bh / p.Hq;
    Elem<T>::st((T *)p.out, b * p.o_bs + h * p.o_hs + sq * p.o_rs + d, ot / lt);
}

int attention_merge_launch(const AttnParams &p, int D, int dtype, hipStream_t s) {
    const size_t n = (size_t)p.B * p.Hq * p.Sq * D;
    return dispatch_dtype(dtype, [&](auto *t) {
        using T = std::remove_pointer_t<decltype(t)>;
        MYNN_LAUNCH(attn_merge_kernel<T>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, p, D);
        return launch_status("attn_merge_kernel");
    });
}

// ---- host side ---------------------------------------------------------------------------------
bool attn_stream_eligible(int B, int Sq, int Hq, int Hkv, int D, int dtype, int kv_int8, int kv_len) {
    const int G = Hq / Hkv;
    return Sq == 1 && !kv_int8 && dtype != MYNN_F32 && (D == 64 || D == 128) && (G == 1 || G == 2 || G == 4 || G == 8) &&
           (long)B * Hkv * kv_len >= 32768;
}

// key rows per workgroup and number of key ranges: as many workgroups as the device holds at once
// (three per CU at the kernel's register count) and no more, so that there is no short second round;
// ranges a multiple of the 64 keys a workgroup takes per step and at least 128 long
void attn_stream_plan(int B, int Hkv, int kv_len, int *slice, int *nsplit) {
    const int step = kStreamWaves * kStreamTile;
    static int slots = 0;
    if (!slots) {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
            (void)hipGetLastError();
            cus = 256;
        }
        slots = 3 * cus;
    }
    int n = slots / (B * Hkv);
    const int nmax = (kv_len + 127) / 128;
    if (n > nmax) n = nmax;
    if (n < 1) n = 1;
    int rows = ((kv_len + n - 1) / n + step - 1) / step * step;
    *slice = rows;
    *nsplit = (kv_len + rows - 1) / rows;
}

template <typename T, int D>
static int stream_g(const AttnParams &p, hipStream_t s) {
    dim3 grid(p.B * p.Hkv, p.nsplit), block(kStreamThreads);
    switch (p.Hq / p.Hkv) {
    case 1: MYNN_LAUNCH((attn_stream_kernel<T, D, 1>), grid, block, 0, s, p); break;
    case 2: MYNN_LAUNCH((attn_stream_kernel<T, D, 2>), grid, block, 0, s, p); break;
    case 4: MYNN_LAUNCH((attn_stream_kernel<T, D, 4>), grid, block, 0, s, p); break;
    case 8: MYNN_LAUNCH((attn_stream_kernel<T, D, 8>), grid, block, 0, s, p); break;
    default: return fail(MYNN_ERR_UNSUPPORTED, "streaming attention: %d query heads per kv head", p.Hq / p.Hkv);
    }
    return launch_status("attn_stream_kernel");
}

int attention_stream_launch(const AttnParams &p, int D, int dtype, hipStream_t s) {
    MYNN_REQUIRE(p.q_rs >= 0 && aligned16(p.q) && aligned16(p.k) && aligned16(p.v) && p.q_bs % 8 == 0 && p.q_hs % 8 == 0,
                 MYNN_ERR_INVALID, "streaming attention: q, k, v must be 16-byte aligned");
    MYNN_REQUIRE(p.nsplit == 1 || (p.part_o && p.part_ml), MYNN_ERR_INVALID,
                 "streaming attention: no scratch for %d key ranges", p.nsplit);
    MYNN_REQUIRE(p.slice % (kStreamWaves * kStreamTile) == 0 && p.nsplit <= 65535, MYNN_ERR_INVALID,
                 "streaming attention: slice %d, %d ranges", p.slice, p.nsplit);
    int rc;
    if (dtype == MYNN_F16) rc = D == 64 ? stream_g<f16_t, 64>(p, s) : stream_g<f16_t, 128>(p, s);
    else rc = D == 64 ? stream_g<bf16_t, 64>(p, s) : stream_g<bf16_t, 128>(p, s);
    if (rc || p.nsplit == 1) return rc;
    return attention_merge_launch(p, D, dtype, s);
}

}  // namespace mynn
