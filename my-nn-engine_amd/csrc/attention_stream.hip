// Streaming GQA decode attention for large (batch x context) products: one query row per sequence,
// 16-bit or int8 (per-token scales) K/V, head_dim 64 or 128, up to 8 query heads per kv head.
//
// attention_decode.hip is built for latency (one pass, everything in flight at once, one workgroup
// per CU); with tens of megabytes of K/V per launch the job is bandwidth instead, and this kernel
// keeps the loads streaming: a workgroup of 4 waves walks its key range in tiles of 32 keys per wave,
// the next tile's K and V already in registers while the current one is used.  Both products run on
// the matrix cores (v_mfma_f32_16x16x32), with the query heads as the 16 columns (zero beyond G):
//   scores   S[keys x heads] = K_tile . Q^T; K rows are the A operand straight from global memory
//            (lane l holds key l%16, dims 8*(l/16)..+7 of each 32-dim block),
//   softmax  online, per head, f32; a lane holds one head (l%16), so rescaling its accumulators is
//            lane-local; the tile's p values go to LDS as [head][key] in the storage type,
//   P.V      O^T[dims x heads] += V^T . P; V needs its keys along the reduction, so the tile is parked
//            in LDS (row stride 136 bytes: conflict-free) and read back two dims at a time, each pair of
//            keys split into an "even dims" and an "odd dims" operand by one v_perm -- the 16 rows of
//            an MFMA tile are dims 32c + 2r (+1),
// then waves are combined through LDS and key ranges by a small second launch (attn_merge_kernel).
// P enters the second product as a sum of two storage-type values.  Replaces the reference's attention_decode (attention.cuh:495-606) for these shapes.
#include <type_traits>

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

constexpr int kStreamWaves = 4, kStreamThreads = kStreamWaves * 64, kStreamTile = 32;
// (sequences x kv heads x keys) from which this kernel is taken instead of the latency kernel of attention_decode.hip:
// measured cross-over (head_dim 64 and 128, 1 .. 32 sequences): below it that kernel's single launch of 9-11 us wins or
// ties, above it this one (two launches, 11 us together, one of 9 us once every CU has a pair) is 25-50 % faster
constexpr long kStreamMinKeys = 8192;

// KVI8: int8 caches with one scale per token row (QuantizingKVCacheUpdate): K and V are widened exactly to
// the 16-bit type in registers, the key's k scale multiplies its score and its v scale its p.
// PAGED: K/V rows are found through a page table (AttnParams::page_table).  A tile of 32 keys never crosses a page
// (pages hold a power of two >= 32 rows, tiles start at multiples of 32), so the page is a wave-uniform value per
// tile: the workgroup's part of the table sits in one register (lane i = the i-th page of its key range, at most 64)
// and a tile picks its entry with v_readlane -- no dependent load in the key loop.
template <typename T, int D, int G, bool KVI8, bool PAGED>
__global__ __launch_bounds__(kStreamThreads) void attn_stream_kernel(AttnParams p) {
    constexpr int KB = D / 32;              // 32-dim blocks of a key row
    constexpr int LPK = D / 8;              // lanes per key row when a tile is loaded 16 bytes per lane
    constexpr int KPP = 64 / LPK;           // key rows per load pass of a wave
    constexpr int NP = kStreamTile / KPP;   // load passes per tile (V)
    constexpr int VST = D + 4;              // V tile row stride in elements (D*2 + 8 bytes)
    constexpr int PST = kStreamTile + 8;    // p tile row stride in elements (16-byte aligned rows)
    __shared__ __align__(16) uint16_t v_s[kStreamWaves][kStreamTile * VST];
    // the storage type keeps 8 (bf16) or 11 (fp16) bits of p, and over thousands of keys that rounding shows
    // in small outputs: a second tile holds the remainder p - T(p) and feeds a second product
    constexpr bool kSplitP = true;
    // fp16 has the bits but not the range: p of a far-away key is subnormal or zero in fp16 while
    // thousands of them still add up, so p is stored times 2^12 and the factor taken out at the end
    constexpr float kPScale = std::is_same<T, f16_t>::value ? 4096.f : 1.f;
    __shared__ __align__(16) uint16_t p_s[kStreamWaves][(kSplitP ? 2 : 1) * 16 * PST];
    __shared__ float m_s[kStreamWaves][G], l_s[kStreamWaves][G];
    __shared__ float o_s[kStreamWaves][G][D];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bhkv = blockIdx.x, split = blockIdx.y;
    const int b = bhkv / p.Hkv, hkv = bhkv % p.Hkv;
    const int head0 = hkv * G;
    const int active = p.d_active ? *p.d_active : p.active;
    const int bound = min(active, p.cache_len);
    const int k0 = split * p.slice, k1 = min(bound, k0 + p.slice);
    const size_t kv_base = PAGED ? 0 : (size_t)bhkv * p.cache_len;
    using TKV = typename std::conditional<KVI8, int8_t, T>::type;
    using Chunk = typename std::conditional<KVI8, uint2, U4>::type;  // 8 elements of a cached row
    const TKV *Kp = (const TKV *)p.k + kv_base * D, *Vp = (const TKV *)p.v + kv_base * D;
    const T *ksc = (const T *)p.k_scale + kv_base, *vsc = (const T *)p.v_scale + kv_base;  // KVI8 only
    // PAGED: pool row (in units of rows of one head) of row `r` of the tile starting at t0 = page's first row + r % P
    const int psh = p.page_shift, pmask = (1 << psh) - 1, pg0 = k0 >> psh;
    int pg_reg = 0;
    if constexpr (PAGED) {
        if (pg0 + lane < p.pages_per_seq) pg_reg = p.page_table[(size_t)b * p.pages_per_seq + pg0 + lane];
    }
    auto page_rows0 = [&](int t0) -> size_t {
        const int pg = __builtin_amdgcn_readlane(pg_reg, __builtin_amdgcn_readfirstlane((t0 >> psh) - pg0));
        return ((size_t)pg * p.Hkv + hkv) << psh;
    };
    auto operand = [](const Chunk &c) -> U4 {
        if constexpr (KVI8) return i8x8_to_operand<T>(c.x, c.y);
        else return c;
    };
    const int col = lane & 15, quad = lane >> 4;  // MFMA column (head) and row/k group of this lane

    // Q^T as the B operand of the score product: column = head, k = dims 8*quad..+7 of each block
    U4 qf[KB];
    {
        const T *qrow = (const T *)p.q + (size_t)b * p.q_bs + (size_t)(head0 + (col < G ? col : 0)) * p.q_hs;
#pragma unroll
        for (int j = 0; j < KB; j++) {
            qf[j] = *(const U4 *)(qrow + j * 32 + quad * 8);
            if (col >= G) qf[j] = U4{0u, 0u, 0u, 0u};
        }
    }

    // running state of head `col`: maximum, partial sum (the 4 quads hold parts), O^T accumulators
    // acc[c][par][e] = dim 32c + 2*(4*quad + e) + par
    float m_run = -INFINITY, l_run = 0.f;
    f4_t acc[KB][2];
#pragma unroll
    for (int c = 0; c < KB; c++)
#pragma unroll
        for (int par = 0; par < 2; par++) acc[c][par] = f4_t{0.f, 0.f, 0.f, 0.f};

    const int vk = lane / LPK, vd = (lane % LPK) * 8;  // V load: key row within a pass, dim offset
    // (KVI8: the scales of the lane's 2 x 4 score keys travel with the tile, 8 bytes per load; the cache
    // length is a multiple of 32 there, so a tile never reaches past its row of scales)
    auto load_tile = [&](int t0, Chunk (*kr)[KB], Chunk *vr, uint2 *sr) {
        size_t po = 0;
        if constexpr (PAGED) po = page_rows0(t0);
        auto at = [&](int row) -> size_t {
            if constexpr (PAGED) return po + (size_t)(row & pmask);
            else return (size_t)row;
        };
        if constexpr (KVI8) {
#pragma unroll
            for (int a = 0; a < 2; a++) {
                sr[a] = *(const uint2 *)(ksc + at(t0 + a * 16 + quad * 4));
                sr[2 + a] = *(const uint2 *)(vsc + at(t0 + a * 16 + quad * 4));
            }
        }
        // rows past the range re-read the last valid row; their scores are masked below
#pragma unroll
        for (int a = 0; a < 2; a++) {
            const int krow = min(t0 + a * 16 + col, k1 - 1);
#pragma unroll
            for (int j = 0; j < KB; j++) kr[a][j] = *(const Chunk *)(Kp + at(krow) * D + j * 32 + quad * 8);
        }
#pragma unroll
        for (int q = 0; q < NP; q++) {
            const int vrow = min(t0 + q * KPP + vk, k1 - 1);
            vr[q] = *(const Chunk *)(Vp + at(vrow) * D + vd);
        }
    };

    uint16_t *vt = v_s[wave], *pt = p_s[wave];
    auto scale_of = [](const uint2 &four, int e) -> float {  // element e of four packed storage-type values
        const uint32_t w = e < 2 ? four.x : four.y;
        const uint16_t b = (uint16_t)((e & 1) ? w >> 16 : w & 0xFFFFu);
        T v = __builtin_bit_cast(T, b);
        return Elem<T>::ld(&v, 0);
    };
    auto process = [&](int t, const Chunk (*kr)[KB], const Chunk *vr, const uint2 *sr) {
        // ---- park V: [key][dim], two 8-byte stores per lane and pass
#pragma unroll
        for (int q = 0; q < NP; q++) {
            uint2 *dst = (uint2 *)&vt[(q * KPP + vk) * VST + vd];
            const U4 v = operand(vr[q]);
            dst[0] = uint2{v.x, v.y};
            dst[1] = uint2{v.z, v.w};
        }
        // ---- scores: lane = head col, keys 16a + 4*quad + e
        float sv[2][4], tmax = -INFINITY;
#pragma unroll
        for (int a = 0; a < 2; a++) {
            f4_t s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < KB; j++) s4 = Mfma16<T>::run(operand(kr[a][j]), qf[j], s4);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int key = t + a * 16 + quad * 4 + e;
                float sc = s4[e];
                if constexpr (KVI8) sc *= scale_of(sr[a], e);
                sv[a][e] = key < k1 ? sc * p.scale : -INFINITY;
                tmax = fmaxf(tmax, sv[a][e]);
            }
        }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const float m_new = fmaxf(m_run, tmax);  // finite: the tile has at least one key in range
        const float alpha = fast_exp(m_run - m_new);
        m_run = m_new;
        float psum = 0.f;
#pragma unroll
        for (int a = 0; a < 2; a++) {
            float pe[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                pe[e] = fast_exp(sv[a][e] - m_new);  // 0 for keys past the range
                psum += pe[e];
                if constexpr (KVI8) pe[e] = t + a * 16 + quad * 4 + e < k1 ? pe[e] * scale_of(sr[2 + a], e) : 0.f;
            }
            // p[head][16a + 4*quad .. +3] in the storage type
            *(uint2 *)&pt[col * PST + a * 16 + quad * 4] =
                uint2{pack2<T>(pe[0] * kPScale, pe[1] * kPScale), pack2<T>(pe[2] * kPScale, pe[3] * kPScale)};
            if constexpr (kSplitP) {
                float lo[4];
#pragma unroll
                for (int e = 0; e < 4; e++) lo[e] = pe[e] * kPScale - Elem<T>::rnd(pe[e] * kPScale);
                *(uint2 *)&pt[16 * PST + col * PST + a * 16 + quad * 4] = uint2{pack2<T>(lo[0], lo[1]), pack2<T>(lo[2], lo[3])};
            }
        }
        l_run = l_run * alpha + psum;
        if (alpha != 1.f) {
#pragma unroll
            for (int c = 0; c < KB; c++)
#pragma unroll
                for (int par = 0; par < 2; par++) acc[c][par] *= alpha;
        }
        __builtin_amdgcn_wave_barrier();
        // ---- O^T += V^T . P: B operand = p[head col][keys 8*quad..+7]; A operands from V dword pairs
        const U4 pf = *(const U4 *)&pt[col * PST + quad * 8];
        U4 pl = U4{0u, 0u, 0u, 0u};
        if constexpr (kSplitP) pl = *(const U4 *)&pt[16 * PST + col * PST + quad * 8];
#pragma unroll
        for (int c = 0; c < KB; c++) {
            uint32_t w[8];
#pragma unroll
            for (int i = 0; i < 8; i++) w[i] = *(const uint32_t *)&vt[(quad * 8 + i) * VST + c * 32 + col * 2];
            U4 ev, od;  // keys 8*quad..+7 at dim 32c + 2*col and at the next dim
            ev.x = __builtin_amdgcn_perm(w[1], w[0], 0x05040100u); od.x = __builtin_amdgcn_perm(w[1], w[0], 0x07060302u);
            ev.y = __builtin_amdgcn_perm(w[3], w[2], 0x05040100u); od.y = __builtin_amdgcn_perm(w[3], w[2], 0x07060302u);
            ev.z = __builtin_amdgcn_perm(w[5], w[4], 0x05040100u); od.z = __builtin_amdgcn_perm(w[5], w[4], 0x07060302u);
            ev.w = __builtin_amdgcn_perm(w[7], w[6], 0x05040100u); od.w = __builtin_amdgcn_perm(w[7], w[6], 0x07060302u);
            acc[c][0] = Mfma16<T>::run(ev, pf, acc[c][0]);
            acc[c][1] = Mfma16<T>::run(od, pf, acc[c][1]);
            if constexpr (kSplitP) {
                acc[c][0] = Mfma16<T>::run(ev, pl, acc[c][0]);
                acc[c][1] = Mfma16<T>::run(od, pl, acc[c][1]);
            }
        }
        __builtin_amdgcn_wave_barrier();
    };

    // two register sets, named so that the wait for one never covers the other; the load of the next tile
    // is issued unconditionally (after the last tile: that tile once more) to keep the loop free of branches
    // around loads
    Chunk kA[2][KB], vA[NP], kB[2][KB], vB[NP];
    uint2 sA[4], sB[4];
    const int tstep = kStreamWaves * kStreamTile;
    // The wave's tiles are k0 + 32 wave + 128 n, n < nt.  The workgroups of different sequences start their walk at
    // different n and wrap around, the kv heads of one sequence stay in step.  Measured over the batch-32 decode step
    // at context 2048 with a paged cache (pages of 256 rows, a sequence's heads 64 KB apart inside a page): every
    // workgroup from n = 0: 53 us per launch; starts one tile apart per sequence: 49 us; one tile apart per
    // workgroup (heads out of step as well): 60 us; a contiguous cache is indifferent to all three (50 us).  The
    // order of the tiles changes nothing but the rounding of the online softmax, and it is a fixed function of the
    // grid.
    const int nt = (k1 - k0 - wave * kStreamTile + tstep - 1) / tstep;
    if (nt > 0) {
        const int rot = (int)((unsigned)(b + split) % (unsigned)nt);
        auto tile_at = [&](int n) {
            n = min(n, nt - 1) + rot;
            if (n >= nt) n -= nt;
            return k0 + wave * kStreamTile + n * tstep;
        };
        int n = 0;
        load_tile(tile_at(0), kA, vA, sA);
        while (true) {
            load_tile(tile_at(n + 1), kB, vB, sB);
            process(tile_at(n), kA, vA, sA);
            if (++n >= nt) break;
            load_tile(tile_at(n + 1), kA, vA, sA);
            process(tile_at(n), kB, vB, sB);
            if (++n >= nt) break;
        }
    }

    // ---- this wave's results to LDS: l over the 4 quads of a head; lane (head col, quad) holds the
    // dims 32c + 2*(4*quad + e) + par of O^T
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
    if (lane < G) {
        m_s[wave][lane] = m_run;
        l_s[wave][lane] = l_run;
    }
    if (col < G) {
#pragma unroll
        for (int c = 0; c < KB; c++)
#pragma unroll
            for (int par = 0; par < 2; par++)
#pragma unroll
                for (int e = 0; e < 4; e++) o_s[wave][col][c * 32 + 2 * (4 * quad + e) + par] = acc[c][par][e] * (1.0f / kPScale);
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
bool attn_stream_eligible(int B, int Sq, int Hq, int Hkv, int D, int dtype, int kv_int8, int kv_len, int cache_len) {
    const int G = Hq / Hkv;
    return Sq == 1 && dtype != MYNN_F32 && (!kv_int8 || cache_len % kStreamTile == 0) && (D == 64 || D == 128) &&
           (G == 1 || G == 2 || G == 4 || G == 8) && cache_len >= kStreamTile && (long)B * Hkv * kv_len >= kStreamMinKeys;
}

// key rows per workgroup and number of key ranges: ONE workgroup per CU (its four waves keep eight tiles in flight,
// which is enough to stream; measured over batch x kv-head counts of 8 .. 384 and contexts of 512 .. 8192, two to
// four workgroups per CU -- what the register count allows -- were 0-25 % slower: shorter sequential runs, more partial
// results to write and to merge, and with at least one (sequence, kv head) per CU the merge launch disappears
// altogether); ranges a multiple of the 128 keys a workgroup takes per step
static int stream_slots() {
    static int slots = 0;
    if (!slots) {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
            (void)hipGetLastError();
            cus = 256;
        }
        slots = cus;
    }
    return slots;
}
void attn_stream_plan(int B, int Hkv, int kv_len, int *slice, int *nsplit) {
    const int step = kStreamWaves * kStreamTile;
    int n = stream_slots() / (B * Hkv);
    const int nmax = (kv_len + 127) / 128;
    if (n > nmax) n = nmax;
    if (n < 1) n = 1;
    int rows = ((kv_len + n - 1) / n + step - 1) / step * step;
    *slice = rows;
    *nsplit = (kv_len + rows - 1) / rows;
}
// The number of key ranges is not monotonic in the length (a longer cache can round to fewer, longer ranges), so a
// workspace is sized for the most ranges ANY length up to kv_len_max can be planned with.
int attn_stream_max_ranges(int B, int Hkv, int kv_len_max) {
    int n = stream_slots() / (B * Hkv);
    const int nmax = (kv_len_max + 127) / 128;
    if (n > nmax) n = nmax;
    return n < 1 ? 1 : n;
}
// Paged caches: the pages of a key range travel in one vector register, a lane each, so a range spans at most 62
// pages (one more at either end for ranges that start inside a page); longer ranges are cut into more of them.
static int paged_slice_cap(int page_shift) {
    const int step = kStreamWaves * kStreamTile;
    return ((62 << page_shift) / step) * step;
}
void attn_stream_plan_paged(int B, int Hkv, int kv_len, int page_shift, int *slice, int *nsplit) {
    attn_stream_plan(B, Hkv, kv_len, slice, nsplit);
    const int cap = paged_slice_cap(page_shift);
    if (*slice > cap) {
        *slice = cap;
        *nsplit = (kv_len + cap - 1) / cap;
    }
}
int attn_stream_max_ranges_paged(int B, int Hkv, int kv_len_max, int page_shift) {
    const int a = attn_stream_max_ranges(B, Hkv, kv_len_max), cap = paged_slice_cap(page_shift);
    const int b = (kv_len_max + cap - 1) / cap;
    return a > b ? a : b;
}
// the conditions of attn_stream_eligible that do not depend on the length of one call
bool attn_stream_possible(int B, int Sq, int Hq, int Hkv, int D, int dtype, int cache_len) {
    const int G = Hq / Hkv;
    return Sq == 1 && dtype != MYNN_F32 && (D == 64 || D == 128) && (G == 1 || G == 2 || G == 4 || G == 8) &&
           cache_len >= kStreamTile && (long)B * Hkv * cache_len >= kStreamMinKeys;
}

template <typename T, int D, bool KVI8, bool PAGED>
static int stream_g(const AttnParams &p, hipStream_t s) {
    dim3 grid(p.B * p.Hkv, p.nsplit), block(kStreamThreads);
    switch (p.Hq / p.Hkv) {
    case 1: MYNN_LAUNCH((attn_stream_kernel<T, D, 1, KVI8, PAGED>), grid, block, 0, s, p); break;
    case 2: MYNN_LAUNCH((attn_stream_kernel<T, D, 2, KVI8, PAGED>), grid, block, 0, s, p); break;
    case 4: MYNN_LAUNCH((attn_stream_kernel<T, D, 4, KVI8, PAGED>), grid, block, 0, s, p); break;
    case 8: MYNN_LAUNCH((attn_stream_kernel<T, D, 8, KVI8, PAGED>), grid, block, 0, s, p); break;
    default: return fail(MYNN_ERR_UNSUPPORTED, "streaming attention: %d query heads per kv head", p.Hq / p.Hkv);
    }
    return launch_status("attn_stream_kernel");
}

template <typename T, int D>
static int stream_kv(const AttnParams &p, int kv_int8, hipStream_t s) {
    if (p.page_table) return kv_int8 ? stream_g<T, D, true, true>(p, s) : stream_g<T, D, false, true>(p, s);
    return kv_int8 ? stream_g<T, D, true, false>(p, s) : stream_g<T, D, false, false>(p, s);
}

// what the paged form needs whatever the sizes: one query row, a 16-bit type, head_dim 64 or 128, 1/2/4/8 query heads
// per kv head, pages of a power of two >= 32 rows
bool attn_stream_paged_supported(int Sq, int Hq, int Hkv, int D, int dtype, int page_rows) {
    const int G = Hkv > 0 ? Hq / Hkv : 0;
    return Sq == 1 && (dtype == MYNN_F16 || dtype == MYNN_BF16) && (D == 64 || D == 128) && (G == 1 || G == 2 || G == 4 || G == 8) &&
           page_rows >= kStreamTile && (page_rows & (page_rows - 1)) == 0;
}

int attention_stream_launch(const AttnParams &p, int D, int dtype, int kv_int8, hipStream_t s) {
    MYNN_REQUIRE(!kv_int8 || (p.k_scale && p.v_scale && p.cache_len % kStreamTile == 0), MYNN_ERR_INVALID,
                 "streaming attention: int8 KV needs scales and a cache length that is a multiple of %d", kStreamTile);
    MYNN_REQUIRE(p.q_rs >= 0 && aligned16(p.q) && aligned16(p.k) && aligned16(p.v) && p.q_bs % 8 == 0 && p.q_hs % 8 == 0,
                 MYNN_ERR_INVALID, "streaming attention: q, k, v must be 16-byte aligned");
    MYNN_REQUIRE(p.nsplit == 1 || (p.part_o && p.part_ml), MYNN_ERR_INVALID,
                 "streaming attention: no scratch for %d key ranges", p.nsplit);
    MYNN_REQUIRE(p.slice % (kStreamWaves * kStreamTile) == 0 && p.nsplit <= 65535, MYNN_ERR_INVALID,
                 "streaming attention: slice %d, %d ranges", p.slice, p.nsplit);
    if (p.page_table) {
        MYNN_REQUIRE(attn_stream_paged_supported(p.Sq, p.Hq, p.Hkv, D, dtype, 1 << p.page_shift), MYNN_ERR_UNSUPPORTED,
                     "paged attention: one query row, 16-bit type, head_dim 64/128, 1/2/4/8 heads per kv head, pages of 2^n >= %d rows",
                     kStreamTile);
        MYNN_REQUIRE(p.cache_len == p.pages_per_seq << p.page_shift, MYNN_ERR_INVALID,
                     "paged attention: cache length %d is not %d pages of %d rows", p.cache_len, p.pages_per_seq, 1 << p.page_shift);
        // a key range's pages travel in one register, a lane each
        MYNN_REQUIRE((p.slice >> p.page_shift) + 2 <= 64, MYNN_ERR_UNSUPPORTED,
                     "paged attention: a key range of %d rows spans more than 62 pages of %d rows", p.slice, 1 << p.page_shift);
    }
    int rc;
    if (dtype == MYNN_F16) rc = D == 64 ? stream_kv<f16_t, 64>(p, kv_int8, s) : stream_kv<f16_t, 128>(p, kv_int8, s);
    else rc = D == 64 ? stream_kv<bf16_t, 64>(p, kv_int8, s) : stream_kv<bf16_t, 128>(p, kv_int8, s);
    if (rc || p.nsplit == 1) return rc;
    return attention_merge_launch(p, D, dtype, s);
}

}  // namespace mynn
