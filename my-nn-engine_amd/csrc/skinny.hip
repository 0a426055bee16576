// DequantMatMul for a few dozen activation rows (16 <= M <= 64: batched decode, short prefill
// chunks): the int8 weight matrix is still the whole cost, so it is streamed ONCE, as int8, and turned
// into matrix-core operands in registers -- unlike the large-M path, which multiplies by a 16-bit
// copy of the weights (twice the bytes) in 256-row tiles that M rows would leave mostly empty.
//
//   out[m,n] = T(scale[n] * sum_k act[m,k] * wq[n,k])   (scale after the f32 sum, as the reference's
//   small-M kernels: dequant_gemv.cuh:12-59, dequant_matmul.cuh:12-51; int8 -> 16-bit is exact)
//
// A wave owns 32 weight rows (the A operand of v_mfma_f32_32x32x16, rows n) against up to two tiles of
// 32 activation rows (B operand, columns m).  The reduction index of an MFMA is free to permute as long
// as both operands agree, so a lane takes 64 CONTIGUOUS bytes of its weight row per step of 128 k
// (a full 128-byte line per row and step across the two lane halves) and the matching activation
// elements (staged through LDS once per workgroup and step).  Two steps' loads are in flight per wave behind the
// one in use; when the matrix has too few rows to fill the device the K range is split over gridDim.y.  Partial sums [ksplit][M][N] (f32) are summed,
// scaled and stored by a second launch that also applies the residual or SwiGLU.
#include <type_traits>

#include "kernels.h"
#include "mfma.h"

namespace mynn {

// (stages: two steps of loads in flight behind the one in use.  Measured over a batch-32 decode step of the 8B shape: 3
// stages 4.18 ms, 4 stages 4.20, 5 stages 4.24-4.26, 6 and 7 stages 4.27-4.31, 2 stages 4.59 -- the weight stream alone,
// taken out of the kernel, also runs faster with fewer requests outstanding: 21.4 us at 3 stages, 22.8 at 5, 24.4 at 8)
constexpr int kSkinnyWaves = 4, kSkinnyThreads = kSkinnyWaves * 64, kSkinnyK = 128, kSkinnyStages = 3;

constexpr int kSkinnyLd = kSkinnyK + 8;  // LDS row stride of the activation chunk (272 bytes: conflict-free 128-bit reads)

// PACKED: wq is the tiled copy made by skinny_pack_kernel -- for every (32 rows, 128 k) tile the 4 KB a
// wave needs, in the order its four load instructions want them (instruction j, lane l -> 16 bytes at
// j*1024 + l*16) instead of 128-byte pieces of 32 rows a row pitch apart (measured 2.3 TB/s for the row-major
// form: DRAM pages are opened for 128 bytes each).  Tiles are ordered K STEP FIRST, [step][row block]: the waves
// of a launch walk their K ranges in step, so what is in flight at any moment is one contiguous stretch of the
// copy (the row blocks of a few consecutive steps) and the launch as a whole sweeps it front to back -- the access
// pattern of the batch-1 GEMV, which streams at 7 TB/s -- and not some 900 separate streams 128 KB apart.
// FEPI < 0: partial sums to `part` (several K ranges, summed by skinny_reduce_kernel).  FEPI = GEMM_*: the
// workgroup covers the whole K range and stores the finished output itself (scale, residual or SwiGLU).
// ABL (measurement aid, mynn_skinny_set_ablation): 1 = the loads alone -- no LDS, no conversion, no MFMA, no barrier; the
// loaded words are folded into the accumulator so that they stay; 2 = everything but the MFMAs.  Results are garbage.
template <typename T, int MT, bool PACKED, int FEPI, int ABL = 0>
__global__ __launch_bounds__(kSkinnyThreads) void skinny_gemm_kernel(float *part, const T *act, const int8_t *wq, int M,
                                                                    int N, int K, int iters_per_split, T *out,
                                                                    const T *scale, const T *res) {
    // the activation chunk [32*MT rows][128 k] of the current step, shared by the four waves
    __shared__ __align__(16) uint16_t a_s[2][MT * 32 * kSkinnyLd];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int n0 = (blockIdx.x * kSkinnyWaves + wave) * 32;
    const int iters = K / kSkinnyK;
    const int it0 = blockIdx.y * iters_per_split, it1 = min(it0 + iters_per_split, iters);
    if (it0 >= it1) return;  // whole workgroup
    // waves past N recompute the last rows (row-major) or read the zero-padded last tile (packed), store nothing
    const size_t step_pitch = (size_t)((N + 31) / 32) * 4096;  // PACKED: bytes of one K step over all row blocks
    const int8_t *wrow = PACKED ? wq + (size_t)min(n0 / 32, (N - 1) / 32) * 4096 + lane * 16
                                : wq + (size_t)min(n0 + r, N - 1) * K + 64 * h;

    f16x_t acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[mt][e] = 0.f;

    // cooperative activation load: 16 lanes per row (256 contiguous bytes), 16 rows per pass of the workgroup
    constexpr int AP = MT * 2;
    const int arow = tid >> 4, acol = (tid & 15) * 8;
    const T *ap[AP];
#pragma unroll
    for (int q = 0; q < AP; q++) ap[q] = act + (size_t)min(arow + 16 * q, M - 1) * K + acol;
    // one step's loads: 64 bytes of this lane's weight row and this thread's share of the activation
    // chunk.  kSkinnyStages - 1 steps are in flight at any time; everything is consumed in the order it was
    // issued, so the counter wait for one step never drains a younger one.  Steps past the range re-read
    // the last one (unused).
    struct Stage {
        U4 w[4], a[AP];
    };
    // Workgroups walk their K range from different starting steps: all rows of the matrix are a multiple of
    // 128 bytes apart, so in lockstep every request in flight would carry the same low address bits and
    // land on the same few memory channels.
    // (the packed copy is read in step by every workgroup on purpose: see PACKED above)
    const int len = it1 - it0, rot = PACKED ? 0 : (int)((blockIdx.x * 7u + blockIdx.y * 3u) % (unsigned)len);
    auto load = [&](int it, Stage &st) {
        int step = min(it, it1 - 1) - it0 + rot;
        if (step >= len) step -= len;
        const size_t k = (size_t)(it0 + step) * kSkinnyK;
        const U4 *src = (const U4 *)(wrow + (PACKED ? (size_t)(it0 + step) * step_pitch : k));
        // the activation share FIRST: loads return in order, and the chunk of step it+1 is wanted (for LDS) one step
        // before that step's weights are -- asked for behind them, the wait for it would drain the weight loads too
        // and leave a single step in flight
#pragma unroll
        for (int q = 0; q < AP; q++) st.a[q] = *(const U4 *)(ap[q] + k);
#pragma unroll
        for (int j = 0; j < 4; j++) st.w[j] = __builtin_nontemporal_load(src + (PACKED ? j * 64 : j));
    };
    auto store_act = [&](int buf, const Stage &st) {
#pragma unroll
        for (int q = 0; q < AP; q++) *(U4 *)&a_s[buf][(arow + 16 * q) * kSkinnyLd + acol] = st.a[q];
    };
    auto compute = [&](int buf, const Stage &st) {
        // all activation operands of the step first (one LDS latency for the step, not one in front of every MFMA;
        // the scheduling barrier keeps the compiler from sinking each read back to its use)
        U4 b[MT][8];
#pragma unroll
        for (int s = 0; s < 8; s++)
#pragma unroll
            for (int mt = 0; mt < MT; mt++) b[mt][s] = *(const U4 *)&a_s[buf][(mt * 32 + r) * kSkinnyLd + 64 * h + 8 * s];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const U4 &q = st.w[s >> 1];
            const U4 a = (s & 1) ? i8x8_to_operand<T>(q.z, q.w) : i8x8_to_operand<T>(q.x, q.y);
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                if constexpr (ABL == 2)
                    acc[mt][s] += __builtin_bit_cast(float, (a.x ^ b[mt][s].x ^ a.y ^ b[mt][s].y ^ a.z ^ b[mt][s].z ^ a.w ^ b[mt][s].w) & 0x3fffffffu);
                else
                    acc[mt] = Mfma<T>::run(a, b[mt][s], acc[mt]);
            }
        }
    };

    constexpr int S = kSkinnyStages;
    Stage st[S];
    int it = it0;
#pragma unroll
    for (int j = 0; j < S - 1; j++) load(it + j, st[j]);
    store_act(0, st[0]);
    __syncthreads();
    int buf = 0;
    auto step = [&](Stage &cur, Stage &next, Stage &refill) {
        load(it + S - 1, refill);
        if constexpr (ABL == 1) {
            uint32_t x = 0;
#pragma unroll
            for (int j = 0; j < 4; j++) x ^= cur.w[j].x ^ cur.w[j].y ^ cur.w[j].z ^ cur.w[j].w;
#pragma unroll
            for (int q = 0; q < AP; q++) x ^= cur.a[q].x;
            acc[0][0] += __builtin_bit_cast(float, x & 0x3fffffffu);
        } else {
            compute(buf, cur);
            store_act(buf ^ 1, next);  // the chunk of step it+1 for the other buffer
            __syncthreads();
        }
        buf ^= 1;
        ++it;
    };
    // Whole groups of S steps in a loop body without branches: every stage index is a constant and the loads that are
    // still in flight at the loop's end sit in the registers they sit in at its start, so the waits inside the body
    // are counted waits.  (With an exit test after every step the compiler could not count across the back edge and
    // drained every load once per group: the stream restarted from empty every S steps.)
    while (it + S <= it1) {
#pragma unroll
        for (int j = 0; j < S; j++) step(st[j], st[(j + 1) % S], st[(j + S - 1) % S]);
    }
    // the remaining steps (fewer than S); the stage indices continue from 0
    const int rest = it1 - it;
#pragma unroll
    for (int j = 0; j < S - 1; j++)
        if (j < rest) step(st[j], st[(j + 1) % S], st[(j + S - 1) % S]);

    // D[n][m]: lane holds column m = lane%32 and rows n = 8*(e/4) + 4*(lane/32) + e%4: four consecutive n
    if (n0 >= N) return;
    if constexpr (FEPI >= 0) {
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            const int m = mt * 32 + r;
            if (m >= M) continue;
#pragma unroll
            for (int e4 = 0; e4 < 4; e4++) {
                const int n = n0 + e4 * 8 + h * 4;
                float y[4];
#pragma unroll
                for (int x = 0; x < 4; x++) y[x] = n + x < N ? acc[mt][e4 * 4 + x] * Elem<T>::ld(scale, n + x) : 0.f;
                if constexpr (FEPI == GEMM_SWIGLU) {
                    // rows 2i / 2i+1 of the weight are gate_i / up_i; out is [M, N/2]
                    T *o = out + (size_t)m * (N >> 1) + (n >> 1);
#pragma unroll
                    for (int x = 0; x < 2; x++) {
                        if (n + 2 * x + 1 < N) {
                            const float g = Elem<T>::rnd(y[2 * x]), u = Elem<T>::rnd(y[2 * x + 1]);
                            const float sig = 1.0f / (1.0f + expf(-g));
                            Elem<T>::st(o, x, (g * sig) * u);
                        }
                    }
                } else {
                    const size_t at = (size_t)m * N + n;
#pragma unroll
                    for (int x = 0; x < 4; x++)
                        if (n + x < N) Elem<T>::st(out, at + x, y[x]);
                }
            }
        }
        return;
    }
    float *dst = part + (size_t)blockIdx.y * M * N;
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
        const int m = mt * 32 + r;
        if (m >= M) continue;
#pragma unroll
        for (int e4 = 0; e4 < 4; e4++) {
            const int n = n0 + e4 * 8 + h * 4;
            float *p = dst + (size_t)m * N + n;
            if (n + 4 <= N && (N & 3) == 0) {
                *(float4 *)p = float4{acc[mt][e4 * 4], acc[mt][e4 * 4 + 1], acc[mt][e4 * 4 + 2], acc[mt][e4 * 4 + 3]};
            } else {
                for (int x = 0; x < 4 && n + x < N; x++) p[x] = acc[mt][e4 * 4 + x];
            }
        }
    }
}

// tile[(it * row_blocks + nb)][j][l] (16 bytes) = W[nb*32 + l%32][it*128 + 64*(l/32) + 16*j ..]; rows past N are zero
__global__ __launch_bounds__(256) void skinny_pack_kernel(U4 *dst, const int8_t *wq, int N, int K, size_t chunks) {
    const size_t c = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (c >= chunks) return;
    const int l = (int)(c & 63), j = (int)((c >> 6) & 3);
    const size_t tile = c >> 8, row_blocks = (size_t)(N + 31) / 32;
    const int it = (int)(tile / row_blocks);
    const size_t row = (tile % row_blocks) * 32 + (l & 31);
    U4 v = U4{0u, 0u, 0u, 0u};
    if (row < (size_t)N) v = *(const U4 *)(wq + row * K + (size_t)it * kSkinnyK + 64 * (l >> 5) + 16 * j);
    dst[c] = v;
}

size_t skinny_packed_bytes(int N, int K) { return (size_t)((N + 31) / 32) * 32 * K; }
int skinny_pack_weight(void *dst, const int8_t *wq, int N, int K, hipStream_t s) {
    MYNN_REQUIRE(dst && wq && K % kSkinnyK == 0 && aligned16(wq) && aligned16(dst), MYNN_ERR_INVALID, "skinny pack: N=%d K=%d", N, K);
    const size_t chunks = skinny_packed_bytes(N, K) / 16;
    MYNN_LAUNCH(skinny_pack_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, s, (U4 *)dst, wq, N, K, chunks);
    return launch_status("skinny_pack_kernel");
}

// sum of the K ranges, scale, store (with the residual or SwiGLU when asked); SWIGLU: rows of the weight
// were gate/up interleaved (row 2i gate_i, 2i+1 up_i) and out is [M, N/2]
template <typename T, int EPI>
__global__ __launch_bounds__(256) void skinny_reduce_kernel(T *out, const float *part, const T *scale, const T *res, int M,
                                                          int N, int ksplit) {
    const int n_out = EPI == GEMM_SWIGLU ? N / 2 : N;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)M * n_out) return;
    const int m = (int)(idx / n_out), c = (int)(idx % n_out);
    auto total = [&](int n) {
        float t = 0.f;
        for (int s = 0; s < ksplit; s++) t += part[((size_t)s * M + m) * N + n];
        return t;
    };
    if (EPI == GEMM_SWIGLU) {
        const float g = Elem<T>::rnd(total(2 * c) * Elem<T>::ld(scale, 2 * c));
        const float u = Elem<T>::rnd(total(2 * c + 1) * Elem<T>::ld(scale, 2 * c + 1));
        const float sig = 1.0f / (1.0f + expf(-g));
        Elem<T>::st(out, idx, (g * sig) * u);
    } else {
        float y = total(c) * Elem<T>::ld(scale, c);
        if (EPI == GEMM_RESIDUAL) y = Elem<T>::rnd(y) + Elem<T>::ld(res, idx);
        Elem<T>::st(out, idx, y);
    }
}

// The residual form of the reduction followed by the RMSNorm of the row it completes (the o projection before
// the MLP's norm, the down projection before the next layer's): one workgroup per output row, four columns per
// thread, every load issued before the first sum; x_out = T(T(sum * scale) + res), nrm_out = T((x * inv) * w)
// with inv = 1 / sqrt(mean(x^2) + eps) over the stored (rounded) x, as the separate operators compute them.
constexpr int kReduceNormThreads = 1024, kReduceNormMaxSplit = 8;
template <typename T>
__global__ __launch_bounds__(kReduceNormThreads) void skinny_reduce_norm_kernel(T *x_out, T *nrm_out, const float *part, const T *scale,
                                                                              const T *res, const T *norm_w, int M, int N, int ksplit,
                                                                              float eps) {
    __shared__ float red[kReduceNormThreads / 64];
    const int m = blockIdx.x, c0 = threadIdx.x * 4;
    const bool live = c0 < N;
    float4 pv[kReduceNormMaxSplit];
    uint2 sc2 = uint2{0u, 0u}, rs2 = sc2, nw2 = sc2;
#pragma unroll
    for (int s = 0; s < kReduceNormMaxSplit; s++) {
        pv[s] = float4{0.f, 0.f, 0.f, 0.f};
        if (live && s < ksplit) pv[s] = *(const float4 *)(part + ((size_t)s * M + m) * N + c0);
    }
    if (live) {
        sc2 = *(const uint2 *)(scale + c0);
        rs2 = *(const uint2 *)(res + (size_t)m * N + c0);
        nw2 = *(const uint2 *)(norm_w + c0);
    }
    float t[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < kReduceNormMaxSplit; s++) {  // the order of skinny_reduce_kernel: K ranges ascending
        if (s < ksplit) {
            t[0] += pv[s].x; t[1] += pv[s].y; t[2] += pv[s].z; t[3] += pv[s].w;
        }
    }
    float sc[8], rs[8], nw[8], x[4];
    widen8<T>(U4{sc2.x, sc2.y, 0u, 0u}, sc);
    widen8<T>(U4{rs2.x, rs2.y, 0u, 0u}, rs);
    widen8<T>(U4{nw2.x, nw2.y, 0u, 0u}, nw);
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        x[i] = Elem<T>::rnd(Elem<T>::rnd(t[i] * sc[i]) + rs[i]);
        ss += x[i] * x[i];
    }
    if (live) *(uint2 *)(x_out + (size_t)m * N + c0) = uint2{pack2<T>(x[0], x[1]), pack2<T>(x[2], x[3])};
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    float tot = 0.f;
#pragma unroll
    for (int w = 0; w < kReduceNormThreads / 64; w++) tot += red[w];
    const float inv = 1.0f / sqrtf(tot / (float)N + eps);
    if (live)
        *(uint2 *)(nrm_out + (size_t)m * N + c0) =
            uint2{pack2<T>((x[0] * inv) * nw[0], (x[1] * inv) * nw[1]), pack2<T>((x[2] * inv) * nw[2], (x[3] * inv) * nw[3])};
}

// The plain form of the reduction for a q|k|v projection, followed by what rope_kv_append_vec_kernel does with
// the stored projection: a thread per (head, 4 rotation pairs) or 4 values of v, a token row's threads spread over
// several two-wave workgroups;
// qkv values are rounded to the storage type before the rotation, exactly as if they had been stored.
// KV8: the caches are int8 with one scale per token row (rope_quant_kv_append_kernel's arithmetic: k after RoPE rounded
// to T, v as stored; s = amax / 127 stored as T, q = trunc(x * 127 / amax +- 0.5) clamped to [-128, 127]); every head
// then takes D/8 threads (4 low + 4 high elements each), an aligned lane group, and the row maximum is a DPP reduction.
constexpr int kReduceRopeThreads = 128;  // two waves: a row's units spread over ~7 workgroups, ~220 workgroups per launch
template <typename T, bool KV8>
__global__ __launch_bounds__(kReduceRopeThreads) void skinny_reduce_rope_kernel(const float *part, const T *scale, int M, int N, int ksplit,
                                                                              T *q_out, void *k_cache_v, void *v_cache_v, T *k_scale,
                                                                              T *v_scale, const T *cos_t, const T *sin_t,
                                                                              const int64_t *position, const int32_t *d_past, int S, int Hq,
                                                                              int Hkv, int D, int max_seq, KvPaging pg) {
    const int m = blockIdx.x, b = m / S, sq = m % S;
    const int half = D / 2, upr = half / 4, upv = KV8 ? upr : D / 4;  // units per rotated head / per v head
    const int rot_units = (Hq + Hkv) * upr, units = rot_units + Hkv * upv;
    const int past = *d_past;
    const size_t tab = (size_t)position[sq] * D;
    auto total4 = [&](int col, float *t) {
        float4 pv[kReduceNormMaxSplit];
#pragma unroll
        for (int s = 0; s < kReduceNormMaxSplit; s++) {
            pv[s] = float4{0.f, 0.f, 0.f, 0.f};
            if (s < ksplit) pv[s] = *(const float4 *)(part + ((size_t)s * M + m) * N + col);
        }
        const uint2 sc2 = *(const uint2 *)(scale + col);
        float sc[8];
        widen8<T>(U4{sc2.x, sc2.y, 0u, 0u}, sc);
        t[0] = t[1] = t[2] = t[3] = 0.f;
#pragma unroll
        for (int s = 0; s < kReduceNormMaxSplit; s++)
            if (s < ksplit) {
                t[0] += pv[s].x; t[1] += pv[s].y; t[2] += pv[s].z; t[3] += pv[s].w;
            }
#pragma unroll
        for (int i = 0; i < 4; i++) t[i] = Elem<T>::rnd(t[i] * sc[i]);
    };
    auto ld4 = [&](const T *p, float *f) {
        const uint2 v = *(const uint2 *)p;
        float w[8];
        widen8<T>(U4{v.x, v.y, 0u, 0u}, w);
#pragma unroll
        for (int i = 0; i < 4; i++) f[i] = w[i];
    };
    // KV8: the lane group's 8 x (D/8) values -> codes and the row's scale
    auto quantise_store = [&](const float *lo, const float *hi, int8_t *cache, T *srow, size_t tok, int j) {
        float amax = 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) amax = fmaxf(amax, fmaxf(fabsf(lo[i]), fabsf(hi[i])));
        amax = D == 128 ? group_max<16>(amax) : group_max<8>(amax);
        const float inv = amax == 0.f ? 0.f : 127.0f / amax;
        if (j == 0) Elem<T>::st(srow, tok, amax * (1.0f / 127.0f));
        auto code = [&](float x) -> uint32_t {
            const float a = x * inv;
            int q = (int)(a + (a >= 0.f ? 0.5f : -0.5f));
            q = q < -128 ? -128 : (q > 127 ? 127 : q);
            return (uint32_t)(q & 0xFF);
        };
        int8_t *dst = cache + tok * D;
        *(uint32_t *)(dst + j) = code(lo[0]) | (code(lo[1]) << 8) | (code(lo[2]) << 16) | (code(lo[3]) << 24);
        *(uint32_t *)(dst + j + half) = code(hi[0]) | (code(hi[1]) << 8) | (code(hi[2]) << 16) | (code(hi[3]) << 24);
    };
    // one unit per thread, a row's units over gridDim.y workgroups (as one workgroup per row, which pulled the row's
    // 150 KB of partial sums through a single CU, the launch took 5.7 us at batch 32; 4.7 us spread over the device)
    const int u = blockIdx.y * kReduceRopeThreads + threadIdx.x;
    if (u >= units) return;
    {
        if (u >= rot_units) {
            if constexpr (KV8) {
                const int hv = (u - rot_units) / upr, j = ((u - rot_units) % upr) * 4;
                float lo[4], hi[4];
                total4((Hq + Hkv + hv) * D + j, lo);
                total4((Hq + Hkv + hv) * D + j + half, hi);
                quantise_store(lo, hi, (int8_t *)v_cache_v, v_scale, kv_cache_row(pg, b, hv, past + sq, Hkv, max_seq), j);
            } else {
                const int hv = (u - rot_units) / upv, j = ((u - rot_units) % upv) * 4;
                float t[4];
                total4((Hq + Hkv + hv) * D + j, t);
                T *dst = (T *)v_cache_v + kv_cache_row(pg, b, hv, past + sq, Hkv, max_seq) * D + j;
                *(uint2 *)dst = uint2{pack2<T>(t[0], t[1]), pack2<T>(t[2], t[3])};
            }
            return;
        }
        const int head = u / upr, j = (u % upr) * 4;
        float xl[4], xh[4], cl[4], ch[4], sl[4], sh[4];
        total4(head * D + j, xl);
        total4(head * D + j + half, xh);
        ld4(cos_t + tab + j, cl);
        ld4(cos_t + tab + j + half, ch);
        ld4(sin_t + tab + j, sl);
        ld4(sin_t + tab + j + half, sh);
        float ol[4], oh[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            ol[i] = xl[i] * cl[i] - xh[i] * sl[i];
            oh[i] = xh[i] * ch[i] + xl[i] * sh[i];
        }
        if constexpr (KV8) {
            if (head >= Hq) {
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    ol[i] = Elem<T>::rnd(ol[i]);
                    oh[i] = Elem<T>::rnd(oh[i]);
                }
                quantise_store(ol, oh, (int8_t *)k_cache_v, k_scale, kv_cache_row(pg, b, head - Hq, past + sq, Hkv, max_seq), j);
                return;
            }
        }
        T *dst = head < Hq ? q_out + (size_t)m * Hq * D + (size_t)head * D
                           : (T *)k_cache_v + kv_cache_row(pg, b, head - Hq, past + sq, Hkv, max_seq) * D;
        *(uint2 *)(dst + j) = uint2{pack2<T>(ol[0], ol[1]), pack2<T>(ol[2], ol[3])};
        *(uint2 *)(dst + j + half) = uint2{pack2<T>(oh[0], oh[1]), pack2<T>(oh[2], oh[3])};
    }
}

// 0 = the product kernel; 1 / 2 = the ablations of skinny_gemm_kernel for the one-launch SwiGLU form (packed weights,
// M <= 32): what bench.py --workload decode_batch --skinny-ablation times
static int g_skinny_ablation = 0;

bool skinny_gemm_supported(int M, int N, int K) { return M >= 16 && M <= 64 && K % kSkinnyK == 0 && K >= 2 * kSkinnyK && N >= 1; }

// K ranges: enough waves to keep ~1000 in flight, each with at least as many steps as it has stages
static int skinny_ksplit(int N, int K) {
    const int waves_n = (N + 31) / 32, iters = K / kSkinnyK;
    if (waves_n >= 768) return 1;  // three waves per CU already: one launch that stores the finished output
    int ks = (1024 + waves_n - 1) / waves_n;  // (768 is as good; 512 and 1536 are 3-5 % slower over a batch-32 step)
    if (ks > iters / kSkinnyStages) ks = iters / kSkinnyStages;
    return ks < 1 ? 1 : ks;  // (ranges of equal length -- 8 of 4 steps instead of five of 6 and one of 2 for N = 6144, K = 4096 -- measured 6 % slower)
}
size_t skinny_scratch_bytes(int M, int N, int K) { return (size_t)skinny_ksplit(N, K) * M * N * sizeof(float); }

// norm_w / nrm_out (optional, residual store only): also write the RMSNorm of the finished rows; *normed tells
// whether this call did (it does when the K range is split, N % 4 == 0 and N <= 4096)
int dequant_gemm_skinny(void *out, const void *act, const int8_t *wq, bool packed, const void *scale, const void *res, int M,
                        int N, int K, int dtype, int epi, float *scratch, hipStream_t s, const void *norm_w, float eps,
                        void *nrm_out, bool *normed, const SkinnyRope *rope, bool *roped) {
    if (normed) *normed = false;
    if (roped) *roped = false;
    MYNN_REQUIRE(out && act && wq && scale && scratch, MYNN_ERR_INVALID, "dequant_matmul: null operand");
    MYNN_REQUIRE(skinny_gemm_supported(M, N, K), MYNN_ERR_UNSUPPORTED, "dequant_matmul (few rows): M=%d N=%d K=%d", M, N, K);
    MYNN_REQUIRE(aligned16(act) && aligned16(wq), MYNN_ERR_INVALID, "dequant_matmul: act and wq must be 16-byte aligned");
    MYNN_REQUIRE(epi != GEMM_RESIDUAL || res, MYNN_ERR_INVALID, "dequant_matmul: residual store without a residual");
    MYNN_REQUIRE(epi != GEMM_SWIGLU || N % 2 == 0, MYNN_ERR_INVALID, "dequant_matmul: SwiGLU store needs row pairs (N=%d)", N);
    const int ksplit = skinny_ksplit(N, K), iters = K / kSkinnyK;
    const int ips = (iters + ksplit - 1) / ksplit;
    const int ks_used = (iters + ips - 1) / ips;
    dim3 grid((N + 32 * kSkinnyWaves - 1) / (32 * kSkinnyWaves), ks_used);
    const size_t n_out = (size_t)M * (epi == GEMM_SWIGLU ? N / 2 : N);
    return dispatch_dtype16(dtype, [&](auto *t) {
        using T = std::remove_pointer_t<decltype(t)>;
        auto gemm = [&](auto fepi) {
            constexpr int FEPI = decltype(fepi)::value;
            T *o = (T *)out;
            const T *sc = (const T *)scale, *rs = (const T *)res;
            if (M <= 32 && packed)
                MYNN_LAUNCH((skinny_gemm_kernel<T, 1, true, FEPI>), grid, dim3(kSkinnyThreads), 0, s, scratch, (const T *)act, wq, M, N, K, ips, o, sc, rs);
            else if (M <= 32)
                MYNN_LAUNCH((skinny_gemm_kernel<T, 1, false, FEPI>), grid, dim3(kSkinnyThreads), 0, s, scratch, (const T *)act, wq, M, N, K, ips, o, sc, rs);
            else if (packed)
                MYNN_LAUNCH((skinny_gemm_kernel<T, 2, true, FEPI>), grid, dim3(kSkinnyThreads), 0, s, scratch, (const T *)act, wq, M, N, K, ips, o, sc, rs);
            else
                MYNN_LAUNCH((skinny_gemm_kernel<T, 2, false, FEPI>), grid, dim3(kSkinnyThreads), 0, s, scratch, (const T *)act, wq, M, N, K, ips, o, sc, rs);
            return launch_status("skinny_gemm_kernel");
        };
        // the whole K range in one workgroup: no partial sums, no second launch (the wide shapes: gate/up and
        // lm_head; a residual store never meets this width, it keeps the two-launch form)
        if (ks_used == 1 && epi == GEMM_SWIGLU && g_skinny_ablation && M <= 32 && packed) {
            T *o = (T *)out;
            if (g_skinny_ablation == 1)
                MYNN_LAUNCH((skinny_gemm_kernel<T, 1, true, GEMM_SWIGLU, 1>), grid, dim3(kSkinnyThreads), 0, s, scratch, (const T *)act, wq, M, N, K, ips, o,
                            (const T *)scale, (const T *)res);
            else
                MYNN_LAUNCH((skinny_gemm_kernel<T, 1, true, GEMM_SWIGLU, 2>), grid, dim3(kSkinnyThreads), 0, s, scratch, (const T *)act, wq, M, N, K, ips, o,
                            (const T *)scale, (const T *)res);
            return launch_status("skinny_gemm_kernel (ablation)");
        }
        if (ks_used == 1 && epi == GEMM_SWIGLU) return gemm(std::integral_constant<int, GEMM_SWIGLU>{});
        if (ks_used == 1 && epi == GEMM_PLAIN) return gemm(std::integral_constant<int, GEMM_PLAIN>{});
        int rc = gemm(std::integral_constant<int, -1>{});
        if (rc) return rc;
        if (epi == GEMM_RESIDUAL && norm_w && nrm_out && normed && N % 4 == 0 && N <= 4 * kReduceNormThreads &&
            ks_used <= kReduceNormMaxSplit && aligned16(out) && aligned16(res) && aligned16(nrm_out) && ((uintptr_t)norm_w & 7) == 0 &&
            ((uintptr_t)scale & 7) == 0) {
            MYNN_LAUNCH(skinny_reduce_norm_kernel<T>, dim3(M), dim3(kReduceNormThreads), 0, s, (T *)out, (T *)nrm_out, scratch,
                        (const T *)scale, (const T *)res, (const T *)norm_w, M, N, ks_used, eps);
            *normed = true;
            return launch_status("skinny_reduce_norm_kernel");
        }
        if (epi == GEMM_PLAIN && rope && roped && rope->D % 8 == 0 && N == (rope->Hq + 2 * rope->Hkv) * rope->D &&
            ks_used <= kReduceNormMaxSplit && ((uintptr_t)scale & 7) == 0 && ((uintptr_t)rope->q_out & 7) == 0 &&
            ((uintptr_t)rope->k_cache & 7) == 0 && ((uintptr_t)rope->v_cache & 7) == 0 && ((uintptr_t)rope->cos_t & 7) == 0 &&
            ((uintptr_t)rope->sin_t & 7) == 0 && (!rope->k_scale || ((rope->D == 64 || rope->D == 128) && rope->v_scale))) {
            const int rope_units = (rope->Hq + rope->Hkv) * (rope->D / 8) + rope->Hkv * (rope->k_scale ? rope->D / 8 : rope->D / 4);
            const dim3 rope_grid(M, (rope_units + kReduceRopeThreads - 1) / kReduceRopeThreads);
            if (rope->k_scale)
                MYNN_LAUNCH((skinny_reduce_rope_kernel<T, true>), rope_grid, dim3(kReduceRopeThreads), 0, s, scratch, (const T *)scale, M, N,
                            ks_used, (T *)rope->q_out, rope->k_cache, rope->v_cache, (T *)rope->k_scale, (T *)rope->v_scale,
                            (const T *)rope->cos_t, (const T *)rope->sin_t, rope->position, rope->d_past, rope->S, rope->Hq, rope->Hkv,
                            rope->D, rope->max_seq, rope->paging);
            else
                MYNN_LAUNCH((skinny_reduce_rope_kernel<T, false>), rope_grid, dim3(kReduceRopeThreads), 0, s, scratch, (const T *)scale, M, N,
                            ks_used, (T *)rope->q_out, rope->k_cache, rope->v_cache, (T *)nullptr, (T *)nullptr, (const T *)rope->cos_t,
                            (const T *)rope->sin_t, rope->position, rope->d_past, rope->S, rope->Hq, rope->Hkv, rope->D, rope->max_seq,
                            rope->paging);
            *roped = true;
            return launch_status("skinny_reduce_rope_kernel");
        }
        const dim3 rg((unsigned)((n_out + 255) / 256));
        if (epi == GEMM_RESIDUAL)
            MYNN_LAUNCH((skinny_reduce_kernel<T, GEMM_RESIDUAL>), rg, dim3(256), 0, s, (T *)out, scratch, (const T *)scale,
                        (const T *)res, M, N, ks_used);
        else if (epi == GEMM_SWIGLU)
            MYNN_LAUNCH((skinny_reduce_kernel<T, GEMM_SWIGLU>), rg, dim3(256), 0, s, (T *)out, scratch, (const T *)scale,
                        (const T *)res, M, N, ks_used);
        else
            MYNN_LAUNCH((skinny_reduce_kernel<T, GEMM_PLAIN>), rg, dim3(256), 0, s, (T *)out, scratch, (const T *)scale,
                        (const T *)res, M, N, ks_used);
        return launch_status("skinny_reduce_kernel");
    });
}

}  // namespace mynn

extern "C" void mynn_skinny_set_ablation(int mode) { mynn::g_skinny_ablation = mode == 1 || mode == 2 ? mode : 0; }
