// Batch-1 decode with Options::quantize_activations: one launch per int8 linear of the layer instead of three or four.
//
//   (RMSNormalization ->) DynamicQuantizeLinear (per row, symmetric) -> QuantizedMatMul (-> Add / SwiGLU)
//   src/transform/optimize/quantize_activations.rs, quantized_gemv_int8.cuh:13-51, qgemv_i8i8.rs:38-80
//
// The structure of dequant_gemv1_kernel with the int8 arithmetic of the operators it replaces: a workgroup stages the
// activation row once -- RMS-normalised if asked (rounded to the storage type, as the separate operator stores it), its
// absolute maximum found, every element quantised to round(x / (amax / 127)) (half away from zero, clamped to +-127) and
// kept in LDS as int8 -- then its waves walk groups of R weight rows: all weight loads of a lane issued before anything
// else, `v_dot4_i32_i8` over 16-byte chunks (a quarter of a vector operation per weight), exact int32 sums, and
// out = T((acc * T(act scale)) * weight scale) as qgemv_i8_kernel computes it; then the residual add or SwiGLU on the
// stored values, as the Add / SwiGLU operators would.
#include <type_traits>

#include "kernels.h"

namespace mynn {

constexpr int kQgThreads = 256, kQgWaves = kQgThreads / 64;

struct QGemvParams {
    void *out;
    float eps;
};

template <typename T, int R, int NC, int EPI, bool NORM>
__global__ __launch_bounds__(kQgThreads) void qgemv1_kernel(const int8_t *wq, const void *act, const void *scale_p, const void *norm_w,
                                                          const void *residual, int N, int K, int groups, int total_waves,
                                                          QGemvParams p) {
    extern __shared__ int8_t act_q[];  // [K]
    __shared__ float red[kQgWaves], redm[kQgWaves];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nchunks = K >> 4;
    int g = blockIdx.x * kQgWaves + wave;

    struct Group {
        U4 w[R][NC];
        T sc, sc1, res;  // as loaded: widening them here would make the wave wait for every load above
    };
    const T *scale = (const T *)scale_p;
    auto load_group = [&](int gg, Group &G) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int row = gg * R + r < N ? gg * R + r : N - 1;
            const U4 *wrow = (const U4 *)(wq + (size_t)row * K);
#pragma unroll
            for (int j = 0; j < NC; j++) G.w[r][j] = __builtin_nontemporal_load(&wrow[min(lane + j * kWave, nchunks - 1)]);
        }
        const int row = min(gg * R + min(lane, R - 1), N - 1);
        G.sc = scale[row];
        if constexpr (EPI == GEMM_SWIGLU) G.sc1 = scale[min(row + 1, N - 1)];
        if constexpr (EPI == GEMM_RESIDUAL) G.res = ((const T *)residual)[row];
    };
    // the activation pieces (and their norm weights) first: loads return in order
    const int npieces = K >> 3;
    constexpr int PMAX = (NC * 1024 / 8 + kQgThreads - 1) / kQgThreads;
    U4 apv[PMAX], nwv[NORM ? PMAX : 1];
#pragma unroll
    for (int q = 0; q < PMAX; q++) {
        const int pc = tid + q * kQgThreads;
        if (pc < npieces) {
            apv[q] = ((const U4 *)act)[pc];
            if constexpr (NORM) nwv[q] = ((const U4 *)norm_w)[pc];
        }
    }
    Group ga;
    load_group(min(g, groups - 1), ga);

    // ---- stage: thread t owns the 8-element pieces t, t + 256, ..
    float asc;  // the activation scale as the quantiser stores it (rounded to T)
    {
        float f[PMAX][8];
        float ss = 0.f;
#pragma unroll
        for (int q = 0; q < PMAX; q++) {
            const int pc = tid + q * kQgThreads;
#pragma unroll
            for (int i = 0; i < 8; i++) f[q][i] = 0.f;
            if (pc < npieces) {
                widen8<T>(apv[q], f[q]);
                if constexpr (NORM) {
#pragma unroll
                    for (int i = 0; i < 8; i++) ss = fmaf(f[q][i], f[q][i], ss);
                }
            }
        }
        if constexpr (NORM) {
            ss = wave_sum(ss);
            if (lane == 0) red[wave] = ss;
            __syncthreads();
            float tot = 0.f;
#pragma unroll
            for (int i = 0; i < kQgWaves; i++) tot += red[i];
            const float inv = 1.0f / sqrtf(tot / (float)K + p.eps);
#pragma unroll
            for (int q = 0; q < PMAX; q++) {
                const int pc = tid + q * kQgThreads;
                if (pc < npieces) {
                    float nw[8];
                    widen8<T>(nwv[q], nw);
#pragma unroll
                    for (int i = 0; i < 8; i++) f[q][i] = Elem<T>::rnd((f[q][i] * inv) * nw[i]);
                }
            }
        }
        float amax = 0.f;
#pragma unroll
        for (int q = 0; q < PMAX; q++)
#pragma unroll
            for (int i = 0; i < 8; i++) amax = fmaxf(amax, fabsf(f[q][i]));
        amax = wave_max(amax);
        if (lane == 0) redm[wave] = amax;
        __syncthreads();
#pragma unroll
        for (int i = 0; i < kQgWaves; i++) amax = fmaxf(amax, redm[i]);
        const float sc = amax > 0.f ? amax / 127.0f : 1.0f;
        const float inv_sc = 1.0f / sc;
        asc = Elem<T>::rnd(sc);
#pragma unroll
        for (int q = 0; q < PMAX; q++) {
            const int pc = tid + q * kQgThreads;
            if (pc < npieces) {
                uint32_t b[2] = {0u, 0u};
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    float r = roundf(f[q][i] * inv_sc);  // half away from zero
                    r = fminf(fmaxf(r, -127.f), 127.f);
                    b[i >> 2] |= ((uint32_t)(int)r & 0xFFu) << (8 * (i & 3));
                }
                *(uint2 *)(act_q + (size_t)pc * 8) = uint2{b[0], b[1]};
            }
        }
    }
    __syncthreads();

    T *out = (T *)p.out;
    bool loaded = true;
    for (; g < groups; g += total_waves) {
        if (!loaded) load_group(g, ga);
        loaded = false;
        int acc[R];
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] = 0;
#pragma unroll
        for (int j = 0; j < NC; j++) {
            const int c = lane + j * kWave;
            if (c < nchunks) {
                const U4 a = *(const U4 *)(act_q + (size_t)c * 16);
#pragma unroll
                for (int r = 0; r < R; r++) {
                    const U4 w = ga.w[r][j];
                    acc[r] = __builtin_amdgcn_sdot4((int)a.x, (int)w.x, acc[r], false);
                    acc[r] = __builtin_amdgcn_sdot4((int)a.y, (int)w.y, acc[r], false);
                    acc[r] = __builtin_amdgcn_sdot4((int)a.z, (int)w.z, acc[r], false);
                    acc[r] = __builtin_amdgcn_sdot4((int)a.w, (int)w.w, acc[r], false);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] = wave_sum_i32(acc[r]);
        const int row0 = g * R;
        // lane r finishes row r (SwiGLU: lane r = 0, 2, .. the pair r, r + 1)
        int mine = acc[0], next = R > 1 ? acc[1] : 0;
#pragma unroll
        for (int r = 1; r < R; r++) {
            if (lane == r) {
                mine = acc[r];
                if (r + 1 < R) next = acc[r + 1];
            }
        }
        if constexpr (EPI == GEMM_SWIGLU) {
            if (lane < R && (lane & 1) == 0 && row0 + lane + 1 < N) {
                const float gt = Elem<T>::rnd(((float)mine * asc) * Elem<T>::ld(&ga.sc, 0));
                const float up = Elem<T>::rnd(((float)next * asc) * Elem<T>::ld(&ga.sc1, 0));
                const float sig = 1.0f / (1.0f + expf(-gt));
                Elem<T>::st(out, (size_t)((row0 + lane) >> 1), (gt * sig) * up);
            }
        } else {
            if (lane < R && row0 + lane < N) {
                float y = ((float)mine * asc) * Elem<T>::ld(&ga.sc, 0);
                if constexpr (EPI == GEMM_RESIDUAL) y = Elem<T>::rnd(y) + Elem<T>::ld(&ga.res, 0);
                Elem<T>::st(out, row0 + lane, y);
            }
        }
    }
}

template <typename T, int R, int NC, int EPI, bool NORM>
static int launch_qgemv1(const void *out, const void *act, const void *norm_w, float eps, const int8_t *wq, const void *scale,
                         const void *residual, int N, int K, hipStream_t s) {
    const int groups = (N + R - 1) / R;
    const int max_waves = 256 * 16;
    const int passes = (groups + max_waves - 1) / max_waves;
    int waves = (groups + passes - 1) / passes;
    const int blocks = (waves + kQgWaves - 1) / kQgWaves;
    waves = blocks * kQgWaves;
    QGemvParams p{(void *)out, eps};
    MYNN_LAUNCH((qgemv1_kernel<T, R, NC, EPI, NORM>), dim3(blocks), dim3(kQgThreads), (size_t)K, s, wq, act, scale, norm_w, residual, N, K,
                groups, waves, p);
    return launch_status("qgemv1_kernel");
}

bool qgemv_fused_supported(const void *act, const void *norm_w, const int8_t *wq, int N, int K) {
    return aligned16(act) && (!norm_w || aligned16(norm_w)) && aligned16(wq) && N > 0 && K % 32 == 0 && (K + 1023) / 1024 <= 14 &&
           K <= 131071;  // (the int32 sums stay exact up to there)
}

template <typename T, int EPI, bool NORM>
static int qgemv1_dispatch(void *out, const void *act, const void *norm_w, float eps, const int8_t *wq, const void *scale,
                           const void *residual, int N, int K, hipStream_t s) {
    MYNN_REQUIRE(out && act && wq && scale && qgemv_fused_supported(act, norm_w, wq, N, K), MYNN_ERR_UNSUPPORTED,
                 "quantised GEMV launch: N=%d K=%d", N, K);
    MYNN_REQUIRE(EPI != GEMM_RESIDUAL || residual, MYNN_ERR_INVALID, "quantised GEMV launch: residual store without a residual");
    MYNN_REQUIRE(EPI != GEMM_SWIGLU || N % 2 == 0, MYNN_ERR_INVALID, "quantised GEMV launch: gate/up rows must come in pairs (N=%d)", N);
    const int nc = (K + 1023) / 1024;
    const bool wide = nc <= 2;  // four rows per wave for short rows, as the dequantising GEMV
#define MYNN_QGEMV1(NC_)                                                                                                          \
    return wide ? launch_qgemv1<T, 4, NC_, EPI, NORM>(out, act, norm_w, eps, wq, scale, residual, N, K, s)                          \
                : launch_qgemv1<T, 2, NC_, EPI, NORM>(out, act, norm_w, eps, wq, scale, residual, N, K, s)
    if (nc <= 1) { MYNN_QGEMV1(1); }
    if (nc <= 2) { MYNN_QGEMV1(2); }
    if (nc <= 4) { MYNN_QGEMV1(4); }
    if (nc <= 6) { MYNN_QGEMV1(6); }
    if (nc <= 8) { MYNN_QGEMV1(8); }
    MYNN_QGEMV1(14);
#undef MYNN_QGEMV1
}

// epi: GEMM_PLAIN / GEMM_RESIDUAL / GEMM_SWIGLU; norm_w: RMS-normalise the row first (null: not)
int qgemv_fused(void *out, const void *act, const void *norm_w, float eps, const int8_t *wq, const void *scale, const void *residual,
                int N, int K, int dtype, int epi, hipStream_t s) {
    return dispatch_dtype16(dtype, [&](auto *t) {
        using T = std::remove_pointer_t<decltype(t)>;
        if (epi == GEMM_SWIGLU) {
            if (norm_w) return qgemv1_dispatch<T, GEMM_SWIGLU, true>(out, act, norm_w, eps, wq, scale, residual, N, K, s);
            return qgemv1_dispatch<T, GEMM_SWIGLU, false>(out, act, norm_w, eps, wq, scale, residual, N, K, s);
        }
        if (epi == GEMM_RESIDUAL) {
            if (norm_w) return qgemv1_dispatch<T, GEMM_RESIDUAL, true>(out, act, norm_w, eps, wq, scale, residual, N, K, s);
            return qgemv1_dispatch<T, GEMM_RESIDUAL, false>(out, act, norm_w, eps, wq, scale, residual, N, K, s);
        }
        if (norm_w) return qgemv1_dispatch<T, GEMM_PLAIN, true>(out, act, norm_w, eps, wq, scale, residual, N, K, s);
        return qgemv1_dispatch<T, GEMM_PLAIN, false>(out, act, norm_w, eps, wq, scale, residual, N, K, s);
    });
}

}  // namespace mynn
