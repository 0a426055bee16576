// QuantizedMatMul (W8A8): acc[m,n] = sum_k lhs[m,k] * rhs[n,k] in exact int32, then
// out[m,n] = T((f32)acc * lhs_scale[m] * rhs_scale[n]) with the products taken left to right.
//
// Replaces quantized_gemv_int8.cuh:13-51 (one 32-lane warp per row, __dp4a) and
// quantized_matmul_int8.cuh:112-269 (mma.m16n8k32.s8, 3-stage cp.async); CPU twin
// src/codegen/cpu/kernels/qgemv_i8i8.rs:38-80.
//   M < 16 : wave64 rows, 16 int8 per lane per load, v_dot4_i32_i8, integer butterfly
//   M >= 16: v_mfma_i32_32x32x32_i8, 128x128 tile per workgroup, K step 32, padded LDS tiles;
//            grids of >= 128 tiles of 256x256 with K % 128 == 0 use the direct-to-LDS kernel of gemm.hip
// Integer accumulation is associative, so both are bit-exact whatever the order.
#include "kernels.h"

namespace mynn {

typedef int i4x_t __attribute__((ext_vector_type(4)));
typedef int i16x_t __attribute__((ext_vector_type(16)));



// ---- small M: one wave per (R rows of rhs) x (MB rows of lhs)
template <typename T, int R, int MB>
__global__ __launch_bounds__(256) void qgemv_i8_kernel(T *out, int32_t *acc_out, const int8_t *lhs, const T *lhs_scale,
                                                       const int8_t *rhs, const T *rhs_scale, int m_base, int N, int K) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row0 = (blockIdx.x * 4 + wave) * R;
    if (row0 >= N) return;
    int acc[R][MB];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int m = 0; m < MB; m++) acc[r][m] = 0;
    const int nchunks = K >> 4;
    for (int c = lane; c < nchunks; c += 64) {
        U4 a[MB];
#pragma unroll
        for (int m = 0; m < MB; m++) a[m] = *((const U4 *)(lhs + (size_t)(m_base + m) * K) + c);
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int row = row0 + r < N ? row0 + r : N - 1;
            const U4 w = __builtin_nontemporal_load((const U4 *)(rhs + (size_t)row * K) + c);
#pragma unroll
            for (int m = 0; m < MB; m++) {
                acc[r][m] = __builtin_amdgcn_sdot4((int)a[m].x, (int)w.x, acc[r][m], false);
                acc[r][m] = __builtin_amdgcn_sdot4((int)a[m].y, (int)w.y, acc[r][m], false);
                acc[r][m] = __builtin_amdgcn_sdot4((int)a[m].z, (int)w.z, acc[r][m], false);
                acc[r][m] = __builtin_amdgcn_sdot4((int)a[m].w, (int)w.w, acc[r][m], false);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int m = 0; m < MB; m++) acc[r][m] = wave_sum_i32(acc[r][m]);
#pragma unroll
    for (int r = 0; r < R; r++) {
        if (lane == r && row0 + r < N) {
#pragma unroll
            for (int m = 0; m < MB; m++) {
                const size_t o = (size_t)(m_base + m) * N + row0 + r;
                if (acc_out) acc_out[o] = acc[r][m];
                if (out) {
                    const float asc = Elem<T>::ld(lhs_scale, m_base + m), wsc = Elem<T>::ld(rhs_scale, row0 + r);
                    Elem<T>::st(out, o, ((float)acc[r][m] * asc) * wsc);
                }
            }
        }
    }
}

// ---- M >= 16: int8 matrix cores
constexpr int QBM = 128, QBN = 128, QBK = 32, QLD = QBK + 16;  // LDS row stride in bytes

template <typename T>
__global__ __launch_bounds__(256) void qgemm_i8_mfma_kernel(T *out, int32_t *acc_out, const int8_t *A, const T *a_scale,
                                                            const int8_t *B, const T *b_scale, int M, int N, int K) {
    __shared__ __align__(16) int8_t As[2][QBM * QLD];
    __shared__ __align__(16) int8_t Bs[2][QBN * QLD];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int tiles_m = (M + QBM - 1) / QBM;
    const int tm = blockIdx.x % tiles_m, tn = blockIdx.x / tiles_m;
    const int m0 = tm * QBM, n0 = tn * QBN;
    // a tile is 128 rows x 32 bytes = 256 chunks of 16 bytes: one per thread and operand
    const int lr = tid >> 1, lc = (tid & 1) * 16;
    U4 ra, rb;
    auto load_tiles = [&](int k0) {
        ra = (m0 + lr < M) ? *(const U4 *)(A + (size_t)(m0 + lr) * K + k0 + lc) : U4{0u, 0u, 0u, 0u};
        rb = (n0 + lr < N) ? *(const U4 *)(B + (size_t)(n0 + lr) * K + k0 + lc) : U4{0u, 0u, 0u, 0u};
    };
    auto store_tiles = [&](int buf) {
        *(U4 *)&As[buf][lr * QLD + lc] = ra;
        *(U4 *)&Bs[buf][lr * QLD + lc] = rb;
    };
    i16x_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0;
    const int fr = lane & 31, fk = (lane >> 5) * 16;
    load_tiles(0);
    store_tiles(0);
    __syncthreads();
    const int nk = K / QBK;
    for (int kt = 0; kt < nk; kt++) {
        const int buf = kt & 1;
        if (kt + 1 < nk) load_tiles((kt + 1) * QBK);
        i4x_t fa[2], fb[2];
#pragma unroll
        for (int i = 0; i < 2; i++) fa[i] = *(const i4x_t *)&As[buf][(wm * 64 + i * 32 + fr) * QLD + fk];
#pragma unroll
        for (int j = 0; j < 2; j++) fb[j] = *(const i4x_t *)&Bs[buf][(wn * 64 + j * 32 + fr) * QLD + fk];
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
        if (kt + 1 < nk) {
            store_tiles(buf ^ 1);
            __syncthreads();
        }
    }
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int col = n0 + wn * 64 + j * 32 + (lane & 31);
            const float wsc = (out && col < N) ? Elem<T>::ld(b_scale, col) : 0.f;
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int row = m0 + wm * 64 + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
                if (row < M && col < N) {
                    const size_t o = (size_t)row * N + col;
                    if (acc_out) acc_out[o] = acc[i][j][e];
                    if (out) Elem<T>::st(out, o, ((float)acc[i][j][e] * Elem<T>::ld(a_scale, row)) * wsc);
                }
            }
        }
}

template <typename T>
static int qmatmul_launch(void *out, int32_t *acc_out, const int8_t *lhs, const void *ls, const int8_t *rhs,
                          const void *rs, int M, int N, int K, hipStream_t s) {
    if (M >= 16) {
        const int tiles = ((M + QBM - 1) / QBM) * ((N + QBN - 1) / QBN);
        MYNN_LAUNCH(qgemm_i8_mfma_kernel<T>, dim3(tiles), dim3(256), 0, s, (T *)out, acc_out, lhs, (const T *)ls, rhs,
                           (const T *)rs, M, N, K);
        return launch_status("qgemm_i8_mfma_kernel");
    }
    const int R = 2;
    const dim3 grid((N + 4 * R - 1) / (4 * R));
    int m = 0;
    while (m < M) {
        const int mb = M - m >= 4 ? 4 : (M - m >= 2 ? 2 : 1);
        if (mb == 4)
            MYNN_LAUNCH((qgemv_i8_kernel<T, R, 4>), grid, dim3(256), 0, s, (T *)out, acc_out, lhs, (const T *)ls, rhs,
                               (const T *)rs, m, N, K);
        else if (mb == 2)
            MYNN_LAUNCH((qgemv_i8_kernel<T, R, 2>), grid, dim3(256), 0, s, (T *)out, acc_out, lhs, (const T *)ls, rhs,
                               (const T *)rs, m, N, K);
        else
            MYNN_LAUNCH((qgemv_i8_kernel<T, R, 1>), grid, dim3(256), 0, s, (T *)out, acc_out, lhs, (const T *)ls, rhs,
                               (const T *)rs, m, N, K);
        int rc = launch_status("qgemv_i8_kernel");
        if (rc) return rc;
        m += mb;
    }
    return 0;
}

}  // namespace mynn

extern "C" int mynn_quantized_matmul(void *out, int32_t *acc_out, const int8_t *lhs, const void *lhs_scale,
                                     const int8_t *rhs, const void *rhs_scale, int M, int N, int K, int dtype,
                                     mynn_stream s) {
    using namespace mynn;
    MYNN_REQUIRE(lhs && rhs && (out || acc_out), MYNN_ERR_INVALID, "quantized_matmul: null operand");
    MYNN_REQUIRE(!out || (lhs_scale && rhs_scale), MYNN_ERR_INVALID, "quantized_matmul: scales are needed for the float output");
    MYNN_REQUIRE(M > 0 && N > 0 && K > 0, MYNN_ERR_INVALID, "quantized_matmul: M=%d N=%d K=%d", M, N, K);
    MYNN_REQUIRE(K % 32 == 0, MYNN_ERR_UNSUPPORTED, "quantized_matmul: K=%d is not a multiple of 32", K);
    MYNN_REQUIRE(aligned16(lhs) && aligned16(rhs), MYNN_ERR_INVALID, "quantized_matmul: operands must be 16-byte aligned");
    // int32 accumulators hold the exact sum as long as K * 128 * 128 < 2^31
    MYNN_REQUIRE(K <= 131071, MYNN_ERR_UNSUPPORTED, "quantized_matmul: K=%d could overflow the int32 accumulator", K);
    // at least half a round of 256-row tiles and whole 128-value K steps: the large direct-to-LDS tiles
    if (dtype != MYNN_F32 && qgemm_dma_supported(M, N, K) && (!out || aligned16(out)))
        return qgemm_dma(out, acc_out, lhs, lhs_scale, rhs, rhs_scale, nullptr, M, N, K, dtype, GEMM_PLAIN, as_stream(s));
    return dispatch_dtype(dtype, [&](auto *t) {
        using T = std::remove_pointer_t<decltype(t)>;
        return qmatmul_launch<T>(out, acc_out, lhs, lhs_scale, rhs, rhs_scale, M, N, K, as_stream(s));
    });
}
