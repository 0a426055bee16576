// DequantMatMul for M > 1 on the CDNA4 matrix cores.
//
// Kernel choice follows the reference (src/codegen/cuda.rs:1518-1652): 16-bit activations and
// scales with M >= 16 take the matrix-core path whose numerics are those of
// dequant_matmul_wmma.cuh:65-76 -- the weight is dequantised to the 16-bit type WITH the scale
// folded in (one rounding) and the products are accumulated in f32; everything else takes the
// scale-after-sum kernels of gemv.hip.
//
// Two launches: (1) W_T[n,k] = T(wq[n,k] * scale[n]) into a library-owned workspace (a pure
// streaming pass, ~3 bytes moved per weight), (2) C = A . W_T^T with v_mfma_f32_32x32x16_{f16,bf16}:
// 128x128 output tile per workgroup of 4 waves (2x2, 64x64 per wave = 2x2 MFMA tiles), K step 32,
// operands staged through padded LDS tiles (conflict-free 128-bit reads), next tile prefetched
// into registers while the current one is multiplied.
#include "kernels.h"
#include "mfma.h"

namespace mynn {

// ---- (1) dequantise: 8 weights per thread; rows are written with stride Kp (K rounded up to the
// GEMM's K step) and zero padding
template <typename T>
__global__ void dequant_rows_kernel(T *out, const int8_t *wq, const T *scale, int K, int Kp, size_t total_chunks) {
    size_t c = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= total_chunks) return;
    const int cpr = Kp >> 3;  // chunks per padded row
    const size_t n = c / cpr;
    const int k = (int)(c % cpr) * 8;
    uint32_t packed[4] = {0u, 0u, 0u, 0u};
    if (k < K) {
        const float s = Elem<T>::ld(scale, n);
        const uint2 w = *(const uint2 *)(wq + n * K + k);
        const uint32_t ww[2] = {w.x, w.y};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float f0 = (float)(int8_t)((ww[i >> 1] >> (16 * (i & 1))) & 0xFF);
            const float f1 = (float)(int8_t)((ww[i >> 1] >> (16 * (i & 1) + 8)) & 0xFF);
            T lo, hi;
            Elem<T>::st(&lo, 0, f0 * s);
            Elem<T>::st(&hi, 0, f1 * s);
            packed[i] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
        }
    }
    *(U4 *)(out + c * 8) = U4{packed[0], packed[1], packed[2], packed[3]};
}

// ---- (2) C[M,N] = A[M,K] . B[N,K]^T, f32 accumulate, one rounding at the store
// 256 x 128 output tile per workgroup of 8 waves (4 x 2, 64 x 64 per wave = 2 x 2 MFMA tiles),
// K step 32, two LDS buffers, next tile prefetched into registers during the multiply.
constexpr int BM = 256, BN = 128, BK = 32, LDT = BK + 8;  // LDS row stride in elements (80 B)
constexpr int kGemmThreads = 512;

// Workgroup -> output tile.  Hardware deals consecutive workgroup ids round-robin over the 8 XCDs
// (each with its own L2), so id b is first turned into a per-XCD contiguous index; inside an XCD
// tiles are walked in bands of 8 tile-rows so that the A rows and the B rows being multiplied at
// one time stay L2-resident.
__device__ inline void tile_of(int b, int nblocks, int tiles_m, int tiles_n, int &tm, int &tn) {
    constexpr int XCD = 8, BAND = 8;
    int l = b;
    if (nblocks % XCD == 0) l = (b % XCD) * (nblocks / XCD) + b / XCD;
    const int band_tiles = BAND * tiles_n;
    const int band = l / band_tiles, in_band = l % band_tiles;
    const int rows_here = min(BAND, tiles_m - band * BAND);
    tm = band * BAND + in_band % rows_here;
    tn = in_band / rows_here;
}

// KTAIL: K is not a multiple of 2*BK, so the last steps mask the columns of A past K.
template <typename T, bool KTAIL>
__global__ __launch_bounds__(kGemmThreads, 2) void gemm_nt_mfma_kernel(T *C, const T *A, const T *B, int M, int N, int K,
                                                                    int Kp) {
    __shared__ __align__(16) uint16_t As[2][BM * LDT];
    __shared__ __align__(16) uint16_t Bs[2][BN * LDT];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;  // wave tile origin: (64*wm, 64*wn)
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    int tm, tn;
    tile_of(blockIdx.x, gridDim.x, tiles_m, tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;

    // global -> register staging: A tile 256 x 32 = 1024 chunks of 8 (2 per thread), B tile 512 (1 per
    // thread).  Two register sets: tile kt+1 waits in one while tile kt+2 is still in flight in the
    // other, so a load has two multiply phases of every resident wave to complete.
    const int lr = tid >> 2, lc = (tid & 3) * 8;  // row (0..127) and element offset within BK
    struct Stage { U4 a0, a1, b; uint32_t mask; };
    // Branch-free: rows past M / N re-read the last row (their products land in rows that are never
    // stored), columns past K are masked to zero.  No branch means the compiler can wait for exactly
    // the older register set (vmcnt(3)) instead of for everything in flight.
    const T *a0p = A + (size_t)min(m0 + lr, M - 1) * K;
    const T *a1p = A + (size_t)min(m0 + lr + 128, M - 1) * K;
    const T *bp = B + (size_t)min(n0 + lr, N - 1) * Kp;
    auto load_tiles = [&](Stage &r, int k0) {
        const int ka = min(k0 + lc, K - 8);
        if (KTAIL) r.mask = k0 + lc < K ? 0xFFFFFFFFu : 0u;  // applied when the registers are consumed
        r.a0 = *(const U4 *)(a0p + ka);
        r.a1 = *(const U4 *)(a1p + ka);
        r.b = *(const U4 *)(bp + k0 + lc);
    };
    auto store_tiles = [&](int buf, const Stage &r) {
        *(U4 *)&As[buf][lr * LDT + lc] = KTAIL ? r.a0 & r.mask : r.a0;
        *(U4 *)&As[buf][(lr + 128) * LDT + lc] = KTAIL ? r.a1 & r.mask : r.a1;
        *(U4 *)&Bs[buf][lr * LDT + lc] = r.b;
    };

    f16x_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

    const int fr = lane & 31, fk = (lane >> 5) * 8;  // fragment row within a 32-row tile, k offset
    auto multiply = [&](int buf) {
#pragma unroll
        for (int ks = 0; ks < BK; ks += 16) {
            U4 fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; i++) fa[i] = *(const U4 *)&As[buf][(wm * 64 + i * 32 + fr) * LDT + ks + fk];
#pragma unroll
            for (int j = 0; j < 2; j++) fb[j] = *(const U4 *)&Bs[buf][(wn * 64 + j * 32 + fr) * LDT + ks + fk];
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) acc[i][j] = Mfma<T>::run(fa[i], fb[j], acc[i][j]);
        }
    };

    const int nk = Kp / BK;  // even: Kp is a multiple of 2*BK
    Stage rA, rB;
    load_tiles(rA, 0);
    store_tiles(0, rA);
    load_tiles(rA, BK);
    load_tiles(rB, min(2, nk - 1) * BK);
    __syncthreads();
    for (int kt = 0; kt < nk; kt += 2) {
        multiply(0);                                   // tile kt
        store_tiles(1, rA);                            // tile kt+1
        load_tiles(rA, min(kt + 3, nk - 1) * BK);      // (a repeat of the last tile near the end; unused)
        __syncthreads();
        multiply(1);                                   // tile kt+1
        store_tiles(0, rB);                            // tile kt+2
        load_tiles(rB, min(kt + 4, nk - 1) * BK);
        __syncthreads();
    }

    // epilogue: D[i][j] of a 32x32 tile sits in lane (j + 32*((i/4)%2)), element 4*(i/8) + i%4
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int col = n0 + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int row = m0 + wm * 64 + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
                if (row < M && col < N) Elem<T>::st(C, (size_t)row * N + col, acc[i][j][e]);
            }
        }
}

// library-owned workspace for the dequantised weight of the call in flight (grown on demand)
static void *g_ws = nullptr;
static size_t g_ws_bytes = 0;

template <typename T>
static int gemm_launch(void *out, const void *act, const int8_t *wq, const void *scale, int M, int N, int K,
                       hipStream_t s) {
    const int Kp = (K + 2 * BK - 1) / (2 * BK) * (2 * BK);  // the GEMM walks K in pairs of steps
    const size_t need = (size_t)N * Kp * sizeof(T);
    if (need > g_ws_bytes) {
        MYNN_HIP(hipStreamSynchronize(s));
        if (g_ws) MYNN_HIP(hipFree(g_ws));
        g_ws = nullptr;
        g_ws_bytes = 0;
        MYNN_HIP(hipMalloc(&g_ws, need));
        g_ws_bytes = need;
    }
    const size_t chunks = (size_t)N * Kp / 8;
    hipLaunchKernelGGL(dequant_rows_kernel<T>, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, s, (T *)g_ws, wq,
                       (const T *)scale, K, Kp, chunks);
    int rc = launch_status("dequant_rows_kernel");
    if (rc) return rc;
    const int tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
    if (K == Kp)
        hipLaunchKernelGGL((gemm_nt_mfma_kernel<T, false>), dim3(tiles), dim3(kGemmThreads), 0, s, (T *)out,
                           (const T *)act, (const T *)g_ws, M, N, K, Kp);
    else
        hipLaunchKernelGGL((gemm_nt_mfma_kernel<T, true>), dim3(tiles), dim3(kGemmThreads), 0, s, (T *)out,
                           (const T *)act, (const T *)g_ws, M, N, K, Kp);
    return launch_status("gemm_nt_mfma_kernel");
}

int dequant_gemm_mfma(void *out, const void *act, const int8_t *wq, const void *scale, int M, int N, int K,
                      int dtype, hipStream_t s) {
    MYNN_REQUIRE(out && act && wq && scale, MYNN_ERR_INVALID, "dequant_matmul: null operand");
    MYNN_REQUIRE(M > 0 && N > 0 && K > 0, MYNN_ERR_INVALID, "dequant_matmul: M=%d N=%d K=%d", M, N, K);
    MYNN_REQUIRE(K % 8 == 0, MYNN_ERR_UNSUPPORTED, "dequant_matmul (matrix cores): K=%d is not a multiple of 8", K);
    MYNN_REQUIRE(aligned16(act) && ((uintptr_t)wq & 7) == 0, MYNN_ERR_INVALID,
                 "dequant_matmul: act must be 16-byte and wq 8-byte aligned");
    return dispatch_dtype16(dtype, [&](auto *t) {
        using T = std::remove_pointer_t<decltype(t)>;
        return gemm_launch<T>(out, act, wq, scale, M, N, K, s);
    });
}

}  // namespace mynn

extern "C" int mynn_dequant_matmul(void *out, const void *act, const int8_t *wq, const void *scale, int M, int N,
                                   int K, int act_dtype, int out_dtype, mynn_stream s) {
    using namespace mynn;
    MYNN_REQUIRE(M >= 1, MYNN_ERR_INVALID, "dequant_matmul: M=%d", M);
    const bool sixteen = act_dtype != MYNN_F32 && out_dtype != MYNN_F32 && act_dtype == out_dtype;
    if (M >= 16 && sixteen && K % 8 == 0 && aligned16(act) && ((uintptr_t)wq & 7) == 0)
        return dequant_gemm_mfma(out, act, wq, scale, M, N, K, out_dtype, as_stream(s));
    return dequant_gemv_dispatch(out, act, wq, scale, M, N, K, act_dtype, out_dtype, as_stream(s));
}
