// DequantMatMul for M > 1 on the CDNA4 matrix cores.
//
// Kernel choice follows the reference (src/codegen/cuda.rs:1518-1652): 16-bit activations and
// scales with M >= 16 take the matrix-core path whose numerics are those of
// dequant_matmul_wmma.cuh:65-76 -- the weight is dequantised to the 16-bit type WITH the scale
// folded in (one rounding) and the products are accumulated in f32; everything else takes the
// scale-after-sum kernels of gemv.hip.
//
// Two steps: (1) W_T[n,k] = T(wq[n,k] * scale[n]) -- a pure streaming pass (~3 bytes moved per
// weight) into a library-owned workspace per call, or once into a resident copy that a prefill
// executor keeps; (2) C = A . W_T^T with v_mfma_f32_32x32x16_{f16,bf16}.  Grids of at least one round
// of 256 x 256 tiles with K % 64 == 0 run gemm_nt_dma_kernel (operand tiles loaded straight into LDS,
// swizzled, 256 x 256 or 256 x 320 per workgroup of 8 waves); the rest runs gemm_nt_mfma_kernel (256 x 128
// or 256 x 256, K step 32, operands staged through registers into padded LDS tiles, any K % 8 == 0).
// The store can add a residual (o_proj, down_proj) or apply SwiGLU to interleaved gate/up columns.
// The int8 form of gemm_nt_dma_kernel is QuantizedMatMul for large grids (qgemm_dma).
#include <map>
#include <mutex>

#include "kernels.h"
#include "mfma.h"

namespace mynn {

// ---- (1) dequantise: 8 weights per thread; rows are written with stride Kp (K rounded up to the
// GEMM's K step) and zero padding
// group > 0: source row r lands in row (r / group) * 2 * group + which * group + r % group of `out`
// (gate rows with which = 0 and up rows with which = 1 interleaved in groups for the SwiGLU store)
template <typename T>
__global__ void dequant_rows_kernel(T *out, const int8_t *wq, const T *scale, int K, int Kp, size_t total_chunks,
                                    int group, int which) {
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
    const size_t dst_row = group > 0 ? (n / group) * 2 * group + (size_t)which * group + n % group : n;
    *(U4 *)(out + dst_row * Kp + k) = U4{packed[0], packed[1], packed[2], packed[3]};
}

// ---- (2) C[M,N] = A[M,K] . B[N,K]^T, f32 accumulate, one rounding at the store
// BM x BN output tile per workgroup of WM x WN waves; a wave owns (BM/WM) x (BN/WN) = TI x TJ MFMA
// tiles of 32 x 32.  K step 32, two LDS buffers, two register stages of global loads in flight.
// Larger wave tiles mean fewer LDS reads per MFMA (TI + TJ fragment reads feed TI * TJ MFMAs).
constexpr int BK = 32, LDT = BK + 8;  // LDS row stride in elements (80 B: conflict-free 128-bit reads)

template <int BM_, int BN_, int WM_, int WN_>
struct GemmTile {
    static constexpr int BM = BM_, BN = BN_, WM = WM_, WN = WN_;
    static constexpr int THREADS = WM * WN * 64;
    static constexpr int TI = BM / WM / 32, TJ = BN / WN / 32;
    static constexpr int CA = BM * 4 / THREADS, CB = BN * 4 / THREADS;  // 16-byte chunks per thread per K step
    static constexpr int ROWS_PER_PASS = THREADS / 4;
    static constexpr int EST = BN / WN + 8;                              // store staging row stride
    static constexpr size_t LDS = (size_t)2 * (BM + BN) * LDT * 2;
    static_assert((size_t)WM * WN * 32 * EST * 2 <= LDS, "store staging must fit the operand buffers");
};
using Tile256x128 = GemmTile<256, 128, 4, 2>;  // 64 x 64 per wave, 61 KB LDS, two workgroups per CU
using Tile256x256 = GemmTile<256, 256, 2, 4>;  // 128 x 64 per wave, 80 KB LDS, one workgroup per CU

// Workgroup -> output tile.  Hardware deals consecutive workgroup ids round-robin over the 8 XCDs
// (each with its own L2), so id b is first turned into a per-XCD contiguous index; inside an XCD
// tiles are walked in bands of 4 tile-rows so that the A rows and the B rows being multiplied at
// one time stay L2-resident.
__device__ inline void tile_of(int b, int nblocks, int tiles_m, int tiles_n, int &tm, int &tn) {
    constexpr int XCD = 8, BAND = 4;  // (bands of 2 / 4 / 8 / 16 / 32 tile rows measured: 4 is best by 0.3-3 % per GEMM, 32 worst)
    int l = b;
    if (nblocks % XCD == 0) l = (b % XCD) * (nblocks / XCD) + b / XCD;
    const int band_tiles = BAND * tiles_n;
    const int band = l / band_tiles, in_band = l % band_tiles;
    const int rows_here = min(BAND, tiles_m - band * BAND);
    tm = band * BAND + in_band % rows_here;
    tn = in_band / rows_here;
}

// ---- store of a workgroup tile.  The MFMAs take the weight fragment as their first operand, so an
// accumulator tile is the transpose of the output tile: lane l holds output row l % 32 and, in elements
// 4q..4q+3, the four neighbouring output columns 8q + 4*(l/32) + 0..3 -- one 8-byte piece of a row.  Each
// wave turns one 32-row strip of its tile at a time into row-major 16-bit values in its own LDS patch (the
// operand buffers are free by now) and writes it out, and reads the residual, 16 bytes per lane, rows
// contiguous.
// at(i, j, e): element e of the accumulator of MFMA tile (i, j), as f32 ready to be rounded.
template <typename T, typename G, int EPI, typename AccAt>
__device__ __forceinline__ void gemm_store(AccAt at, uint16_t *lds, T *C, const T *R, int M, int N, int m0,
                                           int n0, int wrow, int wcol, int lane, int wave) {
    constexpr int TI = G::TI, TJ = G::TJ;
    constexpr int EST = G::EST;
    static_assert(EPI != GEMM_SWIGLU || TJ % 2 == 0, "the SwiGLU store pairs neighbouring column tiles");
    constexpr int OC = EPI == GEMM_SWIGLU ? TJ * 16 : TJ * 32;  // output columns of the wave tile
    constexpr int CPR = OC / 8;                                 // 16-byte chunks per strip row
    const int ldc = EPI == GEMM_SWIGLU ? N >> 1 : N;
    const int c0 = EPI == GEMM_SWIGLU ? (n0 + wcol) >> 1 : n0 + wcol;
    T *patch = (T *)lds + (size_t)wave * 32 * EST;
    const bool vec_ok = (ldc & 7) == 0;
#pragma unroll
    for (int i = 0; i < TI; i++) {
        T *prow = patch + (lane & 31) * EST + (lane >> 5) * 4;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            if (EPI == GEMM_SWIGLU) {
#pragma unroll
                for (int j = 0; j < TJ; j += 2) {
                    float o[4];
#pragma unroll
                    for (int x = 0; x < 4; x++) {
                        const float g = Elem<T>::rnd(at(i, j, 4 * q + x)), u = Elem<T>::rnd(at(i, j + 1, 4 * q + x));
                        // hardware 2^x and reciprocal (about 1 ulp of f32 each, far below the 16-bit rounding that
                        // follows); the exact expf and division cost ~35 instructions per element here
                        const float sig = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g * -1.4426950408889634f));
                        o[x] = (g * sig) * u;
                    }
                    *(uint2 *)(prow + j * 16 + 8 * q) = uint2{pack2<T>(o[0], o[1]), pack2<T>(o[2], o[3])};
                }
            } else {
#pragma unroll
                for (int j = 0; j < TJ; j++)
                    *(uint2 *)(prow + j * 32 + 8 * q) = uint2{pack2<T>(at(i, j, 4 * q), at(i, j, 4 * q + 1)),
                                                              pack2<T>(at(i, j, 4 * q + 2), at(i, j, 4 * q + 3))};
            }
        }
        __builtin_amdgcn_wave_barrier();
        const int row0 = m0 + wrow + i * 32;
#pragma unroll
        for (int q = 0; q < 32 * CPR / 64; q++) {
            const int ch = q * 64 + lane, r = ch / CPR, cc = (ch % CPR) * 8;
            const int row = row0 + r, col = c0 + cc;
            if (row >= M || col >= ldc) continue;
            U4 v = *(const U4 *)&patch[r * EST + cc];
            const size_t at = (size_t)row * ldc + col;
            if (vec_ok && col + 8 <= ldc) {
                if (EPI == GEMM_RESIDUAL) {
                    float fv[8], fr8[8];
                    widen8<T>(v, fv);
                    widen8<T>(*(const U4 *)(R + at), fr8);
                    v = U4{pack2<T>(fr8[0] + fv[0], fr8[1] + fv[1]), pack2<T>(fr8[2] + fv[2], fr8[3] + fv[3]),
                           pack2<T>(fr8[4] + fv[4], fr8[5] + fv[5]), pack2<T>(fr8[6] + fv[6], fr8[7] + fv[7])};
                }
                *(U4 *)(C + at) = v;
            } else {
                for (int x = 0; x < 8 && col + x < ldc; x++) {
                    const float f = Elem<T>::ld(patch, r * EST + cc + x);
                    if (EPI == GEMM_RESIDUAL) Elem<T>::st(C, at + x, Elem<T>::ld(R, at + x) + f);
                    else C[at + x] = patch[r * EST + cc + x];
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
}

// KTAIL: K is not a multiple of 2*BK, so the last steps mask the columns of A past K.
// EPI: GEMM_PLAIN C = T(acc); GEMM_RESIDUAL C = T(R + T(acc)) with R laid out like C;
// GEMM_SWIGLU: B's rows are gate/up interleaved in groups of 32, C is [M, N/2] and
// C = T(swish(T(acc_gate)) * T(acc_up)) -- the roundings of separate linear, Add and SwiGLU ops.
template <typename T, typename G, bool KTAIL, int EPI>
__global__ __launch_bounds__(G::THREADS) void gemm_nt_mfma_kernel(T *C, const T *A, const T *B, const T *R, int M, int N,
                                                                 int K, int Kp) {
    constexpr int BM = G::BM, BN = G::BN, TI = G::TI, TJ = G::TJ, CA = G::CA, CB = G::CB, RPP = G::ROWS_PER_PASS;
    extern __shared__ __align__(16) uint16_t lds[];
    uint16_t *As = lds, *Bs = lds + 2 * BM * LDT;  // As[buf] = As + buf*BM*LDT, Bs[buf] = Bs + buf*BN*LDT
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / G::WN, wn = wave % G::WN;
    const int wrow = wm * TI * 32, wcol = wn * TJ * 32;  // wave tile origin inside the workgroup tile
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    int tm, tn;
    tile_of(blockIdx.x, gridDim.x, tiles_m, tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;

    // global -> register staging, 16 bytes per load.  Two register sets: tile kt+1 waits in one while
    // tile kt+2 is still in flight in the other.  Branch-free: rows past M / N re-read the last row
    // (their products land in rows that are never stored) and columns past K are masked to zero when
    // the registers are consumed, so the compiler can wait for exactly the older set.
    const int lr = tid >> 2, lc = (tid & 3) * 8;
    struct Stage { U4 a[CA], b[CB]; uint32_t mask; };
    const T *ap[CA], *bp[CB];
#pragma unroll
    for (int q = 0; q < CA; q++) ap[q] = A + (size_t)min(m0 + lr + q * RPP, M - 1) * K;
#pragma unroll
    for (int q = 0; q < CB; q++) bp[q] = B + (size_t)min(n0 + lr + q * RPP, N - 1) * Kp;
    auto load_tiles = [&](Stage &r, int k0) {
        const int ka = min(k0 + lc, K - 8);
        if (KTAIL) r.mask = k0 + lc < K ? 0xFFFFFFFFu : 0u;
#pragma unroll
        for (int q = 0; q < CA; q++) r.a[q] = *(const U4 *)(ap[q] + ka);
#pragma unroll
        for (int q = 0; q < CB; q++) r.b[q] = *(const U4 *)(bp[q] + k0 + lc);
    };
    auto store_tiles = [&](int buf, const Stage &r) {
#pragma unroll
        for (int q = 0; q < CA; q++)
            *(U4 *)&As[buf * BM * LDT + (lr + q * RPP) * LDT + lc] = KTAIL ? r.a[q] & r.mask : r.a[q];
#pragma unroll
        for (int q = 0; q < CB; q++) *(U4 *)&Bs[buf * BN * LDT + (lr + q * RPP) * LDT + lc] = r.b[q];
    };

    f16x_t acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; i++)
#pragma unroll
        for (int j = 0; j < TJ; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

    const int fr = lane & 31, fk = (lane >> 5) * 8;  // fragment row within a 32-row tile, k offset
    auto multiply = [&](int buf) {
#pragma unroll
        for (int ks = 0; ks < BK; ks += 16) {
            U4 fa[TI], fb[TJ];
#pragma unroll
            for (int i = 0; i < TI; i++) fa[i] = *(const U4 *)&As[buf * BM * LDT + (wrow + i * 32 + fr) * LDT + ks + fk];
#pragma unroll
            for (int j = 0; j < TJ; j++) fb[j] = *(const U4 *)&Bs[buf * BN * LDT + (wcol + j * 32 + fr) * LDT + ks + fk];
#pragma unroll
            for (int i = 0; i < TI; i++)
#pragma unroll
                for (int j = 0; j < TJ; j++) acc[i][j] = Mfma<T>::run(fb[j], fa[i], acc[i][j]);
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

    gemm_store<T, G, EPI>([&](int i, int j, int e) { return acc[i][j][e]; }, lds, C, R, M, N, m0, n0, wrow, wcol, lane, wave);
}

// ---- the same product with the operand tiles copied global -> LDS by the load unit itself
// (global_load_lds_dwordx4: no register staging, no LDS store instructions).  A wave's load instruction
// fills 1 KB of LDS lane by lane, so padding is impossible; instead the 16-byte chunks of a tile (8 per
// row at K step 64) are placed at position 8*row + (chunk ^ ((row >> 1) & 7)), which keeps the chunks of a
// row together (one full 128-byte line per row in global memory) and makes the 128-bit fragment reads
// conflict-free.  Two LDS stages of 64 KB: the loads of tile kt+2 are issued as soon as everyone has
// finished reading tile kt and fly during tile kt+1; one barrier per K tile, a bare s_barrier with explicit
// counter waits.  Fragments of the next 16-k step are read while the current one multiplies.
// 256 x 256 tile, 8 waves of 128 x 64; or 256 x 320, 8 waves of 64 x 160, for widths that this turns into
// a whole number of rounds over the CUs (N = 2560: 256 tiles instead of 320).  Needs K % 64 == 0.
using TileDma = GemmTile<256, 256, 2, 4>;
using TileDma320 = GemmTile<256, 320, 4, 2>;
constexpr int DBK = 64;
template <typename G> constexpr int dma_stage_elems() { return (G::BM + G::BN) * DBK; }  // A tile then B tile
template <typename G> constexpr size_t dma_lds_bytes() { return (size_t)2 * dma_stage_elems<G>() * 2; }

// I8: the operands are int8 (QuantizedMatMul: A = activations quantised per row, B = the int8 weights), the
// K tile is the same 128 bytes per row = 128 values, the MFMA is v_mfma_i32_32x32x32_i8 over the same 16-byte
// fragments, the sum is exact int32 (optionally written out) and the store applies the two scales.
typedef int i4x_t __attribute__((ext_vector_type(4)));
typedef int i16x_t __attribute__((ext_vector_type(16)));

template <typename T, typename G, int EPI, bool I8>
__global__ __launch_bounds__(G::THREADS) void gemm_nt_dma_kernel(T *C, const void *A_, const void *B_, const T *R, int M, int N,
                                                                 int K, int Kp, const T *a_scale, const T *b_scale,
                                                                 int32_t *acc_out) {
    constexpr int TI = G::TI, TJ = G::TJ, KS = DBK / 16, BM = G::BM, BN = G::BN;
    constexpr int EB = I8 ? 1 : 2;            // bytes per operand value
    constexpr int TILE_B = DBK * 2;           // bytes of one row of a K tile
    const char *A = (const char *)A_, *B = (const char *)B_;
    constexpr int CHA = BM * 8 / G::THREADS, CHB = BN * 8 / G::THREADS;  // 16-byte chunks per thread per operand tile
    constexpr int kDmaStage = dma_stage_elems<G>();
    static_assert(BM * 8 % G::THREADS == 0 && BN * 8 % G::THREADS == 0, "whole load instructions per wave");
    extern __shared__ __align__(16) uint16_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / G::WN, wn = wave % G::WN;
    const int wrow = wm * TI * 32, wcol = wn * TJ * 32;
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    int tm, tn;
    tile_of(blockIdx.x, gridDim.x, tiles_m, tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;

    // this lane's chunks of each operand tile: LDS position P = (CH*wave + i)*64 + lane
    const char *asrc[CHA], *bsrc[CHB];
#pragma unroll
    for (int i = 0; i < CHA; i++) {
        const int P = (CHA * wave + i) * 64 + lane, r = P >> 3, c = (P & 7) ^ ((r >> 1) & 7);
        asrc[i] = A + (size_t)min(m0 + r, M - 1) * K * EB + c * 16;
    }
#pragma unroll
    for (int i = 0; i < CHB; i++) {
        const int P = (CHB * wave + i) * 64 + lane, r = P >> 3, c = (P & 7) ^ ((r >> 1) & 7);
        bsrc[i] = B + (size_t)min(n0 + r, N - 1) * Kp * EB + c * 16;
    }
    auto issue = [&](int kt, int stage) {
        uint16_t *dst = lds + stage * kDmaStage;  // wave-uniform destinations; the lane offset is implicit
#pragma unroll
        for (int i = 0; i < (CHA > CHB ? CHA : CHB); i++) {
            if (i < CHA)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(asrc[i] + (size_t)kt * TILE_B),
                                                 (__attribute__((address_space(3))) void *)(dst + (CHA * wave + i) * 512), 16, 0, 0);
            if (i < CHB)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(bsrc[i] + (size_t)kt * TILE_B),
                                                 (__attribute__((address_space(3))) void *)(dst + BM * DBK + (CHB * wave + i) * 512), 16, 0, 0);
        }
    };

    using acc_t = std::conditional_t<I8, i16x_t, f16x_t>;
    acc_t acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; i++)
#pragma unroll
        for (int j = 0; j < TJ; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0;

    // fragment addresses (elements) inside a stage: row r, chunk c = 2*ks + g  ->  (8r + (c ^ swz)) * 8
    const int fr = lane & 31, g = lane >> 5;
    int arow8[TI], aswz[TI], brow8[TJ], bswz[TJ];
#pragma unroll
    for (int i = 0; i < TI; i++) {
        const int r = wrow + i * 32 + fr;
        arow8[i] = 64 * r;
        aswz[i] = (r >> 1) & 7;
    }
#pragma unroll
    for (int j = 0; j < TJ; j++) {
        const int r = wcol + j * 32 + fr;
        brow8[j] = BM * DBK + 64 * r;
        bswz[j] = (r >> 1) & 7;
    }
    auto read_frags = [&](const uint16_t *st, int ks, U4 *fa, U4 *fb) {
        const int c = 2 * ks + g;
#pragma unroll
        for (int i = 0; i < TI; i++) fa[i] = *(const U4 *)&st[arow8[i] + ((c ^ aswz[i]) << 3)];
#pragma unroll
        for (int j = 0; j < TJ; j++) fb[j] = *(const U4 *)&st[brow8[j] + ((c ^ bswz[j]) << 3)];
    };

    auto multiply = [&](const U4 *fa, const U4 *fb) {
#pragma unroll
        for (int i = 0; i < TI; i++)
#pragma unroll
            for (int j = 0; j < TJ; j++) {
                if constexpr (I8)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i4x_t, fb[j]), __builtin_bit_cast(i4x_t, fa[i]),
                                                                      acc[i][j], 0, 0, 0);
                else
                    acc[i][j] = Mfma<T>::run(fb[j], fa[i], acc[i][j]);
            }
    };

    // Schedule of one K tile (4 steps of 16): steps 0..2 multiply while the fragments of the next step are
    // read; then the one synchronisation point of the tile -- this wave's reads of the tile are complete
    // and its share of the next tile has landed, so after the barrier the next tile is whole and the stage
    // of this one is free; step 3 multiplies while the loads of tile kt+2 are issued into that stage and the
    // first fragments of tile kt+1 are read.  Left alone the instruction scheduler sinks every LDS read to
    // just before its first use and exposes the LDS latency once per step; the sched_group_barrier
    // sequences pin the interleaving (one read or load, then its share of the MFMAs).
    const int nk = K * EB / TILE_B;
    U4 fa[2][TI], fb[2][TJ];
    issue(0, 0);
    issue(min(1, nk - 1), 1);
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    read_frags(lds, 0, fa[0], fb[0]);
    __builtin_amdgcn_sched_barrier(0);
    for (int kt = 0; kt < nk; kt++) {
        const uint16_t *st = lds + (kt & 1) * kDmaStage, *nx = lds + ((kt + 1) & 1) * kDmaStage;
#pragma unroll
        for (int ks = 0; ks + 1 < KS; ks++) {
            read_frags(st, ks + 1, fa[(ks + 1) & 1], fb[(ks + 1) & 1]);
            multiply(fa[ks & 1], fb[ks & 1]);
#pragma unroll
            for (int n = 0; n < TI + TJ; n++) {  // reads early in the step, so the last has landed by its end
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            }
            __builtin_amdgcn_sched_group_barrier(0x008, TI * TJ - (TI + TJ), 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        read_frags(nx, 0, fa[0], fb[0]);     // (after the last tile: stale data, never used)
        issue(min(kt + 2, nk - 1), kt & 1);  // (past the end: a repeat of the last tile, never read)
        multiply(fa[(KS - 1) & 1], fb[(KS - 1) & 1]);
        // LDS reads first (the compiler keeps them ahead of the LDS-writing loads anyway), two per MFMA,
        // then the loads spread over the remaining MFMAs
        constexpr int RD_MFMA = (TI + TJ + 1) / 2, LD_MFMA = TI * TJ - RD_MFMA;
#pragma unroll
        for (int n = 0; n < RD_MFMA; n++) {
            __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
#pragma unroll
        for (int n = 0; n < LD_MFMA; n++) {
            __builtin_amdgcn_sched_group_barrier(0x010, (CHA + CHB + LD_MFMA - 1) / LD_MFMA, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // the repeat of the last tile too, before LDS is reused
    __syncthreads();
    if constexpr (I8) {
        // accumulator tile = transposed output tile: lane l has output row l % 32 of strip i, and in elements
        // 4q..4q+3 the columns 8q + 4*(l/32) + 0..3 of column tile j
        if (acc_out) {
#pragma unroll
            for (int i = 0; i < TI; i++)
#pragma unroll
                for (int j = 0; j < TJ; j++)
#pragma unroll
                    for (int e = 0; e < 16; e++) {
                        const int row = m0 + wrow + i * 32 + (lane & 31);
                        const int col = n0 + wcol + j * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                        if (row < M && col < N) acc_out[(size_t)row * N + col] = acc[i][j][e];
                    }
        }
        if (C) {
            // the column scales of the tile as f32 in the top of LDS (above the store patches), the row scales in
            // registers; out = T(((f32)sum * row scale) * column scale)
            float *bs = (float *)((char *)lds + dma_lds_bytes<G>() - BN * sizeof(float));
            for (int c = tid; c < BN; c += G::THREADS) bs[c] = n0 + c < N ? Elem<T>::ld(b_scale, n0 + c) : 0.f;
            float asc[TI];
#pragma unroll
            for (int i = 0; i < TI; i++) {
                const int row = m0 + wrow + i * 32 + (lane & 31);
                asc[i] = row < M ? Elem<T>::ld(a_scale, row) : 0.f;
            }
            __syncthreads();
            const float *bw = bs + wcol + 4 * (lane >> 5);
            gemm_store<T, G, EPI>([&](int i, int j, int e) { return ((float)acc[i][j][e] * asc[i]) * bw[j * 32 + 8 * (e >> 2) + (e & 3)]; },
                                  lds, C, R, M, N, m0, n0, wrow, wcol, lane, wave);
        }
    } else {
        gemm_store<T, G, EPI>([&](int i, int j, int e) { return acc[i][j][e]; }, lds, C, R, M, N, m0, n0, wrow, wcol, lane, wave);
    }
}

static int gemm_kp(int K) { return (K + 2 * BK - 1) / (2 * BK) * (2 * BK); }  // the GEMM walks K in pairs of steps

size_t gemm_weight_bytes(int N, int K) { return (size_t)N * gemm_kp(K) * 2; }

int dequant_weight_rows(void *dst, const int8_t *wq, const void *scale, int N, int K, int dtype, int group, int which,
                        hipStream_t s) {
    MYNN_REQUIRE(dst && wq && scale, MYNN_ERR_INVALID, "dequant_matmul: null operand");
    MYNN_REQUIRE(N > 0 && K > 0, MYNN_ERR_INVALID, "dequant_matmul: N=%d K=%d", N, K);
    MYNN_REQUIRE(K % 8 == 0, MYNN_ERR_UNSUPPORTED, "dequant_matmul (matrix cores): K=%d is not a multiple of 8", K);
    MYNN_REQUIRE(((uintptr_t)wq & 7) == 0 && aligned16(dst), MYNN_ERR_INVALID, "dequant_matmul: wq must be 8-byte aligned");
    MYNN_REQUIRE(group == 0 || N % group == 0, MYNN_ERR_INVALID, "dequant_matmul: N=%d is not a multiple of the group %d", N, group);
    const int Kp = gemm_kp(K);
    const size_t chunks = (size_t)N * Kp / 8;
    return dispatch_dtype16(dtype, [&](auto *t) {
        using T = std::remove_pointer_t<decltype(t)>;
        MYNN_LAUNCH(dequant_rows_kernel<T>, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, s, (T *)dst, wq,
                           (const T *)scale, K, Kp, chunks, group, which);
        return launch_status("dequant_rows_kernel");
    });
}

template <typename T, typename G, int EPI>
static int gemm_launch_tile(void *out, const void *act, const void *wt, const void *res, int M, int N, int K,
                            hipStream_t s) {
    const int Kp = gemm_kp(K);
    const int tiles = ((M + G::BM - 1) / G::BM) * ((N + G::BN - 1) / G::BN);
    static bool lds_set = false;  // the kernels want more LDS than the 64 KB default
    if (!lds_set) {
        MYNN_HIP(hipFuncSetAttribute((const void *)gemm_nt_mfma_kernel<T, G, false, EPI>,
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)G::LDS));
        MYNN_HIP(hipFuncSetAttribute((const void *)gemm_nt_mfma_kernel<T, G, true, EPI>,
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)G::LDS));
        lds_set = true;
    }
    if (K == Kp)
        MYNN_LAUNCH((gemm_nt_mfma_kernel<T, G, false, EPI>), dim3(tiles), dim3(G::THREADS), G::LDS, s, (T *)out,
                           (const T *)act, (const T *)wt, (const T *)res, M, N, K, Kp);
    else
        MYNN_LAUNCH((gemm_nt_mfma_kernel<T, G, true, EPI>), dim3(tiles), dim3(G::THREADS), G::LDS, s, (T *)out,
                           (const T *)act, (const T *)wt, (const T *)res, M, N, K, Kp);
    return launch_status("gemm_nt_mfma_kernel");
}

template <typename T, typename G, int EPI, bool I8 = false>
static int gemm_launch_dma(void *out, const void *act, const void *wt, const void *res, int M, int N, int K, hipStream_t s,
                           const void *a_scale = nullptr, const void *b_scale = nullptr, int32_t *acc_out = nullptr) {
    static bool lds_set = false;
    if (!lds_set) {
        MYNN_HIP(hipFuncSetAttribute((const void *)gemm_nt_dma_kernel<T, G, EPI, I8>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)dma_lds_bytes<G>()));
        lds_set = true;
    }
    const int tiles = ((M + G::BM - 1) / G::BM) * ((N + G::BN - 1) / G::BN);
    MYNN_LAUNCH((gemm_nt_dma_kernel<T, G, EPI, I8>), dim3(tiles), dim3(G::THREADS), dma_lds_bytes<G>(), s, (T *)out, act, wt,
                (const T *)res, M, N, K, I8 ? K : gemm_kp(K), (const T *)a_scale, (const T *)b_scale, acc_out);
    return launch_status("gemm_nt_dma_kernel");
}

// QuantizedMatMul on the matrix cores for a grid of at least one round of 256-row tiles: K % 128 == 0.
// out (scaled, storage type; optionally + residual) and / or acc_out (exact int32).
bool qgemm_dma_supported(int M, int N, int K) {
    return K % 128 == 0 && (long)((M + 255) / 256) * ((N + 255) / 256) >= 128;
}
int qgemm_dma(void *out, int32_t *acc_out, const int8_t *lhs, const void *lhs_scale, const int8_t *rhs, const void *rhs_scale,
              const void *res, int M, int N, int K, int dtype, int epi, hipStream_t s) {
    MYNN_REQUIRE(qgemm_dma_supported(M, N, K), MYNN_ERR_UNSUPPORTED, "quantized_matmul (large tiles): M=%d N=%d K=%d", M, N, K);
    MYNN_REQUIRE(epi != GEMM_RESIDUAL || res, MYNN_ERR_INVALID, "quantized_matmul: residual store without a residual");
    MYNN_REQUIRE(epi != GEMM_SWIGLU || (N % 64 == 0 && !acc_out), MYNN_ERR_INVALID, "quantized_matmul: SwiGLU store needs N %% 64 == 0, N=%d", N);
    return dispatch_dtype16(dtype, [&](auto *t) {
        using T = std::remove_pointer_t<decltype(t)>;
        const long t256 = (long)((M + 255) / 256) * ((N + 255) / 256), t320 = (long)((M + 255) / 256) * ((N + 319) / 320);
        const bool wide = (t320 + 255) / 256 * 320 < (t256 + 255) / 256 * 256;
        if (epi == GEMM_SWIGLU)
            return gemm_launch_dma<T, TileDma, GEMM_SWIGLU, true>(out, lhs, rhs, nullptr, M, N, K, s, lhs_scale, rhs_scale, nullptr);
        if (epi == GEMM_RESIDUAL) {
            if (wide) return gemm_launch_dma<T, TileDma320, GEMM_RESIDUAL, true>(out, lhs, rhs, res, M, N, K, s, lhs_scale, rhs_scale, acc_out);
            return gemm_launch_dma<T, TileDma, GEMM_RESIDUAL, true>(out, lhs, rhs, res, M, N, K, s, lhs_scale, rhs_scale, acc_out);
        }
        if (wide) return gemm_launch_dma<T, TileDma320, GEMM_PLAIN, true>(out, lhs, rhs, nullptr, M, N, K, s, lhs_scale, rhs_scale, acc_out);
        return gemm_launch_dma<T, TileDma, GEMM_PLAIN, true>(out, lhs, rhs, nullptr, M, N, K, s, lhs_scale, rhs_scale, acc_out);
    });
}

// tile: 0 = heuristic, 1 = 256x128, 2 = 256x256 via registers, 3 = 256x256 / 4 = 256x320 direct to LDS
template <typename T, int EPI>
static int gemm_launch(void *out, const void *act, const void *wt, const void *res, int M, int N, int K, int tile, hipStream_t s) {
    const int g_gemm_tile_override = tile;
    // the large tile needs fewer LDS reads per MFMA (measured 10-25% faster) but runs one workgroup per CU:
    // it is chosen once it fills the 256 CUs at least once (a partly filled second round still wins: the
    // CUs left running clock higher)
    const long big_tiles = (long)((M + 255) / 256) * ((N + 255) / 256);
    bool big = big_tiles >= 256;
    if (g_gemm_tile_override) big = g_gemm_tile_override == 2;
    // the direct-to-LDS kernel is the faster 256 x 256 one (measured +5..20%); it needs whole 64-wide K steps
    const bool dma_ok = K % 64 == 0 && g_gemm_tile_override != 2;
    if (g_gemm_tile_override == 3 || g_gemm_tile_override == 4) big = dma_ok;
    if constexpr (EPI != GEMM_SWIGLU) {
        // 320 columns per tile when that saves rounds over the CUs (rounds x tile width = time)
        const long wide_tiles = (long)((M + 255) / 256) * ((N + 319) / 320);
        const long cost256 = (big_tiles + 255) / 256 * 256, cost320 = (wide_tiles + 255) / 256 * 320;
        const bool wide = g_gemm_tile_override ? g_gemm_tile_override == 4 : (big && cost320 < cost256);
        if (wide && dma_ok) return gemm_launch_dma<T, TileDma320, EPI>(out, act, wt, res, M, N, K, s);
    }
    if (big && dma_ok) return gemm_launch_dma<T, TileDma, EPI>(out, act, wt, res, M, N, K, s);
    if (big) return gemm_launch_tile<T, Tile256x256, EPI>(out, act, wt, res, M, N, K, s);
    return gemm_launch_tile<T, Tile256x128, EPI>(out, act, wt, res, M, N, K, s);
}

int gemm_nt_mfma(void *out, const void *act, const void *wt, const void *res, int M, int N, int K, int dtype, int epi,
                 hipStream_t s, int tile) {
    MYNN_REQUIRE(tile >= 0 && tile <= 4, MYNN_ERR_INVALID,
                 "gemm tile %d is not 0 (automatic), 1 (256x128), 2 (256x256), 3 (256x256, direct-to-LDS loads) or 4 (256x320, direct-to-LDS loads)", tile);
    MYNN_REQUIRE(out && act && wt, MYNN_ERR_INVALID, "dequant_matmul: null operand");
    MYNN_REQUIRE(M > 0 && N > 0 && K > 0 && K % 8 == 0, MYNN_ERR_INVALID, "dequant_matmul: M=%d N=%d K=%d", M, N, K);
    MYNN_REQUIRE(aligned16(act) && aligned16(wt), MYNN_ERR_INVALID, "dequant_matmul: act must be 16-byte aligned");
    MYNN_REQUIRE(epi != GEMM_RESIDUAL || res, MYNN_ERR_INVALID, "dequant_matmul: residual store without a residual");
    MYNN_REQUIRE(epi != GEMM_SWIGLU || N % 64 == 0, MYNN_ERR_INVALID, "dequant_matmul: SwiGLU store needs N %% 64 == 0, N=%d", N);
    return dispatch_dtype16(dtype, [&](auto *t) {
        using T = std::remove_pointer_t<decltype(t)>;
        if (epi == GEMM_RESIDUAL) return gemm_launch<T, GEMM_RESIDUAL>(out, act, wt, res, M, N, K, tile, s);
        if (epi == GEMM_SWIGLU) return gemm_launch<T, GEMM_SWIGLU>(out, act, wt, res, M, N, K, tile, s);
        return gemm_launch<T, GEMM_PLAIN>(out, act, wt, res, M, N, K, tile, s);
    });
}

// ---- library-owned workspaces of the stand-alone entry point: one per stream, so calls on different streams never
// share a dequantised weight; the table is guarded by a mutex.  A workspace only ever grows, and growing waits for
// the stream's earlier work before the old block is released.
struct StreamWs {
    void *ptr = nullptr;
    size_t bytes = 0;
};
static std::mutex g_ws_mu;
static std::map<hipStream_t, StreamWs> g_ws;

static int stream_workspace(hipStream_t s, size_t need, void **out) {
    std::lock_guard<std::mutex> lk(g_ws_mu);
    StreamWs &w = g_ws[s];
    if (need > w.bytes) {
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(s, &cs) == hipSuccess && cs != hipStreamCaptureStatusNone)
            return fail(MYNN_ERR_STATE, "dequant_matmul: the library workspace cannot grow while the stream is being captured; "
                                        "pass a workspace (mynn_dequant_matmul_ws) or a prepared weight");
        MYNN_HIP(hipStreamSynchronize(s));
        if (w.ptr) MYNN_HIP(hipFree(w.ptr));
        w = StreamWs{};
        MYNN_HIP(hipMalloc(&w.ptr, need));
        w.bytes = need;
    }
    *out = w.ptr;
    return 0;
}

int dequant_gemm_mfma(void *out, const void *act, const int8_t *wq, const void *scale, int M, int N, int K, int dtype, void *ws,
                      int tile, hipStream_t s) {
    int rc = dequant_weight_rows(ws, wq, scale, N, K, dtype, 0, 0, s);
    if (rc) return rc;
    return gemm_nt_mfma(out, act, ws, nullptr, M, N, K, dtype, GEMM_PLAIN, s, tile);
}

// the reference's kernel choice (cuda.rs:1518-1652): matrix cores for M >= 16 with 16-bit operands
static bool takes_matrix_cores(const void *act, const int8_t *wq, int M, int K, int act_dtype, int out_dtype) {
    const bool sixteen = act_dtype != MYNN_F32 && out_dtype != MYNN_F32 && act_dtype == out_dtype;
    return M >= 16 && sixteen && K % 8 == 0 && aligned16(act) && ((uintptr_t)wq & 7) == 0;
}

}  // namespace mynn

using namespace mynn;

extern "C" size_t mynn_dequant_matmul_workspace_bytes(int M, int N, int K, int act_dtype, int out_dtype) {
    if (M < 16 || N <= 0 || K <= 0 || K % 8 != 0 || act_dtype == MYNN_F32 || act_dtype != out_dtype) return 0;
    return gemm_weight_bytes(N, K);
}

extern "C" int mynn_dequant_matmul_ws(void *out, const void *act, const int8_t *wq, const void *scale, int M, int N, int K,
                                      int act_dtype, int out_dtype, void *workspace, size_t workspace_bytes, int gemm_tile,
                                      mynn_stream s) {
    MYNN_REQUIRE(M >= 1, MYNN_ERR_INVALID, "dequant_matmul: M=%d", M);
    if (takes_matrix_cores(act, wq, M, K, act_dtype, out_dtype)) {
        MYNN_REQUIRE(N > 0 && K > 0, MYNN_ERR_INVALID, "dequant_matmul: N=%d K=%d", N, K);
        MYNN_REQUIRE(workspace && aligned16(workspace) && workspace_bytes >= gemm_weight_bytes(N, K), MYNN_ERR_INVALID,
                     "dequant_matmul: the workspace must hold %zu bytes (mynn_dequant_matmul_workspace_bytes), 16-byte aligned",
                     gemm_weight_bytes(N, K));
        return dequant_gemm_mfma(out, act, wq, scale, M, N, K, out_dtype, workspace, gemm_tile, as_stream(s));
    }
    return dequant_gemv_dispatch(out, act, wq, scale, M, N, K, act_dtype, out_dtype, as_stream(s));
}

extern "C" int mynn_dequant_matmul(void *out, const void *act, const int8_t *wq, const void *scale, int M, int N,
                                   int K, int act_dtype, int out_dtype, mynn_stream s) {
    MYNN_REQUIRE(M >= 1, MYNN_ERR_INVALID, "dequant_matmul: M=%d", M);
    if (takes_matrix_cores(act, wq, M, K, act_dtype, out_dtype)) {
        MYNN_REQUIRE(N > 0 && K > 0, MYNN_ERR_INVALID, "dequant_matmul: N=%d K=%d", N, K);
        void *ws = nullptr;
        int rc = stream_workspace(as_stream(s), gemm_weight_bytes(N, K), &ws);
        if (rc) return rc;
        return dequant_gemm_mfma(out, act, wq, scale, M, N, K, out_dtype, ws, 0, as_stream(s));
    }
    return dequant_gemv_dispatch(out, act, wq, scale, M, N, K, act_dtype, out_dtype, as_stream(s));
}

extern "C" size_t mynn_dequant_weight_bytes(int N, int K) { return N > 0 && K > 0 ? gemm_weight_bytes(N, K) : 0; }

extern "C" int mynn_dequant_weight_prepare(void *wt, const int8_t *wq, const void *scale, int N, int K, int dtype, mynn_stream s) {
    return dequant_weight_rows(wt, wq, scale, N, K, dtype, 0, 0, as_stream(s));
}

extern "C" int mynn_dequant_matmul_prepared(void *out, const void *act, const void *wt, int M, int N, int K, int dtype,
                                            int gemm_tile, mynn_stream s) {
    MYNN_REQUIRE(M >= 16, MYNN_ERR_UNSUPPORTED, "dequant_matmul_prepared: M=%d (the prepared weight serves the matrix-core path, M >= 16)", M);
    return gemm_nt_mfma(out, act, wt, nullptr, M, N, K, dtype, GEMM_PLAIN, as_stream(s), gemm_tile);
}
