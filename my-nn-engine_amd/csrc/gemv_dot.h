// The inner product of the batch-1 GEMVs: how a workgroup keeps its staged activation row in LDS and how a lane
// multiplies its 16-byte weight chunks against it.  One definition for dequant_gemv1_kernel and the GEMV roles of
// qkv_attention_kernel, whose results must agree bit for bit.
//
// bf16 (and any other T): the row as f32 [K]; a weight byte is converted to f32 and multiplied with an FMA (two
// vector operations per weight).
// fp16: the row as fp16, the first and the second 8 elements of every 16-element chunk in two separate arrays (so that
// the lanes of a wave read consecutive 16-byte words), followed by one f32 bias term for every 8-element piece.  A
// weight byte b, as b ^ 0x80 under an 0x64 high byte, IS the fp16 number 1152 + b, and as b ^ 0x7F under an 0xE4 high
// byte the fp16 number b - 1151: one xor per four weights and one byte permute per two make an (even, odd) pair
// (1152 + b0, b1 - 1151), and v_dot2_f32_f16 multiplies it with two activations with f32 accumulation -- one vector
// operation per weight.  Every product is exact in f32.  The sums carry 1152 * (even activations) - 1151 * (odd
// activations), which is subtracted once per row before the lanes meet; the opposite signs matter: for activations
// with a non-zero mean (SwiGLU outputs, attention outputs) the two halves cancel inside every dot2, so the running
// sum stays near the size of the result instead of growing to 1152 * K/64 * mean and rounding at that magnitude.
// Semantics either way: out[n] = T(scale[n] * sum_k act[k] * wq[n,k]), scale after the f32 sum
// (dequant_gemv.cuh:12-59).
#pragma once
#include <type_traits>

#include "mynn_common.h"
#include "mfma.h"

namespace mynn {

template <typename T> constexpr bool kGemvDot2 = std::is_same<T, f16_t>::value;

// bytes of LDS for a row of K elements (K % 16 == 0)
template <typename T> __host__ __device__ constexpr size_t gemv_stage_bytes(int K) {
    return kGemvDot2<T> ? (size_t)K * 2 + (size_t)(K / 8) * 4 : (size_t)K * 4;
}

// piece pc = elements [8 pc, 8 pc + 8) of the row, values already rounded to T
template <typename T> __device__ inline void gemv_stage_piece(float *lds, int K, int pc, const float *f) {
    if constexpr (kGemvDot2<T>) {
        const U4 v = U4{pack2<T>(f[0], f[1]), pack2<T>(f[2], f[3]), pack2<T>(f[4], f[5]), pack2<T>(f[6], f[7])};
        U4 *half = (U4 *)lds + (pc & 1) * (K >> 4);  // [2][K / 16] words of 16 bytes
        half[pc >> 1] = v;
        // 1152 * (f0 + f2 + f4 + f6) - 1151 * (f1 + f3 + f5 + f7), as 1152 * (even - odd) + odd
        const float ev = (f[0] + f[2]) + (f[4] + f[6]), od = (f[1] + f[3]) + (f[5] + f[7]);
        lds[(K >> 1) + pc] = fmaf(1152.f, ev - od, od);
    } else {
        float4 *dst = (float4 *)(lds + pc * 8);
        dst[0] = float4{f[0], f[1], f[2], f[3]};
        dst[1] = float4{f[4], f[5], f[6], f[7]};
    }
}

// acc += sum over 16 weights of (1152 + w) * a (even elements) and (w - 1151) * a (odd elements)
// (w: 16 int8 of one 128-bit load, a0 / a1: the 16 fp16 activations)
__device__ inline float gemv_dot16_biased(const U4 &w, const U4 &a0, const U4 &a1, float acc) {
    const uint32_t x[4] = {w.x ^ 0x7F807F80u, w.y ^ 0x7F807F80u, w.z ^ 0x7F807F80u, w.w ^ 0x7F807F80u};
    const uint32_t a[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        // high bytes: 0x64 for the even element of a pair, 0xE4 for the odd one (bytes 0 and 1 of the constant)
        const uint32_t lo = __builtin_amdgcn_perm(0x6464E464u, x[i], 0x05010400u);
        const uint32_t hi = __builtin_amdgcn_perm(0x6464E464u, x[i], 0x05030402u);
        acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, a[2 * i]), __builtin_bit_cast(h2_t, lo), acc, false);
        acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, a[2 * i + 1]), __builtin_bit_cast(h2_t, hi), acc, false);
    }
    return acc;
}

// acc[r] = this lane's share of row r: chunks lane, lane + 64, .. of the R rows in w[r][j]
template <typename T, int R, int NC>
__device__ __forceinline__ void gemv_rows_dot(const float *lds, int K, int lane, U4 (*w)[NC], float *acc) {
    const int nchunks = K >> 4;
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.f;
    if constexpr (kGemvDot2<T>) {
        const U4 *lo = (const U4 *)lds, *hi = lo + nchunks;
        const float2 *psum = (const float2 *)(lds + (K >> 1));
        float bias = 0.f;
#pragma unroll
        for (int j = 0; j < NC; j++) {
            const int c = lane + j * kWave;
            if (c < nchunks) {
                const U4 a0 = lo[c], a1 = hi[c];
                const float2 s = psum[c];
                bias += s.x + s.y;
#pragma unroll
                for (int r = 0; r < R; r++) {
                    pin(w[r][j]);
                    acc[r] = gemv_dot16_biased(w[r][j], a0, a1, acc[r]);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] -= bias;
    } else {
#pragma unroll
        for (int j = 0; j < NC; j++) {
            const int c = lane + j * kWave;
            if (c < nchunks) {
                float a[16];
                const float4 *ap = (const float4 *)(lds + c * 16);
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    float4 t = ap[q];
                    a[4 * q] = t.x; a[4 * q + 1] = t.y; a[4 * q + 2] = t.z; a[4 * q + 3] = t.w;
                }
#pragma unroll
                for (int r = 0; r < R; r++) {
                    float wf[16];
                    pin(w[r][j]);
                    widen16_i8(w[r][j], wf);
#pragma unroll
                    for (int i = 0; i < 16; i++) acc[r] = fmaf(a[i], wf[i], acc[r]);
                }
            }
        }
    }
}

}  // namespace mynn
