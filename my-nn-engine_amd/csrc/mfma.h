// Thin wrappers over the gfx950 matrix-core builtins used by the GEMM and attention kernels.
// v_mfma_f32_32x32x16_{f16,bf16}: A is 32 x 16 (lane l holds row l%32, k = 8*(l/32) .. +7),
// B is 16 x 32 (lane l holds column l%32, k = 8*(l/32) .. +7), D is 32 x 32 f32 (lane l holds
// column l%32 and the 16 rows 8*(e/4) + 4*(l/32) + e%4, e = 0..15).
#pragma once
#include <type_traits>

#include "mynn_common.h"

namespace mynn {

typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef __bf16 b8_t __attribute__((ext_vector_type(8)));
typedef float f16x_t __attribute__((ext_vector_type(16)));

template <typename T> struct Mfma;
template <> struct Mfma<f16_t> {
    __device__ static f16x_t run(const U4 &a, const U4 &b, f16x_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8_t, a), __builtin_bit_cast(h8_t, b), c, 0, 0, 0);
    }
};
template <> struct Mfma<bf16_t> {
    __device__ static f16x_t run(const U4 &a, const U4 &b, f16x_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(b8_t, a), __builtin_bit_cast(b8_t, b), c, 0, 0, 0);
    }
};

// two f32 -> one dword of two storage-type values (low half first), round to nearest even: one packed
// convert instruction.  The inputs are values ALREADY rounded to f32 (the empty asm keeps the compiler from
// fusing the producing multiply into a mixed-precision op that would round the exact product once).
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));
template <typename T> __device__ inline uint32_t pack2(float lo, float hi);
template <> __device__ inline uint32_t pack2<f16_t>(float lo, float hi) {
    asm volatile("" : "+v"(lo), "+v"(hi));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2_t){lo, hi}, h2_t));
}
template <> __device__ inline uint32_t pack2<bf16_t>(float lo, float hi) {
    asm volatile("" : "+v"(lo), "+v"(hi));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2_t){lo, hi}, bf2_t));
}

// 8 int8 (two dwords) -> 8 values of T packed in a U4; exact
template <typename T> __device__ inline U4 i8x8_to_operand(uint32_t w0, uint32_t w1) {
    if constexpr (std::is_same<T, f16_t>::value) {
        // byte b + 128 under an 0x64 high byte is the fp16 number 1024 + (b + 128); subtract 1152
        const h2_t bias = {(_Float16)1152.f, (_Float16)1152.f};
        const uint32_t x0 = w0 ^ 0x80808080u, x1 = w1 ^ 0x80808080u;
        auto two = [&](uint32_t x, uint32_t sel) {
            const h2_t h = __builtin_bit_cast(h2_t, __builtin_amdgcn_perm(0x64646464u, x, sel)) - bias;
            return __builtin_bit_cast(uint32_t, h);
        };
        return U4{two(x0, 0x04010400u), two(x0, 0x04030402u), two(x1, 0x04010400u), two(x1, 0x04030402u)};
    } else {
        // |b| <= 128 has at most 8 significant bits: the upper half of its f32 form is the bf16 value
        auto two = [&](uint32_t w, int sh) {
            const float a = (float)(int8_t)((w >> sh) & 0xFF), b = (float)(int8_t)((w >> (sh + 8)) & 0xFF);
            return __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, b), __builtin_bit_cast(uint32_t, a), 0x07060302u);
        };
        return U4{two(w0, 0), two(w0, 16), two(w1, 0), two(w1, 16)};
    }
}

}  // namespace mynn
