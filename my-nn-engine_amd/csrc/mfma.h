// Thin wrappers over the gfx950 matrix-core builtins used by the GEMM and attention kernels.
// v_mfma_f32_32x32x16_{f16,bf16}: A is 32 x 16 (lane l holds row l%32, k = 8*(l/32) .. +7),
// B is 16 x 32 (lane l holds column l%32, k = 8*(l/32) .. +7), D is 32 x 32 f32 (lane l holds
// column l%32 and the 16 rows 8*(e/4) + 4*(l/32) + e%4, e = 0..15).
#pragma once
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

// two f32 -> one dword of two storage-type values (low half first)
template <typename T> __device__ inline uint32_t pack2(float lo, float hi) {
    T a, b;
    Elem<T>::st(&a, 0, lo);
    Elem<T>::st(&b, 0, hi);
    return (uint32_t)__builtin_bit_cast(uint16_t, a) | ((uint32_t)__builtin_bit_cast(uint16_t, b) << 16);
}

}  // namespace mynn
