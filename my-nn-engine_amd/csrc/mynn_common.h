// Shared device/host helpers for the gfx950 kernel library: storage types, conversions with the
// rounding the reference uses, wave64 reductions, launch-error plumbing.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include "../../include/mynn_hip.h"

namespace mynn {

constexpr int kWave = 64;

// ---- storage types -------------------------------------------------------------------------
struct bf16_t { uint16_t bits; };
using f16_t = _Float16;

// f32 -> bf16, round to nearest even: (bits + 0x7fff + lsb) >> 16, NaN -> 0x7FC0
// (reference: src/codegen/cpu/kernels/ftype.rs:41-50, crates/llm/src/quantize.rs:74-81)
__host__ __device__ inline uint16_t f32_to_bf16_bits(float x) {
    uint32_t u = __builtin_bit_cast(uint32_t, x);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}
__host__ __device__ inline float bf16_bits_to_f32(uint16_t b) {
    return __builtin_bit_cast(float, (uint32_t)b << 16);
}

template <typename T> struct Elem;
template <> struct Elem<float> {
    static constexpr int code = MYNN_F32;
    __host__ __device__ static float ld(const float *p, size_t i) { return p[i]; }
    __host__ __device__ static void st(float *p, size_t i, float v) { p[i] = v; }
    __host__ __device__ static float rnd(float v) { return v; }
};
template <> struct Elem<bf16_t> {
    static constexpr int code = MYNN_BF16;
    __host__ __device__ static float ld(const bf16_t *p, size_t i) { return bf16_bits_to_f32(p[i].bits); }
    __host__ __device__ static void st(bf16_t *p, size_t i, float v) { p[i].bits = f32_to_bf16_bits(v); }
    __host__ __device__ static float rnd(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }
};
// f32 -> f16, round to nearest even, of a value that has ALREADY been rounded to f32.  The empty
// asm keeps the compiler from folding the producing multiply into v_fma_mixlo_f16, which rounds
// the exact product straight to f16 (one rounding) and so differs from "f32 result, then narrow"
// (two roundings, what the reference's kernels do) whenever the f32 result is a tie.
__host__ __device__ inline f16_t f32_to_f16(float v) {
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("" : "+v"(v));
#endif
    return (f16_t)v;
}
template <> struct Elem<f16_t> {
    static constexpr int code = MYNN_F16;
    __host__ __device__ static float ld(const f16_t *p, size_t i) { return (float)p[i]; }
    __host__ __device__ static void st(f16_t *p, size_t i, float v) { p[i] = f32_to_f16(v); }
    __host__ __device__ static float rnd(float v) { return (float)f32_to_f16(v); }
};

inline size_t dtype_size(int dt) { return dt == MYNN_F32 ? 4 : 2; }
inline bool dtype_ok(int dt) { return dt == MYNN_F32 || dt == MYNN_BF16 || dt == MYNN_F16; }

// 8 consecutive 16-bit elements (one 128-bit load) widened to f32
typedef uint32_t U4 __attribute__((ext_vector_type(4)));

template <typename T> __device__ inline void widen8(const U4 &v, float *f);
template <> __device__ inline void widen8<bf16_t>(const U4 &v, float *f) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        f[2 * i] = __builtin_bit_cast(float, w[i] << 16);
        f[2 * i + 1] = __builtin_bit_cast(float, w[i] & 0xFFFF0000u);
    }
}
template <> __device__ inline void widen8<f16_t>(const U4 &v, float *f) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        f[2 * i] = (float)__builtin_bit_cast(f16_t, (uint16_t)(w[i] & 0xFFFFu));
        f[2 * i + 1] = (float)__builtin_bit_cast(f16_t, (uint16_t)(w[i] >> 16));
    }
}

// Pins a 128-bit register value at this point of the instruction stream: nothing computed from
// it can be scheduled earlier.  Used to keep int8 -> f32 converts next to their FMAs (left alone,
// the compiler converts every loaded chunk up front and quadruples the register count).
__device__ inline void pin(U4 &v) {
    asm volatile("" : "+v"(v.x), "+v"(v.y), "+v"(v.z), "+v"(v.w));
}

// 16 int8 (one 128-bit load) widened to f32
__device__ inline void widen16_i8(const U4 &v, float *f) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        f[4 * i + 0] = (float)(int8_t)(w[i] & 0xFF);
        f[4 * i + 1] = (float)(int8_t)((w[i] >> 8) & 0xFF);
        f[4 * i + 2] = (float)(int8_t)((w[i] >> 16) & 0xFF);
        f[4 * i + 3] = (float)(int8_t)(w[i] >> 24);
    }
}

// ---- wave64 reductions ------------------------------------------------------------------------
// (value of another lane through the data-parallel-primitive path: no LDS instruction, no wait)
template <int CTRL> __device__ inline float dpp_get(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
// the same for the rows of 16 lanes named by ROWS (bit r = row r); the other rows get `other`
template <int CTRL, int ROWS> __device__ inline float dpp_rows(float v, float other) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, other), __builtin_bit_cast(int, v), CTRL, ROWS, 0xF, false));
}
constexpr int kDppXor1 = 0xB1, kDppXor2 = 0x4E;     // quad_perm [1,0,3,2] / [2,3,0,1]
constexpr int kDppHalfMirror = 0x141, kDppMirror = 0x140, kDppRor8 = 0x128;  // lane i <- 7-i (per 8) / 15-i / i^8
constexpr int kDppBcast15 = 0x142, kDppBcast31 = 0x143;  // lane 15 of a row to the next row / lane 31 to rows 2 and 3
// Sum / maximum over the wave, the same value in every lane: a butterfly inside each row of 16 (after the steps
// inside a quad every lane of a quad holds the quad's sum, so the mirrored lane of the other quad (half row) stands
// for lane ^ 4 (lane ^ 8)), then row 1 += row 0 and row 3 += row 2, rows 2 and 3 += row 1, and lane 63 is read back.
// Every lane of the wave must be active at the call (a DPP read of an inactive lane returns zero, and lane 63 is read).
__device__ inline float wave_sum(float v) {
    v += dpp_get<kDppXor1>(v);
    v += dpp_get<kDppXor2>(v);
    v += dpp_get<kDppHalfMirror>(v);
    v += dpp_get<kDppMirror>(v);
    v += dpp_rows<kDppBcast15, 0xA>(v, 0.f);
    v += dpp_rows<kDppBcast31, 0xC>(v, 0.f);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ inline float wave_max(float v) {
    v = fmaxf(v, dpp_get<kDppXor1>(v));
    v = fmaxf(v, dpp_get<kDppXor2>(v));
    v = fmaxf(v, dpp_get<kDppHalfMirror>(v));
    v = fmaxf(v, dpp_get<kDppMirror>(v));
    v = fmaxf(v, dpp_rows<kDppBcast15, 0xA>(v, v));
    v = fmaxf(v, dpp_rows<kDppBcast31, 0xC>(v, v));
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
// Exchange across rows of 16 lanes without the LDS crossbar: v_permlane16_swap / v_permlane32_swap swap the odd rows
// (the upper half) of one register with the even rows (the lower half) of another.  Applied to two copies of v, one
// copy ends up holding the even-row (lower-half) values in both rows of a pair and the other the odd-row (upper-half)
// values, so their sum / maximum is v[lane] combined with v[lane ^ 16] (v[lane ^ 32]) in every lane.  (Inline
// assembly: the compiler's builtin for these instructions returns the first result twice when both operands hold
// the same value.  The s_nop covers the wait states between a vector write and the swap that reads it.)
__device__ inline void permlane16_swap(float &a, float &b) { asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b)); }
__device__ inline void permlane32_swap(float &a, float &b) { asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b)); }
__device__ inline float xor16_sum(float v) { float a = v, b = v; permlane16_swap(a, b); return a + b; }
__device__ inline float xor32_sum(float v) { float a = v, b = v; permlane32_swap(a, b); return a + b; }
__device__ inline float xor16_max(float v) { float a = v, b = v; permlane16_swap(a, b); return fmaxf(a, b); }
__device__ inline float xor32_max(float v) { float a = v, b = v; permlane32_swap(a, b); return fmaxf(a, b); }
// exact integer sum over the wave, the same value in every lane
__device__ inline int wave_sum_i32(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, kDppXor1, 0xF, 0xF, false);
    v += __builtin_amdgcn_update_dpp(0, v, kDppXor2, 0xF, 0xF, false);
    v += __builtin_amdgcn_update_dpp(0, v, kDppHalfMirror, 0xF, 0xF, false);
    v += __builtin_amdgcn_update_dpp(0, v, kDppMirror, 0xF, 0xF, false);
    v += __builtin_amdgcn_update_dpp(0, v, kDppBcast15, 0xA, 0xF, false);
    v += __builtin_amdgcn_update_dpp(0, v, kDppBcast31, 0xC, 0xF, false);
    return __builtin_amdgcn_readlane(v, 63);
}

// sum over the lanes of an aligned group of `width` lanes (power of two <= 64)
template <int width> __device__ inline float group_sum(float v) {
    if constexpr (width <= 16) {
        // the same pairs as the xor butterfly: after the steps inside a quad every lane of a quad holds the quad's
        // sum, so the mirrored lane of the other quad (half row) stands for lane ^ 4 (lane ^ 8)
        if constexpr (width >= 2) v += dpp_get<kDppXor1>(v);
        if constexpr (width >= 4) v += dpp_get<kDppXor2>(v);
        if constexpr (width >= 8) v += dpp_get<kDppHalfMirror>(v);
        if constexpr (width >= 16) v += dpp_get<kDppMirror>(v);
        return v;
    } else {
        v = group_sum<16>(v);
        v = xor16_sum(v);
        if constexpr (width >= 64) v = xor32_sum(v);
        return v;
    }
}

// maximum over the lanes of an aligned group of `width` lanes (power of two <= 16)
template <int width> __device__ inline float group_max(float v) {
    static_assert(width <= 16, "inside a row of 16 lanes");
    if constexpr (width >= 2) v = fmaxf(v, dpp_get<kDppXor1>(v));
    if constexpr (width >= 4) v = fmaxf(v, dpp_get<kDppXor2>(v));
    if constexpr (width >= 8) v = fmaxf(v, dpp_get<kDppHalfMirror>(v));
    if constexpr (width >= 16) v = fmaxf(v, dpp_get<kDppMirror>(v));
    return v;
}

// greedy-token candidates: (value, index) ordered by value, then index -- of equal maxima the LATER one wins
// (the reference's max_by over the logits, crates/llm/src/session.rs:683-690); index < 0 = no candidate yet
__device__ inline void argmax_take(float &bv, int &bi, float v, int i) {
    if (bi < 0 || v > bv || (v == bv && i > bi)) { bv = v; bi = i; }
}

// exp for softmax / SiLU: one definition for every kernel
__device__ inline float fast_exp(float x) { return __expf(x); }

// cache row of the key with recency rank `rank` in the sink + ring layout (reference common.cuh:55-60)
__host__ __device__ inline int ring_phys_index(int rank, int sink, int window, int start) {
    if (window == 0 || rank < sink) return rank;
    return sink + (start + (rank - sink)) % window;
}

// ---- errors ---------------------------------------------------------------------------------
void set_error(const char *fmt, ...);
int fail(int code, const char *fmt, ...);
int hip_fail(hipError_t e, const char *what);

#define MYNN_REQUIRE(cond, code, ...)                 \
    do {                                              \
        if (!(cond)) return ::mynn::fail((code), __VA_ARGS__); \
    } while (0)

#define MYNN_HIP(expr)                                          \
    do {                                                        \
        hipError_t e__ = (expr);                                \
        if (e__ != hipSuccess) return ::mynn::hip_fail(e__, #expr); \
    } while (0)

// A pair of events that the NEXT kernel launch made by this thread ties to its own start and end
// timestamps (hipExtLaunchKernelGGL); that launch consumes the pair.  The executor's per-launch
// profile sets it; everywhere else it is empty and launches are ordinary.
struct LaunchTimer {
    hipEvent_t start = nullptr, stop = nullptr;
};
LaunchTimer &launch_timer();

#define MYNN_LAUNCH(kernel, grid, block, shmem, stream, ...)                                                       \
    do {                                                                                                           \
        mynn::LaunchTimer &lt_ = mynn::launch_timer();                                                             \
        if (lt_.start) {                                                                                           \
            hipExtLaunchKernelGGL(kernel, grid, block, shmem, stream, lt_.start, lt_.stop, 0, __VA_ARGS__);        \
            lt_.start = lt_.stop = nullptr;                                                                        \
        } else {                                                                                                   \
            hipLaunchKernelGGL(kernel, grid, block, shmem, stream, __VA_ARGS__);                                   \
        }                                                                                                          \
    } while (0)

inline int launch_status(const char *what) {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : hip_fail(e, what);
}

inline hipStream_t as_stream(mynn_stream s) { return (hipStream_t)s; }
inline bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

template <typename F> inline int dispatch_dtype(int dt, F &&f) {
    switch (dt) {
    case MYNN_F32: return f((float *)nullptr);
    case MYNN_BF16: return f((bf16_t *)nullptr);
    case MYNN_F16: return f((f16_t *)nullptr);
    default: return fail(MYNN_ERR_INVALID, "unknown dtype %d", dt);
    }
}
template <typename F> inline int dispatch_dtype16(int dt, F &&f) {
    switch (dt) {
    case MYNN_BF16: return f((bf16_t *)nullptr);
    case MYNN_F16: return f((f16_t *)nullptr);
    default: return fail(MYNN_ERR_UNSUPPORTED, "dtype %d: this kernel needs a 16-bit float type", dt);
    }
}

}  // namespace mynn
