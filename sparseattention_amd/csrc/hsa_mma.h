// MFMA wrappers for the 16-bit element types of gfx950 and the vector types they take.
//
// Operand layouts of a wavefront (lane = 16 * g + r, r < 16, g < 4):
//   k32: D[16x16] += A[16x32] * B[32x16]; lane holds row r of A / column r of B, elements
//        k = 8g .. 8g+7 (16 bytes); D: lane holds column r, rows 4g .. 4g+3.
//   k16: the same with 16-deep operands, elements k = 4g .. 4g+3 (8 bytes).
#pragma once

#include "hsa_common.h"

namespace hsa {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4_t __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

template <typename T> struct Mma;

template <> struct Mma<BF16> {
    static constexpr uint16_t kOne = 0x3f80;
    static __device__ __forceinline__ f32x4 k32(u32x4_t a, u32x4_t b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                       __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 k16(u32x2_t a, u32x2_t b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4_t, a),
                                                         __builtin_bit_cast(s16x4_t, b), c, 0, 0, 0);
    }
    // round-to-nearest-even pair
    static __device__ __forceinline__ uint32_t pack(float a, float b) {
        f32x2 v = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
    }
    // the inputs are exactly representable: keep the high halves
    static __device__ __forceinline__ uint32_t pack_exact(float a, float b) {
        return (__float_as_uint(a) >> 16) | (__float_as_uint(b) & 0xffff0000u);
    }
};

template <> struct Mma<F16> {
    static constexpr uint16_t kOne = 0x3c00;
    static __device__ __forceinline__ f32x4 k32(u32x4_t a, u32x4_t b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a),
                                                      __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 k16(u32x2_t a, u32x2_t b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4_t, a),
                                                     __builtin_bit_cast(f16x4_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack(float a, float b) {
        f32x2 v = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
    }
    static __device__ __forceinline__ uint32_t pack_exact(float a, float b) { return pack(a, b); }
};

}  // namespace hsa
