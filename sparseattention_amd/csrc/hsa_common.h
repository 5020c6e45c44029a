// Shared helpers for the gfx950 kernels: element-type traits, error reporting.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "../../include/hsa_gfx950.h"

namespace hsa {

// ---- error text, one slot per host thread --------------------------------
void set_error(const char *fmt, ...);
int fail(int code, const char *fmt, ...);
int check_launch(const char *what);

#define HSA_REQUIRE(cond, ...)                                    \
    do {                                                          \
        if (!(cond)) return ::hsa::fail(HSA_ERR_INVALID, __VA_ARGS__); \
    } while (0)

// ---- element types ---------------------------------------------------------
// Raw 16-bit storage is handled as uint16_t so that loads stay plain integer
// loads; conversion is explicit.
struct F32 { using storage = float;    static constexpr int id = HSA_F32;  };
struct F16 { using storage = uint16_t; static constexpr int id = HSA_F16;  };
struct BF16 { using storage = uint16_t; static constexpr int id = HSA_BF16; };

template <typename T> __device__ __forceinline__ float to_float(typename T::storage x);
template <> __device__ __forceinline__ float to_float<F32>(float x) { return x; }
template <> __device__ __forceinline__ float to_float<F16>(uint16_t x) {
    return __half2float(__ushort_as_half(x));
}
template <> __device__ __forceinline__ float to_float<BF16>(uint16_t x) {
    return __uint_as_float(((uint32_t)x) << 16);
}

template <typename T> __device__ __forceinline__ typename T::storage from_float(float x);
template <> __device__ __forceinline__ float from_float<F32>(float x) { return x; }
template <> __device__ __forceinline__ uint16_t from_float<F16>(float x) {
    return __half_as_ushort(__float2half_rn(x));
}
// round-to-nearest-even, NaN kept quiet
template <> __device__ __forceinline__ uint16_t from_float<BF16>(float x) {
    uint32_t u = __float_as_uint(x);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static inline int elem_size(int dtype) { return dtype == HSA_F32 ? 4 : 2; }

static inline int ilog2_exact(int n) {
    int l = 0;
    while ((1 << l) < n) ++l;
    return ((1 << l) == n) ? l : -1;
}

// First row of tree level l (l >= 1) in the per-batch node space of N leaves.
__host__ __device__ __forceinline__ int level_offset(int N, int l) {
    return l == 0 ? 0 : 2 * N - (N >> (l - 1));
}

}  // namespace hsa
