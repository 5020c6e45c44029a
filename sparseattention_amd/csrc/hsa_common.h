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

// ---- optional timing of the next kernel launch of this host thread -----------------------------
// hsa_attn_fwd_timed leaves a pair of events here; the launcher that finds them attaches them
// to the kernel dispatch itself (recorded at the kernel's begin and end) and clears the slot.
struct LaunchEvents {
    hipEvent_t start = nullptr, stop = nullptr;
};
void set_launch_events(hipEvent_t start, hipEvent_t stop);
LaunchEvents take_launch_events();

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
// round-to-nearest-even (the hardware conversion of gfx950)
template <> __device__ __forceinline__ uint16_t from_float<BF16>(float x) {
    return __builtin_bit_cast(uint16_t, static_cast<__bf16>(x));
}

// ---- cross-lane sums inside an aligned group of G lanes (G a power of two) --------------
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
// quad swaps, then mirrors inside 8 and 16 lanes (after the quads hold their sums, a mirror
// brings in the other half's sum); wider groups cross the 16-lane rows with a shuffle
__device__ __forceinline__ float group_sum(float v, int G) {
    if (G >= 2) v += dpp_move<0xB1>(v);    // quad_perm [1,0,3,2]
    if (G >= 4) v += dpp_move<0x4E>(v);    // quad_perm [2,3,0,1]
    if (G >= 8) v += dpp_move<0x141>(v);   // row_half_mirror
    if (G >= 16) v += dpp_move<0x140>(v);  // row_mirror
    if (G >= 32) v += __shfl_xor(v, 16, 64);
    if (G >= 64) v += __shfl_xor(v, 32, 64);
    return v;
}

// 3-way softmax with the reference kernel's epsilon in the denominator.  fp32 tensors get
// the accurate exp and division; 16-bit tensors (output precision 2^-9 or 2^-11) use the
// hardware exp2 and reciprocal.
template <typename T>
__device__ __forceinline__ void softmax3(float s0, float s1, float s2, float &w0, float &w1, float &w2) {
    float m = fmaxf(s0, fmaxf(s1, s2));
    if constexpr (sizeof(typename T::storage) == 4) {
        float e0 = expf(s0 - m), e1 = expf(s1 - m), e2 = expf(s2 - m);
        float den = e0 + e1 + e2 + 1e-9f;
        w0 = e0 / den;
        w1 = e1 / den;
        w2 = e2 / den;
    } else {
        constexpr float kLog2e = 1.4426950408889634f;
        float e0 = __builtin_amdgcn_exp2f((s0 - m) * kLog2e);
        float e1 = __builtin_amdgcn_exp2f((s1 - m) * kLog2e);
        float e2 = __builtin_amdgcn_exp2f((s2 - m) * kLog2e);
        float inv = __builtin_amdgcn_rcpf(e0 + e1 + e2 + 1e-9f);
        w0 = e0 * inv;
        w1 = e1 * inv;
        w2 = e2 * inv;
    }
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

// Rows of the initial span nodes of any leaf count N: level l (l >= 1) holds N >> l rows (an odd
// row at the end of a level has no partner and no parent); first row of level l within y.
__host__ __device__ __forceinline__ int span_level_start(int N, int l) {
    int s = 0;
    for (int j = 1; j < l; ++j) s += N >> j;
    return s;
}
static inline int span_levels(int N) {
    int l = 0;
    while ((N >> (l + 1)) >= 1) ++l;
    return l;
}
static inline int span_rows(int N) { return span_level_start(N, span_levels(N) + 1); }

}  // namespace hsa
