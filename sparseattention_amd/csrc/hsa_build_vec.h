// 16-byte (or scalar) row pieces shared by the parent-build kernels.
#pragma once
#include "hsa_common.h"

namespace hsa {

template <typename T, int VEC> struct Pack { typename T::storage e[VEC]; };

template <typename T, int VEC>
__device__ __forceinline__ void load_vec(const typename T::storage *p, float (&f)[VEC]) {
    if constexpr (VEC == 1) {
        f[0] = to_float<T>(p[0]);
    } else {
        // every operand of a level is read once per launch: streaming hint
        using P = Pack<T, VEC>;
        typedef uint32_t u4 __attribute__((ext_vector_type(4)));
        static_assert(sizeof(P) == 16, "vector path moves 16 bytes per lane");
        const P v = __builtin_bit_cast(P, __builtin_nontemporal_load(reinterpret_cast<const u4 *>(p)));
#pragma unroll
        for (int i = 0; i < VEC; ++i) f[i] = to_float<T>(v.e[i]);
    }
}

// STREAM: the store carries the streaming hint (the row does not stay in the caches)
template <typename T, int VEC, bool STREAM = false>
__device__ __forceinline__ void store_vec(typename T::storage *p, const float (&f)[VEC]) {
    if constexpr (VEC == 1) {
        p[0] = from_float<T>(f[0]);
    } else {
        using P = Pack<T, VEC>;
        P v;
#pragma unroll
        for (int i = 0; i < VEC; ++i) v.e[i] = from_float<T>(f[i]);
        static_assert(sizeof(P) == 16, "vector path moves 16 bytes per lane");
        if constexpr (STREAM) {
            typedef uint32_t u4 __attribute__((ext_vector_type(4)));
            __builtin_nontemporal_store(__builtin_bit_cast(u4, v), reinterpret_cast<u4 *>(p));
        } else {
            *reinterpret_cast<P *>(p) = v;
        }
    }
}

// 16-byte load of a row piece that is read once per launch (streaming hint), as a Pack-like P
#ifndef HSA_TREE_NT
#define HSA_TREE_NT 1
#endif
template <typename P> __device__ __forceinline__ P load_once(const void *p) {
    if constexpr (sizeof(P) == 16 && HSA_TREE_NT) {
        typedef uint32_t u4 __attribute__((ext_vector_type(4)));
        const u4 v = __builtin_nontemporal_load(reinterpret_cast<const u4 *>(p));
        return __builtin_bit_cast(P, v);
    } else {
        return *reinterpret_cast<const P *>(p);
    }
}

// 16-byte store of a node row piece, with the streaming hint if STREAM.
template <bool STREAM, typename P> __device__ __forceinline__ void store_node(void *p, const P &v) {
    if constexpr (sizeof(P) == 16 && STREAM) {
        typedef uint32_t u4 __attribute__((ext_vector_type(4)));
        __builtin_nontemporal_store(__builtin_bit_cast(u4, v), reinterpret_cast<u4 *>(p));
    } else {
        *reinterpret_cast<P *>(p) = v;
    }
}

}  // namespace hsa
