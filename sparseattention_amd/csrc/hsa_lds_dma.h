// Global memory -> LDS without a stop in the registers (gfx950: 16 bytes per lane), and the LDS
// reads that go with it, both as inline assembly.
//
// Why by hand: the wavefront that stages its next block's rows this way wants them in flight while
// it reads the current block's rows from another part of the LDS.  The compiler tracks such
// transfers too, but a read of any LDS location then waits for every transfer still in flight,
// which would serialise the prefetch.  Issued from inline assembly the transfers are invisible to
// it; the waits are written out where the data is consumed:
//   * transfers and ordinary loads / stores share one in-order counter (vmcnt), so
//     "s_waitcnt vmcnt(n)" right after issuing n transfers means: everything older has arrived;
//   * what the compiler does not know about can only make its own waits stricter (it allows
//     fewer operations in flight than really are), never too weak, because the counters retire
//     in order.
// A lane's 16 bytes land at (M0 base) + 16 * lane: one instruction fills 1 KiB of LDS row by row
// without padding, so bank conflicts are avoided by permuting, per row, WHICH 16-byte piece of the
// row each lane fetches (an XOR swizzle applied on the global side) instead of by a padded pitch.
#pragma once

#include <cstdint>
#include <type_traits>

#include "hsa_mma.h"

namespace hsa {

// LDS byte address of a pointer into a __shared__ array (the low half of its flat address)
__device__ __forceinline__ uint32_t lds_address(const void *p) { return (uint32_t)(uintptr_t)p; }

// workgroup barrier that orders LDS traffic only: __syncthreads() would also wait for every
// vector-memory operation in flight, the transfers requested ahead included
__device__ __forceinline__ void lds_only_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// one instruction: lane l's 16 bytes from g to LDS[lds_base + 16 l]; lds_base is wavefront-uniform
__device__ __forceinline__ void lds_dma16(const void *g, uint32_t lds_base) {
    uint32_t keep;
    asm volatile(
        "s_mov_b32 %0, m0\n\t"
        "s_mov_b32 m0, %2\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %1, off\n\t"
        "s_mov_b32 m0, %0"
        : "=&s"(keep)
        : "v"(g), "s"(lds_base)
        : "memory");
}
// two instructions, the second STRIDE bytes further in the LDS
__device__ __forceinline__ void lds_dma16_pair(const void *g0, const void *g1, uint32_t lds_base, uint32_t lds_base1) {
    uint32_t keep;
    asm volatile(
        "s_mov_b32 %0, m0\n\t"
        "s_mov_b32 m0, %3\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %1, off\n\t"
        "s_mov_b32 m0, %4\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %2, off\n\t"
        "s_mov_b32 m0, %0"
        : "=&s"(keep)
        : "v"(g0), "v"(g1), "s"(lds_base), "s"(lds_base1)
        : "memory");
}

// everything but the youngest N vector-memory operations has completed
template <int N>
__device__ __forceinline__ void wait_vmem_all_but() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// 16-byte LDS reads the compiler does not see, issued together and waited for inside the one
// statement (a value the compiler could touch between its read and the wait would be garbage).
// Addresses are per-lane byte addresses, the offsets compile-time constants below 64 KiB.
template <int O0, int O1, int O2, int O3>
__device__ __forceinline__ void lds_read16_x4(uint32_t a0, uint32_t a1, uint32_t a2, uint32_t a3, u32x4_t &r0,
                                              u32x4_t &r1, u32x4_t &r2, u32x4_t &r3) {
    asm volatile(
        "ds_read_b128 %0, %4 offset:%8\n\t"
        "ds_read_b128 %1, %5 offset:%9\n\t"
        "ds_read_b128 %2, %6 offset:%10\n\t"
        "ds_read_b128 %3, %7 offset:%11\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3)
        : "v"(a0), "v"(a1), "v"(a2), "v"(a3), "n"(O0), "n"(O1), "n"(O2), "n"(O3)
        : "memory");
}
// six staged blocks of ARR bytes each, starting OFF bytes behind the addresses: operand pieces of
// two contraction steps (addresses a0, a1) of each block
template <int OFF, int ARR>
__device__ __forceinline__ void lds_read16_6x2(uint32_t a0, uint32_t a1, u32x4_t (&b0)[2], u32x4_t (&b1)[2],
                                               u32x4_t (&b2)[2], u32x4_t (&b3)[2], u32x4_t (&b4)[2],
                                               u32x4_t (&b5)[2]) {
    asm volatile(
        "ds_read_b128 %0, %12 offset:%14\n\t"
        "ds_read_b128 %1, %13 offset:%14\n\t"
        "ds_read_b128 %2, %12 offset:%15\n\t"
        "ds_read_b128 %3, %13 offset:%15\n\t"
        "ds_read_b128 %4, %12 offset:%16\n\t"
        "ds_read_b128 %5, %13 offset:%16\n\t"
        "ds_read_b128 %6, %12 offset:%17\n\t"
        "ds_read_b128 %7, %13 offset:%17\n\t"
        "ds_read_b128 %8, %12 offset:%18\n\t"
        "ds_read_b128 %9, %13 offset:%18\n\t"
        "ds_read_b128 %10, %12 offset:%19\n\t"
        "ds_read_b128 %11, %13 offset:%19\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&v"(b0[0]), "=&v"(b0[1]), "=&v"(b1[0]), "=&v"(b1[1]), "=&v"(b2[0]), "=&v"(b2[1]), "=&v"(b3[0]),
          "=&v"(b3[1]), "=&v"(b4[0]), "=&v"(b4[1]), "=&v"(b5[0]), "=&v"(b5[1])
        : "v"(a0), "v"(a1), "n"(OFF), "n"(OFF + ARR), "n"(OFF + 2 * ARR), "n"(OFF + 3 * ARR), "n"(OFF + 4 * ARR),
          "n"(OFF + 5 * ARR)
        : "memory");
}
// the same with one contraction step per block
template <int OFF, int ARR>
__device__ __forceinline__ void lds_read16_6x1(uint32_t a0, u32x4_t (&b0)[1], u32x4_t (&b1)[1], u32x4_t (&b2)[1],
                                               u32x4_t (&b3)[1], u32x4_t (&b4)[1], u32x4_t (&b5)[1]) {
    asm volatile(
        "ds_read_b128 %0, %6 offset:%7\n\t"
        "ds_read_b128 %1, %6 offset:%8\n\t"
        "ds_read_b128 %2, %6 offset:%9\n\t"
        "ds_read_b128 %3, %6 offset:%10\n\t"
        "ds_read_b128 %4, %6 offset:%11\n\t"
        "ds_read_b128 %5, %6 offset:%12\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&v"(b0[0]), "=&v"(b1[0]), "=&v"(b2[0]), "=&v"(b3[0]), "=&v"(b4[0]), "=&v"(b5[0])
        : "v"(a0), "n"(OFF), "n"(OFF + ARR), "n"(OFF + 2 * ARR), "n"(OFF + 3 * ARR), "n"(OFF + 4 * ARR),
          "n"(OFF + 5 * ARR)
        : "memory");
}

}  // namespace hsa
