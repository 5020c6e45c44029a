// The whole bottom-up tree in ONE launch.
//
//   Out_l = build_parent_nodes(Qp_l, Kp_l, Vp_l, Out_{l-1}, Out_{l-1}),  level 1 from the leaf K / V.
//
// Three phases inside the kernel, no second launch and no waiting on other workgroups:
//   A  a group of G lanes (G * 16 bytes = one head row) owns one (batch, head) and a subtree of
//      2^TL leaves: every row it needs is requested up front, the TL levels stay in registers;
//   B  a workgroup covers S consecutive subtrees of all H heads (so its wavefronts still read
//      whole token rows); their roots are exchanged through LDS and the next log2 S levels are
//      finished inside the workgroup (parent rows were requested together with phase A's and wait
//      in LDS);
//   C  what is left per batch element -- one node per workgroup -- is finished by "the last one to
//      arrive": each workgroup publishes its node, increments an arrival counter shared by a group
//      of 2^g neighbouring workgroups and exits unless it was the last of the group; the last one
//      reads the group's 2^g nodes, computes g more levels and repeats one level of grouping
//      further up, until the root.  Nobody spins: every workgroup exits after at most one pass
//      over its own data plus the groups it happened to close.
// The second copy of the result (out2) is written after the arrival: until then the launch is
// almost purely reading, and the copy drains while the closing workgroups finish the top levels.
// Arrival counters live in a device array that is part of the library image; they count with
// wrap-around (the closing arrival resets the counter), so they are zero whenever no launch
// is using them, and each stream has its own slice, so launches that may run concurrently
// never share a counter.
#include "hsa_build_vec.h"

#include <atomic>
#include <mutex>

namespace hsa {

template <typename T, int VEC> struct alignas(sizeof(typename T::storage) * VEC) VPack {
    typename T::storage e[VEC];
};

struct TreeArgs {
    const void *qp, *kp, *vp, *kleaf, *vleaf;
    void *out, *out2;
    unsigned *counters;  // this launch's slice: counters_per_batch per batch element, all zero
    int N, H, D, L;
    int lgG, lgH;        // lanes per head row, heads (both powers of two)
    int lgS;             // subtrees per workgroup (phase B finishes lgS levels)
    int lg_nsub;         // subtrees per (batch, head) = N >> TL
    int gcap;            // most levels one phase-C stage takes
    int counters_per_batch;
    int64_t qp_bs, kp_bs, vp_bs, kleaf_bs, vleaf_bs, out_bs, out2_bs;
    float scale;
};

constexpr int ilog2_const(int x) { return x <= 1 ? 0 : 1 + ilog2_const(x >> 1); }

#ifndef TREE_DOT2
#define TREE_DOT2 1
#endif
constexpr int TREE_NLMAX = 4;               // phase B: at most 16 subtrees per workgroup
constexpr int TREE_GCAP_MAX = TREE_NLMAX + 2;  // phase C: at most 64 nodes per group

__device__ __forceinline__ void lds_barrier() {
    // workgroup barrier that orders LDS traffic only: __syncthreads() would also wait for the
    // global loads that were requested ahead on purpose
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// A row piece that another workgroup will read during this launch is written and read with
// device-scope atomic accesses (two 8-byte halves): they go through to memory instead of
// staying in the L2 of the writer's XCD, so publishing costs no cache write-back.  (A
// device-scope release fence writes back every dirty line of that L2 and serialises the
// workgroups: measured 0.1 - 0.6 us per workgroup.)
template <typename P> __device__ __forceinline__ void publish_piece(void *dst, const P &v) {
    static_assert(sizeof(P) == 16, "two 8-byte halves");
    const unsigned long long *w = reinterpret_cast<const unsigned long long *>(&v);
    unsigned long long *d = reinterpret_cast<unsigned long long *>(dst);
    __hip_atomic_store(d, w[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(d + 1, w[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <typename P> __device__ __forceinline__ P fetch_published(const void *src) {
    unsigned long long *s = reinterpret_cast<unsigned long long *>(const_cast<void *>(src));
    unsigned long long w[2];
    w[0] = __hip_atomic_load(s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    w[1] = __hip_atomic_load(s + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return *reinterpret_cast<const P *>(w);
}

// acc + <a, b> for two packed 16-bit elements with the two-element dot instruction: the products
// are exact in fp32, the three-term sum is formed in fp32 (a level's dot products take a fifth of
// the instructions of unpack + multiply-add; the levels of the launch's tail are bound by their
// instruction count)
template <typename T> __device__ __forceinline__ float dot2_acc(uint32_t a, uint32_t b, float acc);
template <> __device__ __forceinline__ float dot2_acc<BF16>(uint32_t a, uint32_t b, float acc) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), acc, false);
}
template <> __device__ __forceinline__ float dot2_acc<F16>(uint32_t a, uint32_t b, float acc) {
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), acc, false);
}

// VEC floats -> a row piece, two elements per conversion where the type has a packed one
template <typename T, int VEC> __device__ __forceinline__ VPack<T, VEC> pack_piece(const float (&o)[VEC]) {
    VPack<T, VEC> r;
    if constexpr (sizeof(typename T::storage) == 2 && VEC % 2 == 0) {
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        uint32_t *w = reinterpret_cast<uint32_t *>(&r);
#pragma unroll
        for (int i = 0; i < VEC / 2; ++i) {
            const f32x2 v = {o[2 * i], o[2 * i + 1]};
            if constexpr (T::id == HSA_BF16) {
                typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
                w[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
            } else {
                typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
                w[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
            }
        }
    } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) r.e[e] = from_float<T>(o[e]);
    }
    return r;
}

// the three scores of a parent: <q, k>, <q, c0>, <q, c1> over this lane's piece
template <typename T, int VEC>
__device__ __forceinline__ void scores3(const VPack<T, VEC> &q, const VPack<T, VEC> &k, const VPack<T, VEC> &c0,
                                        const VPack<T, VEC> &c1, float &s0, float &s1, float &s2) {
    s0 = 0.f; s1 = 0.f; s2 = 0.f;
    if constexpr (sizeof(typename T::storage) == 2 && VEC % 2 == 0 && TREE_DOT2) {
        const uint32_t *qw = reinterpret_cast<const uint32_t *>(&q), *kw = reinterpret_cast<const uint32_t *>(&k);
        const uint32_t *aw = reinterpret_cast<const uint32_t *>(&c0), *bw = reinterpret_cast<const uint32_t *>(&c1);
#pragma unroll
        for (int w = 0; w < VEC / 2; ++w) {
            s0 = dot2_acc<T>(qw[w], kw[w], s0);
            s1 = dot2_acc<T>(qw[w], aw[w], s1);
            s2 = dot2_acc<T>(qw[w], bw[w], s2);
        }
    } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const float fq = to_float<T>(q.e[e]);
            s0 = fmaf(fq, to_float<T>(k.e[e]), s0);
            s1 = fmaf(fq, to_float<T>(c0.e[e]), s1);
            s2 = fmaf(fq, to_float<T>(c1.e[e]), s2);
        }
    }
}

// one parent from its q/k/v row pieces and its two children's pieces (children are both key and value)
template <typename T, int VEC>
__device__ __forceinline__ VPack<T, VEC> combine(const VPack<T, VEC> &q, const VPack<T, VEC> &k,
                                                  const VPack<T, VEC> &v, const VPack<T, VEC> &c0,
                                                  const VPack<T, VEC> &c1, int G, float scale) {
    float s0, s1, s2;
    scores3<T, VEC>(q, k, c0, c1, s0, s1, s2);
    s0 = group_sum(s0, G);
    s1 = group_sum(s1, G);
    s2 = group_sum(s2, G);
    float w0, w1, w2;
    softmax3<T>(s0 * scale, s1 * scale, s2 * scale, w0, w1, w2);
    float o[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) o[e] = w0 * to_float<T>(v.e[e]) + w1 * to_float<T>(c0.e[e]) + w2 * to_float<T>(c1.e[e]);
    return pack_piece<T, VEC>(o);
}


// LGG / LGH: log2 of the lanes per head row and of the head count when known at compile time
// (-1: taken from the arguments).  With both fixed, the subtrees per workgroup, every slot
// index and the cross-lane sums become constants: about half the instructions per level.
struct VPackBits { uint32_t x, y, z, w; };

template <typename T, int VEC, int TL, int THREADS, int LGG, int LGH>
__global__ void __launch_bounds__(THREADS) build_tree_fused_kernel(TreeArgs a) {
    using S = typename T::storage;
    using P = VPack<T, VEC>;
    constexpr int NC = 1 << TL;
    constexpr int PB = (int)sizeof(P);  // 16 bytes
    // Node rows leave with the streaming hint in the small-workgroup variants, i.e. when the
    // launch leaves half the chip's wavefront slots empty: there it takes 2-3 us off the launch
    // (measured at B16 N512 .. B2 N4096, 8 heads of 64), while at 512 threads the launch gains
    // nothing and the span attention that follows loses the node rows the memory-side cache kept.
    constexpr bool STREAM = THREADS <= 256;
    // LDS: two exchange buffers (2 * THREADS and THREADS pieces) and the staged parent rows
    // (three tensors, 2 * THREADS pieces each): 144 bytes per thread
    __shared__ __align__(16) unsigned char tree_lds[9 * THREADS * PB];
    unsigned char *bufX = tree_lds;                       // 2 * THREADS pieces
    unsigned char *bufY = tree_lds + 2 * THREADS * PB;    // THREADS pieces
    __shared__ int s_last;

    const int lgG = LGG >= 0 ? LGG : a.lgG, lgH = LGH >= 0 ? LGH : a.lgH;
    const int lgS = (LGG >= 0 && LGH >= 0) ? ilog2_const(THREADS) - LGG - LGH : a.lgS;
    const int gcap = lgS + 2 < TREE_GCAP_MAX ? lgS + 2 : TREE_GCAP_MAX;
    const int N = a.N, H = 1 << lgH, G = 1 << lgG, D = a.D;
    const int u_local = (int)threadIdx.x >> lgG;        // (subtree, head) slot inside the workgroup
    const int gl = (int)threadIdx.x & (G - 1);
    const int h = u_local & (H - 1);
    const int p_local = u_local >> lgH;                 // subtree inside the workgroup
    const int lg_wpb = a.lg_nsub - lgS;                 // workgroups per batch element (log2)
    const int wg = (int)blockIdx.x & ((1 << lg_wpb) - 1);
    const int b = (int)blockIdx.x >> lg_wpb;
    const int sub = (wg << lgS) + p_local;
    const size_t rs = (size_t)H * D;
    const size_t hd = (size_t)h * D + (size_t)gl * VEC;
    const S *Qp = (const S *)a.qp + (size_t)b * a.qp_bs + hd;
    const S *Kp = (const S *)a.kp + (size_t)b * a.kp_bs + hd;
    const S *Vp = (const S *)a.vp + (size_t)b * a.vp_bs + hd;
    S *Out = (S *)a.out + (size_t)b * a.out_bs + hd;
    S *Out2 = a.out2 ? (S *)a.out2 + (size_t)b * a.out2_bs + hd : nullptr;
    auto node_row = [&](int level, int idx) { return (size_t)(level_offset(N, level) - N + idx) * rs; };

    // ---- phase A: TL levels in registers; every row is requested before the first use --------
    // Requests go out tensor by tensor (a wavefront's eight leaf K rows are 8 KiB in a row, then
    // the four level-1 q rows, ...): contiguous runs are served faster than the same rows
    // requested in the order of use (measured on the bare request pattern at 8 x 2048 rows of
    // 1 KiB: 12.6 against 13.4 us).  Loads return in order, so the first parents are computed
    // while the upper levels' rows are still arriving.
    P rck[NC], rcv[NC], rq[NC - 1], rk[NC - 1], rv[NC - 1];
    {
        const S *kc = (const S *)a.kleaf + (size_t)b * a.kleaf_bs + (size_t)sub * NC * rs + hd;
        const S *vc = (const S *)a.vleaf + (size_t)b * a.vleaf_bs + (size_t)sub * NC * rs + hd;
        const size_t row1 = node_row(1, sub * (NC / 2));
#pragma unroll
        for (int i = 0; i < NC; ++i) rck[i] = load_once<P>(kc + (size_t)i * rs);
#pragma unroll
        for (int i = 0; i < NC / 2; ++i) rq[i] = load_once<P>(Qp + row1 + (size_t)i * rs);
#pragma unroll
        for (int i = 0; i < NC / 2; ++i) rk[i] = load_once<P>(Kp + row1 + (size_t)i * rs);
#pragma unroll
        for (int i = 0; i < NC; ++i) rcv[i] = load_once<P>(vc + (size_t)i * rs);
#pragma unroll
        for (int i = 0; i < NC / 2; ++i) rv[i] = load_once<P>(Vp + row1 + (size_t)i * rs);
    }
#pragma unroll
    for (int j = 2; j <= TL; ++j) {
        const int np = NC >> j;
        const int base = NC - 2 * np;
        const size_t row = node_row(j, sub * np);
#pragma unroll
        for (int i = 0; i < NC / 4; ++i)
            if (i < np) rq[base + i] = load_once<P>(Qp + row + (size_t)i * rs);
#pragma unroll
        for (int i = 0; i < NC / 4; ++i)
            if (i < np) rk[base + i] = load_once<P>(Kp + row + (size_t)i * rs);
#pragma unroll
        for (int i = 0; i < NC / 4; ++i)
            if (i < np) rv[base + i] = load_once<P>(Vp + row + (size_t)i * rs);
    }
    // phase B's parent rows, one piece per thread and tensor: thread t fetches what staging slot t
    // holds (levels back to back, each level's (parent, head, lane) slots in order; the last
    // H * G slots stay unused and re-read the top row).  The loads are unconditional, because a
    // load under a branch is waited for at the end of the branch, and with it every load
    // requested before it.
    constexpr int LGT = ilog2_const(THREADS);
    P sq, sk, sv;
    {
        const int m = THREADS - 1 - (int)threadIdx.x;
        int jj = LGT - (31 - __clz(m | 1));     // slot t belongs to run level jj
        jj = jj < lgS ? jj : lgS;
        jj = jj > 0 ? jj : 0;                   // lgS == 0: no run; the subtree's own root row
        const int first = jj > 0 ? THREADS - (THREADS >> (jj - 1)) : 0;
        const int np = 1 << (lgS - jj);
        int pp = ((int)threadIdx.x - first) >> (lgH + lgG);
        pp = pp < np ? pp : np - 1;
        const size_t row = node_row(TL + jj, ((wg << lgS) >> jj) + pp);
        sq = load_once<P>(Qp + row);
        sk = load_once<P>(Kp + row);
        sv = load_once<P>(Vp + row);
    }
    // The parent rows of the levels above the workgroups' own (phase C) are read by whichever
    // workgroup closes a group, right after its arrival and on the critical path of the launch's
    // tail.  The workgroups of a batch element share them out and touch them now, last in the
    // request order and with regular loads, so that the closing workgroup finds them in the caches.
    P touch;
    {
        const int first_lvl = TL + lgS + 1;
        const long rows_top = (long)(N >> (first_lvl - 1)) - 1;   // nodes of levels first_lvl .. root
        const long ppr = (long)(rs / VEC);                        // 16-byte pieces per row
        const long n_pieces = rows_top > 0 ? 3 * rows_top * ppr : 1;
        long t = (long)wg * THREADS + (long)threadIdx.x;
        if (t >= n_pieces) t = n_pieces - 1;
        const long per = rows_top > 0 ? rows_top * ppr : 1;
        const int which = (int)(t / per);
        const long rem = t - (long)which * per;
        const S *base = which == 0 ? (const S *)a.qp + (size_t)b * a.qp_bs
                      : which == 1 ? (const S *)a.kp + (size_t)b * a.kp_bs
                                   : (const S *)a.vp + (size_t)b * a.vp_bs;
        const size_t first_row = rows_top > 0 ? (size_t)(level_offset(N, first_lvl) - N) : 0;
        touch = *reinterpret_cast<const P *>(base + first_row * rs + (size_t)rem * VEC);
    }
    __builtin_amdgcn_sched_barrier(0);

    // Every row is stored to `out` as it is produced and kept in registers for the second copy,
    // which is written after the arrival (see `second_copy`).
    P keep[NC - 1];
    {
        // level 1: keys and values are different rows
#pragma unroll
        for (int i = 0; i < NC / 2; ++i) {
            float s0, s1, s2;
            scores3<T, VEC>(rq[i], rk[i], rck[2 * i], rck[2 * i + 1], s0, s1, s2);
            s0 = group_sum(s0, G);
            s1 = group_sum(s1, G);
            s2 = group_sum(s2, G);
            float w0, w1, w2;
            softmax3<T>(s0 * a.scale, s1 * a.scale, s2 * a.scale, w0, w1, w2);
            float o[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e)
                o[e] = w0 * to_float<T>(rv[i].e[e]) + w1 * to_float<T>(rcv[2 * i].e[e]) + w2 * to_float<T>(rcv[2 * i + 1].e[e]);
            keep[i] = pack_piece<T, VEC>(o);
            store_node<STREAM>(Out + node_row(1, sub * (NC / 2) + i), keep[i]);
        }
        // levels 2..TL
#pragma unroll
        for (int j = 2; j <= TL; ++j) {
            const int np = NC >> j;
            const int base = NC - 2 * np;
            const int cbase = NC - 4 * np;  // the level below
#pragma unroll
            for (int i = 0; i < NC / 4; ++i) {
                if (i < np) {
                    const P r = combine<T, VEC>(rq[base + i], rk[base + i], rv[base + i], keep[cbase + 2 * i],
                                                keep[cbase + 2 * i + 1], G, a.scale);
                    keep[base + i] = r;
                    const size_t row = node_row(j, sub * np + i);
                    if (j == TL && lgS == 0 && lg_wpb > 0) publish_piece(Out + row, r);  // the workgroup's node
                    else store_node<STREAM>(Out + row, r);
                }
            }
        }
        // the subtree's root goes to LDS, slot = (subtree, head): piece threadIdx.x
        *reinterpret_cast<P *>(bufX + (size_t)threadIdx.x * PB) = keep[NC - 2];
    }

    // ---- phases B and C share one loop ----------------------------------------------------------
    // A "run" finishes n_lds levels inside the workgroup: the children sit in LDS (bufX), the
    // parents' q/k/v pieces wait in LDS as well (stg), one level per iteration of a loop that is
    // not unrolled: phase B's levels and the levels of every closing stage of phase C are the
    // same instructions.  A level costs a wavefront about 220 instructions; the levels of the
    // launch's tail are bound by that (two wavefronts per SIMD at the first level of a stage:
    // 1.1 us, one: 0.5 us), not by memory.
    // Staging slot of (run level jj, thread t): w1x2 - (w1x2 >> (jj-1)) + t, where w1x2 is twice
    // the number of lanes busy at the run's first level: levels back to back, so that slot s of
    // the whole run is fetched by thread s mod THREADS (no row is fetched twice).
    unsigned char *stgQ = tree_lds + 3 * THREADS * PB;   // 2 * THREADS pieces each
    unsigned char *stgK = stgQ + 2 * THREADS * PB;
    unsigned char *stgV = stgK + 2 * THREADS * PB;
    *reinterpret_cast<P *>(stgQ + (size_t)threadIdx.x * PB) = sq;
    *reinterpret_cast<P *>(stgK + (size_t)threadIdx.x * PB) = sk;
    *reinterpret_cast<P *>(stgV + (size_t)threadIdx.x * PB) = sv;

    // The second copy of phase A's rows.  Stored as they are produced, these writes compete with
    // the reads that every workgroup still has under way; stored after the arrival they overlap
    // the closing workgroups' top levels instead (headline shape: 28.7 -> 26 us per launch;
    // deferring `out` as well loses again: the closing workgroups then work inside twice the
    // write traffic).  A closing workgroup writes its own after its last stage.
    auto second_copy = [&]() {
        if (!Out2) return;
#pragma unroll
        for (int j = 1; j <= TL; ++j) {
            const int np = NC >> j;
            const int base = NC - 2 * np;
#pragma unroll
            for (int i = 0; i < NC / 2; ++i)
                if (i < np) store_node<STREAM>(Out2 + node_row(j, sub * np + i), keep[base + i]);
        }
    };

    int n_lds = lgS;             // levels of the coming run
    int lvl_base = TL;           // level of the run's children
    int idx_base = wg << lgS;    // index (within the batch element) of the run's first child
    int w1x2 = THREADS;          // twice the lanes busy at the run's first level
    int level = TL + lgS;        // after the run this workgroup holds node `idx` of that level (all heads)
    int idx = wg;
    int lg_width = lg_wpb;       // nodes of that level per batch element (log2)
    unsigned *cnt = a.counters + (size_t)b * a.counters_per_batch;
    const int upb = THREADS >> lgG;  // (node, head) slots one pass of the workgroup covers
    asm volatile("" : "+s"(n_lds));  // one copy of the loop for every run: nothing specialised for the first
    if (n_lds > 0) lds_barrier();
    for (;;) {
        const bool more = lg_width > 0;  // another stage follows: the run's last level is published
        unsigned char *src = bufX, *dst = bufY;
#pragma unroll 1
        for (int jj = 1; jj <= n_lds; ++jj) {
            if ((int)threadIdx.x < (w1x2 >> jj)) {
                const size_t slot = (size_t)(w1x2 - (w1x2 >> (jj - 1))) + threadIdx.x;
                const P q = *reinterpret_cast<const P *>(stgQ + slot * PB);
                const P k = *reinterpret_cast<const P *>(stgK + slot * PB);
                const P v = *reinterpret_cast<const P *>(stgV + slot * PB);
                const size_t c_off = ((size_t)(((2 * p_local) << lgH) + h) << lgG) + gl;
                const P c0 = *reinterpret_cast<const P *>(src + c_off * PB);
                const P c1 = *reinterpret_cast<const P *>(src + (c_off + ((size_t)1 << (lgH + lgG))) * PB);
                const P r = combine<T, VEC>(q, k, v, c0, c1, G, a.scale);
                const size_t row = node_row(lvl_base + jj, (idx_base >> jj) + p_local);
                if (jj == n_lds && more) publish_piece(Out + row, r);  // read by the stage that follows
                else store_node<STREAM>(Out + row, r);
                if (Out2) store_node<STREAM>(Out2 + row, r);
                if (jj < n_lds) *reinterpret_cast<P *>(dst + (size_t)threadIdx.x * PB) = r;
            }
            if (jj < n_lds) lds_barrier();
            unsigned char *t = src;
            src = dst;
            dst = t;
        }
        if (!more) break;

        // ---- arrival: the last workgroup of a group to arrive continues upwards ----------------
        const int g = lg_width < gcap ? lg_width : gcap;
        const int grp = idx >> g;
        // Where the closing workgroup will read: worked out by every workgroup before it waits
        // for its stores, so that whoever closes the group has nothing left to do after the
        // counter's answer but to request the rows.  The stage's first level takes its children
        // (the group's published nodes) and parents from registers, maybe in two passes over the
        // slots; the parents of the levels above go to LDS slots t and t + THREADS of the run that
        // follows.  Slots and levels that do not exist re-read the nearest one.
        const bool two = ((1 << (g - 1)) << lgH) > upb;
        const int lgw = g - 1 + lgH + lgG;   // log2 of the next run's w1x2
        size_t o_child[2], o_par[2], o_up[2];
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
            const int p = (u_local + pass * upb) >> lgH;
            const int np = 1 << (g - 1);
            const int pc = p < np ? p : np - 1;
            o_child[pass] = node_row(level, (grp << g) + 2 * pc);
            o_par[pass] = node_row(level + 1, (grp << (g - 1)) + pc);
            const int sl = (int)threadIdx.x + pass * THREADS;
            const int m = (1 << lgw) - 1 - sl;
            int jj = lgw - (31 - __clz((m > 0 ? m : 0) | 1));
            jj = jj < g - 1 ? jj : g - 1;
            jj = jj > 0 ? jj : 0;               // g == 1: no run; the stage's own parent row
            const int first = jj > 0 ? (1 << lgw) - ((1 << lgw) >> (jj - 1)) : 0;
            const int npu = 1 << (g - 1 - jj);
            int pp = (sl - first) >> (lgH + lgG);
            pp = pp < npu ? pp : npu - 1;
            pp = pp > 0 ? pp : 0;
            o_up[pass] = node_row(level + 1 + jj, (grp << (g - 1 - jj)) + pp);
            asm volatile("" : "+v"(o_child[pass]), "+v"(o_par[pass]), "+v"(o_up[pass]));  // computed here, not after the wait
        }
        // This workgroup's node has been written with device-scope (sc1) stores, which the L2
        // writes through to memory; such a store is acknowledged -- the wavefront's vmcnt drops --
        // only when the write has reached the memory side, the point where every XCD's L2 misses
        // meet.  So: wait for vmcnt = 0 in every wavefront, meet at the workgroup barrier, and only
        // then count the arrival (a device-scope atomic, executed at the memory side as well).  The
        // closing workgroup reads the nodes with device-scope (sc1) loads, which miss in its own
        // L2, after it has seen the counter's closing value: it reads what the stores left.
        // A release on the increment would be the portable spelling, but at device scope it makes
        // the compiler write back the whole L2 (0.1 - 0.6 us per workgroup, serialised).  The
        // wait is an asm statement with a memory clobber, so the compiler moves no store below it
        // and no load above it; a second compiler barrier follows the "am I last" branch.
        asm volatile("" ::"v"(__builtin_bit_cast(VPackBits, touch).x));  // keeps the touching load alive
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __syncthreads();
        if (threadIdx.x == 0) {
            const unsigned last = (1u << g) - 1u;
            s_last = atomicInc(cnt + grp, last) == last;
        }
        __syncthreads();
        if (!s_last) {
            second_copy();
            return;
        }
        asm volatile("" ::: "memory");

        // ---- the closing workgroup ---------------------------------------------------------------
        P cq[2], ckk[2], cvv[2], ch0[2], ch1[2];
        typedef uint32_t u4 __attribute__((ext_vector_type(4)));
        u4 uq[2], uk[2], uv[2];
        w1x2 = 1 << lgw;
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
            ch0[pass] = fetch_published<P>(Out + o_child[pass]);
            ch1[pass] = fetch_published<P>(Out + o_child[pass] + rs);
            cq[pass] = *reinterpret_cast<const P *>(Qp + o_par[pass]);
            ckk[pass] = *reinterpret_cast<const P *>(Kp + o_par[pass]);
            cvv[pass] = *reinterpret_cast<const P *>(Vp + o_par[pass]);
        }
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
            uq[pass] = *reinterpret_cast<const u4 *>(Qp + o_up[pass]);
            uk[pass] = *reinterpret_cast<const u4 *>(Kp + o_up[pass]);
            uv[pass] = *reinterpret_cast<const u4 *>(Vp + o_up[pass]);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
            if (pass == 0 || two) {
                const int u = u_local + pass * upb;
                const int p = u >> lgH;
                if (p < (1 << (g - 1))) {
                    const P r = combine<T, VEC>(cq[pass], ckk[pass], cvv[pass], ch0[pass], ch1[pass], G, a.scale);
                    const size_t row = node_row(level + 1, (grp << (g - 1)) + p);
                    if (g == 1 && lg_width > g) publish_piece(Out + row, r);  // read by the next stage
                    else store_node<STREAM>(Out + row, r);
                    if (Out2) store_node<STREAM>(Out2 + row, r);
                    if (g > 1) *reinterpret_cast<P *>(bufX + (((size_t)u << lgG) + gl) * PB) = r;
                }
            }
        }
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
            const size_t slot = (size_t)threadIdx.x + (size_t)pass * THREADS;
            *reinterpret_cast<u4 *>(stgQ + slot * PB) = uq[pass];
            *reinterpret_cast<u4 *>(stgK + slot * PB) = uk[pass];
            *reinterpret_cast<u4 *>(stgV + slot * PB) = uv[pass];
        }
        if (g > 1) lds_barrier();
        n_lds = g - 1;
        lvl_base = level + 1;
        idx_base = grp << (g - 1);
        cnt += (size_t)1 << (lg_width - g);
        lg_width -= g;
        level += g;
        idx = grp;
    }
    second_copy();  // the workgroups that closed the last stage (or a batch element's only workgroup)
}

// ---- arrival counters ------------------------------------------------------------------------
// One slice per (device, stream): launches on one stream run in order, so they can share a slice;
// launches on different streams may overlap and never do.  Counters wrap to zero on the closing
// arrival, so a slice is all zero between launches.  The last slice is not a stream's: launches
// recorded into a graph take their counters from it, each its own and for good (see below).
constexpr int TREE_SLICES = 32;
constexpr int TREE_SLICE_COUNTERS = 1 << 16;
}  // namespace hsa

static __device__ __align__(256) unsigned tree_counters[hsa::TREE_SLICES * hsa::TREE_SLICE_COUNTERS];

namespace hsa {

constexpr int TREE_MAX_DEVICES = 64;
static std::mutex g_tree_mu;
static unsigned *g_tree_base[TREE_MAX_DEVICES];
struct SliceOwner { int dev; hipStream_t stream; };
static SliceOwner g_tree_owner[TREE_SLICES];
static int g_tree_owners = 0;

// The slice of the current device's counter array that belongs to `st`, or nullptr when every
// slice has an owner (the caller then takes the path that needs no counters).
static unsigned *tree_counter_slice(hipStream_t st) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= TREE_MAX_DEVICES) return nullptr;
    std::lock_guard<std::mutex> lock(g_tree_mu);
    if (!g_tree_base[dev]) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(tree_counters)) != hipSuccess || !p) {
            (void)hipGetLastError();
            return nullptr;
        }
        g_tree_base[dev] = (unsigned *)p;
    }
    int slot = -1;
    for (int i = 0; i < g_tree_owners; ++i)
        if (g_tree_owner[i].dev == dev && g_tree_owner[i].stream == st) { slot = i; break; }
    if (slot < 0) {
        if (g_tree_owners == TREE_SLICES - 1) return nullptr;
        slot = g_tree_owners++;
        g_tree_owner[slot] = {dev, st};
    }
    return g_tree_base[dev] + (size_t)slot * TREE_SLICE_COUNTERS;
}

// Counters of a launch that is being recorded into a graph.  The recorded launch may replay on any
// stream, next to anything, so it cannot borrow a stream's slice: it gets `need` counters of the
// last slice that no other launch will ever use (a graph does not run concurrently with itself).
// They are never handed back; once the slice is used up, and while the array's address on this
// device is still unknown (resolving a symbol is no call to make during a capture), recorded
// launches take the path that needs no counters.
static unsigned g_tree_graph_used[TREE_MAX_DEVICES];
static unsigned *tree_counters_for_capture(long need) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= TREE_MAX_DEVICES) return nullptr;
    std::lock_guard<std::mutex> lock(g_tree_mu);
    if (!g_tree_base[dev]) return nullptr;
    if ((long)g_tree_graph_used[dev] + need > TREE_SLICE_COUNTERS) return nullptr;
    unsigned *p = g_tree_base[dev] + (size_t)(TREE_SLICES - 1) * TREE_SLICE_COUNTERS + g_tree_graph_used[dev];
    g_tree_graph_used[dev] += (unsigned)need;
    return p;
}

// compute units of the current device (queried once per device)
static int device_compute_units() {
    static std::atomic<int> cached[TREE_MAX_DEVICES];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= TREE_MAX_DEVICES) return 256;
    int n = cached[dev];
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev] = n;
    }
    return n;
}

static int ilog2_pow2(int x) {
    int l = 0;
    while ((1 << l) < x) ++l;
    return ((1 << l) == x) ? l : -1;
}

// Launches the one-kernel tree build, or returns HSA_ERR_UNSUPPORTED when the shape or the counter
// pool does not allow it.
template <typename T>
static int build_tree_fused_typed(const void *qp, const void *kp, const void *vp, const void *k_leaf,
                                  const void *v_leaf, void *out, void *out2, int B, int N, int H, int D,
                                  int64_t qp_bs, int64_t kp_bs, int64_t vp_bs, int64_t kleaf_bs, int64_t vleaf_bs,
                                  int64_t out_bs, int64_t out2_bs, int threads_pref, bool force, hipStream_t st) {
    using S = typename T::storage;
    constexpr int VEC = 16 / (int)sizeof(S);
    constexpr int TL = 3;
    const uintptr_t align = (uintptr_t)qp | (uintptr_t)kp | (uintptr_t)vp | (uintptr_t)k_leaf | (uintptr_t)v_leaf |
                            (uintptr_t)out | (uintptr_t)out2;
    const int64_t strides = qp_bs | kp_bs | vp_bs | kleaf_bs | vleaf_bs | out_bs | out2_bs;
    if (D % VEC != 0 || (align & 15) != 0 || (strides % VEC) != 0) return HSA_ERR_UNSUPPORTED;
    const int lgG = ilog2_pow2(D / VEC), lgH = ilog2_pow2(H), L = ilog2_exact(N);
    if (lgG < 0 || lgG > 6 || lgH < 0 || L < TL) return HSA_ERR_UNSUPPORTED;
    const int lg_nsub = L - TL;
    // workgroup size: the preferred one, shrunk until a workgroup stays inside one batch element
    // and finishes at most TREE_NLMAX levels; it must hold whole (subtree, all heads) slots
    const int lg_slot = lgG + lgH;  // lanes one subtree's heads take
    if (lg_slot > 9) return HSA_ERR_UNSUPPORTED;
    if (threads_pref == 0) {
        // automatic: one resident round of workgroups is where the single launch pays (its
        // arrival step costs every workgroup a memory round trip, which only a kernel whose
        // workgroups all run at once does not feel): 512 threads when that fills the chip,
        // 256 when it would leave half the compute units idle, the multi-launch path beyond
        const long wg512 = ((long)B << lg_nsub) >> (9 - lg_slot);  // subtrees of all batch elements / subtrees per workgroup
        const int cus = device_compute_units();
        if (!force && wg512 > cus) return HSA_ERR_UNSUPPORTED;
        threads_pref = wg512 * 2 <= cus ? 256 : 512;
    }
    int lgT = ilog2_pow2(threads_pref);
    if (lgT < 0) return HSA_ERR_UNSUPPORTED;
    if (lgT < lg_slot) lgT = lg_slot;
    if (lgT - lg_slot > lg_nsub) lgT = lg_slot + lg_nsub;
    if (lgT - lg_slot > TREE_NLMAX) lgT = lg_slot + TREE_NLMAX;
    if (lgT > 9) lgT = 9;  // 1024 threads leave 128 registers per lane: not enough for phase A
    if (lgT < 6 || lgT < lg_slot) return HSA_ERR_UNSUPPORTED;  // less than a wavefront: tiny trees go level by level
    const int threads = 1 << lgT;
    const int lgS = ilog2_pow2(threads >> (lgG + lgH));
    const int lg_wpb = lg_nsub - lgS;
    const long blocks = (long)B << lg_wpb;
    if (blocks > 0x7fffffffL) return HSA_ERR_UNSUPPORTED;
    TreeArgs a;
    a.qp = qp; a.kp = kp; a.vp = vp; a.kleaf = k_leaf; a.vleaf = v_leaf; a.out = out; a.out2 = out2;
    a.N = N; a.H = H; a.D = D; a.L = L; a.lgG = lgG; a.lgH = lgH; a.lgS = lgS; a.lg_nsub = lg_nsub;
    a.gcap = lgS + 2 < TREE_GCAP_MAX ? lgS + 2 : TREE_GCAP_MAX;
    a.qp_bs = qp_bs; a.kp_bs = kp_bs; a.vp_bs = vp_bs; a.kleaf_bs = kleaf_bs; a.vleaf_bs = vleaf_bs;
    a.out_bs = out_bs; a.out2_bs = out2_bs;
    a.scale = 1.0f / sqrtf((float)D);
    long per_batch = 0;
    for (int w = lg_wpb; w > 0;) {
        const int g = w < a.gcap ? w : a.gcap;
        w -= g;
        per_batch += 1L << w;
    }
    a.counters_per_batch = (int)per_batch;
    a.counters = nullptr;
    if (per_batch > 0) {
        if (per_batch * B > TREE_SLICE_COUNTERS) return HSA_ERR_UNSUPPORTED;
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(st, &cap) != hipSuccess) {
            (void)hipGetLastError();
            return HSA_ERR_UNSUPPORTED;
        }
        a.counters = cap != hipStreamCaptureStatusNone ? tree_counters_for_capture(per_batch * B) : tree_counter_slice(st);
        if (!a.counters) return HSA_ERR_UNSUPPORTED;
    }
#define HSA_TREE_LAUNCH(THR, GG, HH) \
    build_tree_fused_kernel<T, VEC, TL, THR, GG, HH><<<(unsigned)blocks, THR, 0, st>>>(a)
    // the common head layouts get their own instantiation at the two larger workgroup sizes
    const int key = lgG * 16 + lgH;
    if (threads == 512 && key == 3 * 16 + 3) HSA_TREE_LAUNCH(512, 3, 3);        // 8 heads, 8 lanes per row
    else if (threads == 512 && key == 4 * 16 + 4) HSA_TREE_LAUNCH(512, 4, 4);   // 16 heads, 16 lanes per row
    else if (threads == 512 && key == 4 * 16 + 3) HSA_TREE_LAUNCH(512, 4, 3);   // 8 heads, 16 lanes per row
    else if (threads == 512 && key == 3 * 16 + 4) HSA_TREE_LAUNCH(512, 3, 4);   // 16 heads, 8 lanes per row
    else if (threads == 256 && key == 3 * 16 + 3) HSA_TREE_LAUNCH(256, 3, 3);
    else if (threads == 256 && key == 4 * 16 + 3) HSA_TREE_LAUNCH(256, 4, 3);
    else if (threads == 256 && key == 3 * 16 + 4) HSA_TREE_LAUNCH(256, 3, 4);
    else if (threads == 512) HSA_TREE_LAUNCH(512, -1, -1);
    else if (threads == 256) HSA_TREE_LAUNCH(256, -1, -1);
    else if (threads == 128) HSA_TREE_LAUNCH(128, -1, -1);
    else HSA_TREE_LAUNCH(64, -1, -1);
#undef HSA_TREE_LAUNCH
    return check_launch("build_tree_fused_kernel");
}

static std::atomic<int> g_tree_threads{0};  // 0 = by problem size
static std::atomic<int> g_tree_mode{1};     // 0 = never the single launch, 1 = where it pays, 2 = wherever possible

int build_tree_tune(int mode, int threads) {
    if (!(threads == -1 || threads == 0 || threads == 64 || threads == 128 || threads == 256 || threads == 512))
        return fail(HSA_ERR_INVALID, "workgroup size %d", threads);
    if (mode > 2) return fail(HSA_ERR_INVALID, "mode %d", mode);
    if (mode >= 0) g_tree_mode = mode;
    if (threads >= 0) g_tree_threads = threads;
    return HSA_OK;
}

int build_tree_fused_dispatch(const void *qp, const void *kp, const void *vp, const void *k_leaf, const void *v_leaf,
                              void *out, void *out2, int B, int N, int H, int D, int64_t qp_bs, int64_t kp_bs,
                              int64_t vp_bs, int64_t kleaf_bs, int64_t vleaf_bs, int64_t out_bs, int64_t out2_bs,
                              int dtype, hipStream_t st) {
    const int mode = g_tree_mode;
    if (mode == 0) return HSA_ERR_UNSUPPORTED;
    const int t = g_tree_threads;
    const bool force = mode == 2;
    switch (dtype) {
        case HSA_F32: return build_tree_fused_typed<F32>(qp, kp, vp, k_leaf, v_leaf, out, out2, B, N, H, D, qp_bs, kp_bs, vp_bs, kleaf_bs, vleaf_bs, out_bs, out2_bs, t, force, st);
        case HSA_F16: return build_tree_fused_typed<F16>(qp, kp, vp, k_leaf, v_leaf, out, out2, B, N, H, D, qp_bs, kp_bs, vp_bs, kleaf_bs, vleaf_bs, out_bs, out2_bs, t, force, st);
        case HSA_BF16: return build_tree_fused_typed<BF16>(qp, kp, vp, k_leaf, v_leaf, out, out2, B, N, H, D, qp_bs, kp_bs, vp_bs, kleaf_bs, vleaf_bs, out_bs, out2_bs, t, force, st);
    }
    return HSA_ERR_UNSUPPORTED;
}

}  // namespace hsa
