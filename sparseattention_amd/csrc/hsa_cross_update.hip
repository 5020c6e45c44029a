// Upper levels of the span-node update in one launch (16-bit element types).
//
// In the module each level l of the bottom-up pass is
//     [k_c | v_c] = src_l * W_kv^T              (projection of the children, all heads)
//     out_l       = parent build(q_l, k_l, v_l, k_c, v_c)     (3-way softmax per parent and head)
//     src_{l+1}   = out_l
// Near the root a level is a few rows, so a launch per projection and per parent build costs
// far more than the work.  Here one workgroup per batch element walks the last levels: the
// level's rows live in LDS, a wavefront owns a head, multiplies the rows by the head's 2*Dh
// weight rows with MFMA (weights streamed from L2 in a pre-packed operand order, so that every
// load instruction of a wavefront reads 1 KiB of consecutive bytes; the rows read from LDS),
// rounds the result to
// the element type as the separate projection would, and finishes the parent build from the
// accumulator registers: in the MFMA result layout a lane holds four consecutive rows of one
// column, i.e. both children of two parents, so the three scores need only a sum over the 16
// lanes that share those rows.  The level's output goes to the result tensor and to the other
// LDS buffer, which is the next level's input.
#include "hsa_mma.h"
#include "hsa_lds_dma.h"

#include <stdlib.h>

#include <atomic>

namespace hsa {

namespace {

constexpr int TOP_WAVES = 8;      // two per SIMD: up to 256 VGPRs each
constexpr int TOP_LDS_MAX = 160 * 1024;

struct TopParams {
    const uint16_t *src;  // [B, C0, Dm]  children of the first level handled here, dense rows
    const uint16_t *qkv;  // parents' q | k | v: row j of this pointer = j-th parent handled here
    const uint16_t *w;    // packed key / value projection weights (see pack_kv_kernel)
    uint16_t *out;        // result rows, numbered like qkv's
    int64_t src_bs, qkv_bs, qkv_rs, out_bs, out_rs;
    int B, H, Dm, C0;
    float scale;
};

template <typename T> __device__ __forceinline__ float rounded(float x) {
    return to_float<T>(from_float<T>(x));
}

// One head of one level: C children (rows of `cur`, `pitch` bytes apart, in LDS or in memory),
// C/2 parents out.  Two passes over the level's rows: the key columns give the softmax weights,
// the value columns the output, so only Dh accumulator columns are live at a time.  Row tiles
// reach past the level's last row when it has fewer than 16*RT children: those lanes re-read the
// last row, and what they compute belongs to no parent and is dropped.
// PD = weight k-steps in flight (divides Dm / 32).
// `tile0`: first 16-row tile of the level this call covers (RT tiles from there).
template <typename T, int CT2, int RT, bool TO_LDS, int PD>
__device__ __forceinline__ void top_level_head(const TopParams &p, int b, int h, int C, int row,
                                               const unsigned char *cur, unsigned char *nxt, int64_t pitch,
                                               int tile0 = 0) {
    // no implicit fusing of multiplies and adds: every instantiation of this function (row tiles
    // in turn or side by side) rounds at the same places; the fused ones are written as fmaf
#pragma clang fp contract(off)
    using M_ = Mma<T>;
    constexpr int Dh = 16 * CT2;
    constexpr bool EARLY = RT * CT2 <= 8;   // registers allow the parents' rows to be requested before the projection
    const int lane = threadIdx.x & 63;
    const int r16 = lane & 15, g = lane >> 4;
    const int Dm = p.Dm, NK = Dm / 32, P = C >> 1;
    const unsigned char *arow[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int r = 16 * (tile0 + rt) + r16;
        arow[rt] = cur + (int64_t)(r < C ? r : C - 1) * pitch + 16 * g;
    }

    {
        // parent e of row tile rt in this lane: 8rt + 2g + e, children = accumulator rows 2e, 2e+1
        const uint16_t *prow[RT][2];
        bool valid[RT][2];
        int prel[RT][2];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const int pe = 8 * (tile0 + rt) + 2 * g + e;
                valid[rt][e] = pe < P;
                prel[rt][e] = valid[rt][e] ? pe : P - 1;
                prow[rt][e] = p.qkv + (size_t)b * p.qkv_bs + (size_t)(row + prel[rt][e]) * p.qkv_rs + h * Dh + r16;
            }

        // acc[rt][ct] = rows 16rt.. of `cur` times weight rows wbase + 16ct + (0..15):
        // lane (r16, g) ends with column r16 of tile ct, rows 16rt + 4g .. +3.
        // The weights of PD k-steps are in flight while one step is multiplied; the scheduling
        // barriers keep the compiler from sinking those loads down to their first use.
        f32x4 acc[RT][CT2];
        auto project = [&](int half) {
            // packed weights: [half][head][k-step][column tile][lane][8 elements]
            const uint16_t *wp = p.w + ((size_t)(half * p.H + h) * NK * CT2 * 64 + lane) * 8;
            int aofs = 0;
            u32x4_t bq[PD][CT2];
            // rows that come from memory travel with the weights; rows in LDS are read at use
            u32x4_t aq[TO_LDS ? 1 : PD][RT];
            auto load_b = [&](int u, int kofs) {
#pragma unroll
                for (int ct = 0; ct < CT2; ++ct)
                    bq[u][ct] = *reinterpret_cast<const u32x4_t *>(wp + (kofs * CT2 + ct) * 512);
                if constexpr (!TO_LDS) {
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt)
                        aq[u][rt] = *reinterpret_cast<const u32x4_t *>(arow[rt] + aofs + 64 * kofs);
                }
            };
            auto step = [&](int u, bool prefetch) {
                u32x4_t a[RT];
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    if constexpr (TO_LDS) a[rt] = *reinterpret_cast<const u32x4_t *>(arow[rt] + aofs + 64 * u);
                    else a[rt] = aq[u][rt];
                }
#pragma unroll
                for (int ct = 0; ct < CT2; ++ct)
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) acc[rt][ct] = M_::k32(a[rt], bq[u][ct], acc[rt][ct]);
                if (prefetch) load_b(u, u + PD);
                __builtin_amdgcn_sched_barrier(0);
            };
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int ct = 0; ct < CT2; ++ct) acc[rt][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int u = 0; u < PD; ++u) load_b(u, u);  // NK >= PD (Dm is a multiple of 128)
            __builtin_amdgcn_sched_barrier(0);
            for (int ks0 = 0; ks0 + PD < NK; ks0 += PD) {
#pragma unroll
                for (int u = 0; u < PD; ++u) step(u, true);
                wp += PD * CT2 * 512;
                aofs += 64 * PD;
            }
#pragma unroll
            for (int u = 0; u < PD; ++u) step(u, false);
        };

        // ---- keys: the three scores and the softmax weights ----
        uint16_t rq[RT][2][CT2], rk[RT][2][CT2];
        auto load_qk = [&]() {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int e = 0; e < 2; ++e)
#pragma unroll
                    for (int c = 0; c < CT2; ++c) {
                        rq[rt][e][c] = prow[rt][e][16 * c];
                        rk[rt][e][c] = prow[rt][e][Dm + 16 * c];
                    }
            __builtin_amdgcn_sched_barrier(0);
        };
        if (EARLY) load_qk();
        project(0);
        if (!EARLY) load_qk();
        float wgt[RT][2][3];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                float s0 = 0.f, s1 = 0.f, s2 = 0.f;
#pragma unroll
                for (int c = 0; c < CT2; ++c) {
                    const float fq = to_float<T>(rq[rt][e][c]);
                    s0 = fmaf(fq, to_float<T>(rk[rt][e][c]), s0);
                    s1 = fmaf(fq, rounded<T>(acc[rt][c][2 * e]), s1);
                    s2 = fmaf(fq, rounded<T>(acc[rt][c][2 * e + 1]), s2);
                }
                s0 = group_sum(s0, 16);
                s1 = group_sum(s1, 16);
                s2 = group_sum(s2, 16);
                softmax3<T>(s0 * p.scale, s1 * p.scale, s2 * p.scale, wgt[rt][e][0], wgt[rt][e][1], wgt[rt][e][2]);
            }
        }

        // ---- values: the weighted sum, to the result tensor and to the next level's rows ----
        uint16_t rv[RT][2][CT2];
        auto load_v = [&]() {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int e = 0; e < 2; ++e)
#pragma unroll
                    for (int c = 0; c < CT2; ++c) rv[rt][e][c] = prow[rt][e][2 * Dm + 16 * c];
            __builtin_amdgcn_sched_barrier(0);
        };
        if (EARLY) load_v();
        project(1);
        if (!EARLY) load_v();
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                uint16_t *orow = p.out + (size_t)b * p.out_bs + (size_t)(row + prel[rt][e]) * p.out_rs + h * Dh + r16;
                uint16_t *lrow = TO_LDS ? reinterpret_cast<uint16_t *>(nxt + prel[rt][e] * pitch) + h * Dh + r16 : nullptr;
#pragma unroll
                for (int c = 0; c < CT2; ++c) {
                    // explicit fused multiply-adds: every instantiation rounds at the same places
                    const float o = fmaf(wgt[rt][e][2], rounded<T>(acc[rt][c][2 * e + 1]),
                                         fmaf(wgt[rt][e][1], rounded<T>(acc[rt][c][2 * e]),
                                              wgt[rt][e][0] * to_float<T>(rv[rt][e][c])));
                    const uint16_t r = from_float<T>(o);
                    if (valid[rt][e]) {
                        orow[16 * c] = r;
                        if (TO_LDS) lrow[16 * c] = r;
                    }
                }
            }
        }
    }
}

// a workgroup's wavefronts share out the heads of one level whose rows are in LDS
template <typename T, int CT2, int RT>
__device__ __forceinline__ void top_level(const TopParams &p, int b, int C, int row, const unsigned char *cur,
                                          unsigned char *nxt, int pitch) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    constexpr int PD = CT2 >= 8 ? 2 : 4;  // eight wavefronts per workgroup: 256 registers each
    for (int h = wave; h < p.H; h += TOP_WAVES) top_level_head<T, CT2, RT, true, PD>(p, b, h, C, row, cur, nxt, pitch);
}

// One level per launch, one wavefront per (batch element, head): the level's rows are read from
// memory (the previous launch's output, or the first level's children), so all B*H heads stream
// their weights on different CUs at once instead of H heads taking turns on one.  The launch
// boundary is what orders the levels.
// A lone wavefront per workgroup has 512 registers: PD weight k-steps (PD * Dh/16 KiB) are in
// flight, which is what bounds a wavefront that streams its head's weights from L2.  A level of
// more than 16 children is shared out in 16-row tiles (blockIdx.z), each streaming the weights
// again: the tiles run side by side instead of one wavefront multiplying them in turn.
// RT = 16-row tiles one wavefront multiplies side by side: with two, a level that would start more
// wavefronts than the chip has SIMDs streams its weights half as often and runs in one round.
template <typename T, int CT2, int PD, int RT = 1>
__global__ void __launch_bounds__(64) cross_update_level_kernel(TopParams p, int C, int row, const uint16_t *lsrc,
                                                                int64_t lsrc_bs, int64_t lsrc_rs) {
    const int b = blockIdx.x, h = blockIdx.y;
    top_level_head<T, CT2, RT, false, PD>(p, b, h, C, row,
                                          reinterpret_cast<const unsigned char *>(lsrc + (size_t)b * lsrc_bs), nullptr,
                                          lsrc_rs * 2, RT * (int)blockIdx.z);
}


// One level per launch for the LARGE levels: a workgroup of WAVES wavefronts shares one (batch
// element, head) and WAVES * RT row tiles of 16 children.  The head's key and value projection
// weights are staged in LDS once per workgroup (chunks of KC k-steps, both halves, two buffers:
// the next chunk is transferred global -> LDS without a stop in the registers while the current
// one is multiplied), so they are fetched once per WAVES * RT * 16 rows instead of once per
// wavefront, and both projections run in one pass over the children's rows (accumulators of both
// halves live side by side), so those rows are read once.  In the packed order a lane's operand of
// (half, k-step, column tile) is 16 consecutive bytes and a wavefront's 1 KiB: the transfer puts
// it at 16 * lane, which is also a conflict-free read.  The 3-way softmax and the weighted sum
// finish from the accumulators exactly like top_level_head (same rounding points), so the level
// needs no projection GEMM, no [rows, 2 Dm] intermediate and no separate parent build.
// OCC = workgroups per CU the kernel is compiled for (2: at most 256 registers; the weights'
// operands are then read a k-step at a time, the other workgroup covers the wait)
template <typename T, int CT2, int RT, int WAVES, int KC, int OCC = 1>
__global__ void __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(OCC)))
cross_update_level_wg_kernel(TopParams p, int C, int row,
                                                                           const uint16_t *lsrc, int64_t lsrc_bs,
                                                                           int64_t lsrc_rs) {
#pragma clang fp contract(off)
    using M_ = Mma<T>;
    extern __shared__ __align__(16) unsigned char wlds[];
    constexpr int Dh = 16 * CT2;
    constexpr int CHB = 2 * KC * CT2 * 1024;     // one buffer: [half][k-step][column tile][lane][16 bytes]
    const int b = blockIdx.x, h = blockIdx.y;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63, r16 = lane & 15, g = lane >> 4;
    const int Dm = p.Dm, NK = Dm / 32, NCH = NK / KC, P = C >> 1;
    const int tile0 = ((int)blockIdx.z * WAVES + wave) * RT;
    const unsigned char *cur = reinterpret_cast<const unsigned char *>(lsrc + (size_t)b * lsrc_bs);
    const int64_t pitch = lsrc_rs * 2;
    const unsigned char *arow[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int r = 16 * (tile0 + rt) + r16;
        arow[rt] = cur + (int64_t)(r < C ? r : C - 1) * pitch + 16 * g;
    }
    // parent e of row tile rt in this lane: 8(tile0 + rt) + 2g + e, children = accumulator rows 2e, 2e+1
    const uint16_t *prow[RT][2];
    bool valid[RT][2];
    int prel[RT][2];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int pe = 8 * (tile0 + rt) + 2 * g + e;
            valid[rt][e] = pe < P;
            prel[rt][e] = valid[rt][e] ? pe : P - 1;
            prow[rt][e] = p.qkv + (size_t)b * p.qkv_bs + (size_t)(row + prel[rt][e]) * p.qkv_rs + h * Dh + r16;
        }

    // the head's packed weights: [half][head][k-step][column tile][lane][8 elements]
    const uint16_t *wsrc[2];
#pragma unroll
    for (int half = 0; half < 2; ++half) wsrc[half] = p.w + ((size_t)(half * p.H + h) * NK * CT2 * 64 + lane) * 8;
    const uint32_t lbase = lds_address(wlds);
    // chunk c -> buffer c & 1: 2 * KC * CT2 pieces of 1 KiB, dealt to the wavefronts in turn
    auto issue = [&](int c) {
        const uint32_t dst = lbase + (c & 1) * CHB;
        for (int i = wave; i < 2 * KC * CT2; i += WAVES) {
            const int half = i / (KC * CT2), j = i - half * (KC * CT2);
            lds_dma16(wsrc[half] + (size_t)(c * KC * CT2 + j) * 512, dst + i * 1024);
        }
    };

    f32x4 accK[RT][CT2], accV[RT][CT2];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int ct = 0; ct < CT2; ++ct) {
            accK[rt][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
            accV[rt][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    // The children's rows of a whole chunk are requested a chunk ahead (a ring of KC k-steps in
    // registers), the weights' operands of a k-step one k-step ahead (from LDS): with one
    // wavefront per SIMD nothing else hides those latencies.
    u32x4_t aq[KC][RT];
    auto load_a = [&](int u, int kg) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) aq[u][rt] = *reinterpret_cast<const u32x4_t *>(arow[rt] + 64 * kg);
    };
    auto load_b = [&](u32x4_t (&bq)[2 * CT2], const unsigned char *wb, int ks) {
#pragma unroll
        for (int ct = 0; ct < CT2; ++ct) {
            bq[ct] = *reinterpret_cast<const u32x4_t *>(wb + ((0 * KC + ks) * CT2 + ct) * 1024);
            bq[CT2 + ct] = *reinterpret_cast<const u32x4_t *>(wb + ((1 * KC + ks) * CT2 + ct) * 1024);
        }
    };
    // the parents' own q, k, v (needed after the projection) are requested first: they arrive
    // behind the main loop
    uint16_t rq[RT][2][CT2], rk[RT][2][CT2], rv[RT][2][CT2];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int e = 0; e < 2; ++e)
#pragma unroll
            for (int c = 0; c < CT2; ++c) {
                rq[rt][e][c] = prow[rt][e][16 * c];
                rk[rt][e][c] = prow[rt][e][Dm + 16 * c];
                rv[rt][e][c] = prow[rt][e][2 * Dm + 16 * c];
            }
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::: "memory");
    issue(0);
#pragma unroll
    for (int u = 0; u < KC; ++u) load_a(u, u);  // NK >= KC
    __builtin_amdgcn_sched_barrier(0);

    for (int c = 0; c < NCH; ++c) {
        // this chunk's transfers (requested a chunk ago) are complete in every wavefront, and
        // every wavefront has finished reading the buffer the next chunk goes to
        // (younger than those transfers: the KC * RT row loads issued since, which stay in flight)
        asm volatile("" ::: "memory");
        wait_vmem_all_but<KC * RT>();
        lds_only_barrier();
        const bool more = c + 1 < NCH;
        if (more) issue(c + 1);
        const unsigned char *wb = wlds + (c & 1) * CHB + lane * 16;
        constexpr int NBQ = OCC >= 2 ? 1 : 2;
        u32x4_t bq[NBQ][2 * CT2];
        if constexpr (NBQ == 2) load_b(bq[0], wb, 0);
#pragma unroll
        for (int ks = 0; ks < KC; ++ks) {
            u32x4_t a[RT];
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) a[rt] = aq[ks][rt];
            if (more) load_a(ks, (c + 1) * KC + ks);
            if constexpr (NBQ == 2) {
                if (ks + 1 < KC) load_b(bq[(ks + 1) & 1], wb, ks + 1);
            } else {
                load_b(bq[0], wb, ks);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ct = 0; ct < CT2; ++ct)
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    accK[rt][ct] = M_::k32(a[rt], bq[ks & (NBQ - 1)][ct], accK[rt][ct]);
                    accV[rt][ct] = M_::k32(a[rt], bq[ks & (NBQ - 1)][CT2 + ct], accV[rt][ct]);
                }
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // ---- the three scores and the softmax weights, then the weighted sum of the values ----
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            float s0 = 0.f, s1 = 0.f, s2 = 0.f;
#pragma unroll
            for (int c = 0; c < CT2; ++c) {
                const float fq = to_float<T>(rq[rt][e][c]);
                s0 = fmaf(fq, to_float<T>(rk[rt][e][c]), s0);
                s1 = fmaf(fq, rounded<T>(accK[rt][c][2 * e]), s1);
                s2 = fmaf(fq, rounded<T>(accK[rt][c][2 * e + 1]), s2);
            }
            s0 = group_sum(s0, 16);
            s1 = group_sum(s1, 16);
            s2 = group_sum(s2, 16);
            float w0, w1, w2;
            softmax3<T>(s0 * p.scale, s1 * p.scale, s2 * p.scale, w0, w1, w2);
            uint16_t *orow = p.out + (size_t)b * p.out_bs + (size_t)(row + prel[rt][e]) * p.out_rs + h * Dh + r16;
#pragma unroll
            for (int c = 0; c < CT2; ++c) {
                // explicit fused multiply-adds: every variant of the level rounds at the same places
                const float o = fmaf(w2, rounded<T>(accV[rt][c][2 * e + 1]),
                                     fmaf(w1, rounded<T>(accV[rt][c][2 * e]), w0 * to_float<T>(rv[rt][e][c])));
                if (valid[rt][e]) orow[16 * c] = from_float<T>(o);
            }
        }
    }
}

// The LARGEST levels: the same fused level, with the head's whole key and value weights resident
// in LDS (2 * Dm/32 * Dh/16 KiB: 128 KiB at Dm 512, Dh 64) while a workgroup of eight wavefronts
// (two per SIMD: one's epilogue runs under the other's multiplications) walks several groups of
// 16 row tiles.  The weights are transferred once per workgroup and there is no barrier after the
// first; the children's rows travel through a ring of PD k-steps in registers that runs across
// the groups, so only a workgroup's very first rows are waited for.
template <typename T, int CT2, int PD>
__global__ void __launch_bounds__(512) cross_update_level_pw_kernel(TopParams p, int C, int row, const uint16_t *lsrc,
                                                                    int64_t lsrc_bs, int64_t lsrc_rs) {
#pragma clang fp contract(off)
    using M_ = Mma<T>;
    extern __shared__ __align__(16) unsigned char wlds[];
    constexpr int Dh = 16 * CT2, RT = 2, WAVES = 8;
    const int b = blockIdx.x, h = blockIdx.y, part = blockIdx.z, parts = gridDim.z;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63, r16 = lane & 15, g = lane >> 4;
    const int Dm = p.Dm, NK = Dm / 32, P = C >> 1;
    const int tiles = (C + 15) / 16, groups = (tiles + WAVES * RT - 1) / (WAVES * RT);
    const int mine = part < groups ? (groups - part + parts - 1) / parts : 0;  // this workgroup's groups
    const unsigned char *cur = reinterpret_cast<const unsigned char *>(lsrc + (size_t)b * lsrc_bs);
    const int64_t pitch = lsrc_rs * 2;

    // the head's packed weights, [half][k-step][column tile][lane][16 bytes], dealt to the wavefronts
    {
        const uint32_t lbase = lds_address(wlds);
        for (int i = wave; i < 2 * NK * CT2; i += WAVES) {
            const int half = i / (NK * CT2), j = i - half * (NK * CT2);
            lds_dma16(p.w + ((size_t)(half * p.H + h) * NK * CT2 * 64 + (size_t)j * 64 + lane) * 8, lbase + i * 1024);
        }
    }
    auto rows_of = [&](int gi, const unsigned char *(&ar)[RT]) {  // group gi of this workgroup
        const int tile0 = ((part + gi * parts) * WAVES + wave) * RT;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            const int r = 16 * (tile0 + rt) + r16;
            ar[rt] = cur + (int64_t)(r < C ? r : C - 1) * pitch + 16 * g;
        }
        return tile0;
    };
    const unsigned char *arow[RT], *anext[RT];
    u32x4_t aq[PD][RT];
    if (mine > 0) {
        rows_of(0, arow);
#pragma unroll
        for (int u = 0; u < PD; ++u)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) aq[u][rt] = *reinterpret_cast<const u32x4_t *>(arow[rt] + 64 * u);  // NK >= PD
    }
    asm volatile("" ::: "memory");
    // the transfers are older than the PD * RT row loads just issued (none if this workgroup has no group)
    if (mine > 0) wait_vmem_all_but<PD * RT>();
    else wait_vmem_all_but<0>();
    lds_only_barrier();
    const unsigned char *wb = wlds + lane * 16;

    for (int gi = 0; gi < mine; ++gi) {
        const int tile0 = rows_of(gi, arow);
        const bool has_next = gi + 1 < mine;
        if (has_next) rows_of(gi + 1, anext);
        // parent e of row tile rt in this lane: 8(tile0 + rt) + 2g + e, children = accumulator rows 2e, 2e+1
        const uint16_t *prow[RT][2];
        bool valid[RT][2];
        int prel[RT][2];
        uint16_t rq[RT][2][CT2], rk[RT][2][CT2], rv[RT][2][CT2];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const int pe = 8 * (tile0 + rt) + 2 * g + e;
                valid[rt][e] = pe < P;
                prel[rt][e] = valid[rt][e] ? pe : P - 1;
                prow[rt][e] = p.qkv + (size_t)b * p.qkv_bs + (size_t)(row + prel[rt][e]) * p.qkv_rs + h * Dh + r16;
#pragma unroll
                for (int c = 0; c < CT2; ++c) {  // needed after the projection: they arrive behind it
                    rq[rt][e][c] = prow[rt][e][16 * c];
                    rk[rt][e][c] = prow[rt][e][Dm + 16 * c];
                    rv[rt][e][c] = prow[rt][e][2 * Dm + 16 * c];
                }
            }
        f32x4 accK[RT][CT2], accV[RT][CT2];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int ct = 0; ct < CT2; ++ct) {
                accK[rt][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
                accV[rt][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
        __builtin_amdgcn_sched_barrier(0);
        for (int ks0 = 0; ks0 < NK; ks0 += PD) {
#pragma unroll
            for (int u = 0; u < PD; ++u) {
                const int ks = ks0 + u;
                u32x4_t a[RT];
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) a[rt] = aq[u][rt];
                // the ring runs on into the next group's rows
                const int kn = ks + PD;
                if (kn < NK) {
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) aq[u][rt] = *reinterpret_cast<const u32x4_t *>(arow[rt] + 64 * kn);
                } else if (has_next) {
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) aq[u][rt] = *reinterpret_cast<const u32x4_t *>(anext[rt] + 64 * (kn - NK));
                }
                u32x4_t bq[2 * CT2];
#pragma unroll
                for (int ct = 0; ct < CT2; ++ct) {
                    bq[ct] = *reinterpret_cast<const u32x4_t *>(wb + ((size_t)(0 * NK + ks) * CT2 + ct) * 1024);
                    bq[CT2 + ct] = *reinterpret_cast<const u32x4_t *>(wb + ((size_t)(1 * NK + ks) * CT2 + ct) * 1024);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int ct = 0; ct < CT2; ++ct)
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) {
                        accK[rt][ct] = M_::k32(a[rt], bq[ct], accK[rt][ct]);
                        accV[rt][ct] = M_::k32(a[rt], bq[CT2 + ct], accV[rt][ct]);
                    }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // ---- the three scores and the softmax weights, then the weighted sum of the values ----
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                float s0 = 0.f, s1 = 0.f, s2 = 0.f;
#pragma unroll
                for (int c = 0; c < CT2; ++c) {
                    const float fq = to_float<T>(rq[rt][e][c]);
                    s0 = fmaf(fq, to_float<T>(rk[rt][e][c]), s0);
                    s1 = fmaf(fq, rounded<T>(accK[rt][c][2 * e]), s1);
                    s2 = fmaf(fq, rounded<T>(accK[rt][c][2 * e + 1]), s2);
                }
                s0 = group_sum(s0, 16);
                s1 = group_sum(s1, 16);
                s2 = group_sum(s2, 16);
                float w0, w1, w2;
                softmax3<T>(s0 * p.scale, s1 * p.scale, s2 * p.scale, w0, w1, w2);
                uint16_t *orow = p.out + (size_t)b * p.out_bs + (size_t)(row + prel[rt][e]) * p.out_rs + h * Dh + r16;
#pragma unroll
                for (int c = 0; c < CT2; ++c) {
                    // explicit fused multiply-adds: every variant of the level rounds at the same places
                    const float o = fmaf(w2, rounded<T>(accV[rt][c][2 * e + 1]),
                                         fmaf(w1, rounded<T>(accV[rt][c][2 * e]), w0 * to_float<T>(rv[rt][e][c])));
                    if (valid[rt][e]) orow[16 * c] = from_float<T>(o);
                }
            }
        }
    }
}

template <typename T, int CT2, int RT0>
__global__ void __launch_bounds__(TOP_WAVES * 64) cross_update_top_kernel(TopParams p) {
    extern __shared__ __align__(16) unsigned char top_smem[];
    const int b = blockIdx.x;
    const int Dm = p.Dm;
    const int pitch = Dm * 2 + 16;
    unsigned char *buf0 = top_smem;
    unsigned char *buf1 = top_smem + 16 * RT0 * pitch;
    {
        // The MFMA passes always read whole 16-row tiles: rows that hold no node (fewer than 16
        // children in a level) are zero, never uninitialised memory.
        constexpr int ROWS = 16 * RT0 + (RT0 >= 2 ? 8 * RT0 : 16);
        const int cpr = (Dm + 8) / 8;  // 16-byte pieces per padded row
        const uint16_t *src = p.src + (size_t)b * p.src_bs;
        for (int i = threadIdx.x; i < ROWS * cpr; i += TOP_WAVES * 64) {
            const int r = i / cpr, c = i - r * cpr;
            u32x4_t val = {0u, 0u, 0u, 0u};
            if (r < p.C0 && 8 * c < Dm) val = *reinterpret_cast<const u32x4_t *>(src + (size_t)r * Dm + 8 * c);
            *reinterpret_cast<u32x4_t *>(top_smem + r * pitch + 16 * c) = val;
        }
    }
    __syncthreads();
    int C = p.C0, row = 0;
    unsigned char *cur = buf0, *nxt = buf1;
    auto advance = [&]() {
        __syncthreads();
        row += C >> 1;
        C >>= 1;
        unsigned char *t = cur;
        cur = nxt;
        nxt = t;
    };
    if constexpr (RT0 >= 4) {
        top_level<T, CT2, 4>(p, b, C, row, cur, nxt, pitch);
        advance();
    }
    if constexpr (RT0 >= 2) {
        top_level<T, CT2, 2>(p, b, C, row, cur, nxt, pitch);
        advance();
    }
    while (C >= 2) {
        top_level<T, CT2, 1>(p, b, C, row, cur, nxt, pitch);
        advance();
    }
}

// Weights into MFMA operand order: packed[half][h][ks][ct][lane = 16g + r][0..7] =
// W_half[h*Dh + 16ct + r][32ks + 8g + 0..7], half 0 = keys, 1 = values.  One thread per
// 16-byte piece.
__global__ void __launch_bounds__(256) pack_kv_kernel(const uint16_t *__restrict__ wk, const uint16_t *__restrict__ wv,
                                                      uint16_t *__restrict__ packed, int H, int Dh, int Dm) {
    const int CT2 = Dh / 16, NK = Dm / 32;
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= 2L * Dm * Dm / 8) return;
    const int lane = (int)(idx & 63);
    long t = idx >> 6;
    const int ct = (int)(t % CT2); t /= CT2;
    const int ks = (int)(t % NK); t /= NK;
    const int h = (int)(t % H);
    const int half = (int)(t / H);
    const int r = lane & 15, g = lane >> 4;
    const uint16_t *src = (half ? wv : wk) + (size_t)(h * Dh + 16 * ct + r) * Dm + 32 * ks + 8 * g;
    *reinterpret_cast<u32x4_t *>(packed + idx * 8) = *reinterpret_cast<const u32x4_t *>(src);
}

// row tiles the first level may have: registers first, then LDS
int top_row_tiles(int H, int Dh) {
    int rt = 16 / (Dh / 16);  // RT * (Dh/16) accumulator tiles <= 16
    if (rt > 4) rt = 4;
    const long pitch = (long)H * Dh * 2 + 16;
    while (rt >= 1 && (16L * rt + (rt >= 2 ? 8L * rt : 16L)) * pitch > TOP_LDS_MAX) rt >>= 1;
    return rt;
}

bool top_shape_ok(int H, int Dh, int dtype) {
    if (dtype != HSA_F16 && dtype != HSA_BF16) return false;
    if (Dh != 32 && Dh != 64 && Dh != 128) return false;
    if (H < 1 || ((long)H * Dh) % 128 != 0) return false;
    return top_row_tiles(H, Dh) >= 1;
}

template <typename T, int CT2, int RT0>
int top_launch_rt(const TopParams &p, hipStream_t st) {
    const int pitch = p.Dm * 2 + 16;
    const size_t lds = (size_t)(16 * RT0 + (RT0 >= 2 ? 8 * RT0 : 16)) * pitch;
    auto kern = cross_update_top_kernel<T, CT2, RT0>;
    if (lds > 64 * 1024) {
        // raising the limit is slow: once per kernel and device, for the largest size it is asked for
        static std::atomic<size_t> allowed[64];
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return fail(HSA_ERR_LAUNCH, "no current device");
        if (allowed[dev].load(std::memory_order_acquire) < lds) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return fail(HSA_ERR_LAUNCH, "LDS size %zu refused: %s", lds, hipGetErrorString(e));
            allowed[dev].store(lds, std::memory_order_release);
        }
    }
    kern<<<p.B, TOP_WAVES * 64, lds, st>>>(p);
    return check_launch("cross_update_top_kernel");
}

// 0 = one launch per level where the result rows allow 16-byte reads, 1 = always the single launch.
// Initialised once from HSA_CROSS_TOP_SINGLE, changed afterwards through hsa_cross_update_top_tune.
static std::atomic<int> &top_single_launch() {
    static std::atomic<int> v{[] { const char *e = getenv("HSA_CROSS_TOP_SINGLE"); return e && atoi(e) != 0 ? 1 : 0; }()};
    return v;
}

// one launch per level reads the previous level's result rows 16 bytes at a time
static bool top_levels_eligible(const TopParams &p) {
    // the per-level kernel moves 16-byte pieces of the children's rows and of the result rows
    return !top_single_launch().load() && ((uintptr_t)p.out & 15) == 0 && p.out_rs % 8 == 0 && p.out_bs % 8 == 0 &&
           ((uintptr_t)p.src & 15) == 0 && p.src_bs % 8 == 0 && p.Dm % 8 == 0;
}

// knob for experiments: levels with at least this many 16-row tiles take the workgroup kernel
// (0: never)
static std::atomic<int> &level_wg_min_tiles() {
    static std::atomic<int> v{[] { const char *e = getenv("HSA_CROSS_WG_MIN_TILES"); return e ? atoi(e) : 8; }()};
    return v;
}

// batch size times children of the largest level the per-level launches take over from the GEMMs
// (0: chosen by shape)
static std::atomic<long> &level_rows_limit() {
    static std::atomic<long> v{[] { const char *e = getenv("HSA_CROSS_LEVEL_ROWS_LIMIT"); return e ? atol(e) : 0L; }()};
    return v;
}

// whether the kernel with the head's weights resident in LDS is built for this head layout
static bool level_pw_capable(int H, int Dh) {
    const long Dm = (long)H * Dh;
    return Dh <= 64 && 2 * (Dm / 32) * (Dh / 16) * 1024 <= 128 * 1024;
}

constexpr int LEVEL_WG_WAVES = 4;

template <typename T, int CT2, int RT, int KC, int OCC = 1>
int launch_level_wg(const TopParams &p, int C, int row, const uint16_t *lsrc, int64_t lbs, int64_t lrs, hipStream_t st) {
    const size_t lds = 2 * (size_t)(2 * KC * CT2 * 1024);
    auto kern = cross_update_level_wg_kernel<T, CT2, RT, LEVEL_WG_WAVES, KC, OCC>;
    if (lds > 64 * 1024) {
        // raising the limit is slow: once per kernel and device
        static std::atomic<bool> allowed[64];
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return fail(HSA_ERR_LAUNCH, "no current device");
        if (!allowed[dev].load(std::memory_order_acquire)) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return fail(HSA_ERR_LAUNCH, "LDS size %zu refused: %s", lds, hipGetErrorString(e));
            allowed[dev].store(true, std::memory_order_release);
        }
    }
    const int tiles = (C + 15) / 16;
    const dim3 grid((unsigned)p.B, (unsigned)p.H, (unsigned)((tiles + LEVEL_WG_WAVES * RT - 1) / (LEVEL_WG_WAVES * RT)));
    kern<<<grid, LEVEL_WG_WAVES * 64, lds, st>>>(p, C, row, lsrc, lbs, lrs);
    return HSA_OK;
}

// the variant with the head's weights resident in LDS: where they fit and a workgroup has at
// least two groups of 16 row tiles to walk
template <typename T, int CT2>
int launch_level_pw(const TopParams &p, int C, int row, const uint16_t *lsrc, int64_t lbs, int64_t lrs, hipStream_t st,
                    bool &taken) {
    taken = false;
    const int NK = p.Dm / 32;
    const size_t lds = (size_t)2 * NK * CT2 * 1024;
    if (!level_pw_capable(p.H, 16 * CT2)) return HSA_OK;
    const long tiles = (C + 15) / 16, groups = (tiles + 15) / 16, bh = (long)p.B * p.H;
    long parts = 256 / bh;
    if (parts < 1) parts = 1;
    if (parts > groups) parts = groups;
    if (groups < 2 * parts) return HSA_OK;
    if constexpr (CT2 > 4) return HSA_OK;
    taken = true;
    auto launch = [&](auto kern) -> int {
        static std::atomic<bool> allowed[64];
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return fail(HSA_ERR_LAUNCH, "no current device");
        if (lds > 64 * 1024 && !allowed[dev].load(std::memory_order_acquire)) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
            if (e != hipSuccess) return fail(HSA_ERR_LAUNCH, "LDS size %zu refused: %s", lds, hipGetErrorString(e));
            allowed[dev].store(true, std::memory_order_release);
        }
        kern<<<dim3((unsigned)p.B, (unsigned)p.H, (unsigned)parts), 512, lds, st>>>(p, C, row, lsrc, lbs, lrs);
        return HSA_OK;
    };
    if constexpr (CT2 <= 2) {
        if (NK % 8 == 0) return launch(cross_update_level_pw_kernel<T, CT2, 8>);
    }
    if constexpr (CT2 <= 4) {
        return launch(cross_update_level_pw_kernel<T, CT2, 4>);
    } else {
        taken = false;  // 128 channels per head: the accumulators of both halves do not fit two wavefronts per SIMD
        return HSA_OK;
    }
}

// Which variant: two row tiles per wavefront where that still starts a workgroup per CU (else
// one); two workgroups per CU (chunks of four k-steps: 64 KB of LDS) where there are at least two
// per CU to start.  Measured at B8 H8 Dh64 (us per level of 4096 / 2048 / 1024 / 512 / 256 / 128
// children): 68 / 34 / 18.5 / 10.9 / 7.2 / 6.7; a GEMM plus the parent build take 71 / 36 / 26,
// the launch per wavefront and row tile 18 / 10.4 / 7.2 from 512 children down.
template <typename T, int CT2>
int launch_level_wg_any(const TopParams &p, int C, int row, const uint16_t *lsrc, int64_t lbs, int64_t lrs, hipStream_t st) {
    const int NK = p.Dm / 32;
    const long tiles = (C + 15) / 16, bh = (long)p.B * p.H;
    {
        bool taken = false;
        const int rc = launch_level_pw<T, CT2>(p, C, row, lsrc, lbs, lrs, st, taken);
        if (taken || rc != HSA_OK) return rc;
    }
    auto wgs = [&](int rt) { return bh * ((tiles + LEVEL_WG_WAVES * rt - 1) / (LEVEL_WG_WAVES * rt)); };
    if constexpr (CT2 <= 4) {
        if (wgs(2) >= 512) return launch_level_wg<T, CT2, 2, 4, 2>(p, C, row, lsrc, lbs, lrs, st);
        if (NK % 8 == 0) {
            if (wgs(2) >= 256) return launch_level_wg<T, CT2, 2, 8>(p, C, row, lsrc, lbs, lrs, st);
            return launch_level_wg<T, CT2, 1, 8>(p, C, row, lsrc, lbs, lrs, st);
        }
    }
    if (wgs(2) >= 256) return launch_level_wg<T, CT2, 2, 4>(p, C, row, lsrc, lbs, lrs, st);  // Dm is a multiple of 128
    return launch_level_wg<T, CT2, 1, 4>(p, C, row, lsrc, lbs, lrs, st);
}

template <typename T, int CT2, int PD>
int top_launch_levels_pd(const TopParams &p, hipStream_t st) {
    int C = p.C0, row = 0;
    const uint16_t *lsrc = p.src;
    int64_t lbs = p.src_bs, lrs = p.Dm;
    const int wg_min = level_wg_min_tiles().load();
    while (C >= 2) {
        const int tiles = (C + 15) / 16;
        if (wg_min > 0 && tiles >= wg_min) {
            const int rc = launch_level_wg_any<T, CT2>(p, C, row, lsrc, lbs, lrs, st);
            if (rc != HSA_OK) return rc;
            lsrc = p.out + (size_t)row * p.out_rs;
            lbs = p.out_bs;
            lrs = p.out_rs;
            row += C >> 1;
            C >>= 1;
            continue;
        }
        // two row tiles per wavefront where single tiles would need a second round of wavefronts
        // (1024 SIMDs; a lone wavefront's registers hold two tiles' operands up to 64 channels)
        if (CT2 <= 4 && tiles % 2 == 0 && (long)p.B * p.H * tiles >= 2048) {
            const dim3 grid((unsigned)p.B, (unsigned)p.H, (unsigned)(tiles / 2));
            cross_update_level_kernel<T, CT2, PD, 2><<<grid, 64, 0, st>>>(p, C, row, lsrc, lbs, lrs);
        } else {
            const dim3 grid((unsigned)p.B, (unsigned)p.H, (unsigned)tiles);
            cross_update_level_kernel<T, CT2, PD><<<grid, 64, 0, st>>>(p, C, row, lsrc, lbs, lrs);
        }
        // the next level's children are the rows just written
        lsrc = p.out + (size_t)row * p.out_rs;
        lbs = p.out_bs;
        lrs = p.out_rs;
        row += C >> 1;
        C >>= 1;
    }
    return check_launch("cross_update_level_kernel");
}

template <typename T, int CT2>
int top_launch_levels(const TopParams &p, hipStream_t st) {
    constexpr int DEEP = CT2 >= 8 ? 4 : 8;
    if ((p.Dm / 32) % DEEP == 0) return top_launch_levels_pd<T, CT2, DEEP>(p, st);
    return top_launch_levels_pd<T, CT2, DEEP / 2>(p, st);
}

template <typename T, int CT2>
int top_launch_ct(const TopParams &p, hipStream_t st) {
    if (top_levels_eligible(p)) return top_launch_levels<T, CT2>(p, st);
    const int rt0 = p.C0 >= 64 ? 4 : (p.C0 >= 32 ? 2 : 1);
    if constexpr (CT2 <= 4) {
        if (rt0 == 4) return top_launch_rt<T, CT2, 4>(p, st);
    }
    if (rt0 == 2) return top_launch_rt<T, CT2, 2>(p, st);
    if (rt0 == 1) return top_launch_rt<T, CT2, 1>(p, st);
    return fail(HSA_ERR_UNSUPPORTED, "too many rows (%d) for head_dim %d", p.C0, 16 * CT2);
}

template <typename T>
int top_launch(const TopParams &p, int Dh, hipStream_t st) {
    switch (Dh) {
        case 32: return top_launch_ct<T, 2>(p, st);
        case 64: return top_launch_ct<T, 4>(p, st);
        case 128: return top_launch_ct<T, 8>(p, st);
    }
    return fail(HSA_ERR_UNSUPPORTED, "head_dim %d", Dh);
}

}  // namespace

}  // namespace hsa

extern "C" {

int hsa_cross_update_top_tune(int single_launch) {
    if (single_launch < -1 || single_launch > 1) return hsa::fail(HSA_ERR_INVALID, "single_launch %d", single_launch);
    if (single_launch >= 0) hsa::top_single_launch().store(single_launch);
    return HSA_OK;
}

int hsa_cross_update_level_tune(int wg_min_tiles, long rows_limit) {
    if (wg_min_tiles < -1 || rows_limit < -1) return hsa::fail(HSA_ERR_INVALID, "knob below -1");
    if (wg_min_tiles >= 0) hsa::level_wg_min_tiles().store(wg_min_tiles);
    if (rows_limit >= 0) hsa::level_rows_limit().store(rows_limit);
    return HSA_OK;
}

int hsa_cross_update_top_rows(int H, int Dh, int dtype) {
    if (!hsa::top_shape_ok(H, Dh, dtype)) return 0;
    return 16 * hsa::top_row_tiles(H, Dh);
}

int hsa_cross_update_level_rows(int B, int H, int Dh, int dtype) {
    if (B < 1 || !hsa::top_shape_ok(H, Dh, dtype)) return 0;
    const int held = 16 * hsa::top_row_tiles(H, Dh);
    if (hsa::top_single_launch().load()) return held;
    // one launch per level re-reads a head's weights for every 16 rows: it beats a GEMM and a
    // parent build per level while the batch's rows of a level are few (measured on the LM forward
    // at 4096 tokens: up to 4096 rows at batch 1, 1024 at 4, 512 at 8, no gain from 32 on)
    int rows = held;
    // Measured on the LM forward at 4096 tokens, batch 8, 8 heads of 64 channels (us per level of
    // 4096 / 2048 / 1024 children): a GEMM plus the parent build 71 / 36 / 26, the fused level with
    // the weights resident in LDS 51 / 29 / -, with the weights staged in chunks 68 / 34 / 18.5:
    // where the resident variant is built every level is handed over, elsewhere B * C <= 8192.
    long limit = hsa::level_rows_limit().load();
    if (limit <= 0) limit = hsa::level_pw_capable(H, Dh) ? (1L << 40) : 8192L;
    while ((long)B * rows * 2 <= limit && rows * 2 <= (1 << 20)) rows *= 2;
    return rows;
}

int hsa_cross_update_pack_weights(const void *wk, const void *wv, void *packed, int H, int Dh, int dtype,
                                  void *stream) {
    HSA_REQUIRE(wk && wv && packed, "null pointer");
    if (!hsa::top_shape_ok(H, Dh, dtype))
        return hsa::fail(HSA_ERR_UNSUPPORTED, "shape H=%d Dh=%d dtype=%d not handled by the fused levels", H, Dh, dtype);
    HSA_REQUIRE((((uintptr_t)wk | (uintptr_t)wv | (uintptr_t)packed) & 15) == 0, "weights must be 16-byte aligned");
    const int Dm = H * Dh;
    const long pieces = 2L * Dm * Dm / 8;
    hsa::pack_kv_kernel<<<(unsigned)((pieces + 255) / 256), 256, 0, (hipStream_t)stream>>>(
        (const uint16_t *)wk, (const uint16_t *)wv, (uint16_t *)packed, H, Dh, Dm);
    return hsa::check_launch("pack_kv_kernel");
}

int hsa_cross_update_top_fwd(const void *src, const void *qkv, const void *w_kv, void *out, int B, int C,
                             int H, int Dh, int64_t src_bs, int64_t qkv_bs, int64_t qkv_rs, int64_t out_bs,
                             int64_t out_rs, int dtype, void *stream) {
    HSA_REQUIRE(src && qkv && w_kv && out, "null pointer");
    HSA_REQUIRE(B >= 1 && H >= 1 && Dh >= 1, "bad shape B=%d H=%d Dh=%d", B, H, Dh);
    HSA_REQUIRE(C >= 2 && hsa::ilog2_exact(C) >= 0, "row count must be a power of two >= 2 (got %d)", C);
    HSA_REQUIRE(C <= (1 << 20) && H <= 65535, "C=%d or H=%d beyond what one grid covers", C, H);
    if (!hsa::top_shape_ok(H, Dh, dtype))
        return hsa::fail(HSA_ERR_UNSUPPORTED, "shape H=%d Dh=%d dtype=%d not handled by the fused levels", H, Dh, dtype);
    const int64_t Dm = (int64_t)H * Dh;
    if (!src_bs) src_bs = (int64_t)C * Dm;
    if (!qkv_rs) qkv_rs = 3 * Dm;
    if (!out_rs) out_rs = Dm;
    if (!qkv_bs) qkv_bs = (int64_t)(C - 1) * qkv_rs;
    if (!out_bs) out_bs = (int64_t)(C - 1) * out_rs;
    HSA_REQUIRE(qkv_rs >= 3 * Dm && out_rs >= Dm, "row strides below the row length");
    HSA_REQUIRE((((uintptr_t)src | (uintptr_t)w_kv) & 15) == 0 && src_bs % 8 == 0,
                "src and w_kv must be 16-byte aligned");
    hsa::TopParams p;
    p.src = (const uint16_t *)src;
    p.qkv = (const uint16_t *)qkv;
    p.w = (const uint16_t *)w_kv;
    p.out = (uint16_t *)out;
    p.src_bs = src_bs; p.qkv_bs = qkv_bs; p.qkv_rs = qkv_rs; p.out_bs = out_bs; p.out_rs = out_rs;
    p.B = B; p.H = H; p.Dm = (int)Dm; p.C0 = C;
    p.scale = 1.0f / sqrtf((float)Dh);
    // the single launch holds a level in registers and LDS; a launch per level takes any size
    if (C > 16 * hsa::top_row_tiles(H, Dh) && !hsa::top_levels_eligible(p))
        return hsa::fail(HSA_ERR_UNSUPPORTED, "%d rows exceed the %d the single launch holds", C,
                         16 * hsa::top_row_tiles(H, Dh));
    if (dtype == HSA_BF16) return hsa::top_launch<hsa::BF16>(p, Dh, (hipStream_t)stream);
    return hsa::top_launch<hsa::F16>(p, Dh, (hipStream_t)stream);
}

}  // extern "C"
