// Bottom-up parent build: each parent attends over {itself, child 2i, child 2i+1}.
//
// Streaming kernel: a group of G lanes owns one (batch, parent, head) row and
// reads it in 16-byte pieces, so a wavefront covers 64/G consecutive head rows
// (one or more whole token rows) per load instruction.  The three dot products
// are reduced inside the group with xor shuffles; the 3-way softmax and the
// weighted sum of the value rows stay in fp32 registers.
#include "hsa_build_vec.h"

namespace hsa {

// Batch and row strides (in elements) of the seven operands of one level, in the order
// qp, kp, vp, kc, vc, out, out2.  A row stride wider than H*D reads a column slice of a
// wider matrix, e.g. one third of a fused q/k/v projection.
struct LevelStrides {
    int64_t bs[7];
    int64_t rs[7];
};

// CH = number of VEC-chunks each lane holds (D <= G * VEC * CH).
template <typename T, int VEC, int CH>
__global__ void __launch_bounds__(256)
build_parents_kernel(const typename T::storage *__restrict__ Qp, const typename T::storage *__restrict__ Kp,
                     const typename T::storage *__restrict__ Vp, const typename T::storage *__restrict__ Kc,
                     const typename T::storage *__restrict__ Vc, typename T::storage *__restrict__ Out,
                     typename T::storage *__restrict__ Out2, typename T::storage *__restrict__ Wt, int B,
                     int P, int H, int D, int G, LevelStrides sd, float scale) {
    const long tid = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long unit = tid / G;
    const int gl = (int)(tid % G);
    const long units = (long)B * P * H;
    const bool active = unit < units;
    const long u = active ? unit : units - 1;  // keep every lane in the shuffles
    const int h = (int)(u % H);
    const int i = (int)((u / H) % P);
    const int b = (int)(u / ((long)H * P));
    const size_t hd = (size_t)h * D;
    const typename T::storage *q = Qp + (size_t)b * sd.bs[0] + (size_t)i * sd.rs[0] + hd;
    const typename T::storage *kp = Kp + (size_t)b * sd.bs[1] + (size_t)i * sd.rs[1] + hd;
    const typename T::storage *vp = Vp + (size_t)b * sd.bs[2] + (size_t)i * sd.rs[2] + hd;
    const typename T::storage *k0 = Kc + (size_t)b * sd.bs[3] + (size_t)(2 * i) * sd.rs[3] + hd;
    const typename T::storage *k1 = k0 + sd.rs[3];
    const typename T::storage *v0 = Vc + (size_t)b * sd.bs[4] + (size_t)(2 * i) * sd.rs[4] + hd;
    const typename T::storage *v1 = v0 + sd.rs[4];

    float fvp[CH][VEC], fv0[CH][VEC], fv1[CH][VEC];
    float s0 = 0.f, s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int d = (c * G + gl) * VEC;
        if (d < D) {
            float fq[VEC], fk[VEC];
            load_vec<T, VEC>(q + d, fq);
            load_vec<T, VEC>(kp + d, fk);
#pragma unroll
            for (int e = 0; e < VEC; ++e) s0 = fmaf(fq[e], fk[e], s0);
            load_vec<T, VEC>(k0 + d, fk);
#pragma unroll
            for (int e = 0; e < VEC; ++e) s1 = fmaf(fq[e], fk[e], s1);
            load_vec<T, VEC>(k1 + d, fk);
#pragma unroll
            for (int e = 0; e < VEC; ++e) s2 = fmaf(fq[e], fk[e], s2);
            load_vec<T, VEC>(vp + d, fvp[c]);
            load_vec<T, VEC>(v0 + d, fv0[c]);
            load_vec<T, VEC>(v1 + d, fv1[c]);
        }
    }
    s0 = group_sum(s0, G);
    s1 = group_sum(s1, G);
    s2 = group_sum(s2, G);
    float w0, w1, w2;
    softmax3<T>(s0 * scale, s1 * scale, s2 * scale, w0, w1, w2);
    if (!active) return;
    typename T::storage *o = Out + (size_t)b * sd.bs[5] + (size_t)i * sd.rs[5] + hd;
    typename T::storage *o2 = Out2 ? Out2 + (size_t)b * sd.bs[6] + (size_t)i * sd.rs[6] + hd : nullptr;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int d = (c * G + gl) * VEC;
        if (d < D) {
            float r[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) r[e] = w0 * fvp[c][e] + w1 * fv0[c][e] + w2 * fv1[c][e];
            store_vec<T, VEC>(o + d, r);
            if (o2) store_vec<T, VEC>(o2 + d, r);
        }
    }
    if (Wt && gl == 0) {
        typename T::storage *wp = Wt + (((size_t)b * P + i) * H + h) * 3;
        wp[0] = from_float<T>(w0);
        wp[1] = from_float<T>(w1);
        wp[2] = from_float<T>(w2);
    }
}

template <typename T, int VEC>
static int build_parents_launch(const void *qp, const void *kp, const void *vp, const void *kc,
                                const void *vc, void *out, void *out2, void *weights, int B, int P, int H, int D,
                                const LevelStrides &sd, hipStream_t st) {
    using S = typename T::storage;
    const int chunks = (D + VEC - 1) / VEC;  // D % VEC == 0 guaranteed by the caller when VEC > 1
    int G = 1;
    while (G < chunks && G < 64) G <<= 1;
    const int CH = (chunks + G - 1) / G;
    const long threads = (long)B * P * H * G;
    const int block = 256;
    const long blocks = (threads + block - 1) / block;
    if (blocks > 0x7fffffffL) return fail(HSA_ERR_UNSUPPORTED, "problem too large for one launch");
    const float scale = 1.0f / sqrtf((float)D);
#define HSA_BPN_LAUNCH(CHN)                                                                        \
    build_parents_kernel<T, VEC, CHN><<<(unsigned)blocks, block, 0, st>>>(                         \
        (const S *)qp, (const S *)kp, (const S *)vp, (const S *)kc, (const S *)vc, (S *)out,       \
        (S *)out2, (S *)weights, B, P, H, D, G, sd, scale)
    if (CH == 1) HSA_BPN_LAUNCH(1);
    else if (CH == 2) HSA_BPN_LAUNCH(2);
    else if (CH <= 4) HSA_BPN_LAUNCH(4);
    else if (CH <= 8) HSA_BPN_LAUNCH(8);
    else return fail(HSA_ERR_UNSUPPORTED, "head_dim %d too large", D);
#undef HSA_BPN_LAUNCH
    return check_launch("build_parents_kernel");
}

// ---- several levels per launch ----------------------------------------------------------
// A group of G lanes owns one (batch, head) and a subtree of 2^TL consecutive children
// (leaves, or the outputs of the previous pass).  The children's K/V pieces and every
// intermediate level stay in registers; each level's output is rounded to the element
// type before it feeds the next level, exactly as if the levels had been separate calls.
// With G * VEC == D a wavefront reads whole token rows (all heads) per load instruction.
// SHARED: the children's keys and values are the same rows (every pass after the first),
// loaded once.  Passes of four levels run one wavefront per workgroup (up to 512 VGPRs).
template <int TL> constexpr int subtree_block() { return TL >= 4 ? 64 : 256; }

// STREAM: node rows are stored with the streaming hint.  Regular stores leave them in the caches
// for the kernels that read them next, which pays as long as the memory-side cache (256 MB) can
// hold them; beyond that the rows are dirty lines the next kernel has to wait for, and the
// build itself is 6-8 % faster without them (B1 H16 N65536 D128: 375 -> 355 us, and the span
// attention after it 346 -> 311 us).
template <typename T, int VEC, int TL, bool SHARED, bool STREAM>
__global__ void __launch_bounds__(subtree_block<TL>())
build_subtree_kernel(const typename T::storage *__restrict__ Qp, const typename T::storage *__restrict__ Kp,
                     const typename T::storage *__restrict__ Vp, const typename T::storage *__restrict__ Kc,
                     const typename T::storage *__restrict__ Vc, typename T::storage *__restrict__ Out,
                     typename T::storage *__restrict__ Out2, int B, int N, int H, int D, int G, int lvl0,
                     int64_t qp_bs, int64_t kp_bs, int64_t vp_bs, int64_t kc_bs, int64_t vc_bs,
                     int64_t out_bs, int64_t out2_bs, float scale) {
    using S = typename T::storage;
    constexpr int NC = 1 << TL;
    // 32-bit index arithmetic (the launcher guarantees the thread count fits); G and the
    // number of subtrees per sequence are powers of two
    const int tid = (int)(blockIdx.x * blockDim.x + threadIdx.x);
    const int lg = 31 - __builtin_clz(G);
    const int unit = tid >> lg;
    const int gl = tid & (G - 1);
    const int n_sub = (N >> lvl0) >> TL;  // subtrees per (batch, head)
    const int lsub = 31 - __builtin_clz(n_sub);
    const int units = (B * H) << lsub;
    const bool active = unit < units;
    const int u = active ? unit : units - 1;
    const int h = u % H;
    const int bs = u / H;  // batch * n_sub + sub
    const int sub = bs & (n_sub - 1);
    const int b = bs >> lsub;
    const int d = gl * VEC;
    const bool dok = d < D;
    const size_t rs = (size_t)H * D;
    const size_t hd = (size_t)h * D + (dok ? d : 0);

    // Every row this subtree needs is requested up front, in the order the results are used
    // (first level parent by parent: its two children and its own q/k/v; then the upper levels).
    // Loads return in order, so the first parents are computed while later rows still arrive.
    using P = Pack<T, VEC>;
    P rck[NC], rcv[SHARED ? 1 : NC], rq[NC - 1], rk[NC - 1], rv[NC - 1];
    {
        const S *kc = Kc + (size_t)b * kc_bs + (size_t)sub * NC * rs + hd;
        const S *vc = Vc + (size_t)b * vc_bs + (size_t)sub * NC * rs + hd;
        const size_t lrow = (size_t)(level_offset(N, lvl0 + 1) - N) + (size_t)sub * (NC / 2);
        const S *q = Qp + (size_t)b * qp_bs + lrow * rs + hd;
        const S *kp = Kp + (size_t)b * kp_bs + lrow * rs + hd;
        const S *vp = Vp + (size_t)b * vp_bs + lrow * rs + hd;
#pragma unroll
        for (int i = 0; i < NC / 2; ++i) {
            rq[i] = load_once<P>(q + (size_t)i * rs);
            rck[2 * i] = load_once<P>(kc + (size_t)(2 * i) * rs);
            rck[2 * i + 1] = load_once<P>(kc + (size_t)(2 * i + 1) * rs);
            rk[i] = load_once<P>(kp + (size_t)i * rs);
            if (!SHARED) {
                rcv[2 * i] = load_once<P>(vc + (size_t)(2 * i) * rs);
                rcv[2 * i + 1] = load_once<P>(vc + (size_t)(2 * i + 1) * rs);
            }
            rv[i] = load_once<P>(vp + (size_t)i * rs);
        }
    }
#pragma unroll
    for (int j = 2; j <= TL; ++j) {
        const int np = NC >> j;
        const int base = NC - 2 * np;  // slot of this level's first parent: NC/2, 3NC/4, ...
        const size_t lrow = (size_t)(level_offset(N, lvl0 + j) - N) + (size_t)sub * np;
        const S *q = Qp + (size_t)b * qp_bs + lrow * rs + hd;
        const S *kp = Kp + (size_t)b * kp_bs + lrow * rs + hd;
        const S *vp = Vp + (size_t)b * vp_bs + lrow * rs + hd;
#pragma unroll
        for (int i = 0; i < NC / 4; ++i) {
            if (i < np) {
                rq[base + i] = load_once<P>(q + (size_t)i * rs);
                rk[base + i] = load_once<P>(kp + (size_t)i * rs);
                rv[base + i] = load_once<P>(vp + (size_t)i * rs);
            }
        }
    }

    // keep every request ahead of the first use
    __builtin_amdgcn_sched_barrier(0);

    // previous level's outputs (as floats, already rounded to the element type); the first level
    // converts its children's pieces where it uses them, so that its first parents do not wait
    // for the last rows
    float lk[NC / 2][VEC];
#pragma unroll
    for (int j = 1; j <= TL; ++j) {
        const int np = NC >> j;
        const int base = NC - 2 * np;
        const size_t lrow = (size_t)(level_offset(N, lvl0 + j) - N) + (size_t)sub * np;
        S *o = Out + (size_t)b * out_bs + lrow * rs + hd;
        S *o2 = Out2 ? Out2 + (size_t)b * out2_bs + lrow * rs + hd : nullptr;
#pragma unroll
        for (int i = 0; i < NC / 2; ++i) {
            if (i < np) {
                float fq[VEC], fk[VEC], fv[VEC], k0[VEC], k1[VEC], v0[VEC], v1[VEC];
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    fq[e] = to_float<T>(rq[base + i].e[e]);
                    fk[e] = to_float<T>(rk[base + i].e[e]);
                    fv[e] = to_float<T>(rv[base + i].e[e]);
                    if (j == 1) {
                        k0[e] = to_float<T>(rck[2 * i].e[e]);
                        k1[e] = to_float<T>(rck[2 * i + 1].e[e]);
                        v0[e] = SHARED ? k0[e] : to_float<T>(rcv[SHARED ? 0 : 2 * i].e[e]);
                        v1[e] = SHARED ? k1[e] : to_float<T>(rcv[SHARED ? 0 : 2 * i + 1].e[e]);
                    } else {
                        k0[e] = v0[e] = lk[2 * i][e];
                        k1[e] = v1[e] = lk[2 * i + 1][e];
                    }
                }
                float s0 = 0.f, s1 = 0.f, s2 = 0.f;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    s0 = fmaf(fq[e], fk[e], s0);
                    s1 = fmaf(fq[e], k0[e], s1);
                    s2 = fmaf(fq[e], k1[e], s2);
                }
                if (!dok) { s0 = 0.f; s1 = 0.f; s2 = 0.f; }
                s0 = group_sum(s0, G);
                s1 = group_sum(s1, G);
                s2 = group_sum(s2, G);
                float w0, w1, w2;
                softmax3<T>(s0 * scale, s1 * scale, s2 * scale, w0, w1, w2);
                float r[VEC];
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    float x = w0 * fv[e] + w1 * v0[e] + w2 * v1[e];
                    r[e] = to_float<T>(from_float<T>(x));  // the stored value feeds the next level
                }
                if (active && dok) {
                    store_vec<T, VEC, STREAM>(o + (size_t)i * rs, r);
                    if (o2) store_vec<T, VEC, STREAM>(o2 + (size_t)i * rs, r);
                }
#pragma unroll
                for (int e = 0; e < VEC; ++e) lk[i][e] = r[e];
            }
        }
    }
}

template <typename T, int VEC>
static int build_subtree_launch(const void *qp, const void *kp, const void *vp, const void *kc,
                                const void *vc, void *out, void *out2, int B, int N, int H, int D, int lvl0,
                                int tl, int64_t qp_bs, int64_t kp_bs, int64_t vp_bs, int64_t kc_bs,
                                int64_t vc_bs, int64_t out_bs, int64_t out2_bs, hipStream_t st) {
    using S = typename T::storage;
    const int chunks = (D + VEC - 1) / VEC;
    int G = 1;
    while (G < chunks) G <<= 1;  // caller guarantees chunks <= 64
    const long units = (long)B * ((N >> lvl0) >> tl) * H;
    const long threads = units * G;
    const int block = tl >= 4 ? subtree_block<4>() : subtree_block<1>();
    const long blocks = (threads + block - 1) / block;
    if (threads + block > 0x7fffffffL) return HSA_ERR_UNSUPPORTED;  // 32-bit indexing in the kernel
    const float scale = 1.0f / sqrtf((float)D);
    const bool shared = (kc == vc && kc_bs == vc_bs);
    // node rows written by the whole tree build, both copies: past 1.5 times the memory-side cache
    // they are stored with the streaming hint
    const size_t node_bytes = (size_t)B * (N - 1) * H * D * sizeof(S) * (out2 ? 2 : 1);
    const bool stream = node_bytes >= ((size_t)384 << 20);
#define HSA_SUBTREE_(TLN, SH, STR)                                                                   \
    build_subtree_kernel<T, VEC, TLN, SH, STR><<<(unsigned)blocks, block, 0, st>>>(                 \
        (const S *)qp, (const S *)kp, (const S *)vp, (const S *)kc, (const S *)vc, (S *)out, (S *)out2, B, \
        N, H, D, G, lvl0, qp_bs, kp_bs, vp_bs, kc_bs, vc_bs, out_bs, out2_bs, scale)
#define HSA_SUBTREE(TLN, SH)                     \
    do {                                         \
        if (stream) HSA_SUBTREE_(TLN, SH, true); \
        else HSA_SUBTREE_(TLN, SH, false);       \
    } while (0)
    if (tl == 4 && shared) HSA_SUBTREE(4, true);
    else if (tl == 1 && shared) HSA_SUBTREE(1, true);
    else if (tl == 2 && shared) HSA_SUBTREE(2, true);
    else if (tl == 3 && shared) HSA_SUBTREE(3, true);
    else if (tl == 1) HSA_SUBTREE(1, false);
    else if (tl == 2) HSA_SUBTREE(2, false);
    else if (tl == 3) HSA_SUBTREE(3, false);
    else return fail(HSA_ERR_INVALID, "internal: bad subtree pass");
#undef HSA_SUBTREE_
#undef HSA_SUBTREE
    return check_launch("build_subtree_kernel");
}

// ---- the top of the tree in one launch ------------------------------------------------------
// One workgroup per (batch, head) finishes every remaining level once at most TOP_MAX_CHILDREN
// nodes are left per sequence.  A group of G lanes owns one parent per level; the q/k/v rows
// of all levels are requested at the start (they do not depend on the children), each level's
// outputs go to global memory and, rounded to the element type, to LDS for the next level.
constexpr int TOP_MAX_LEVELS = 8;
constexpr int TOP_THREADS = 1024;

// GT: lanes per parent row when known at compile time (the reductions then need no branches), 0 = use G
template <typename T, int VEC, int GT>
__global__ void __launch_bounds__(TOP_THREADS)
build_top_kernel(const typename T::storage *__restrict__ Qp, const typename T::storage *__restrict__ Kp,
                 const typename T::storage *__restrict__ Vp, typename T::storage *__restrict__ Out,
                 typename T::storage *__restrict__ Out2, int N, int H, int D, int G, int lvl0, int nlev,
                 int64_t qp_bs, int64_t kp_bs, int64_t vp_bs, int64_t out_bs, int64_t out2_bs, float scale) {
    if (GT) G = GT;
    using S = typename T::storage;
    using P = Pack<T, VEC>;
    extern __shared__ __align__(16) unsigned char top_lds[];
    const int lg = 31 - __builtin_clz(G);
    const int grp = threadIdx.x >> lg;  // parent slot
    const int gl = threadIdx.x & (G - 1);
    const int b = blockIdx.x / H, h = blockIdx.x % H;
    const int nc = N >> lvl0;  // children of the first level
    const size_t rs = (size_t)H * D;
    const size_t hd = (size_t)h * D + (size_t)gl * VEC;
    const size_t row_bytes = (size_t)D * sizeof(S);
    // ping-pong level buffers in LDS: [nc/2 rows] and [nc/4 rows]
    unsigned char *buf0 = top_lds, *buf1 = top_lds + (size_t)(nc / 2) * row_bytes;

    // parent rows are requested TOP_AHEAD levels before they are used (they do not depend on
    // the children), which bounds the registers to a few levels' worth
    constexpr int TOP_AHEAD = 3;
    P rq[TOP_MAX_LEVELS], rk[TOP_MAX_LEVELS], rv[TOP_MAX_LEVELS], c0, c1;
    // Loads are unconditional (idle groups re-read the level's last row, levels past the root
    // re-read the root's): a load under a lane-dependent branch would be waited for at the end
    // of its branch, one memory round trip per level.
    auto request = [&](int j) {  // j = 1-based level of this pass
        const int je = j <= nlev ? j : nlev;
        const int np = nc >> je;
        const size_t lrow = (size_t)(level_offset(N, lvl0 + je) - N) + (grp < np ? grp : np - 1);
        rq[j - 1] = *reinterpret_cast<const P *>(Qp + (size_t)b * qp_bs + lrow * rs + hd);
        rk[j - 1] = *reinterpret_cast<const P *>(Kp + (size_t)b * kp_bs + lrow * rs + hd);
        rv[j - 1] = *reinterpret_cast<const P *>(Vp + (size_t)b * vp_bs + lrow * rs + hd);
    };
    {
        const int np = nc >> 1;
        const S *ch = Out + (size_t)b * out_bs +
                      ((size_t)(level_offset(N, lvl0) - N) + 2 * (grp < np ? grp : np - 1)) * rs + hd;
        c0 = *reinterpret_cast<const P *>(ch);
        c1 = *reinterpret_cast<const P *>(ch + rs);
    }
#pragma unroll
    for (int j = 1; j <= TOP_AHEAD; ++j) request(j);
    __builtin_amdgcn_sched_barrier(0);

#pragma unroll
    for (int j = 1; j <= TOP_MAX_LEVELS; ++j) {
        if (j <= nlev) {
            const int np = nc >> j;
            unsigned char *src = (j & 1) ? buf1 : buf0;  // level j-1 outputs (j >= 2)
            unsigned char *dst = (j & 1) ? buf0 : buf1;
            if (j + TOP_AHEAD <= TOP_MAX_LEVELS) request(j + TOP_AHEAD);
            if (grp < np) {
                if (j >= 2) {
                    c0 = *reinterpret_cast<const P *>(src + (size_t)(2 * grp) * row_bytes + (size_t)gl * VEC * sizeof(S));
                    c1 = *reinterpret_cast<const P *>(src + (size_t)(2 * grp + 1) * row_bytes + (size_t)gl * VEC * sizeof(S));
                }
                float s0 = 0.f, s1 = 0.f, s2 = 0.f;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float q = to_float<T>(rq[j - 1].e[e]);
                    s0 = fmaf(q, to_float<T>(rk[j - 1].e[e]), s0);
                    s1 = fmaf(q, to_float<T>(c0.e[e]), s1);
                    s2 = fmaf(q, to_float<T>(c1.e[e]), s2);
                }
                s0 = group_sum(s0, GT ? GT : G);
                s1 = group_sum(s1, GT ? GT : G);
                s2 = group_sum(s2, GT ? GT : G);
                float w0, w1, w2;
                softmax3<T>(s0 * scale, s1 * scale, s2 * scale, w0, w1, w2);
                P r;
#pragma unroll
                for (int e = 0; e < VEC; ++e)
                    r.e[e] = from_float<T>(w0 * to_float<T>(rv[j - 1].e[e]) + w1 * to_float<T>(c0.e[e]) +
                                           w2 * to_float<T>(c1.e[e]));
                const size_t lrow = (size_t)(level_offset(N, lvl0 + j) - N) + grp;
                *reinterpret_cast<P *>(Out + (size_t)b * out_bs + lrow * rs + hd) = r;
                if (Out2) *reinterpret_cast<P *>(Out2 + (size_t)b * out2_bs + lrow * rs + hd) = r;
                if (j < nlev)
                    *reinterpret_cast<P *>(dst + (size_t)grp * row_bytes + (size_t)gl * VEC * sizeof(S)) = r;
            }
            if (j < nlev) {
                // LDS-only barrier: __syncthreads() would also drain the outstanding global loads
                // (requested levels ahead on purpose) and stores
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
            }
        }
    }
}

template <typename T, int VEC>
static int build_top_launch(const void *qp, const void *kp, const void *vp, void *out, void *out2, int B,
                            int N, int H, int D, int lvl0, int64_t qp_bs, int64_t kp_bs, int64_t vp_bs,
                            int64_t out_bs, int64_t out2_bs, hipStream_t st) {
    using S = typename T::storage;
    const int G = D / VEC;
    const int nc = N >> lvl0;
    const int nlev = ilog2_exact(N) - lvl0;
    const size_t lds = (size_t)(nc / 2 + nc / 4 + 1) * D * sizeof(S);
    const float scale = 1.0f / sqrtf((float)D);
    int threads = (nc / 2) * G;
    if (threads < 64) threads = 64;
#define HSA_TOP_LAUNCH(GT)                                                                              \
    build_top_kernel<T, VEC, GT><<<B * H, threads, lds, st>>>((const S *)qp, (const S *)kp, (const S *)vp, \
                                                              (S *)out, (S *)out2, N, H, D, G, lvl0, nlev, \
                                                              qp_bs, kp_bs, vp_bs, out_bs, out2_bs, scale)
    if (G == 8) HSA_TOP_LAUNCH(8);
    else if (G == 16) HSA_TOP_LAUNCH(16);
    else HSA_TOP_LAUNCH(0);
#undef HSA_TOP_LAUNCH
    return check_launch("build_top_kernel");
}

// Whole tree, up to three levels per launch.  Returns HSA_ERR_UNSUPPORTED when the shape
// does not fit the subtree kernel (the caller then goes level by level).
template <typename T>
static int build_tree_typed(const void *qp, const void *kp, const void *vp, const void *k_leaf,
                            const void *v_leaf, void *out, void *out2, int B, int N, int H, int D,
                            int64_t qp_bs, int64_t kp_bs, int64_t vp_bs, int64_t kleaf_bs, int64_t vleaf_bs,
                            int64_t out_bs, int64_t out2_bs, hipStream_t st) {
    constexpr int VEC16 = 16 / (int)sizeof(typename T::storage);
    const uintptr_t align = (uintptr_t)qp | (uintptr_t)kp | (uintptr_t)vp | (uintptr_t)k_leaf |
                            (uintptr_t)v_leaf | (uintptr_t)out | (uintptr_t)out2;
    const int64_t strides = qp_bs | kp_bs | vp_bs | kleaf_bs | vleaf_bs | out_bs | out2_bs;
    const bool vec_ok = D % VEC16 == 0 && (align & 15) == 0 && (strides % VEC16) == 0;
    const int vec = vec_ok ? VEC16 : 1;
    if ((D + vec - 1) / vec > 64) return HSA_ERR_UNSUPPORTED;
    const int L = ilog2_exact(N);
    const size_t row = (size_t)H * D * sizeof(typename T::storage);
    int lvl0 = 0;
    while (lvl0 < L) {
        // once few enough nodes are left, one launch finishes the tree
        if (lvl0 > 0 && vec_ok && D % VEC16 == 0 && ((D / VEC16) & (D / VEC16 - 1)) == 0 && D / VEC16 <= 64 &&
            L - lvl0 <= TOP_MAX_LEVELS && (long)((N >> lvl0) / 2) * (D / VEC16) <= TOP_THREADS &&
            (long)B * H <= 0x7fffffffL)
            return build_top_launch<T, VEC16>(qp, kp, vp, out, out2, B, N, H, D, lvl0, qp_bs, kp_bs, vp_bs, out_bs,
                                              out2_bs, st);
        // three levels from the leaves (keys and values are different rows), then four at a time
        const int cap = lvl0 == 0 ? 3 : 4;
        const int tl = L - lvl0 >= cap ? cap : L - lvl0;
        const void *kc = k_leaf, *vc = v_leaf;
        int64_t kc_bs = kleaf_bs, vc_bs = vleaf_bs;
        if (lvl0 > 0) {
            kc = vc = (const char *)out + (size_t)(level_offset(N, lvl0) - N) * row;
            kc_bs = vc_bs = out_bs;
        }
        int rc = vec_ok ? build_subtree_launch<T, VEC16>(qp, kp, vp, kc, vc, out, out2, B, N, H, D, lvl0, tl,
                                                         qp_bs, kp_bs, vp_bs, kc_bs, vc_bs, out_bs, out2_bs, st)
                        : build_subtree_launch<T, 1>(qp, kp, vp, kc, vc, out, out2, B, N, H, D, lvl0, tl, qp_bs,
                                                     kp_bs, vp_bs, kc_bs, vc_bs, out_bs, out2_bs, st);
        if (rc != HSA_OK) return rc;
        lvl0 += tl;
    }
    return HSA_OK;
}

int build_tree_dispatch(const void *qp, const void *kp, const void *vp, const void *k_leaf, const void *v_leaf,
                        void *out, void *out2, int B, int N, int H, int D, int64_t qp_bs, int64_t kp_bs,
                        int64_t vp_bs, int64_t kleaf_bs, int64_t vleaf_bs, int64_t out_bs, int64_t out2_bs,
                        int dtype, hipStream_t st) {
    switch (dtype) {
        case HSA_F32: return build_tree_typed<F32>(qp, kp, vp, k_leaf, v_leaf, out, out2, B, N, H, D, qp_bs, kp_bs, vp_bs, kleaf_bs, vleaf_bs, out_bs, out2_bs, st);
        case HSA_F16: return build_tree_typed<F16>(qp, kp, vp, k_leaf, v_leaf, out, out2, B, N, H, D, qp_bs, kp_bs, vp_bs, kleaf_bs, vleaf_bs, out_bs, out2_bs, st);
        case HSA_BF16: return build_tree_typed<BF16>(qp, kp, vp, k_leaf, v_leaf, out, out2, B, N, H, D, qp_bs, kp_bs, vp_bs, kleaf_bs, vleaf_bs, out_bs, out2_bs, st);
    }
    return fail(HSA_ERR_INVALID, "unknown dtype %d", dtype);
}

template <typename T>
static int build_parents_typed(const void *qp, const void *kp, const void *vp, const void *kc,
                               const void *vc, void *out, void *out2, void *weights, int B, int P, int H,
                               int D, const LevelStrides &sd, hipStream_t st) {
    constexpr int VEC = 16 / (int)sizeof(typename T::storage);
    const uintptr_t align = (uintptr_t)qp | (uintptr_t)kp | (uintptr_t)vp | (uintptr_t)kc | (uintptr_t)vc |
                            (uintptr_t)out | (uintptr_t)out2;
    int64_t strides = 0;
    for (int i = 0; i < 7; ++i) strides |= sd.bs[i] | sd.rs[i];
    if (D % VEC == 0 && (align & 15) == 0 && (strides % VEC) == 0)
        return build_parents_launch<T, VEC>(qp, kp, vp, kc, vc, out, out2, weights, B, P, H, D, sd, st);
    return build_parents_launch<T, 1>(qp, kp, vp, kc, vc, out, out2, weights, B, P, H, D, sd, st);
}

int build_parents_strided(const void *qp, const void *kp, const void *vp, const void *kc, const void *vc,
                          void *out, void *out2, void *weights, int B, int P, int H, int D,
                          const LevelStrides &in, int dtype, hipStream_t st) {
    // zero = dense: rows H*D apart, batches rows * row stride apart
    LevelStrides sd = in;
    for (int i = 0; i < 7; ++i) {
        const int64_t rows = (i == 3 || i == 4) ? 2 * (int64_t)P : (int64_t)P;
        if (!sd.rs[i]) sd.rs[i] = (int64_t)H * D;
        if (sd.rs[i] < (int64_t)H * D) return fail(HSA_ERR_INVALID, "row stride %lld below H*D", (long long)sd.rs[i]);
        if (!sd.bs[i]) sd.bs[i] = rows * sd.rs[i];
    }
    switch (dtype) {
        case HSA_F32: return build_parents_typed<F32>(qp, kp, vp, kc, vc, out, out2, weights, B, P, H, D, sd, st);
        case HSA_F16: return build_parents_typed<F16>(qp, kp, vp, kc, vc, out, out2, weights, B, P, H, D, sd, st);
        case HSA_BF16: return build_parents_typed<BF16>(qp, kp, vp, kc, vc, out, out2, weights, B, P, H, D, sd, st);
    }
    return fail(HSA_ERR_INVALID, "unknown dtype %d", dtype);
}

int build_parents_dispatch(const void *qp, const void *kp, const void *vp, const void *kc, const void *vc,
                           void *out, void *out2, void *weights, int B, int P, int H, int D, int64_t qp_bs,
                           int64_t kp_bs, int64_t vp_bs, int64_t kc_bs, int64_t vc_bs, int64_t out_bs,
                           int64_t out2_bs, int dtype, hipStream_t st) {
    LevelStrides sd = {{qp_bs, kp_bs, vp_bs, kc_bs, vc_bs, out_bs, out2_bs}, {0, 0, 0, 0, 0, 0, 0}};
    return build_parents_strided(qp, kp, vp, kc, vc, out, out2, weights, B, P, H, D, sd, dtype, st);
}

int build_tree_fused_dispatch(const void *qp, const void *kp, const void *vp, const void *k_leaf, const void *v_leaf,
                              void *out, void *out2, int B, int N, int H, int D, int64_t qp_bs, int64_t kp_bs,
                              int64_t vp_bs, int64_t kleaf_bs, int64_t vleaf_bs, int64_t out_bs, int64_t out2_bs,
                              int dtype, hipStream_t st);  // hsa_build_tree.hip
int build_tree_tune(int mode, int threads);

}  // namespace hsa

extern "C" {

int hsa_build_tree_tune(int mode, int workgroup_threads) {
    return hsa::build_tree_tune(mode, workgroup_threads);
}

int hsa_build_parents_fwd(const void *qp, const void *kp, const void *vp, const void *kc,
                          const void *vc, void *out, void *weights, int B, int P, int H, int D,
                          int64_t qp_bs, int64_t kp_bs, int64_t vp_bs, int64_t kc_bs, int64_t vc_bs,
                          int64_t out_bs, int dtype, void *stream) {
    HSA_REQUIRE(qp && kp && vp && kc && vc && out, "null pointer");
    HSA_REQUIRE(B >= 1 && P >= 1 && H >= 1 && D >= 1, "bad shape B=%d P=%d H=%d D=%d", B, P, H, D);
    return hsa::build_parents_dispatch(qp, kp, vp, kc, vc, out, nullptr, weights, B, P, H, D, qp_bs, kp_bs,
                                       vp_bs, kc_bs, vc_bs, out_bs, 0, dtype, (hipStream_t)stream);
}

int hsa_build_parents_strided_fwd(const void *qp, const void *kp, const void *vp, const void *kc,
                                  const void *vc, void *out, void *out2, int B, int P, int H, int D,
                                  const int64_t *batch_strides, const int64_t *row_strides, int dtype,
                                  void *stream) {
    HSA_REQUIRE(qp && kp && vp && kc && vc && out, "null pointer");
    HSA_REQUIRE(B >= 1 && P >= 1 && H >= 1 && D >= 1, "bad shape B=%d P=%d H=%d D=%d", B, P, H, D);
    hsa::LevelStrides sd = {};
    for (int i = 0; i < 7; ++i) {
        if (batch_strides) sd.bs[i] = batch_strides[i];
        if (row_strides) sd.rs[i] = row_strides[i];
        HSA_REQUIRE(sd.bs[i] >= 0 && sd.rs[i] >= 0, "negative stride");
    }
    return hsa::build_parents_strided(qp, kp, vp, kc, vc, out, out2, nullptr, B, P, H, D, sd, dtype,
                                      (hipStream_t)stream);
}

int hsa_build_tree_fwd(const void *qp, const void *kp, const void *vp, const void *k_leaf,
                       const void *v_leaf, void *out, void *out2, int B, int N, int H, int D, int64_t qp_bs,
                       int64_t kp_bs, int64_t vp_bs, int64_t kleaf_bs, int64_t vleaf_bs, int64_t out_bs,
                       int64_t out2_bs, int dtype, void *stream) {
    HSA_REQUIRE(qp && kp && vp && k_leaf && v_leaf && out, "null pointer");
    HSA_REQUIRE(B >= 1 && H >= 1 && D >= 1, "bad shape B=%d H=%d D=%d", B, H, D);
    HSA_REQUIRE(N >= 2 && hsa::ilog2_exact(N) >= 0, "N must be a power of two >= 2 (got %d)", N);
    const int64_t tree = (int64_t)(N - 1) * H * D, leaf = (int64_t)N * H * D;
    if (!qp_bs) qp_bs = tree;
    if (!kp_bs) kp_bs = tree;
    if (!vp_bs) vp_bs = tree;
    if (!out_bs) out_bs = tree;
    if (!out2_bs) out2_bs = tree;
    if (!kleaf_bs) kleaf_bs = leaf;
    if (!vleaf_bs) vleaf_bs = leaf;
    HSA_REQUIRE(dtype == HSA_F32 || dtype == HSA_F16 || dtype == HSA_BF16, "unknown dtype %d", dtype);
    {
        // one launch for the whole tree where the shape, the stream and the counter pool allow it
        int rc = hsa::build_tree_fused_dispatch(qp, kp, vp, k_leaf, v_leaf, out, out2, B, N, H, D, qp_bs, kp_bs,
                                                vp_bs, kleaf_bs, vleaf_bs, out_bs, out2_bs, dtype,
                                                (hipStream_t)stream);
        if (rc != HSA_ERR_UNSUPPORTED) return rc;
    }
    {
        int rc = hsa::build_tree_dispatch(qp, kp, vp, k_leaf, v_leaf, out, out2, B, N, H, D, qp_bs, kp_bs, vp_bs,
                                          kleaf_bs, vleaf_bs, out_bs, out2_bs, dtype, (hipStream_t)stream);
        if (rc != HSA_ERR_UNSUPPORTED) return rc;
    }
    const size_t es = hsa::elem_size(dtype);
    const size_t row = (size_t)H * D * es;
    // shapes the subtree kernel does not take: level by level; each level reads the previous
    // level's rows of `out`
    const char *kc = (const char *)k_leaf, *vc = (const char *)v_leaf;
    int64_t kc_bs = kleaf_bs, vc_bs = vleaf_bs;
    size_t off = 0;
    for (int P = N / 2; P >= 1; P /= 2) {
        int rc = hsa::build_parents_dispatch((const char *)qp + off * row, (const char *)kp + off * row,
                                             (const char *)vp + off * row, kc, vc, (char *)out + off * row,
                                             out2 ? (char *)out2 + off * row : nullptr, nullptr, B, P, H, D,
                                             qp_bs, kp_bs, vp_bs, kc_bs, vc_bs, out_bs, out2_bs, dtype,
                                             (hipStream_t)stream);
        if (rc != HSA_OK) return rc;
        kc = vc = (const char *)out + off * row;
        kc_bs = vc_bs = out_bs;
        off += P;
    }
    return HSA_OK;
}

}  // extern "C"
