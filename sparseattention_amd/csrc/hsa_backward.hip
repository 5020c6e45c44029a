// Backward passes of the two ops and of the initial span nodes.
//
//  parent build   one lane group per (batch, parent, head) recomputes the three weights from
//                 q and the keys (nothing but the inputs has to be saved by the forward) and
//                 writes every gradient row exactly once: children 2i, 2i+1 belong to parent i.
//  span attention two launches, no atomics, deterministic:
//                 (1) per (batch, query, head): recompute the slot weights P, form
//                     dP_t = <dO, V_t>, dS_t = P_t (dP_t - sum_u P_u dP_u) / sqrt(D), store P and
//                     dS (fp32, [B,N,H,2R+1+L], window slots first) and dQ = sum_t dS_t K_t;
//                 (2) per (batch, key row, head): gather the queries that attend the row --
//                     window neighbours and the level-0 sibling for a leaf, the 2^l leaves under
//                     the sibling subtree for a level-l node -- and accumulate
//                     dK = sum dS Q, dV = sum P dO in fp32, written once in the element type.
//                 Canonical complete-binary-tree tables only.
//  span nodes     dx[n] = sum_l 2^-l dY[level l, n >> l].
#include <mutex>

#include "hsa_attn_bwd_tile.h"

namespace hsa {

template <typename T, int D>
int attn_bwd_tile_launch_td(const BwdTileParams &p, int nbw, bool causal, int sb, hipStream_t st);

// ---------------------------------------------------------------- parent build
template <typename T, int VEC> struct BPack { typename T::storage e[VEC]; };

template <typename T, int VEC>
__device__ __forceinline__ void bload(const typename T::storage *p, float (&f)[VEC]) {
    if constexpr (VEC == 1) {
        f[0] = to_float<T>(p[0]);
    } else {
        BPack<T, VEC> v = *reinterpret_cast<const BPack<T, VEC> *>(p);
#pragma unroll
        for (int i = 0; i < VEC; ++i) f[i] = to_float<T>(v.e[i]);
    }
}
template <typename T, int VEC>
__device__ __forceinline__ void bstore(typename T::storage *p, const float (&f)[VEC]) {
    if constexpr (VEC == 1) {
        p[0] = from_float<T>(f[0]);
    } else {
        BPack<T, VEC> v;
#pragma unroll
        for (int i = 0; i < VEC; ++i) v.e[i] = from_float<T>(f[i]);
        *reinterpret_cast<BPack<T, VEC> *>(p) = v;
    }
}

// Batch and row strides (in elements) of the eleven operands, in the order
// dout, qp, kp, vp, kc, vc, dqp, dkp, dvp, dkc, dvc.
struct BwdStrides {
    int64_t bs[11];
    int64_t rs[11];
};

template <typename T, int VEC, int CH>
__global__ void __launch_bounds__(256)
build_parents_bwd_kernel(const typename T::storage *__restrict__ dO, const typename T::storage *__restrict__ Qp,
                         const typename T::storage *__restrict__ Kp, const typename T::storage *__restrict__ Vp,
                         const typename T::storage *__restrict__ Kc, const typename T::storage *__restrict__ Vc,
                         typename T::storage *__restrict__ dQ, typename T::storage *__restrict__ dKp,
                         typename T::storage *__restrict__ dVp, typename T::storage *__restrict__ dKc,
                         typename T::storage *__restrict__ dVc, int B, int P, int H, int D, int G, BwdStrides sd,
                         float scale) {
    const long tid = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long unit = tid / G;
    const int gl = (int)(tid % G);
    const long units = (long)B * P * H;
    const bool active = unit < units;
    const long u = active ? unit : units - 1;
    const int h = (int)(u % H);
    const int i = (int)((u / H) % P);
    const int b = (int)(u / ((long)H * P));
    // element offset of this (batch, row, head) in operand o; children: rows 2i and 2i+1
    auto at = [&](int o, int row) { return (size_t)b * sd.bs[o] + (size_t)row * sd.rs[o] + (size_t)h * D; };
    dO += at(0, i); Qp += at(1, i); Kp += at(2, i); Vp += at(3, i);
    dQ += at(6, i); dKp += at(7, i); dVp += at(8, i);
    const typename T::storage *Kc1 = Kc + at(4, 2 * i + 1), *Vc1 = Vc + at(5, 2 * i + 1);
    typename T::storage *dKc1 = dKc + at(9, 2 * i + 1), *dVc1 = dVc + at(10, 2 * i + 1);
    Kc += at(4, 2 * i); Vc += at(5, 2 * i); dKc += at(9, 2 * i); dVc += at(10, 2 * i);

    float q[CH][VEC], kp[CH][VEC], k0[CH][VEC], k1[CH][VEC], vp[CH][VEC], v0[CH][VEC], v1[CH][VEC], g[CH][VEC];
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, p0 = 0.f, p1 = 0.f, p2 = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int d = (c * G + gl) * VEC;
        if (d < D) {
            bload<T, VEC>(Qp + d, q[c]);
            bload<T, VEC>(Kp + d, kp[c]);
            bload<T, VEC>(Kc + d, k0[c]);
            bload<T, VEC>(Kc1 + d, k1[c]);
            bload<T, VEC>(Vp + d, vp[c]);
            bload<T, VEC>(Vc + d, v0[c]);
            bload<T, VEC>(Vc1 + d, v1[c]);
            bload<T, VEC>(dO + d, g[c]);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                s0 = fmaf(q[c][e], kp[c][e], s0);
                s1 = fmaf(q[c][e], k0[c][e], s1);
                s2 = fmaf(q[c][e], k1[c][e], s2);
                p0 = fmaf(g[c][e], vp[c][e], p0);
                p1 = fmaf(g[c][e], v0[c][e], p1);
                p2 = fmaf(g[c][e], v1[c][e], p2);
            }
        }
    }
    s0 = group_sum(s0, G); s1 = group_sum(s1, G); s2 = group_sum(s2, G);
    p0 = group_sum(p0, G); p1 = group_sum(p1, G); p2 = group_sum(p2, G);
    s0 *= scale; s1 *= scale; s2 *= scale;
    const float m = fmaxf(s0, fmaxf(s1, s2));
    const float e0 = expf(s0 - m), e1 = expf(s1 - m), e2 = expf(s2 - m);
    const float den = e0 + e1 + e2 + 1e-9f;
    const float w0 = e0 / den, w1 = e1 / den, w2 = e2 / den;
    const float dot = w0 * p0 + w1 * p1 + w2 * p2;
    const float ds0 = w0 * (p0 - dot) * scale, ds1 = w1 * (p1 - dot) * scale, ds2 = w2 * (p2 - dot) * scale;
    if (!active) return;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int d = (c * G + gl) * VEC;
        if (d < D) {
            float r[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) r[e] = ds0 * kp[c][e] + ds1 * k0[c][e] + ds2 * k1[c][e];
            bstore<T, VEC>(dQ + d, r);
#pragma unroll
            for (int e = 0; e < VEC; ++e) r[e] = ds0 * q[c][e];
            bstore<T, VEC>(dKp + d, r);
#pragma unroll
            for (int e = 0; e < VEC; ++e) r[e] = ds1 * q[c][e];
            bstore<T, VEC>(dKc + d, r);
#pragma unroll
            for (int e = 0; e < VEC; ++e) r[e] = ds2 * q[c][e];
            bstore<T, VEC>(dKc1 + d, r);
#pragma unroll
            for (int e = 0; e < VEC; ++e) r[e] = w0 * g[c][e];
            bstore<T, VEC>(dVp + d, r);
#pragma unroll
            for (int e = 0; e < VEC; ++e) r[e] = w1 * g[c][e];
            bstore<T, VEC>(dVc + d, r);
#pragma unroll
            for (int e = 0; e < VEC; ++e) r[e] = w2 * g[c][e];
            bstore<T, VEC>(dVc1 + d, r);
        }
    }
}

template <typename T>
static int build_parents_bwd_typed(const void *dout, const void *qp, const void *kp, const void *vp, const void *kc,
                                   const void *vc, void *dqp, void *dkp, void *dvp, void *dkc, void *dvc, int B,
                                   int P, int H, int D, const BwdStrides &sd, hipStream_t st) {
    using S = typename T::storage;
    constexpr int VEC16 = 16 / (int)sizeof(S);
    const uintptr_t al = (uintptr_t)dout | (uintptr_t)qp | (uintptr_t)kp | (uintptr_t)vp | (uintptr_t)kc |
                         (uintptr_t)vc | (uintptr_t)dqp | (uintptr_t)dkp | (uintptr_t)dvp | (uintptr_t)dkc |
                         (uintptr_t)dvc;
    int64_t strides = 0;
    for (int o = 0; o < 11; ++o) strides |= sd.bs[o] | sd.rs[o];
    const bool vec_ok = D % VEC16 == 0 && (al & 15) == 0 && (strides % VEC16) == 0;
    const int vec = vec_ok ? VEC16 : 1;
    const int chunks = (D + vec - 1) / vec;
    int G = 1;
    while (G < chunks && G < 64) G <<= 1;
    const int CH = (chunks + G - 1) / G;
    const long threads = (long)B * P * H * G;
    const long blocks = (threads + 255) / 256;
    if (blocks > 0x7fffffffL) return fail(HSA_ERR_UNSUPPORTED, "problem too large for one launch");
    const float scale = 1.0f / sqrtf((float)D);
#define HSA_BWD(VECN, CHN)                                                                                  \
    build_parents_bwd_kernel<T, VECN, CHN><<<(unsigned)blocks, 256, 0, st>>>(                               \
        (const S *)dout, (const S *)qp, (const S *)kp, (const S *)vp, (const S *)kc, (const S *)vc, (S *)dqp, \
        (S *)dkp, (S *)dvp, (S *)dkc, (S *)dvc, B, P, H, D, G, sd, scale)
    if (vec_ok) {
        if (CH == 1) HSA_BWD(VEC16, 1);
        else if (CH == 2) HSA_BWD(VEC16, 2);
        else return fail(HSA_ERR_UNSUPPORTED, "head_dim %d too large", D);
    } else {
        if (CH == 1) HSA_BWD(1, 1);
        else if (CH == 2) HSA_BWD(1, 2);
        else if (CH <= 4) HSA_BWD(1, 4);
        else if (CH <= 8) HSA_BWD(1, 8);
        else return fail(HSA_ERR_UNSUPPORTED, "head_dim %d too large", D);
    }
#undef HSA_BWD
    return check_launch("build_parents_bwd_kernel");
}

// ---------------------------------------------------------------- span attention, pass 1
constexpr int BWD_MAX_CHUNKS = 4;

__device__ __forceinline__ float bwd_wave_max(float v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ float bwd_wave_sum(float v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

template <typename T>
__global__ void __launch_bounds__(256)
attn_bwd_query_kernel(const typename T::storage *__restrict__ Q, const typename T::storage *__restrict__ K,
                      const typename T::storage *__restrict__ V, const typename T::storage *__restrict__ dO,
                      typename T::storage *__restrict__ dQ, float *__restrict__ Pw, float *__restrict__ DS, int B,
                      int N, int M, int H, int D, int L, int R, int causal, float scale,
                      const int32_t *__restrict__ idx = nullptr, const uint8_t *__restrict__ mask = nullptr) {
    const int lane = threadIdx.x & 63;
    const long unit = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (unit >= (long)B * N * H) return;
    const int h = (int)(unit % H);
    const int n = (int)((unit / H) % N);
    const int b = (int)(unit / ((long)H * N));
    const int Wn = 2 * R + 1, S = Wn + L;
    const size_t rs = (size_t)H * D;
    const typename T::storage *q = Q + (((size_t)b * N + n) * H + h) * D;
    const typename T::storage *go = dO + (((size_t)b * N + n) * H + h) * D;
    const typename T::storage *kb = K + (size_t)b * M * rs + (size_t)h * D;
    const typename T::storage *vb = V + (size_t)b * M * rs + (size_t)h * D;

    int row[BWD_MAX_CHUNKS];
    float sc[BWD_MAX_CHUNKS], dp[BWD_MAX_CHUNKS];
    float mx = -INFINITY;
#pragma unroll
    for (int c = 0; c < BWD_MAX_CHUNKS; ++c) {
        const int t = c * 64 + lane;
        int r = -1;
        if (t < Wn) {
            const int j = n + t - R;
            if (j >= 0 && j < N && (!causal || j <= n)) r = j;
        } else if (t < S) {
            const int l = t - Wn;
            if (idx) {
                // the caller's tables: an entry outside [0, M) or a set mask byte is a dead slot
                const int e = idx[(size_t)n * L + l];
                if (e >= 0 && e < M && !(mask && mask[(size_t)n * L + l])) r = e;
            } else if (!(causal && (((n >> l) & 1) == 0))) {
                r = level_offset(N, l) + ((n >> l) ^ 1);
            }
        }
        row[c] = r;
        float s = -INFINITY, g = 0.f;
        if (r >= 0) {
            const typename T::storage *kr = kb + (size_t)r * rs;
            const typename T::storage *vr = vb + (size_t)r * rs;
            float a = 0.f;
            for (int d = 0; d < D; ++d) {
                a = fmaf(to_float<T>(q[d]), to_float<T>(kr[d]), a);
                g = fmaf(to_float<T>(go[d]), to_float<T>(vr[d]), g);
            }
            s = a * scale;
        }
        sc[c] = s;
        dp[c] = g;
        mx = fmaxf(mx, s);
    }
    mx = bwd_wave_max(mx);
    float den = 0.f;
#pragma unroll
    for (int c = 0; c < BWD_MAX_CHUNKS; ++c) {
        sc[c] = row[c] >= 0 ? expf(sc[c] - mx) : 0.f;
        den += sc[c];
    }
    den = fmaxf(bwd_wave_sum(den), 1.0e-5f);
    float dot = 0.f;
#pragma unroll
    for (int c = 0; c < BWD_MAX_CHUNKS; ++c) {
        sc[c] /= den;
        dot += sc[c] * dp[c];
    }
    dot = bwd_wave_sum(dot);
    float *pw = Pw + (((size_t)b * N + n) * H + h) * S;
    float *ds = DS + (((size_t)b * N + n) * H + h) * S;
#pragma unroll
    for (int c = 0; c < BWD_MAX_CHUNKS; ++c) {
        dp[c] = sc[c] * (dp[c] - dot) * scale;  // dS
        const int t = c * 64 + lane;
        if (t < S) { pw[t] = sc[c]; ds[t] = dp[c]; }
    }
    typename T::storage *o = dQ + (((size_t)b * N + n) * H + h) * D;
    for (int d0 = 0; d0 < D; d0 += 64) {
        const int d = d0 + lane;
        float acc = 0.f;
#pragma unroll
        for (int c = 0; c < BWD_MAX_CHUNKS; ++c) {
            const int lim = S - c * 64 < 64 ? S - c * 64 : 64;
            for (int t = 0; t < lim; ++t) {
                const int r = __shfl(row[c], t, 64);
                const float w = __shfl(dp[c], t, 64);
                if (r >= 0 && d < D) acc = fmaf(w, to_float<T>(kb[(size_t)r * rs + d]), acc);
            }
        }
        if (d < D) o[d] = from_float<T>(acc);
    }
}

// ---------------------------------------------------------------- span attention, pass 2
// One wavefront per (batch, key row, head); lanes own channels.
template <typename T>
__global__ void __launch_bounds__(256)
attn_bwd_key_kernel(const typename T::storage *__restrict__ Q, const typename T::storage *__restrict__ dO,
                    const float *__restrict__ Pw, const float *__restrict__ DS,
                    typename T::storage *__restrict__ dK, typename T::storage *__restrict__ dV, int B, int N, int M,
                    int H, int D, int L, int R, int causal, const int32_t *__restrict__ gather = nullptr) {
    const int lane = threadIdx.x & 63;
    const long unit = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (unit >= (long)B * M * H) return;
    const int h = (int)(unit % H);
    const int row = (int)((unit / H) % M);
    const int b = (int)(unit / ((long)H * M));
    const int Wn = 2 * R + 1, S = Wn + L;
    const size_t rs = (size_t)H * D;
    const typename T::storage *qb = Q + (size_t)b * N * rs + (size_t)h * D;
    const typename T::storage *gb = dO + (size_t)b * N * rs + (size_t)h * D;
    const float *pw = Pw + (size_t)b * N * H * S + (size_t)h * S;
    const float *ds = DS + (size_t)b * N * H * S + (size_t)h * S;
    const size_t ws = (size_t)H * S;  // weights stride between queries
    typename T::storage *ok = dK + (((size_t)b * M + row) * H + h) * D;
    typename T::storage *ov = dV + (((size_t)b * M + row) * H + h) * D;

    for (int d0 = 0; d0 < D; d0 += 64) {
        const int d = d0 + lane;
        const bool dok = d < D;
        float ak = 0.f, av = 0.f;
        auto add = [&](int n, int slot) {
            const float w = pw[(size_t)n * ws + slot];
            const float s = ds[(size_t)n * ws + slot];
            if (dok) {
                ak = fmaf(s, to_float<T>(qb[(size_t)n * rs + d]), ak);
                av = fmaf(w, to_float<T>(gb[(size_t)n * rs + d]), av);
            }
        };
        if (row < N) {
            const int lo = causal ? row : (row - R < 0 ? 0 : row - R);
            const int hi = row + R >= N ? N - 1 : row + R;
            for (int n = lo; n <= hi; ++n) add(n, row - n + R);
            if (L > 0) {
                const int sib = row ^ 1;  // the query whose level-0 neighbour is this leaf
                if (sib < N && (!causal || (sib & 1))) add(sib, Wn);
            }
        } else if (row < 2 * N - 2) {  // tree node below the root
            int lvl = 1;
            while (row >= level_offset(N, lvl + 1)) ++lvl;
            const int pidx = row - level_offset(N, lvl);
            if (gather) {
                // the caller's table: first of the 2^lvl queries that attend this node through their
                // slot of level lvl, or -1 (what the reference's kernels read from it,
                // ops/triton/sparse_attn.py:389-470); masked queries carry zero weights
                const int first = gather[(size_t)row * 3];
                if (lvl < L && first >= 0 && first + (1 << lvl) <= N)
                    for (int n = first; n < first + (1 << lvl); ++n) add(n, Wn + lvl);
            } else if (!causal || (pidx & 1) == 0) {
                const int first = (pidx ^ 1) << lvl;
                for (int n = first; n < first + (1 << lvl); ++n) add(n, Wn + lvl);
            }
        }
        if (dok) {
            ok[d] = from_float<T>(ak);
            ov[d] = from_float<T>(av);
        }
    }
}

// ---- vector variants of the two passes (D a multiple of 16 bytes of elements) ----------------
// Same lane mapping as the vector forward gather kernel: D/VEC lanes share a row and read it as
// one contiguous piece.  Pass 1: a wavefront owns one query, 64*VEC/D slots per pass.  Pass 2: a
// wavefront owns 64*VEC/D consecutive key rows, each lane group walks the queries of its row.
constexpr int BWD_MAX_PASSES = 40;

template <typename T, int VEC, int LPS>
__global__ void __launch_bounds__(256)
attn_bwd_query_vec_kernel(const typename T::storage *__restrict__ Q, const typename T::storage *__restrict__ K,
                          const typename T::storage *__restrict__ V, const typename T::storage *__restrict__ dO,
                          typename T::storage *__restrict__ dQ, float *__restrict__ Pw, float *__restrict__ DS,
                          int B, int N, int M, int H, int L, int R, int causal, float scale) {
    constexpr int D = VEC * LPS;
    constexpr int SPW = 64 / LPS;
    struct alignas(16) Pk { typename T::storage e[VEC]; };
    const int lane = threadIdx.x & 63;
    const int sub = lane / LPS, gl = lane % LPS;
    const long unit = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (unit >= (long)B * N * H) return;
    const int h = (int)(unit % H);
    const int n = (int)((unit / H) % N);
    const int b = (int)(unit / ((long)H * N));
    const int Wn = 2 * R + 1, S = Wn + L;
    const int passes = (S + SPW - 1) / SPW;
    const size_t rs = (size_t)H * D;
    const typename T::storage *kb = K + (size_t)b * M * rs + (size_t)h * D + gl * VEC;
    const typename T::storage *vb = V + (size_t)b * M * rs + (size_t)h * D + gl * VEC;
    const size_t qoff = (((size_t)b * N + n) * H + h) * D + gl * VEC;
    float q[VEC], g[VEC];
    {
        Pk a = *reinterpret_cast<const Pk *>(Q + qoff), c = *reinterpret_cast<const Pk *>(dO + qoff);
#pragma unroll
        for (int e = 0; e < VEC; ++e) { q[e] = to_float<T>(a.e[e]) * scale; g[e] = to_float<T>(c.e[e]); }
    }
    auto slot_row = [&](int t) {
        int r = -1;
        if (t < Wn) {
            const int j = n + t - R;
            if (j >= 0 && j < N && (!causal || j <= n)) r = j;
        } else if (t < S) {
            const int l = t - Wn;
            if (!(causal && (((n >> l) & 1) == 0))) r = level_offset(N, l) + ((n >> l) ^ 1);
        }
        return r;
    };
    // eight passes at a time: key and value pieces requested together and unconditionally
    // (a dead slot re-reads the query's own leaf row)
    constexpr int CHUNK = 8;
    float sc[BWD_MAX_PASSES], dp[BWD_MAX_PASSES];
    float mx = -INFINITY;
#pragma unroll
    for (int c = 0; c < BWD_MAX_PASSES / CHUNK; ++c) {
#pragma unroll
        for (int p = 0; p < CHUNK; ++p) { sc[c * CHUNK + p] = -INFINITY; dp[c * CHUNK + p] = 0.f; }
        if (c * CHUNK < passes) {  // uniform
            int rr[CHUNK];
            Pk kk[CHUNK], vv[CHUNK];
#pragma unroll
            for (int p = 0; p < CHUNK; ++p) {
                rr[p] = slot_row((c * CHUNK + p) * SPW + sub);
                const size_t ro = (size_t)(rr[p] < 0 ? n : rr[p]) * rs;
                kk[p] = *reinterpret_cast<const Pk *>(kb + ro);
                vv[p] = *reinterpret_cast<const Pk *>(vb + ro);
            }
#pragma unroll
            for (int p = 0; p < CHUNK; ++p) {
                float a = 0.f, cc = 0.f;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    a = fmaf(q[e], to_float<T>(kk[p].e[e]), a);
                    cc = fmaf(g[e], to_float<T>(vv[p].e[e]), cc);
                }
                a = group_sum(a, LPS);
                cc = group_sum(cc, LPS);
                if (rr[p] >= 0) { sc[c * CHUNK + p] = a; dp[c * CHUNK + p] = cc; }
                mx = fmaxf(mx, sc[c * CHUNK + p]);
            }
        }
    }
    for (int o = LPS; o < 64; o <<= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    float den = 0.f;
#pragma unroll
    for (int p = 0; p < BWD_MAX_PASSES; ++p)
        if ((p / CHUNK) * CHUNK < passes) { sc[p] = sc[p] == -INFINITY ? 0.f : expf(sc[p] - mx); den += sc[p]; }
    for (int o = LPS; o < 64; o <<= 1) den += __shfl_xor(den, o, 64);
    den = fmaxf(den, 1.0e-5f);
    float dot = 0.f;
#pragma unroll
    for (int p = 0; p < BWD_MAX_PASSES; ++p)
        if ((p / CHUNK) * CHUNK < passes) { sc[p] /= den; dot += sc[p] * dp[p]; }
    for (int o = LPS; o < 64; o <<= 1) dot += __shfl_xor(dot, o, 64);
    float *pw = Pw + (((size_t)b * N + n) * H + h) * S;
    float *ds = DS + (((size_t)b * N + n) * H + h) * S;
    float acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
#pragma unroll
    for (int c = 0; c < BWD_MAX_PASSES / CHUNK; ++c) {
        if (c * CHUNK < passes) {  // uniform
            Pk kk[CHUNK];
#pragma unroll
            for (int p = 0; p < CHUNK; ++p) {
                const int r = slot_row((c * CHUNK + p) * SPW + sub);
                kk[p] = *reinterpret_cast<const Pk *>(kb + (size_t)(r < 0 ? n : r) * rs);
            }
#pragma unroll
            for (int p = 0; p < CHUNK; ++p) {
                const int t = (c * CHUNK + p) * SPW + sub;
                const float s = sc[c * CHUNK + p] * (dp[c * CHUNK + p] - dot) * scale;  // zero for dead slots
                if (gl == 0 && t < S) { pw[t] = sc[c * CHUNK + p]; ds[t] = s; }
#pragma unroll
                for (int e = 0; e < VEC; ++e) acc[e] = fmaf(s, to_float<T>(kk[p].e[e]), acc[e]);
            }
        }
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e)
        for (int o = LPS; o < 64; o <<= 1) acc[e] += __shfl_xor(acc[e], o, 64);
    if (sub == 0) {
        Pk o;
#pragma unroll
        for (int e = 0; e < VEC; ++e) o.e[e] = from_float<T>(acc[e]);
        *reinterpret_cast<Pk *>(dQ + qoff) = o;
    }
}

template <typename T, int VEC, int LPS>
__global__ void __launch_bounds__(256)
attn_bwd_key_vec_kernel(const typename T::storage *__restrict__ Q, const typename T::storage *__restrict__ dO,
                        const float *__restrict__ Pw, const float *__restrict__ DS,
                        typename T::storage *__restrict__ dK, typename T::storage *__restrict__ dV, int B, int N,
                        int M, int H, int L, int R, int causal) {
    constexpr int D = VEC * LPS;
    constexpr int SPW = 64 / LPS;
    struct alignas(16) Pk { typename T::storage e[VEC]; };
    const int lane = threadIdx.x & 63;
    const int sub = lane / LPS, gl = lane % LPS;
    // unit = (batch, row group, head): SPW consecutive rows of one head per wavefront
    const int groups = (M + SPW - 1) / SPW;
    const long unit = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (unit >= (long)B * groups * H) return;
    const int h = (int)(unit % H);
    const int grp = (int)((unit / H) % groups);
    const int b = (int)(unit / ((long)H * groups));
    const int row = grp * SPW + sub;
    if (row >= M) return;
    const int Wn = 2 * R + 1, S = Wn + L;
    const size_t rs = (size_t)H * D;
    const typename T::storage *qb = Q + (size_t)b * N * rs + (size_t)h * D + gl * VEC;
    const typename T::storage *gb = dO + (size_t)b * N * rs + (size_t)h * D + gl * VEC;
    const float *pw = Pw + (size_t)b * N * H * S + (size_t)h * S;
    const float *ds = DS + (size_t)b * N * H * S + (size_t)h * S;
    const size_t ws = (size_t)H * S;
    float ak[VEC], av[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) { ak[e] = 0.f; av[e] = 0.f; }
    auto add = [&](int n, int slot) {
        const float w = pw[(size_t)n * ws + slot];
        const float s = ds[(size_t)n * ws + slot];
        Pk qq = *reinterpret_cast<const Pk *>(qb + (size_t)n * rs);
        Pk gg = *reinterpret_cast<const Pk *>(gb + (size_t)n * rs);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            ak[e] = fmaf(s, to_float<T>(qq.e[e]), ak[e]);
            av[e] = fmaf(w, to_float<T>(gg.e[e]), av[e]);
        }
    };
    if (row < N) {
        const int lo = causal ? row : (row - R < 0 ? 0 : row - R);
        const int hi = row + R >= N ? N - 1 : row + R;
#pragma unroll 4
        for (int n = lo; n <= hi; ++n) add(n, row - n + R);
        if (L > 0) {
            const int sib = row ^ 1;
            if (!causal || (sib & 1)) add(sib, Wn);
        }
    } else if (row < 2 * N - 2) {
        int lvl = 1;
        while (row >= level_offset(N, lvl + 1)) ++lvl;
        const int pidx = row - level_offset(N, lvl);
        if (!causal || (pidx & 1) == 0) {
            const int first = (pidx ^ 1) << lvl;
#pragma unroll 4
            for (int n = first; n < first + (1 << lvl); ++n) add(n, Wn + lvl);
        }
    }
    Pk ok, ov;
#pragma unroll
    for (int e = 0; e < VEC; ++e) { ok.e[e] = from_float<T>(ak[e]); ov.e[e] = from_float<T>(av[e]); }
    const size_t off = (((size_t)b * M + row) * H + h) * D + gl * VEC;
    *reinterpret_cast<Pk *>(dK + off) = ok;
    *reinterpret_cast<Pk *>(dV + off) = ov;
}

template <typename T, int LPS>
static int attn_bwd_vec_launch(const void *q, const void *k, const void *v, const void *dout, void *dq, void *dk,
                               void *dv, float *ws_p, float *ws_ds, int B, int N, int M, int H, int L, int R,
                               int causal, hipStream_t st) {
    using S = typename T::storage;
    constexpr int VEC = 16 / (int)sizeof(S);
    constexpr int SPW = 64 / LPS;
    const float scale = 1.0f / sqrtf((float)(VEC * LPS));
    long units = (long)B * N * H;
    long blocks = (units + 3) / 4;
    if (blocks > 0x7fffffffL) return fail(HSA_ERR_UNSUPPORTED, "problem too large for one launch");
    attn_bwd_query_vec_kernel<T, VEC, LPS><<<(unsigned)blocks, 256, 0, st>>>(
        (const S *)q, (const S *)k, (const S *)v, (const S *)dout, (S *)dq, ws_p, ws_ds, B, N, M, H, L, R, causal,
        scale);
    int rc = check_launch("attn_bwd_query_vec_kernel");
    if (rc != HSA_OK) return rc;
    units = (long)B * ((M + SPW - 1) / SPW) * H;
    blocks = (units + 3) / 4;
    if (blocks > 0x7fffffffL) return fail(HSA_ERR_UNSUPPORTED, "problem too large for one launch");
    attn_bwd_key_vec_kernel<T, VEC, LPS><<<(unsigned)blocks, 256, 0, st>>>(
        (const S *)q, (const S *)dout, ws_p, ws_ds, (S *)dk, (S *)dv, B, N, M, H, L, R, causal);
    return check_launch("attn_bwd_key_vec_kernel");
}

template <typename T>
static int attn_bwd_vec_try(const void *q, const void *k, const void *v, const void *dout, void *dq, void *dk,
                            void *dv, float *ws_p, float *ws_ds, int B, int N, int M, int H, int D, int L, int R,
                            int causal, hipStream_t st) {
    constexpr int VEC = 16 / (int)sizeof(typename T::storage);
    if (D % VEC != 0) return HSA_ERR_UNSUPPORTED;
    const uintptr_t al = (uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)dout | (uintptr_t)dq |
                         (uintptr_t)dk | (uintptr_t)dv;
    if ((al & 15) != 0) return HSA_ERR_UNSUPPORTED;
    const int S = 2 * R + 1 + L;
#define HSA_BV(LPSN)                                                                                          \
    case LPSN:                                                                                                \
        if ((S + 64 / LPSN - 1) / (64 / LPSN) > BWD_MAX_PASSES) return HSA_ERR_UNSUPPORTED;                   \
        return attn_bwd_vec_launch<T, LPSN>(q, k, v, dout, dq, dk, dv, ws_p, ws_ds, B, N, M, H, L, R, causal, st)
    switch (D / VEC) {
        HSA_BV(2);
        HSA_BV(4);
        HSA_BV(8);
        HSA_BV(16);
        HSA_BV(32);
    }
#undef HSA_BV
    return HSA_ERR_UNSUPPORTED;
}

template <typename T>
static int attn_bwd_typed(const void *q, const void *k, const void *v, const void *dout, void *dq, void *dk,
                          void *dv, float *ws_p, float *ws_ds, int B, int N, int M, int H, int D, int L, int R,
                          int causal, hipStream_t st, const int32_t *idx = nullptr, const uint8_t *mask = nullptr,
                          const int32_t *gather = nullptr) {
    using S = typename T::storage;
    if (!idx) {
        int rc = attn_bwd_vec_try<T>(q, k, v, dout, dq, dk, dv, ws_p, ws_ds, B, N, M, H, D, L, R, causal, st);
        if (rc != HSA_ERR_UNSUPPORTED) return rc;
    }
    const float scale = 1.0f / sqrtf((float)D);
    long units = (long)B * N * H;
    long blocks = (units + 3) / 4;
    if (blocks > 0x7fffffffL) return fail(HSA_ERR_UNSUPPORTED, "problem too large for one launch");
    attn_bwd_query_kernel<T><<<(unsigned)blocks, 256, 0, st>>>((const S *)q, (const S *)k, (const S *)v,
                                                               (const S *)dout, (S *)dq, ws_p, ws_ds, B, N, M, H, D,
                                                               L, R, causal, scale, idx, mask);
    int rc = check_launch("attn_bwd_query_kernel");
    if (rc != HSA_OK) return rc;
    units = (long)B * M * H;
    blocks = (units + 3) / 4;
    if (blocks > 0x7fffffffL) return fail(HSA_ERR_UNSUPPORTED, "problem too large for one launch");
    attn_bwd_key_kernel<T><<<(unsigned)blocks, 256, 0, st>>>((const S *)q, (const S *)dout, ws_p, ws_ds, (S *)dk,
                                                             (S *)dv, B, N, M, H, D, L, R, causal, gather);
    return check_launch("attn_bwd_key_kernel");
}

// ---------------------------------------------------------------- initial span nodes
// One thread per (batch, leaf, VEC channels): VEC = 16 bytes of elements when the channel count and
// the pointers allow it, else 1.
template <typename T, int VEC>
__global__ void span_y_bwd_kernel(const typename T::storage *__restrict__ dY, typename T::storage *__restrict__ dX,
                                  int B, int N, int C, int L) {
    using S = typename T::storage;
    struct alignas(sizeof(S) * VEC) Pk { S e[VEC]; };
    const int CV = C / VEC;
    const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t total = (size_t)B * N * CV;
    if (t >= total) return;
    const int c = (int)(t % CV) * VEC;
    const int n = (int)((t / CV) % N);
    const int b = (int)(t / ((size_t)CV * N));
    // level l holds N >> l rows; a leaf under an unpaired row contributes to no level above it
    int start = 0;
    for (int l = 1; l <= L; ++l) start += N >> l;
    const S *dy = dY + (size_t)b * start * C + c;
    float acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
    float w = 1.f;
    start = 0;
    for (int l = 1; l <= L; ++l) {
        w *= 0.5f;
        const int rows = N >> l;
        if ((n >> l) >= rows) break;
        const Pk v = *reinterpret_cast<const Pk *>(dy + (size_t)(start + (n >> l)) * C);
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] = fmaf(w, to_float<T>(v.e[e]), acc[e]);
        start += rows;
    }
    Pk o;
#pragma unroll
    for (int e = 0; e < VEC; ++e) o.e[e] = from_float<T>(acc[e]);
    *reinterpret_cast<Pk *>(dX + ((size_t)b * N + n) * C + c) = o;
}

template <typename T>
static int span_y_bwd_launch(const void *dy, void *dx, int B, int N, int C, int L, hipStream_t st) {
    using S = typename T::storage;
    constexpr int VEC16 = 16 / (int)sizeof(S);
    const bool vec = C % VEC16 == 0 && ((((uintptr_t)dy | (uintptr_t)dx)) & 15) == 0;
    const size_t total = (size_t)B * N * (vec ? C / VEC16 : C);
    const size_t blocks = (total + 255) / 256;
    if (blocks > 0x7fffffffUL) return fail(HSA_ERR_UNSUPPORTED, "problem too large for one launch");
    if (vec) span_y_bwd_kernel<T, VEC16><<<(unsigned)blocks, 256, 0, st>>>((const S *)dy, (S *)dx, B, N, C, L);
    else span_y_bwd_kernel<T, 1><<<(unsigned)blocks, 256, 0, st>>>((const S *)dy, (S *)dx, B, N, C, L);
    return check_launch("span_y_bwd_kernel");
}

// ---------------------------------------------------------------- tile backward dispatch
bool attn_bwd_tile_f32_eligible(int N, int M, int D, int L, int R);  // hsa_attn_bwd_tile_f32.hip
int attn_bwd_tile_f32_dispatch(const void *q, const void *k, const void *v, const void *dout, void *dq, void *dk,
                               void *dv, float *ws, int B, int N, int M, int H, int D, int L, int R, int causal,
                               hipStream_t st);

// 16-bit types take R <= 64 (the workspace does not depend on the causal flag).
static bool attn_bwd_tile_eligible(int N, int M, int D, int L, int R, int dtype, int causal) {
    (void)causal;
    if (dtype == HSA_F32) return attn_bwd_tile_f32_eligible(N, M, D, L, R);
    if (dtype != HSA_F16 && dtype != HSA_BF16) return false;
    if (D != 32 && D != 64 && D != 128) return false;
    if (N < TILE_Q || ilog2_exact(N) != L || L > TILE_MAX_LEVELS || M < 2 * N - 1) return false;
    const int nbw = (R + TILE_Q - 1) / TILE_Q;
    return nbw <= 4;
}

static size_t bwd_gather_ws_floats(int B, int N, int H, int L, int R) {
    return 2 * (size_t)B * N * H * (2 * R + 1 + L);
}
// statistics [B,N,H,2] + partial rows of dK and dV: levels 4 and 5 per query block, levels >= 6 per
// strip (sized for strips of one block)
static size_t bwd_tile_ws_floats(int B, int N, int H, int D, int L) {
    const size_t lv = 2 + (L > 6 ? L - 6 : 0);
    return (size_t)B * N * H * 2 + 2 * (size_t)B * (N / TILE_Q) * H * lv * D;
}

template <typename T>
static int attn_bwd_tile_typed(const void *q, const void *k, const void *v, const void *dout, void *dq, void *dk,
                               void *dv, float *ws, int B, int N, int M, int H, int D, int L, int R, int causal,
                               hipStream_t st) {
    BwdTileParams p;
    p.q = (const uint16_t *)q; p.k = (const uint16_t *)k; p.v = (const uint16_t *)v; p.dout = (const uint16_t *)dout;
    p.dq = (uint16_t *)dq; p.dk = (uint16_t *)dk; p.dv = (uint16_t *)dv;
    p.stats = ws;
    p.partial = ws + (size_t)B * N * H * 2;
    p.B = B; p.N = N; p.M = M; p.H = H; p.L = L; p.R = R;
    const long units = (long)B * (N / TILE_Q) * H;
    if (units > 0x3fffffffL) return fail(HSA_ERR_UNSUPPORTED, "problem too large for one launch");
    p.n_units = (int)units;
    p.scale = 1.0f / sqrtf((float)D);
    p.scale_log2e = 1.4426950408889634f * p.scale;
    const int nbw = (R + TILE_Q - 1) / TILE_Q;
    const int NB = N / TILE_Q;
    // seven or nine leaf blocks per query block at 128 channels: one block per wavefront
    const bool wide128 = nbw > 2 && !causal && D > 64;
    const int sb = (NB % BWD_STRIP == 0 && !wide128) ? BWD_STRIP : 1;
    // The query pass finishes levels 1..4 (1..5 when it walks strips); the rows above them, the
    // root row and the rows past 2N-1 are summed from its partial rows by the trailing workgroups
    // of the key pass, one thread per four channels.
    int first = level_offset(N, sb == BWD_STRIP ? 6 : 5);
    if (first > 2 * N - 2) first = 2 * N - 2;
    const size_t red_threads = (size_t)B * (M - first) * H * (D / 4);
    const size_t red_wgs = (red_threads + BWD_WPB * 64 - 1) / (BWD_WPB * 64);
    if (red_wgs > 0x3fffffffUL) return fail(HSA_ERR_UNSUPPORTED, "problem too large for one launch");
    p.causal = causal != 0;
    p.red_first_row = first;
    p.red_wgs = (int)red_wgs;
    return D == 32 ? attn_bwd_tile_launch_td<T, 32>(p, nbw, causal != 0, sb, st)
         : D == 64 ? attn_bwd_tile_launch_td<T, 64>(p, nbw, causal != 0, sb, st)
                   : attn_bwd_tile_launch_td<T, 128>(p, nbw, causal != 0, sb, st);
}

// ---- one-pass backward on saved forward state (hsa_attn_bwd_fused.h) ---------------------------
int &bwd_fused_strip_knob() {
    static int v = 0;
    return v;
}
template <typename T, int D>
int attn_bwd_fused_launch_td(const BwdFusedParams &fp, bool causal, hipStream_t st);

static bool attn_bwd_fused_eligible(int N, int M, int D, int L, int R, int dtype, int causal) {
    if (dtype != HSA_F16 && dtype != HSA_BF16) return false;
    if (D != 32 && D != 64 && D != 128) return false;
    if (N < TILE_Q * BWD_STRIP || ilog2_exact(N) != L || L > TILE_MAX_LEVELS || M < 2 * N - 1) return false;
    // 128 channels (two wavefronts per head) only with the causal mask: without it the exchange
    // buffers leave room for one workgroup per CU
    if (D == 128 && causal == 0) return false;
    // one block of neighbours to either side, or two with the causal mask
    return R <= TILE_Q || (R <= 2 * TILE_Q && causal != 0);
}
// partial rows of dK and dV for levels >= 6, laid out like the two-pass workspace without its
// statistics
static size_t bwd_fused_ws_floats(int B, int N, int H, int D, int L) {
    const size_t lv = 2 + (L > 6 ? L - 6 : 0);
    return 2 * (size_t)B * (N / TILE_Q) * H * lv * D;
}

template <typename T>
static int attn_bwd_fused_typed(const void *q, const void *k, const void *v, const void *out, const float *lse,
                                const void *dout, void *dq, void *dk, void *dv, float *ws, int B, int N, int M,
                                int H, int D, int L, int R, int causal, hipStream_t st) {
    BwdFusedParams fp;
    BwdTileParams &p = fp.t;
    p.q = (const uint16_t *)q; p.k = (const uint16_t *)k; p.v = (const uint16_t *)v; p.dout = (const uint16_t *)dout;
    p.dq = (uint16_t *)dq; p.dk = (uint16_t *)dk; p.dv = (uint16_t *)dv;
    p.stats = nullptr;
    p.partial = ws;
    fp.out = (const uint16_t *)out;
    fp.lse = lse;
    p.B = B; p.N = N; p.M = M; p.H = H; p.L = L; p.R = R;
    const long units = (long)B * (N / TILE_Q) * H;
    if (units > 0x3fffffffL) return fail(HSA_ERR_UNSUPPORTED, "problem too large for one launch");
    p.n_units = (int)units;
    p.scale = 1.0f / sqrtf((float)D);
    p.scale_log2e = 1.4426950408889634f * p.scale;
    // the strips finish levels 1..6 (..7 with strips of eight blocks); the rows above them, the root
    // row and the rows past 2N-1 are summed from the strips' partial rows by a second, small
    // launch, whose first row the launcher sets once it knows the strip length
    int first = level_offset(N, 6);
    if (first > 2 * N - 2) first = 2 * N - 2;
    const size_t red_threads = (size_t)B * (M - first) * H * (D / 4) * BWD_FUSED_RED_SPLIT;
    const size_t red_wgs = (red_threads + BWD_WPB * 64 - 1) / (BWD_WPB * 64);
    if (red_wgs > 0x3fffffffUL) return fail(HSA_ERR_UNSUPPORTED, "problem too large for one launch");
    p.causal = causal != 0;
    p.red_first_row = first;
    p.red_wgs = (int)red_wgs;
    p.red_lg_sb = 2;
    return D == 32 ? attn_bwd_fused_launch_td<T, 32>(fp, causal != 0, st)
         : D == 64 ? attn_bwd_fused_launch_td<T, 64>(fp, causal != 0, st)
                   : attn_bwd_fused_launch_td<T, 128>(fp, causal != 0, st);
}

}  // namespace hsa

extern "C" {

static int build_parents_bwd_any(const void *dout, const void *qp, const void *kp, const void *vp, const void *kc,
                                 const void *vc, void *dqp, void *dkp, void *dvp, void *dkc, void *dvc, int B, int P,
                                 int H, int D, const int64_t *batch_strides, const int64_t *row_strides, int dtype,
                                 void *stream) {
    HSA_REQUIRE(dout && qp && kp && vp && kc && vc && dqp && dkp && dvp && dkc && dvc, "null pointer");
    HSA_REQUIRE(B >= 1 && P >= 1 && H >= 1 && D >= 1, "bad shape B=%d P=%d H=%d D=%d", B, P, H, D);
    hsa::BwdStrides sd;
    for (int o = 0; o < 11; ++o) {
        const bool child = o == 4 || o == 5 || o == 9 || o == 10;
        sd.rs[o] = row_strides && row_strides[o] ? row_strides[o] : (int64_t)H * D;
        HSA_REQUIRE(sd.rs[o] >= (int64_t)H * D, "row stride %lld below H*D", (long long)sd.rs[o]);
        sd.bs[o] = batch_strides && batch_strides[o] ? batch_strides[o] : (child ? 2 : 1) * (int64_t)P * sd.rs[o];
        HSA_REQUIRE(sd.bs[o] >= 0, "negative stride");
    }
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case HSA_F32: return hsa::build_parents_bwd_typed<hsa::F32>(dout, qp, kp, vp, kc, vc, dqp, dkp, dvp, dkc, dvc, B, P, H, D, sd, st);
        case HSA_F16: return hsa::build_parents_bwd_typed<hsa::F16>(dout, qp, kp, vp, kc, vc, dqp, dkp, dvp, dkc, dvc, B, P, H, D, sd, st);
        case HSA_BF16: return hsa::build_parents_bwd_typed<hsa::BF16>(dout, qp, kp, vp, kc, vc, dqp, dkp, dvp, dkc, dvc, B, P, H, D, sd, st);
    }
    return hsa::fail(HSA_ERR_INVALID, "unknown dtype %d", dtype);
}

int hsa_build_parents_bwd(const void *dout, const void *qp, const void *kp, const void *vp, const void *kc,
                          const void *vc, void *dqp, void *dkp, void *dvp, void *dkc, void *dvc, int B, int P,
                          int H, int D, int dtype, void *stream) {
    return build_parents_bwd_any(dout, qp, kp, vp, kc, vc, dqp, dkp, dvp, dkc, dvc, B, P, H, D, nullptr, nullptr,
                                 dtype, stream);
}

int hsa_build_parents_strided_bwd(const void *dout, const void *qp, const void *kp, const void *vp, const void *kc,
                                  const void *vc, void *dqp, void *dkp, void *dvp, void *dkc, void *dvc, int B,
                                  int P, int H, int D, const int64_t *batch_strides, const int64_t *row_strides,
                                  int dtype, void *stream) {
    return build_parents_bwd_any(dout, qp, kp, vp, kc, vc, dqp, dkp, dvp, dkc, dvc, B, P, H, D, batch_strides,
                                 row_strides, dtype, stream);
}

size_t hsa_attn_bwd_workspace_bytes(int B, int N, int M, int H, int D, int L, int R, int dtype, int algo) {
    const bool tile = algo != HSA_ATTN_GATHER && hsa::attn_bwd_tile_eligible(N, M, D, L, R, dtype, -1);
    const size_t tile_fl = hsa::bwd_tile_ws_floats(B, N, H, D, L), gather_fl = hsa::bwd_gather_ws_floats(B, N, H, L, R);
    const size_t fl = tile ? tile_fl : gather_fl;
    return fl * sizeof(float);
}

int hsa_attn_bwd(const void *q, const void *k, const void *v, const void *dout, void *dq, void *dk, void *dv,
                 void *workspace, size_t workspace_bytes, int B, int N, int M, int H, int D, int L, int R,
                 int causal, int dtype, int algo, void *stream) {
    HSA_REQUIRE(q && k && v && dout && dq && dk && dv && workspace, "null pointer");
    HSA_REQUIRE(B >= 1 && N >= 1 && H >= 1 && D >= 1, "bad shape B=%d N=%d H=%d D=%d", B, N, H, D);
    HSA_REQUIRE(hsa::ilog2_exact(N) == L, "canonical table needs L == log2 N (N=%d L=%d)", N, L);
    HSA_REQUIRE(M >= 2 * N - 1, "canonical table needs M >= 2N-1 (N=%d M=%d)", N, M);
    HSA_REQUIRE(R >= 0, "bad R=%d", R);
    HSA_REQUIRE(dtype == HSA_F32 || dtype == HSA_F16 || dtype == HSA_BF16, "unknown dtype %d", dtype);
    HSA_REQUIRE(workspace_bytes >= hsa_attn_bwd_workspace_bytes(B, N, M, H, D, L, R, dtype, algo),
                "workspace too small (%zu bytes)", workspace_bytes);
    hipStream_t st = (hipStream_t)stream;
    float *ws = (float *)workspace;
    bool tile_ok = hsa::attn_bwd_tile_eligible(N, M, D, L, R, dtype, causal ? 1 : 0);
    if (algo == HSA_ATTN_TILE && !tile_ok)
        return hsa::fail(HSA_ERR_UNSUPPORTED, "tile backward not available for N=%d D=%d L=%d R=%d causal=%d dtype=%d", N, D, L, R, causal ? 1 : 0, dtype);
    // the tile kernels move 16-byte pieces: tensors that are not aligned to that run on the gather
    // kernels (whose scalar variant takes any address), given a workspace of their size
    const bool aligned = (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)dout | (uintptr_t)dq |
                           (uintptr_t)dk | (uintptr_t)dv | (uintptr_t)workspace) & 15) == 0;
    if (tile_ok && algo != HSA_ATTN_GATHER && !aligned) {
        if (algo == HSA_ATTN_TILE) return hsa::fail(HSA_ERR_INVALID, "tile backward needs 16-byte aligned tensors");
        const size_t need = hsa::bwd_gather_ws_floats(B, N, H, L, R) * sizeof(float);
        if (workspace_bytes < need)
            return hsa::fail(HSA_ERR_INVALID, "tensors are not 16-byte aligned: they run on the gather kernels, which "
                             "need a workspace of %zu bytes (hsa_attn_bwd_workspace_bytes with HSA_ATTN_GATHER)", need);
        tile_ok = false;
    }
    if (tile_ok && algo != HSA_ATTN_GATHER) {
        if (dtype == HSA_F32)
            return hsa::attn_bwd_tile_f32_dispatch(q, k, v, dout, dq, dk, dv, ws, B, N, M, H, D, L, R, causal, st);
        if (dtype == HSA_BF16)
            return hsa::attn_bwd_tile_typed<hsa::BF16>(q, k, v, dout, dq, dk, dv, ws, B, N, M, H, D, L, R, causal, st);
        return hsa::attn_bwd_tile_typed<hsa::F16>(q, k, v, dout, dq, dk, dv, ws, B, N, M, H, D, L, R, causal, st);
    }
    if (2 * R + 1 + L > 64 * hsa::BWD_MAX_CHUNKS)
        return hsa::fail(HSA_ERR_UNSUPPORTED, "2R+1+L = %d slots exceeds %d", 2 * R + 1 + L, 64 * hsa::BWD_MAX_CHUNKS);
    float *ws_p = ws, *ws_ds = ws + (size_t)B * N * H * (2 * R + 1 + L);
    switch (dtype) {
        case HSA_F32: return hsa::attn_bwd_typed<hsa::F32>(q, k, v, dout, dq, dk, dv, ws_p, ws_ds, B, N, M, H, D, L, R, causal ? 1 : 0, st);
        case HSA_F16: return hsa::attn_bwd_typed<hsa::F16>(q, k, v, dout, dq, dk, dv, ws_p, ws_ds, B, N, M, H, D, L, R, causal ? 1 : 0, st);
        case HSA_BF16: return hsa::attn_bwd_typed<hsa::BF16>(q, k, v, dout, dq, dk, dv, ws_p, ws_ds, B, N, M, H, D, L, R, causal ? 1 : 0, st);
    }
    return hsa::fail(HSA_ERR_INVALID, "unknown dtype %d", dtype);
}

int hsa_attn_bwd_tables(const void *q, const void *k, const void *v, const void *dout, const int32_t *idx,
                        const uint8_t *mask, const int32_t *gather, void *dq, void *dk, void *dv, void *workspace,
                        size_t workspace_bytes, int B, int N, int M, int H, int D, int L, int R, int causal, int dtype,
                        void *stream) {
    HSA_REQUIRE(q && k && v && dout && idx && gather && dq && dk && dv && workspace, "null pointer");
    HSA_REQUIRE(B >= 1 && N >= 1 && H >= 1 && D >= 1 && L >= 0, "bad shape B=%d N=%d H=%d D=%d L=%d", B, N, H, D, L);
    HSA_REQUIRE(M >= N, "key rows M=%d below the leaf count N=%d", M, N);
    HSA_REQUIRE(R >= 0, "bad R=%d", R);
    HSA_REQUIRE(dtype == HSA_F32 || dtype == HSA_F16 || dtype == HSA_BF16, "unknown dtype %d", dtype);
    const size_t need = hsa::bwd_gather_ws_floats(B, N, H, L, R) * sizeof(float);
    HSA_REQUIRE(workspace_bytes >= need, "workspace too small (%zu bytes, %zu needed)", workspace_bytes, need);
    if (2 * R + 1 + L > 64 * hsa::BWD_MAX_CHUNKS)
        return hsa::fail(HSA_ERR_UNSUPPORTED, "2R+1+L = %d slots exceeds %d", 2 * R + 1 + L, 64 * hsa::BWD_MAX_CHUNKS);
    hipStream_t st = (hipStream_t)stream;
    float *ws_p = (float *)workspace, *ws_ds = ws_p + (size_t)B * N * H * (2 * R + 1 + L);
    const int c = causal ? 1 : 0;
    switch (dtype) {
        case HSA_F32: return hsa::attn_bwd_typed<hsa::F32>(q, k, v, dout, dq, dk, dv, ws_p, ws_ds, B, N, M, H, D, L, R, c, st, idx, mask, gather);
        case HSA_F16: return hsa::attn_bwd_typed<hsa::F16>(q, k, v, dout, dq, dk, dv, ws_p, ws_ds, B, N, M, H, D, L, R, c, st, idx, mask, gather);
        default: return hsa::attn_bwd_typed<hsa::BF16>(q, k, v, dout, dq, dk, dv, ws_p, ws_ds, B, N, M, H, D, L, R, c, st, idx, mask, gather);
    }
}

int hsa_attn_bwd_saved_tune(int strip_blocks) {
    if (strip_blocks != 0 && strip_blocks != 4 && strip_blocks != 8 && strip_blocks != 16 && strip_blocks != 32)
        return hsa::fail(HSA_ERR_INVALID, "strip length %d (0, 4, 8, 16 or 32)", strip_blocks);
    hsa::bwd_fused_strip_knob() = strip_blocks;
    return HSA_OK;
}

size_t hsa_attn_bwd_saved_workspace_bytes(int B, int N, int M, int H, int D, int L, int R, int causal, int dtype) {
    if (!hsa::attn_bwd_fused_eligible(N, M, D, L, R, dtype, causal)) return 0;
    return hsa::bwd_fused_ws_floats(B, N, H, D, L) * sizeof(float);
}

int hsa_attn_bwd_saved(const void *q, const void *k, const void *v, const void *out, const float *lse,
                       const void *dout, void *dq, void *dk, void *dv, void *workspace, size_t workspace_bytes, int B,
                       int N, int M, int H, int D, int L, int R, int causal, int dtype, void *stream) {
    HSA_REQUIRE(q && k && v && out && lse && dout && dq && dk && dv && workspace, "null pointer");
    HSA_REQUIRE(B >= 1 && N >= 1 && H >= 1 && D >= 1, "bad shape B=%d N=%d H=%d D=%d", B, N, H, D);
    HSA_REQUIRE(hsa::ilog2_exact(N) == L, "canonical table needs L == log2 N (N=%d L=%d)", N, L);
    HSA_REQUIRE(M >= 2 * N - 1, "canonical table needs M >= 2N-1 (N=%d M=%d)", N, M);
    HSA_REQUIRE(R >= 0, "bad R=%d", R);
    if (!hsa::attn_bwd_fused_eligible(N, M, D, L, R, dtype, causal))
        return hsa::fail(HSA_ERR_UNSUPPORTED, "one-pass backward not available for N=%d D=%d L=%d R=%d causal=%d dtype=%d "
                         "(16-bit types, 32, 64 or 128 channels per head, radius up to 16, or up to 32 with the causal mask, "
                         "at least 64 leaves)", N, D, L, R, causal ? 1 : 0, dtype);
    const bool aligned = (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out | (uintptr_t)dout |
                           (uintptr_t)dq | (uintptr_t)dk | (uintptr_t)dv | (uintptr_t)workspace) & 15) == 0;
    if (!aligned) return hsa::fail(HSA_ERR_UNSUPPORTED, "one-pass backward needs 16-byte aligned tensors");
    HSA_REQUIRE(workspace_bytes >= hsa_attn_bwd_saved_workspace_bytes(B, N, M, H, D, L, R, causal, dtype),
                "workspace too small (%zu bytes)", workspace_bytes);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == HSA_BF16)
        return hsa::attn_bwd_fused_typed<hsa::BF16>(q, k, v, out, lse, dout, dq, dk, dv, (float *)workspace, B, N, M, H,
                                                    D, L, R, causal, st);
    return hsa::attn_bwd_fused_typed<hsa::F16>(q, k, v, out, lse, dout, dq, dk, dv, (float *)workspace, B, N, M, H, D,
                                               L, R, causal, st);
}

// ---- hsa_attn_bwd for callers that must not allocate ---------------------------------------------
// The workspace of hsa_attn_bwd lives in this file-scope device array instead of caller memory.
// Every device the library's code object is loaded on holds its own copy at its own address;
// host code never uses the array's name as an address, only what hipGetSymbolAddress returned
// for the device that is current.
static __device__ __align__(256) unsigned char scratch[HSA_ATTN_BWD_STATIC_BYTES];

namespace hsa {
static constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mu;
static void *g_scratch_ptr[kMaxDevices];  // per device, filled on the first call there

// `may_resolve` false: only an address that is already known is returned (a stream that is being
// captured must not see the symbol lookup, which is no stream operation and may fail or end the
// capture)
static int scratch_for_current_device(void **out, bool may_resolve) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(HSA_ERR_LAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return fail(HSA_ERR_UNSUPPORTED, "device ordinal %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        if (!may_resolve)
            return fail(HSA_ERR_UNSUPPORTED,
                        "hsa_attn_bwd_static: first use on device %d while the stream is being captured; call "
                        "hsa_attn_bwd_static_capacity() (or hsa_attn_bwd_static once) on this device before the capture",
                        dev);
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return fail(HSA_ERR_LAUNCH, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return HSA_OK;
}
}  // namespace hsa

// Also the set-up call: resolves the buffer's address on the current device, so that a later
// hsa_attn_bwd_static there does nothing but launch (what a captured stream needs).
size_t hsa_attn_bwd_static_capacity(void) {
    void *ws = nullptr;
    (void)hsa::scratch_for_current_device(&ws, true);
    return (size_t)HSA_ATTN_BWD_STATIC_BYTES;
}

int hsa_attn_bwd_static(const void *q, const void *k, const void *v, const void *dout, void *dq, void *dk,
                        void *dv, int B, int N, int M, int H, int D, int L, int R, int causal, int dtype,
                        int algo, void *stream) {
    HSA_REQUIRE(B >= 1 && N >= 1 && H >= 1 && D >= 1, "bad shape B=%d N=%d H=%d D=%d", B, N, H, D);
    HSA_REQUIRE(L >= 0 && R >= 0, "bad L=%d R=%d", L, R);
    const size_t need = hsa_attn_bwd_workspace_bytes(B, N, M, H, D, L, R, dtype, algo);
    if (need > (size_t)HSA_ATTN_BWD_STATIC_BYTES)
        return hsa::fail(HSA_ERR_UNSUPPORTED,
                         "problem needs %zu bytes of scratch, the built-in buffer holds %zu: use hsa_attn_bwd "
                         "with a caller-provided workspace", need, (size_t)HSA_ATTN_BWD_STATIC_BYTES);
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing((hipStream_t)stream, &cap) != hipSuccess) {
        (void)hipGetLastError();
        cap = hipStreamCaptureStatusNone;
    }
    void *ws = nullptr;
    const int rc = hsa::scratch_for_current_device(&ws, cap == hipStreamCaptureStatusNone);
    if (rc != HSA_OK) return rc;
    // the kernels write every workspace entry before they read it: nothing to clear between calls
    return hsa_attn_bwd(q, k, v, dout, dq, dk, dv, ws, (size_t)HSA_ATTN_BWD_STATIC_BYTES, B, N, M, H, D, L, R,
                        causal, dtype, algo, stream);
}

int hsa_span_input_y_bwd(const void *dy, void *dx, int B, int N, int C, int dtype, void *stream) {
    HSA_REQUIRE(dy && dx, "null pointer");
    HSA_REQUIRE(B >= 1 && C >= 1, "bad shape B=%d C=%d", B, C);
    HSA_REQUIRE(N >= 2 && N <= (1 << 26), "N must lie in [2, 2^26] (got %d)", N);
    const int L = hsa::span_levels(N);
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case HSA_F32: return hsa::span_y_bwd_launch<hsa::F32>(dy, dx, B, N, C, L, st);
        case HSA_F16: return hsa::span_y_bwd_launch<hsa::F16>(dy, dx, B, N, C, L, st);
        case HSA_BF16: return hsa::span_y_bwd_launch<hsa::BF16>(dy, dx, B, N, C, L, st);
    }
    return hsa::fail(HSA_ERR_INVALID, "unknown dtype %d", dtype);
}

}  // extern "C"
