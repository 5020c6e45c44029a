// Bottom-up parent build: each parent attends over {itself, child 2i, child 2i+1}.
//
// Streaming kernel: a group of G lanes owns one (batch, parent, head) row and
// reads it in 16-byte pieces, so a wavefront covers 64/G consecutive head rows
// (one or more whole token rows) per load instruction.  The three dot products
// are reduced inside the group with xor shuffles; the 3-way softmax and the
// weighted sum of the value rows stay in fp32 registers.
#include "hsa_common.h"

namespace hsa {

template <typename T, int VEC> struct Pack { typename T::storage e[VEC]; };

template <typename T, int VEC>
__device__ __forceinline__ void load_vec(const typename T::storage *p, float (&f)[VEC]) {
    if constexpr (VEC == 1) {
        f[0] = to_float<T>(p[0]);
    } else {
        using P = Pack<T, VEC>;
        P v = *reinterpret_cast<const P *>(p);
#pragma unroll
        for (int i = 0; i < VEC; ++i) f[i] = to_float<T>(v.e[i]);
    }
}

template <typename T, int VEC>
__device__ __forceinline__ void store_vec(typename T::storage *p, const float (&f)[VEC]) {
    if constexpr (VEC == 1) {
        p[0] = from_float<T>(f[0]);
    } else {
        using P = Pack<T, VEC>;
        P v;
#pragma unroll
        for (int i = 0; i < VEC; ++i) v.e[i] = from_float<T>(f[i]);
        *reinterpret_cast<P *>(p) = v;
    }
}

// 3-way softmax with the reference kernel's epsilon in the denominator.
__device__ __forceinline__ void softmax3(float s0, float s1, float s2, float &w0, float &w1, float &w2) {
    float m = fmaxf(s0, fmaxf(s1, s2));
    float e0 = expf(s0 - m), e1 = expf(s1 - m), e2 = expf(s2 - m);
    float den = e0 + e1 + e2 + 1e-9f;
    w0 = e0 / den;
    w1 = e1 / den;
    w2 = e2 / den;
}

// CH = number of VEC-chunks each lane holds (D <= G * VEC * CH).
template <typename T, int VEC, int CH>
__global__ void __launch_bounds__(256)
build_parents_kernel(const typename T::storage *__restrict__ Qp, const typename T::storage *__restrict__ Kp,
                     const typename T::storage *__restrict__ Vp, const typename T::storage *__restrict__ Kc,
                     const typename T::storage *__restrict__ Vc, typename T::storage *__restrict__ Out,
                     typename T::storage *__restrict__ Out2, typename T::storage *__restrict__ Wt, int B,
                     int P, int H, int D, int G, int64_t qp_bs, int64_t kp_bs, int64_t vp_bs, int64_t kc_bs,
                     int64_t vc_bs, int64_t out_bs, int64_t out2_bs, float scale) {
    const long tid = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long unit = tid / G;
    const int gl = (int)(tid % G);
    const long units = (long)B * P * H;
    const bool active = unit < units;
    const long u = active ? unit : units - 1;  // keep every lane in the shuffles
    const int h = (int)(u % H);
    const int i = (int)((u / H) % P);
    const int b = (int)(u / ((long)H * P));
    const size_t prow = ((size_t)i * H + h) * D;
    const size_t c0row = ((size_t)(2 * i) * H + h) * D;
    const size_t c1row = c0row + (size_t)H * D;
    const typename T::storage *q = Qp + (size_t)b * qp_bs + prow;
    const typename T::storage *kp = Kp + (size_t)b * kp_bs + prow;
    const typename T::storage *vp = Vp + (size_t)b * vp_bs + prow;
    const typename T::storage *k0 = Kc + (size_t)b * kc_bs + c0row;
    const typename T::storage *k1 = Kc + (size_t)b * kc_bs + c1row;
    const typename T::storage *v0 = Vc + (size_t)b * vc_bs + c0row;
    const typename T::storage *v1 = Vc + (size_t)b * vc_bs + c1row;

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
    for (int o = G >> 1; o >= 1; o >>= 1) {
        s0 += __shfl_xor(s0, o, 64);
        s1 += __shfl_xor(s1, o, 64);
        s2 += __shfl_xor(s2, o, 64);
    }
    float w0, w1, w2;
    softmax3(s0 * scale, s1 * scale, s2 * scale, w0, w1, w2);
    if (!active) return;
    typename T::storage *o = Out + (size_t)b * out_bs + prow;
    typename T::storage *o2 = Out2 ? Out2 + (size_t)b * out2_bs + prow : nullptr;
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
                                int64_t qp_bs, int64_t kp_bs, int64_t vp_bs, int64_t kc_bs, int64_t vc_bs,
                                int64_t out_bs, int64_t out2_bs, hipStream_t st) {
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
        (S *)out2, (S *)weights, B, P, H, D, G, qp_bs, kp_bs, vp_bs, kc_bs, vc_bs, out_bs, out2_bs, scale)
    if (CH == 1) HSA_BPN_LAUNCH(1);
    else if (CH == 2) HSA_BPN_LAUNCH(2);
    else if (CH <= 4) HSA_BPN_LAUNCH(4);
    else if (CH <= 8) HSA_BPN_LAUNCH(8);
    else return fail(HSA_ERR_UNSUPPORTED, "head_dim %d too large", D);
#undef HSA_BPN_LAUNCH
    return check_launch("build_parents_kernel");
}

template <typename T>
static int build_parents_typed(const void *qp, const void *kp, const void *vp, const void *kc,
                               const void *vc, void *out, void *out2, void *weights, int B, int P, int H,
                               int D, int64_t qp_bs, int64_t kp_bs, int64_t vp_bs, int64_t kc_bs,
                               int64_t vc_bs, int64_t out_bs, int64_t out2_bs, hipStream_t st) {
    constexpr int VEC = 16 / (int)sizeof(typename T::storage);
    const uintptr_t align = (uintptr_t)qp | (uintptr_t)kp | (uintptr_t)vp | (uintptr_t)kc | (uintptr_t)vc |
                            (uintptr_t)out | (uintptr_t)out2;
    const int64_t strides = qp_bs | kp_bs | vp_bs | kc_bs | vc_bs | out_bs | out2_bs;
    if (D % VEC == 0 && (align & 15) == 0 && (strides % VEC) == 0)
        return build_parents_launch<T, VEC>(qp, kp, vp, kc, vc, out, out2, weights, B, P, H, D, qp_bs, kp_bs,
                                            vp_bs, kc_bs, vc_bs, out_bs, out2_bs, st);
    return build_parents_launch<T, 1>(qp, kp, vp, kc, vc, out, out2, weights, B, P, H, D, qp_bs, kp_bs, vp_bs,
                                      kc_bs, vc_bs, out_bs, out2_bs, st);
}

int build_parents_dispatch(const void *qp, const void *kp, const void *vp, const void *kc, const void *vc,
                           void *out, void *out2, void *weights, int B, int P, int H, int D, int64_t qp_bs,
                           int64_t kp_bs, int64_t vp_bs, int64_t kc_bs, int64_t vc_bs, int64_t out_bs,
                           int64_t out2_bs, int dtype, hipStream_t st) {
    const int64_t prow = (int64_t)P * H * D, crow = 2 * prow;
    if (!qp_bs) qp_bs = prow;
    if (!kp_bs) kp_bs = prow;
    if (!vp_bs) vp_bs = prow;
    if (!out_bs) out_bs = prow;
    if (!out2_bs) out2_bs = prow;
    if (!kc_bs) kc_bs = crow;
    if (!vc_bs) vc_bs = crow;
    switch (dtype) {
        case HSA_F32: return build_parents_typed<F32>(qp, kp, vp, kc, vc, out, out2, weights, B, P, H, D, qp_bs, kp_bs, vp_bs, kc_bs, vc_bs, out_bs, out2_bs, st);
        case HSA_F16: return build_parents_typed<F16>(qp, kp, vp, kc, vc, out, out2, weights, B, P, H, D, qp_bs, kp_bs, vp_bs, kc_bs, vc_bs, out_bs, out2_bs, st);
        case HSA_BF16: return build_parents_typed<BF16>(qp, kp, vp, kc, vc, out, out2, weights, B, P, H, D, qp_bs, kp_bs, vp_bs, kc_bs, vc_bs, out_bs, out2_bs, st);
    }
    return fail(HSA_ERR_INVALID, "unknown dtype %d", dtype);
}

}  // namespace hsa

extern "C" {

int hsa_build_parents_fwd(const void *qp, const void *kp, const void *vp, const void *kc,
                          const void *vc, void *out, void *weights, int B, int P, int H, int D,
                          int64_t qp_bs, int64_t kp_bs, int64_t vp_bs, int64_t kc_bs, int64_t vc_bs,
                          int64_t out_bs, int dtype, void *stream) {
    HSA_REQUIRE(qp && kp && vp && kc && vc && out, "null pointer");
    HSA_REQUIRE(B >= 1 && P >= 1 && H >= 1 && D >= 1, "bad shape B=%d P=%d H=%d D=%d", B, P, H, D);
    return hsa::build_parents_dispatch(qp, kp, vp, kc, vc, out, nullptr, weights, B, P, H, D, qp_bs, kp_bs,
                                       vp_bs, kc_bs, vc_bs, out_bs, 0, dtype, (hipStream_t)stream);
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
    const size_t es = hsa::elem_size(dtype);
    const size_t row = (size_t)H * D * es;
    // level by level; each level reads the previous level's rows of `out`
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
