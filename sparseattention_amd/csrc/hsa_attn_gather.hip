// Span attention forward, per-query gather kernel.
//
// One wavefront owns one (batch, query, head).  Lanes first act as "one lane per
// attention slot" (window slots 0..2R, then the L tree slots): each lane fetches
// its key row and forms the full dot product, so the softmax statistics need
// only wave-wide max / sum reductions.  For the value pass the lanes switch to
// "one lane per output channel": the slot weights and rows are broadcast lane by
// lane and V rows are read coalesced.  Works for any element type, any D, any
// neighbour table (including -1 entries) and writes the optional fp32 weights.
// It is the reference-shaped kernel; the MFMA tile kernel is the fast path.
#include "hsa_common.h"

namespace hsa {

constexpr int GATHER_MAX_CHUNKS = 4;  // slots <= 64 * 4

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

template <typename T>
__global__ void __launch_bounds__(256)
attn_gather_kernel(const typename T::storage *__restrict__ Q, const typename T::storage *__restrict__ K,
                   const typename T::storage *__restrict__ V, const int32_t *__restrict__ idx,
                   const uint8_t *__restrict__ mask, typename T::storage *__restrict__ Out,
                   float *__restrict__ W, int B, int N, int M, int H, int D, int L, int R, int causal,
                   float scale) {
    const int lane = threadIdx.x & 63;
    const long unit = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const long units = (long)B * N * H;
    if (unit >= units) return;  // whole wave leaves together
    const int h = (int)(unit % H);
    const int n = (int)((unit / H) % N);
    const int b = (int)(unit / ((long)H * N));
    const int Wn = 2 * R + 1;
    const int S = Wn + L;

    const typename T::storage *q = Q + (((size_t)b * N + n) * H + h) * D;
    const typename T::storage *kb = K + (size_t)b * M * H * D + (size_t)h * D;
    const typename T::storage *vb = V + (size_t)b * M * H * D + (size_t)h * D;
    const size_t row_stride = (size_t)H * D;

    int row[GATHER_MAX_CHUNKS];
    float sc[GATHER_MAX_CHUNKS];
    float mx = -INFINITY;
#pragma unroll
    for (int c = 0; c < GATHER_MAX_CHUNKS; ++c) {
        const int t = c * 64 + lane;
        int r = -1;
        if (t < Wn) {
            int j = n + t - R;
            if (j >= 0 && j < N && (!causal || j <= n)) r = j;
        } else if (t < S) {
            int l = t - Wn;
            int m;
            bool dead;
            if (idx) {
                m = idx[(size_t)n * L + l];
                dead = (m == -1) || (mask && mask[(size_t)n * L + l] != 0);
            } else {
                m = level_offset(N, l) + ((n >> l) ^ 1);
                dead = causal && (((n >> l) & 1) == 0);
            }
            if (!dead) r = m;
        }
        row[c] = r;
        float s = -INFINITY;
        if (r >= 0) {
            const typename T::storage *kr = kb + (size_t)r * row_stride;
            float acc = 0.f;
            for (int d = 0; d < D; ++d) acc = fmaf(to_float<T>(q[d]), to_float<T>(kr[d]), acc);
            s = acc * scale;
        }
        sc[c] = s;
        mx = fmaxf(mx, s);
    }
    mx = wave_max(mx);
    float den = 0.f;
#pragma unroll
    for (int c = 0; c < GATHER_MAX_CHUNKS; ++c) {
        float e = (row[c] >= 0) ? expf(sc[c] - mx) : 0.f;
        sc[c] = e;
        den += e;
    }
    den = wave_sum(den);
    den = fmaxf(den, 1.0e-5f);
#pragma unroll
    for (int c = 0; c < GATHER_MAX_CHUNKS; ++c) sc[c] = sc[c] / den;

    if (W) {
        float *wp = W + (((size_t)b * N + n) * H + h) * S;
#pragma unroll
        for (int c = 0; c < GATHER_MAX_CHUNKS; ++c) {
            int t = c * 64 + lane;
            if (t < S) wp[t] = sc[c];
        }
    }

    typename T::storage *o = Out + (((size_t)b * N + n) * H + h) * D;
    for (int d0 = 0; d0 < D; d0 += 64) {
        const int d = d0 + lane;
        float acc = 0.f;
#pragma unroll
        for (int c = 0; c < GATHER_MAX_CHUNKS; ++c) {
            const int lim = S - c * 64 < 64 ? S - c * 64 : 64;
            for (int t = 0; t < lim; ++t) {
                int r = __shfl(row[c], t, 64);
                float p = __shfl(sc[c], t, 64);
                if (r >= 0 && d < D) acc = fmaf(p, to_float<T>(vb[(size_t)r * row_stride + d]), acc);
            }
        }
        if (d < D) o[d] = from_float<T>(acc);
    }
}

// ---- vector variant ---------------------------------------------------------------------------
// D/VEC lanes (VEC = 16 bytes of elements) share one attention slot and read its key / value row
// as one contiguous piece, so a wavefront covers SPW = 64*VEC/D slots per pass and every load is
// a whole head-row.  Each lane keeps its VEC channels of q and of the output accumulator; scores
// are reduced inside the lane group, the output across the SPW groups at the end.
constexpr int GATHER_MAX_PASSES = 40;

template <typename T, int VEC, int LPS /* lanes per slot = D / VEC */>
__global__ void __launch_bounds__(256)
attn_gather_vec_kernel(const typename T::storage *__restrict__ Q, const typename T::storage *__restrict__ K,
                       const typename T::storage *__restrict__ V, const int32_t *__restrict__ idx,
                       const uint8_t *__restrict__ mask, typename T::storage *__restrict__ Out,
                       float *__restrict__ W, int B, int N, int M, int H, int L, int R, int causal, float scale) {
    constexpr int D = VEC * LPS;
    constexpr int SPW = 64 / LPS;  // slots per pass
    struct alignas(16) Pk { typename T::storage e[VEC]; };
    const int lane = threadIdx.x & 63;
    const int sub = lane / LPS;    // slot inside a pass
    const int gl = lane % LPS;     // channel piece
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

    float q[VEC];
    {
        Pk t = *reinterpret_cast<const Pk *>(Q + (((size_t)b * N + n) * H + h) * D + gl * VEC);
#pragma unroll
        for (int e = 0; e < VEC; ++e) q[e] = to_float<T>(t.e[e]) * scale;
    }
    auto slot_row = [&](int t) {
        int r = -1;
        if (t < Wn) {
            const int j = n + t - R;
            if (j >= 0 && j < N && (!causal || j <= n)) r = j;
        } else if (t < S) {
            const int l = t - Wn;
            if (idx) {
                const int m = idx[(size_t)n * L + l];
                if (m != -1 && !(mask && mask[(size_t)n * L + l] != 0)) r = m;
            } else if (!(causal && (((n >> l) & 1) == 0))) {
                r = level_offset(N, l) + ((n >> l) ^ 1);
            }
        }
        return r;
    };
    // pass 1: scores of this lane group's slots, eight passes at a time: the eight key pieces are
    // requested together and unconditionally (a dead slot re-reads the query's own leaf row, which
    // is hot), so one memory round trip serves eight passes
    constexpr int CHUNK = 8;
    float sc[GATHER_MAX_PASSES];
    float mx = -INFINITY;
#pragma unroll
    for (int c = 0; c < GATHER_MAX_PASSES / CHUNK; ++c) {
#pragma unroll
        for (int p = 0; p < CHUNK; ++p) sc[c * CHUNK + p] = -INFINITY;
        if (c * CHUNK < passes) {  // uniform
            int rr[CHUNK];
            Pk kk[CHUNK];
#pragma unroll
            for (int p = 0; p < CHUNK; ++p) {
                rr[p] = slot_row((c * CHUNK + p) * SPW + sub);
                kk[p] = *reinterpret_cast<const Pk *>(kb + (size_t)(rr[p] < 0 ? n : rr[p]) * rs);
            }
#pragma unroll
            for (int p = 0; p < CHUNK; ++p) {
                float a = 0.f;
#pragma unroll
                for (int e = 0; e < VEC; ++e) a = fmaf(q[e], to_float<T>(kk[p].e[e]), a);
                a = group_sum(a, LPS);
                if (rr[p] >= 0) sc[c * CHUNK + p] = a;
                mx = fmaxf(mx, sc[c * CHUNK + p]);
            }
        }
    }
    for (int o = LPS; o < 64; o <<= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    float den = 0.f;
#pragma unroll
    for (int p = 0; p < GATHER_MAX_PASSES; ++p) {
        if ((p / CHUNK) * CHUNK < passes) {  // every pass of an active chunk (dead slots become 0)
            sc[p] = sc[p] == -INFINITY ? 0.f : expf(sc[p] - mx);
            den += sc[p];
        }
    }
    for (int o = LPS; o < 64; o <<= 1) den += __shfl_xor(den, o, 64);
    den = fmaxf(den, 1.0e-5f);
    float acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
    float *wp = W ? W + (((size_t)b * N + n) * H + h) * S : nullptr;
#pragma unroll
    for (int c = 0; c < GATHER_MAX_PASSES / CHUNK; ++c) {
        if (c * CHUNK < passes) {  // uniform
            int rr[CHUNK];
            Pk vv[CHUNK];
#pragma unroll
            for (int p = 0; p < CHUNK; ++p) {
                rr[p] = slot_row((c * CHUNK + p) * SPW + sub);
                vv[p] = *reinterpret_cast<const Pk *>(vb + (size_t)(rr[p] < 0 ? n : rr[p]) * rs);
            }
#pragma unroll
            for (int p = 0; p < CHUNK; ++p) {
                const int t = (c * CHUNK + p) * SPW + sub;
                const float w = sc[c * CHUNK + p] / den;  // zero for dead slots
                if (wp && gl == 0 && t < S) wp[t] = w;
#pragma unroll
                for (int e = 0; e < VEC; ++e) acc[e] = fmaf(w, to_float<T>(vv[p].e[e]), acc[e]);
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
        *reinterpret_cast<Pk *>(Out + (((size_t)b * N + n) * H + h) * D + gl * VEC) = o;
    }
}

template <typename T, int LPS>
static int attn_gather_vec_launch(const void *q, const void *k, const void *v, const int32_t *idx,
                                  const uint8_t *mask, void *out, float *weights, int B, int N, int M, int H,
                                  int L, int R, int causal, hipStream_t st) {
    using S = typename T::storage;
    constexpr int VEC = 16 / (int)sizeof(S);
    const long units = (long)B * N * H;
    const long blocks = (units + 3) / 4;
    if (blocks > 0x7fffffffL) return fail(HSA_ERR_UNSUPPORTED, "problem too large for one launch");
    const float scale = 1.0f / sqrtf((float)(VEC * LPS));
    attn_gather_vec_kernel<T, VEC, LPS><<<(unsigned)blocks, 256, 0, st>>>(
        (const S *)q, (const S *)k, (const S *)v, idx, mask, (S *)out, weights, B, N, M, H, L, R, causal, scale);
    return check_launch("attn_gather_vec_kernel");
}

// returns HSA_ERR_UNSUPPORTED when the shape does not fit (the scalar kernel then runs)
template <typename T>
static int attn_gather_vec_try(const void *q, const void *k, const void *v, const int32_t *idx, const uint8_t *mask,
                               void *out, float *weights, int B, int N, int M, int H, int D, int L, int R,
                               int causal, hipStream_t st) {
    constexpr int VEC = 16 / (int)sizeof(typename T::storage);
    if (D % VEC != 0) return HSA_ERR_UNSUPPORTED;
    if ((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15) != 0) return HSA_ERR_UNSUPPORTED;
    const int lps = D / VEC;
    const int S = 2 * R + 1 + L;
#define HSA_GV(LPSN)                                                                                         \
    case LPSN:                                                                                               \
        if ((S + 64 / LPSN - 1) / (64 / LPSN) > GATHER_MAX_PASSES) return HSA_ERR_UNSUPPORTED;               \
        return attn_gather_vec_launch<T, LPSN>(q, k, v, idx, mask, out, weights, B, N, M, H, L, R, causal, st)
    switch (lps) {
        HSA_GV(2);
        HSA_GV(4);
        HSA_GV(8);
        HSA_GV(16);
        HSA_GV(32);
    }
#undef HSA_GV
    return HSA_ERR_UNSUPPORTED;
}

template <typename T>
int attn_gather_launch(const void *q, const void *k, const void *v, const int32_t *idx,
                       const uint8_t *mask, void *out, float *weights, int B, int N, int M, int H,
                       int D, int L, int R, int causal, hipStream_t st) {
    using S = typename T::storage;
    const long units = (long)B * N * H;
    const int waves_per_block = 4;
    const long blocks = (units + waves_per_block - 1) / waves_per_block;
    if (blocks > 0x7fffffffL) return fail(HSA_ERR_UNSUPPORTED, "problem too large for one launch");
    const float scale = 1.0f / sqrtf((float)D);
    attn_gather_kernel<T><<<(unsigned)blocks, waves_per_block * 64, 0, st>>>(
        (const S *)q, (const S *)k, (const S *)v, idx, mask, (S *)out, weights, B, N, M, H, D, L, R,
        causal, scale);
    return check_launch("attn_gather_kernel");
}

int attn_gather_dispatch(const void *q, const void *k, const void *v, const int32_t *idx,
                         const uint8_t *mask, void *out, float *weights, int B, int N, int M, int H,
                         int D, int L, int R, int causal, int dtype, hipStream_t st) {
    if (2 * R + 1 + L > 64 * GATHER_MAX_CHUNKS)
        return fail(HSA_ERR_UNSUPPORTED, "2R+1+L = %d slots exceeds %d", 2 * R + 1 + L,
                    64 * GATHER_MAX_CHUNKS);
    {
        int rc = HSA_ERR_UNSUPPORTED;
        if (dtype == HSA_F32) rc = attn_gather_vec_try<F32>(q, k, v, idx, mask, out, weights, B, N, M, H, D, L, R, causal, st);
        else if (dtype == HSA_F16) rc = attn_gather_vec_try<F16>(q, k, v, idx, mask, out, weights, B, N, M, H, D, L, R, causal, st);
        else if (dtype == HSA_BF16) rc = attn_gather_vec_try<BF16>(q, k, v, idx, mask, out, weights, B, N, M, H, D, L, R, causal, st);
        if (rc != HSA_ERR_UNSUPPORTED) return rc;
    }
    switch (dtype) {
        case HSA_F32: return attn_gather_launch<F32>(q, k, v, idx, mask, out, weights, B, N, M, H, D, L, R, causal, st);
        case HSA_F16: return attn_gather_launch<F16>(q, k, v, idx, mask, out, weights, B, N, M, H, D, L, R, causal, st);
        case HSA_BF16: return attn_gather_launch<BF16>(q, k, v, idx, mask, out, weights, B, N, M, H, D, L, R, causal, st);
    }
    return fail(HSA_ERR_INVALID, "unknown dtype %d", dtype);
}

}  // namespace hsa
