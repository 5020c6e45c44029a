// hsa_attn_fwd: argument checks and kernel selection for the span attention forward.
#include "hsa_common.h"

namespace hsa {

int attn_gather_dispatch(const void *q, const void *k, const void *v, const int32_t *idx,
                         const uint8_t *mask, void *out, float *weights, int B, int N, int M, int H,
                         int D, int L, int R, int causal, int dtype, hipStream_t st);

bool attn_tile_eligible(int N, int M, int H, int D, int L, int R, int dtype, bool canonical,
                        bool want_weights, bool causal);
int attn_tile_dispatch(const void *q, const void *k, const void *v, void *out, float *weights, float *lse, int B,
                       int N, int M, int H, int D, int L, int R, int causal, int dtype, hipStream_t st);
int attn_tile_tune(int sb, int wpb, int swizzle, int alternate);
bool attn_tile_f32_eligible(int N, int M, int D, int L, int R, bool canonical, bool want_weights);
int attn_tile_f32_dispatch(const void *q, const void *k, const void *v, void *out, int B, int N, int M, int H,
                           int D, int L, int R, int causal, hipStream_t st);

// the MFMA tile kernels: 16-bit element types, or fp32 on the fp32 matrix instructions
static bool tile_ok_for(int N, int M, int H, int D, int L, int R, int dtype, bool canonical, bool want_weights,
                        bool causal) {
    if (dtype == HSA_F32) return attn_tile_f32_eligible(N, M, D, L, R, canonical, want_weights);
    return attn_tile_eligible(N, M, H, D, L, R, dtype, canonical, want_weights, causal);
}

}  // namespace hsa

extern "C" {

int hsa_attn_tile_tune(int strip_blocks, int waves_per_group, int xcd_remap, int alternate) {
    return hsa::attn_tile_tune(strip_blocks, waves_per_group, xcd_remap, alternate);
}

int hsa_attn_fwd_uses_tile(int N, int M, int H, int D, int L, int R, int dtype, int canonical_tables,
                           int want_weights) {
    return hsa::tile_ok_for(N, M, H, D, L, R, dtype, canonical_tables != 0, want_weights != 0,
                            canonical_tables == 2) ? 1 : 0;
}

int hsa_attn_fwd(const void *q, const void *k, const void *v, const int32_t *idx,
                 const uint8_t *mask, void *out, float *weights, int B, int N, int M, int H, int D,
                 int L, int R, int causal, int dtype, int algo, void *stream) {
    HSA_REQUIRE(q && k && v && out, "null pointer");
    HSA_REQUIRE(B >= 1 && N >= 1 && H >= 1 && D >= 1, "bad shape B=%d N=%d H=%d D=%d", B, N, H, D);
    HSA_REQUIRE(M >= N, "key rows M=%d < N=%d", M, N);
    HSA_REQUIRE(L >= 0 && R >= 0, "bad L=%d R=%d", L, R);
    HSA_REQUIRE(dtype == HSA_F32 || dtype == HSA_F16 || dtype == HSA_BF16, "unknown dtype %d", dtype);
    const bool canonical = (idx == nullptr);
    if (canonical) {
        HSA_REQUIRE(mask == nullptr, "mask must be NULL when idx is NULL (use `causal`)");
        HSA_REQUIRE(hsa::ilog2_exact(N) == L, "canonical table needs L == log2 N (N=%d L=%d)", N, L);
        HSA_REQUIRE(M >= 2 * N - 1, "canonical table needs M >= 2N-1 (N=%d M=%d)", N, M);
    } else {
        causal = (mask != nullptr);
    }
    hipStream_t st = (hipStream_t)stream;
    bool tile_ok = hsa::tile_ok_for(N, M, H, D, L, R, dtype, canonical, weights != nullptr, causal != 0);
    // the tile kernels move 16-byte pieces: tensors at other addresses (a view at an odd element
    // offset) go to the gather kernel unless the tile kernel was asked for by name
    const bool aligned = (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15) == 0;
    if (!aligned && algo != HSA_ATTN_TILE) tile_ok = false;
    if (!aligned && algo == HSA_ATTN_TILE && tile_ok)
        return hsa::fail(HSA_ERR_INVALID, "tile kernel needs 16-byte aligned tensors");
    if (algo == HSA_ATTN_TILE && !tile_ok)
        return hsa::fail(HSA_ERR_UNSUPPORTED,
                         "tile kernel not available for N=%d H=%d D=%d L=%d R=%d dtype=%d canonical=%d",
                         N, H, D, L, R, dtype, (int)canonical);
    if (tile_ok && algo != HSA_ATTN_GATHER) {
        if (dtype == HSA_F32) {
            // dispatch events are attached by the 16-bit launcher only: record around this one
            const hsa::LaunchEvents ev = hsa::take_launch_events();
            if (ev.start && ev.stop) (void)hipEventRecord(ev.start, st);
            const int rc = hsa::attn_tile_f32_dispatch(q, k, v, out, B, N, M, H, D, L, R, causal ? 1 : 0, st);
            if (ev.start && ev.stop) (void)hipEventRecord(ev.stop, st);
            return rc;
        }
        return hsa::attn_tile_dispatch(q, k, v, out, weights, nullptr, B, N, M, H, D, L, R, causal ? 1 : 0, dtype, st);
    }
    // the gather kernels take no dispatch events: record around the call instead
    const hsa::LaunchEvents ev = hsa::take_launch_events();
    if (ev.start && ev.stop) (void)hipEventRecord(ev.start, st);
    const int rc = hsa::attn_gather_dispatch(q, k, v, idx, mask, out, weights, B, N, M, H, D, L, R,
                                             causal ? 1 : 0, dtype, st);
    if (ev.start && ev.stop) (void)hipEventRecord(ev.stop, st);
    return rc;
}

int hsa_attn_fwd_lse(const void *q, const void *k, const void *v, void *out, float *lse, int B, int N, int M,
                     int H, int D, int L, int R, int causal, int dtype, void *stream) {
    HSA_REQUIRE(q && k && v && out && lse, "null pointer");
    HSA_REQUIRE(B >= 1 && N >= 1 && H >= 1 && D >= 1, "bad shape B=%d N=%d H=%d D=%d", B, N, H, D);
    HSA_REQUIRE(L >= 0 && R >= 0, "bad L=%d R=%d", L, R);
    if ((dtype != HSA_F16 && dtype != HSA_BF16) || R > (causal ? 32 : 16) ||
        !hsa::attn_tile_eligible(N, M, H, D, L, R, dtype, true, false, causal != 0) ||
        ((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15) != 0))
        return hsa::fail(HSA_ERR_UNSUPPORTED, "the log-sum-exp output comes from the 16-bit tile kernel only "
                         "(N=%d H=%d D=%d L=%d R=%d dtype=%d)", N, H, D, L, R, dtype);
    return hsa::attn_tile_dispatch(q, k, v, out, nullptr, lse, B, N, M, H, D, L, R, causal ? 1 : 0, dtype,
                                   (hipStream_t)stream);
}

int hsa_attn_fwd_timed(const void *q, const void *k, const void *v, const int32_t *idx,
                       const uint8_t *mask, void *out, float *weights, int B, int N, int M, int H, int D,
                       int L, int R, int causal, int dtype, int algo, void *stream, void *start_event,
                       void *stop_event) {
    HSA_REQUIRE(start_event && stop_event, "null event");
    hsa::set_launch_events((hipEvent_t)start_event, (hipEvent_t)stop_event);
    const int rc = hsa_attn_fwd(q, k, v, idx, mask, out, weights, B, N, M, H, D, L, R, causal, dtype, algo, stream);
    (void)hsa::take_launch_events();  // an argument error returns before any launcher looks
    return rc;
}

}  // extern "C"
