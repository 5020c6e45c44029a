// Eligibility test and launch parameters of the MFMA tile kernel.
#include "hsa_attn_tile.h"

#include <stdlib.h>

namespace hsa {

constexpr int TILE_MAX_NBW = 2;

bool attn_tile_eligible(int N, int M, int H, int D, int L, int R, int dtype, bool canonical,
                        bool want_weights) {
    (void)H;
    if (!canonical || want_weights) return false;
    if (dtype != HSA_F16 && dtype != HSA_BF16) return false;
    if (D != 32 && D != 64 && D != 128) return false;
    if (N < TILE_Q || ilog2_exact(N) != L || L > TILE_MAX_LEVELS) return false;
    if (M < 2 * N - 1) return false;
    if ((R + TILE_Q - 1) / TILE_Q > TILE_MAX_NBW) return false;
    return true;
}

int attn_tile_dispatch(const void *q, const void *k, const void *v, void *out, float *weights, int B,
                       int N, int M, int H, int D, int L, int R, int causal, int dtype, hipStream_t st) {
    (void)weights;
    if ((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15) != 0)
        return fail(HSA_ERR_INVALID, "tile kernel needs 16-byte aligned tensors");
    TileParams p;
    p.q = (const uint16_t *)q; p.k = (const uint16_t *)k; p.v = (const uint16_t *)v;
    p.out = (uint16_t *)out;
    p.B = B; p.N = N; p.M = M; p.H = H; p.L = L; p.R = R;
    const int NB = N / TILE_Q;
    // strip length: long enough to amortise the halo and to prefetch, short enough to give
    // every SIMD of the 256 CUs at least two wavefronts
    const long block_units = (long)B * H * NB;
    int sb = block_units >= 4 * 2048 ? 4 : (block_units >= 2 * 2048 ? 2 : 1);
    if (const char *e = getenv("HSA_ATTN_TILE_SB")) { int x = atoi(e); if (x == 1 || x == 2 || x == 4) sb = x; }
    if (!causal && (R + TILE_Q - 1) / TILE_Q >= 2 && sb > 2) sb = 2;  // five leaf blocks: registers
    while (sb > NB) sb >>= 1;  // NB is a power of two
    p.NS = NB / sb;
    const long units = (long)B * p.NS * H;
    if (units > 0x3fffffffL) return fail(HSA_ERR_UNSUPPORTED, "problem too large for one launch");
    p.n_units = (int)units;
    p.xcd_swizzle = 1;
    if (const char *e = getenv("HSA_ATTN_TILE_SWZ")) p.xcd_swizzle = atoi(e);
    p.alternate = 1;
    if (const char *e = getenv("HSA_ATTN_TILE_ALT")) p.alternate = atoi(e);
    p.scale_log2e = 1.4426950408889634f / sqrtf((float)D);
    int wpb = 8;
    if (const char *e = getenv("HSA_ATTN_TILE_WPB")) { int x = atoi(e); if (x >= 1 && x <= 8) wpb = x; }
    const int nbw = (R + TILE_Q - 1) / TILE_Q;
    if (dtype == HSA_BF16) {
        if (D == 32) return attn_tile_launch_td<BF16, 32>(p, nbw, causal != 0, sb, wpb, st);
        if (D == 64) return attn_tile_launch_td<BF16, 64>(p, nbw, causal != 0, sb, wpb, st);
        return attn_tile_launch_td<BF16, 128>(p, nbw, causal != 0, sb, wpb, st);
    }
    if (D == 32) return attn_tile_launch_td<F16, 32>(p, nbw, causal != 0, sb, wpb, st);
    if (D == 64) return attn_tile_launch_td<F16, 64>(p, nbw, causal != 0, sb, wpb, st);
    return attn_tile_launch_td<F16, 128>(p, nbw, causal != 0, sb, wpb, st);
}

}  // namespace hsa
