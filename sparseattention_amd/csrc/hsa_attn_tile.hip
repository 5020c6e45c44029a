// Eligibility test and launch parameters of the MFMA tile kernel.
#include "hsa_attn_tile.h"

#include <stdlib.h>

#include <atomic>

namespace hsa {

// window radius in 16-row leaf blocks: up to 4 (R <= 64) when causal, where a query block sees
// NBW + 1 leaf blocks; up to 2 (R <= 32) otherwise, where it sees 2 NBW + 1
constexpr int TILE_MAX_NBW_CAUSAL = 4;
constexpr int TILE_MAX_NBW = 2;
constexpr int TILE_MAX_NBW_WIDE = 4;

// Experiment knobs of the tile launch: strip length in query blocks (0 = by problem size),
// wavefronts per workgroup (0 = by head count), XCD remap on/off, alternating strip direction on/off.  Initialised
// once per process from HSA_ATTN_TILE_SB / _WPB / _SWZ / _ALT, changed afterwards only through
// hsa_attn_tile_tune; a launch reads four atomics, never the environment.
struct TileKnobs {
    std::atomic<int> sb{0}, wpb{0}, swizzle{1}, alternate{1};
    TileKnobs() {
        if (const char *e = getenv("HSA_ATTN_TILE_SB")) { int x = atoi(e); if (x == 1 || x == 2 || x == 4 || x == 8) sb = x; }
        if (const char *e = getenv("HSA_ATTN_TILE_SWZ")) swizzle = atoi(e) != 0;
        if (const char *e = getenv("HSA_ATTN_TILE_ALT")) alternate = atoi(e) != 0;
        if (const char *e = getenv("HSA_ATTN_TILE_WPB")) { int x = atoi(e); if (x >= 1 && x <= 8) wpb = x; }
    }
};
static TileKnobs &tile_knobs() {
    static TileKnobs k;
    return k;
}

// the two knobs the fp32 tile launch shares
void attn_tile_knobs_sb_swizzle(int *sb, int *swizzle) {
    *sb = tile_knobs().sb > 4 ? 4 : (int)tile_knobs().sb;  // strips of more than four blocks: 16-bit kernels only
    *swizzle = tile_knobs().swizzle;
}

int attn_tile_tune(int sb, int wpb, int swizzle, int alternate) {
    if (!(sb == -1 || sb == 0 || sb == 1 || sb == 2 || sb == 4 || sb == 8))
        return fail(HSA_ERR_INVALID, "strip length %d", sb);
    if (!(wpb == -1 || (wpb >= 0 && wpb <= 8))) return fail(HSA_ERR_INVALID, "wavefronts per workgroup %d", wpb);
    TileKnobs &k = tile_knobs();
    if (sb >= 0) k.sb = sb;
    if (wpb >= 0) k.wpb = wpb;
    if (swizzle >= 0) k.swizzle = swizzle != 0;
    if (alternate >= 0) k.alternate = alternate != 0;
    return HSA_OK;
}

bool attn_tile_eligible(int N, int M, int H, int D, int L, int R, int dtype, bool canonical,
                        bool want_weights, bool causal) {
    (void)H;
    if (!canonical) return false;
    // the weights of a query block are assembled in the wavefront's LDS region: a row of
    // 2R+1+L floats has to fit the operand pitch
    if (want_weights && 2 * R + 1 + L > D * 2 + 16) return false;
    if (dtype != HSA_F16 && dtype != HSA_BF16) return false;
    if (D != 32 && D != 64 && D != 128) return false;
    if (N < TILE_Q || ilog2_exact(N) != L || L > TILE_MAX_LEVELS) return false;
    if (M < 2 * N - 1) return false;
    const int nbw = (R + TILE_Q - 1) / TILE_Q;
    if (causal) return nbw <= TILE_MAX_NBW_CAUSAL;
    // without the causal mask: up to five leaf blocks everywhere, seven or nine with one query
    // block per wavefront
    return nbw <= TILE_MAX_NBW || nbw <= TILE_MAX_NBW_WIDE;
}

int attn_tile_dispatch(const void *q, const void *k, const void *v, void *out, float *weights, float *lse, int B,
                       int N, int M, int H, int D, int L, int R, int causal, int dtype, hipStream_t st) {
    if ((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15) != 0)
        return fail(HSA_ERR_INVALID, "tile kernel needs 16-byte aligned tensors");
    TileParams p;
    p.q = (const uint16_t *)q; p.k = (const uint16_t *)k; p.v = (const uint16_t *)v;
    p.out = (uint16_t *)out;
    p.weights = weights;
    p.lse = lse;
    p.B = B; p.N = N; p.M = M; p.H = H; p.L = L; p.R = R;
    const int NB = N / TILE_Q;
    TileKnobs &knobs = tile_knobs();
    // strip length: long enough to amortise the halo and to prefetch, short enough to fill every
    // wavefront slot of the 256 CUs once (two per SIMD up to 64 channels, one at 128: there a
    // second round of shorter strips loses to one round of longer ones, B1 H16 N4096 D128 R32
    // 26.1 -> 24.0 us)
    const long block_units = (long)B * H * NB;
    const long slots = D > 64 ? 1024 : 2048;
    int sb = block_units >= 4 * slots ? 4 : (block_units >= 2 * slots ? 2 : 1);
    // long sequences with the causal mask: a wavefront walks two runs of four blocks, the window's
    // neighbouring leaf blocks are then fetched once per eight blocks.  From eight blocks per
    // wavefront slot on (us, strips of 4 -> 8): B1 H16 N65536 D128 R32 302 -> 286, N16384 80.0 ->
    // 73.5, N8192 42.6 -> 39.1; B8 H8 N4096 D64 R16 40.2 -> 38.2, B1 H16 N65536 D64 156 -> 146; the
    // headline shape (four blocks per slot) 20.4 -> 23.8, so not there.  Without the mask (three
    // leaf blocks per query block in 256 registers) it loses: B8 H8 N8192 D64 84.3 -> 89.8.  Four
    // runs gain nothing more at 64 channels and at 128 their code no longer fits the instruction
    // cache (1465 us).
    int runs = (causal && block_units >= 8 * slots) ? 2 : 1;
    if (const int forced = knobs.sb) {
        sb = forced > 4 ? 4 : forced;
        runs = forced > 4 ? forced / 4 : 1;
    }
    // four or five leaf blocks per query block: shorter strips keep the operands in registers
    if ((R + TILE_Q - 1) / TILE_Q >= (causal ? 3 : 2) && sb > 2) sb = 2;
    if ((R + TILE_Q - 1) / TILE_Q >= 4 && !knobs.sb) sb = 1;  // longer strips spill at five leaf blocks + halo
    if (!causal && (R + TILE_Q - 1) / TILE_Q > TILE_MAX_NBW) sb = 1;  // seven or nine leaf blocks: one block per wavefront
    while (sb > NB) sb >>= 1;  // NB is a power of two
    // runs: strips of four blocks, one or two blocks of neighbours to either side (two: causal), no weights output
    const int nbw_ = (R + TILE_Q - 1) / TILE_Q;
    if (sb != 4 || weights || nbw_ < 1 || nbw_ > (causal ? 2 : 1)) runs = 1;
    while (sb * runs > NB) runs >>= 1;
    p.runs = runs;
    p.NS = NB / (sb * runs);
    sb *= runs;  // the launchers switch on the strip length
    const long units = (long)B * p.NS * H;
    if (units > 0x3fffffffL) return fail(HSA_ERR_UNSUPPORTED, "problem too large for one launch");
    p.n_units = (int)units;
    p.xcd_swizzle = knobs.swizzle;
    p.alternate = knobs.alternate;
    p.scale_log2e = 1.4426950408889634f / sqrtf((float)D);
    // wavefronts per workgroup: as many as the variant allows, but a divisor of the head count
    // where one at least half that large exists, so that a workgroup's wavefronts are heads of one
    // strip and read whole contiguous token rows together (12 heads: 6 per workgroup, 35 -> 32 us
    // at B8 N2048 D64)
    int wpb = knobs.wpb;
    if (wpb == 0) {
        const int maxw = D > 64 ? 4 : 8;
        wpb = maxw;
        if (H % maxw != 0)
            for (int d = maxw - 1; d >= maxw / 2; --d)
                if (H % d == 0) { wpb = d; break; }
    }
    const int nbw = (R + TILE_Q - 1) / TILE_Q;
    if (weights) {
        // one query block per wavefront
        p.NS = NB;
        const long wunits = (long)B * NB * H;
        if (wunits > 0x3fffffffL) return fail(HSA_ERR_UNSUPPORTED, "problem too large for one launch");
        p.n_units = (int)wunits;
        if (dtype == HSA_BF16) {
            if (D == 32) return attn_tile_weights_launch_td<BF16, 32>(p, nbw, causal != 0, wpb, st);
            if (D == 64) return attn_tile_weights_launch_td<BF16, 64>(p, nbw, causal != 0, wpb, st);
            return attn_tile_weights_launch_td<BF16, 128>(p, nbw, causal != 0, wpb, st);
        }
        if (D == 32) return attn_tile_weights_launch_td<F16, 32>(p, nbw, causal != 0, wpb, st);
        if (D == 64) return attn_tile_weights_launch_td<F16, 64>(p, nbw, causal != 0, wpb, st);
        return attn_tile_weights_launch_td<F16, 128>(p, nbw, causal != 0, wpb, st);
    }
    if (lse) {
        if (weights) return fail(HSA_ERR_UNSUPPORTED, "weights and log-sum-exp outputs together are not built");
        if (dtype == HSA_BF16) {
            if (D == 32) return attn_tile_lse_launch_td<BF16, 32>(p, nbw, causal != 0, sb, wpb, st);
            if (D == 64) return attn_tile_lse_launch_td<BF16, 64>(p, nbw, causal != 0, sb, wpb, st);
            return attn_tile_lse_launch_td<BF16, 128>(p, nbw, causal != 0, sb, wpb, st);
        }
        if (D == 32) return attn_tile_lse_launch_td<F16, 32>(p, nbw, causal != 0, sb, wpb, st);
        if (D == 64) return attn_tile_lse_launch_td<F16, 64>(p, nbw, causal != 0, sb, wpb, st);
        return attn_tile_lse_launch_td<F16, 128>(p, nbw, causal != 0, sb, wpb, st);
    }
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
