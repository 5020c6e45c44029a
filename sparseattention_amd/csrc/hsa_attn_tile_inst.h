// Instantiates the tile kernels of one (element type, head_dim) pair; included by the
// hsa_attn_tile_<type>_d<D>.hip files so that they compile in parallel.
#pragma once
#include "hsa_attn_tile.h"

#include <hip/hip_ext.h>

namespace hsa {

template <typename T, int D, int NBW, bool CAUSAL, int SB>
static int tile_launch_one(const TileParams &p, int wpb, hipStream_t st) {
    constexpr int MAXW = tile_max_wpb<D, (CAUSAL ? NBW + 1 : 2 * NBW + 1)>();
    if (wpb > MAXW) wpb = MAXW;
    const int nwg = (p.n_units + wpb - 1) / wpb;
    const LaunchEvents ev = take_launch_events();
    if (ev.start && ev.stop)
        hipExtLaunchKernelGGL((attn_tile_kernel<T, D, NBW, CAUSAL, SB>), dim3(nwg), dim3(wpb * 64), 0, st, ev.start,
                              ev.stop, 0, p);
    else
        attn_tile_kernel<T, D, NBW, CAUSAL, SB><<<nwg, wpb * 64, 0, st>>>(p);
    return check_launch("attn_tile_kernel");
}

// strips of eight blocks: two runs of four (one or two blocks of neighbours, two with the causal mask)
template <typename T, int D, int NBW, bool CAUSAL, bool LSE, int RUNS>
static int tile_launch_runs(const TileParams &p, int wpb, hipStream_t st) {
    if constexpr (NBW >= 1 && NBW <= (CAUSAL ? 2 : 1)) {
        constexpr int MAXW = tile_max_wpb<D, (CAUSAL ? NBW + 1 : 2 * NBW + 1)>();
        if (wpb > MAXW) wpb = MAXW;
        const int nwg = (p.n_units + wpb - 1) / wpb;
        const LaunchEvents ev = take_launch_events();
        if (ev.start && ev.stop)
            hipExtLaunchKernelGGL((attn_tile_kernel<T, D, NBW, CAUSAL, 4, false, LSE, RUNS>), dim3(nwg), dim3(wpb * 64), 0,
                                  st, ev.start, ev.stop, 0, p);
        else
            attn_tile_kernel<T, D, NBW, CAUSAL, 4, false, LSE, RUNS><<<nwg, wpb * 64, 0, st>>>(p);
        return check_launch("attn_tile_kernel (runs)");
    } else {
        return fail(HSA_ERR_UNSUPPORTED, "strips of more than four blocks are not built for this window radius");
    }
}

// the variant that also writes the queries' log-sum-exp (window radius up to 16, or 32 with the
// causal mask)
template <typename T, int D, int NBW, bool CAUSAL>
static int tile_launch_lse(const TileParams &p, int sb, int wpb, hipStream_t st) {
    constexpr int MAXW = tile_max_wpb<D, (CAUSAL ? NBW + 1 : 2 * NBW + 1)>();
    if (wpb > MAXW) wpb = MAXW;
    const int nwg = (p.n_units + wpb - 1) / wpb;
    switch (sb) {
        case 1: attn_tile_kernel<T, D, NBW, CAUSAL, 1, false, true><<<nwg, wpb * 64, 0, st>>>(p); break;
        case 2: attn_tile_kernel<T, D, NBW, CAUSAL, 2, false, true><<<nwg, wpb * 64, 0, st>>>(p); break;
        case 4: attn_tile_kernel<T, D, NBW, CAUSAL, 4, false, true><<<nwg, wpb * 64, 0, st>>>(p); break;
        case 8: return tile_launch_runs<T, D, NBW, CAUSAL, true, 2>(p, wpb, st);
        default: return fail(HSA_ERR_UNSUPPORTED, "strip length %d not built", sb);
    }
    return check_launch("attn_tile_kernel (log-sum-exp)");
}

template <typename T, int D, int NBW, bool CAUSAL>
static int tile_launch_weights(const TileParams &p, int wpb, hipStream_t st) {
    constexpr int MAXW = tile_max_wpb<D, (CAUSAL ? NBW + 1 : 2 * NBW + 1)>();
    if (wpb > MAXW) wpb = MAXW;
    const int nwg = (p.n_units + wpb - 1) / wpb;
    attn_tile_kernel<T, D, NBW, CAUSAL, 1, true><<<nwg, wpb * 64, 0, st>>>(p);
    return check_launch("attn_tile_kernel (weights)");
}

template <typename T, int D, int NBW, bool CAUSAL>
static int tile_launch_sb(const TileParams &p, int sb, int wpb, hipStream_t st) {
    switch (sb) {
        case 1: return tile_launch_one<T, D, NBW, CAUSAL, 1>(p, wpb, st);
        case 2: return tile_launch_one<T, D, NBW, CAUSAL, 2>(p, wpb, st);
        case 4: return tile_launch_one<T, D, NBW, CAUSAL, 4>(p, wpb, st);
        case 8: return tile_launch_runs<T, D, NBW, CAUSAL, false, 2>(p, wpb, st);
    }
    return fail(HSA_ERR_UNSUPPORTED, "strip length %d not built", sb);
}

// seven or nine leaf blocks per query block (window radius 33..64 without the causal mask): one
// block per wavefront, one wavefront per SIMD (at 128 channels per head part of the operands
// lives in per-lane scratch memory)
template <typename T, int D, int NBW>
static int tile_launch_wide(const TileParams &p, int wpb, hipStream_t st) {
    return tile_launch_one<T, D, NBW, false, 1>(p, wpb, st);
}
// the same with the weights output
template <typename T, int D, int NBW>
static int tile_launch_wide_weights(const TileParams &p, int wpb, hipStream_t st) {
    return tile_launch_weights<T, D, NBW, false>(p, wpb, st);
}

#define HSA_TILE_INSTANTIATE(T, D)                                                              \
    template <>                                                                                 \
    int attn_tile_launch_td<T, D>(const TileParams &p, int nbw, bool causal, int sb, int wpb,  \
                                  hipStream_t st) {                                             \
        switch (nbw * 2 + (causal ? 1 : 0)) {                                                   \
            case 0: return tile_launch_sb<T, D, 0, false>(p, sb, wpb, st);                      \
            case 1: return tile_launch_sb<T, D, 0, true>(p, sb, wpb, st);                       \
            case 2: return tile_launch_sb<T, D, 1, false>(p, sb, wpb, st);                      \
            case 3: return tile_launch_sb<T, D, 1, true>(p, sb, wpb, st);                       \
            case 4: return tile_launch_sb<T, D, 2, false>(p, sb, wpb, st);                      \
            case 5: return tile_launch_sb<T, D, 2, true>(p, sb, wpb, st);                       \
            case 6: return tile_launch_wide<T, D, 3>(p, wpb, st);                               \
            case 8: return tile_launch_wide<T, D, 4>(p, wpb, st);                               \
            case 7: return tile_launch_sb<T, D, 3, true>(p, sb, wpb, st);                       \
            case 9: return tile_launch_sb<T, D, 4, true>(p, sb, wpb, st);                       \
        }                                                                                       \
        return fail(HSA_ERR_UNSUPPORTED, "window radius too large for the tile kernel");       \
    }                                                                                           \
    template <>                                                                                 \
    int attn_tile_lse_launch_td<T, D>(const TileParams &p, int nbw, bool causal, int sb,       \
                                      int wpb, hipStream_t st) {                                \
        switch (nbw * 2 + (causal ? 1 : 0)) {                                                   \
            case 0: return tile_launch_lse<T, D, 0, false>(p, sb, wpb, st);                     \
            case 1: return tile_launch_lse<T, D, 0, true>(p, sb, wpb, st);                      \
            case 2: return tile_launch_lse<T, D, 1, false>(p, sb, wpb, st);                     \
            case 3: return tile_launch_lse<T, D, 1, true>(p, sb, wpb, st);                      \
            case 5: return tile_launch_lse<T, D, 2, true>(p, sb, wpb, st);                      \
        }                                                                                       \
        return fail(HSA_ERR_UNSUPPORTED, "the log-sum-exp output is built for window radius up to 16, or 32 with the causal mask"); \
    }                                                                                           \
    template <>                                                                                 \
    int attn_tile_weights_launch_td<T, D>(const TileParams &p, int nbw, bool causal, int wpb,  \
                                          hipStream_t st) {                                     \
        switch (nbw * 2 + (causal ? 1 : 0)) {                                                   \
            case 0: return tile_launch_weights<T, D, 0, false>(p, wpb, st);                     \
            case 1: return tile_launch_weights<T, D, 0, true>(p, wpb, st);                      \
            case 2: return tile_launch_weights<T, D, 1, false>(p, wpb, st);                     \
            case 3: return tile_launch_weights<T, D, 1, true>(p, wpb, st);                      \
            case 4: return tile_launch_weights<T, D, 2, false>(p, wpb, st);                     \
            case 5: return tile_launch_weights<T, D, 2, true>(p, wpb, st);                      \
            case 6: return tile_launch_wide_weights<T, D, 3>(p, wpb, st);                       \
            case 8: return tile_launch_wide_weights<T, D, 4>(p, wpb, st);                       \
            case 7: return tile_launch_weights<T, D, 3, true>(p, wpb, st);                      \
            case 9: return tile_launch_weights<T, D, 4, true>(p, wpb, st);                      \
        }                                                                                       \
        return fail(HSA_ERR_UNSUPPORTED, "window radius too large for the tile kernel");       \
    }

}  // namespace hsa
