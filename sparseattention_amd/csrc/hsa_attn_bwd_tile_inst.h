// Instantiates the tile backward kernels of one (element type, head_dim) pair.
#pragma once
#include "hsa_attn_bwd_tile.h"

namespace hsa {

// p.n_units counts 16-row blocks; a wavefront takes SB of them
template <typename T, int D, int NBW, bool CAUSAL, int SB>
static int bwd_tile_launch_sb(const BwdTileParams &p, hipStream_t st) {
    BwdTileParams q = p;
    q.n_units = p.n_units / SB;
    q.red_lg_sb = SB == BWD_STRIP ? 2 : 0;
    const int nwg = (q.n_units + BWD_WPB - 1) / BWD_WPB;
    attn_bwd_tile_query_kernel<T, D, NBW, CAUSAL, SB><<<nwg, BWD_WPB * 64, 0, st>>>(q);
    int rc = check_launch("attn_bwd_tile_query_kernel");
    if (rc != HSA_OK) return rc;
    // same strip length for the key blocks (shorter strips re-read more query rows: 54 / 55 us
    // with two / one block against 52; eight blocks change nothing)
    attn_bwd_tile_key_kernel<T, D, NBW, CAUSAL, SB><<<nwg + q.red_wgs, BWD_WPB * 64, 0, st>>>(q);
    return check_launch("attn_bwd_tile_key_kernel");
}

template <typename T, int D, int NBW, bool CAUSAL>
static int bwd_tile_launch_one(const BwdTileParams &p, int sb, hipStream_t st) {
    if (sb == BWD_STRIP) return bwd_tile_launch_sb<T, D, NBW, CAUSAL, BWD_STRIP>(p, st);
    if (sb != 1) return fail(HSA_ERR_INVALID, "internal: strip length %d not built", sb);
    return bwd_tile_launch_sb<T, D, NBW, CAUSAL, 1>(p, st);
}

// Windows of 33..64 neighbours to either side without the causal mask (seven or nine leaf blocks
// per query block): head sizes up to 64 hold that many blocks in registers, one wavefront per SIMD;
// at 128 channels only one block per wavefront is built (the caller passes sb = 1), and the key
// pass keeps part of its operands in per-lane scratch memory.
template <typename T, int D, int NBW>
static int bwd_tile_launch_wide(const BwdTileParams &p, int sb, hipStream_t st) {
    if constexpr (D <= 64) return bwd_tile_launch_one<T, D, NBW, false>(p, sb, st);
    else {
        if (sb != 1) return fail(HSA_ERR_INVALID, "internal: strip length %d not built at this radius and head size", sb);
        return bwd_tile_launch_sb<T, D, NBW, false, 1>(p, st);
    }
}

template <typename T, int D>
int attn_bwd_tile_launch_td(const BwdTileParams &p, int nbw, bool causal, int sb, hipStream_t st);

#define HSA_BWD_TILE_INSTANTIATE(T, D)                                                           \
    template <>                                                                                  \
    int attn_bwd_tile_launch_td<T, D>(const BwdTileParams &p, int nbw, bool causal, int sb,      \
                                      hipStream_t st) {                                          \
        switch (nbw * 2 + (causal ? 1 : 0)) {                                                    \
            case 0: return bwd_tile_launch_one<T, D, 0, false>(p, sb, st);                       \
            case 1: return bwd_tile_launch_one<T, D, 0, true>(p, sb, st);                        \
            case 2: return bwd_tile_launch_one<T, D, 1, false>(p, sb, st);                       \
            case 3: return bwd_tile_launch_one<T, D, 1, true>(p, sb, st);                        \
            case 4: return bwd_tile_launch_one<T, D, 2, false>(p, sb, st);                       \
            case 5: return bwd_tile_launch_one<T, D, 2, true>(p, sb, st);                        \
            case 6: return bwd_tile_launch_wide<T, D, 3>(p, sb, st);                             \
            case 7: return bwd_tile_launch_one<T, D, 3, true>(p, sb, st);                        \
            case 8: return bwd_tile_launch_wide<T, D, 4>(p, sb, st);                             \
            case 9: return bwd_tile_launch_one<T, D, 4, true>(p, sb, st);                        \
        }                                                                                        \
        return fail(HSA_ERR_UNSUPPORTED, "window radius too large for the tile backward");       \
    }

}  // namespace hsa
