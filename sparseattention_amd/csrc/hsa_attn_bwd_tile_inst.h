// Instantiates the tile backward kernels of one (element type, head_dim) pair.
#pragma once
#include "hsa_attn_bwd_tile.h"

namespace hsa {

// p.n_units counts 16-row blocks; a wavefront of the query pass takes sbq of them, one of the key
// pass sbk (4 when the sequence has a multiple of four blocks and the variant's operands fit the
// registers, else 1)
template <typename T, int D, int NBW, bool CAUSAL, int SBQ, int SBK>
static int bwd_tile_launch_sb(const BwdTileParams &p, hipStream_t st) {
    BwdTileParams q = p;
    q.n_units = p.n_units / SBQ;
    attn_bwd_tile_query_kernel<T, D, NBW, CAUSAL, SBQ><<<(q.n_units + BWD_WPB - 1) / BWD_WPB, BWD_WPB * 64, 0, st>>>(q);
    int rc = check_launch("attn_bwd_tile_query_kernel");
    if (rc != HSA_OK) return rc;
    q.n_units = p.n_units / SBK;
    attn_bwd_tile_key_kernel<T, D, NBW, CAUSAL, SBK><<<(q.n_units + BWD_WPB - 1) / BWD_WPB, BWD_WPB * 64, 0, st>>>(q);
    return check_launch("attn_bwd_tile_key_kernel");
}

template <typename T, int D, int NBW, bool CAUSAL>
static int bwd_tile_launch_one(const BwdTileParams &p, int sbq, int sbk, hipStream_t st) {
    constexpr int MQ = BWD_QUERY_STRIP, MK = bwd_key_strip(D, NBW, CAUSAL);
    if (sbq == 1 && sbk == 1) return bwd_tile_launch_sb<T, D, NBW, CAUSAL, 1, 1>(p, st);
    if (sbq == MQ && sbk == 1) return bwd_tile_launch_sb<T, D, NBW, CAUSAL, MQ, 1>(p, st);
    if constexpr (MK > 1) {
        if (sbq == MQ && sbk == MK) return bwd_tile_launch_sb<T, D, NBW, CAUSAL, MQ, MK>(p, st);
    }
    return fail(HSA_ERR_INVALID, "internal: strip lengths %d / %d not built for this variant", sbq, sbk);
}

template <typename T, int D>
int attn_bwd_tile_launch_td(const BwdTileParams &p, int nbw, bool causal, int sbq, int sbk, hipStream_t st);

#define HSA_BWD_TILE_INSTANTIATE(T, D)                                                           \
    template <>                                                                                  \
    int attn_bwd_tile_launch_td<T, D>(const BwdTileParams &p, int nbw, bool causal, int sbq,     \
                                      int sbk, hipStream_t st) {                                 \
        switch (nbw * 2 + (causal ? 1 : 0)) {                                                    \
            case 0: return bwd_tile_launch_one<T, D, 0, false>(p, sbq, sbk, st);                 \
            case 1: return bwd_tile_launch_one<T, D, 0, true>(p, sbq, sbk, st);                  \
            case 2: return bwd_tile_launch_one<T, D, 1, false>(p, sbq, sbk, st);                 \
            case 3: return bwd_tile_launch_one<T, D, 1, true>(p, sbq, sbk, st);                  \
            case 4: return bwd_tile_launch_one<T, D, 2, false>(p, sbq, sbk, st);                 \
            case 5: return bwd_tile_launch_one<T, D, 2, true>(p, sbq, sbk, st);                  \
        }                                                                                        \
        return fail(HSA_ERR_UNSUPPORTED, "window radius too large for the tile backward");       \
    }

}  // namespace hsa
