#include "hsa_attn_bwd_tile_inst.h"
namespace hsa {
HSA_BWD_TILE_INSTANTIATE(BF16, 32)
}  // namespace hsa
