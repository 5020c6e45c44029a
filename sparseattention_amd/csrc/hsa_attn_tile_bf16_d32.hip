#include "hsa_attn_tile_inst.h"
namespace hsa {
HSA_TILE_INSTANTIATE(BF16, 32)
}  // namespace hsa
