#include "hsa_attn_tile_inst.h"
namespace hsa {
HSA_TILE_INSTANTIATE(F16, 64)
}  // namespace hsa
