#include "hsa_attn_bwd_fused.h"
namespace hsa {
HSA_BWD_FUSED_INSTANTIATE(F16, 128)
}  // namespace hsa
