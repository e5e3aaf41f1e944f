// bf16 instantiations of the backward attention kernel.
#include "attn_bwd_impl.h"

namespace slapo {
int attn_bwd_mfma_bf16(const AttnArgs& a, hipStream_t st) { return bwd::dispatch<bf16_t>(a, st); }
}  // namespace slapo
