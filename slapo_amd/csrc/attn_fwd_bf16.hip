// bf16 instantiations of the forward attention kernel.
#include "attn_fwd_impl.h"

namespace slapo {
int attn_fwd_mfma_bf16(const AttnArgs& a, hipStream_t st) { return fwd::dispatch<bf16_t>(a, st); }
}  // namespace slapo
