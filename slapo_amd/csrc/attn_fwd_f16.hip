// fp16 instantiations of the forward attention kernel.
#include "attn_fwd_impl.h"

namespace slapo {
int attn_fwd_mfma_f16(const AttnArgs& a, hipStream_t st) { return fwd::dispatch<f16_t>(a, st); }
}  // namespace slapo
