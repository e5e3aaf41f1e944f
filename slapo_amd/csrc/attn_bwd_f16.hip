// fp16 instantiations of the backward attention kernel.
#include "attn_bwd_impl.h"

namespace slapo {
int attn_bwd_mfma_f16(const AttnArgs& a, hipStream_t st) { return bwd::dispatch<f16_t>(a, st); }
}  // namespace slapo
