// f16 instantiation of the dQ backward kernel (one translation unit per element type keeps the
// builds parallel).
#include "attn_bwd_dq_impl.h"

namespace slapo {
int attn_bwd_dq_mfma_f16(const AttnArgs& a, hipStream_t st) { return bwd_dq::dispatch<f16_t>(a, st); }
}  // namespace slapo
