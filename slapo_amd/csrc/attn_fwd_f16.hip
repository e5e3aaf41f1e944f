// fp16 instantiations of the forward attention kernel.
#include "attn_fwd_impl.h"
#include "attn_fwd_lean_impl.h"

namespace slapo {
int attn_fwd_mfma_f16(const AttnArgs& a, hipStream_t st) {
    // head_dim <= 64: the register-lean kernel (three workgroups per CU); above: the pipelined one
    if (a.d <= 64) return fwd_lean::dispatch_flags<f16_t, 64>(a, st);
    return fwd::dispatch<f16_t>(a, st);
}
}  // namespace slapo
