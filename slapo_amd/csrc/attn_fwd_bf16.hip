// bf16 instantiations of the forward attention kernel.
#include "attn_fwd_impl.h"
#include "attn_fwd_lean_impl.h"

namespace slapo {
int attn_fwd_mfma_bf16(const AttnArgs& a, hipStream_t st) {
    // head_dim <= 64: the register-lean kernel (three workgroups per CU); above: the pipelined one
    if (a.d <= 64) return fwd_lean::dispatch_flags<bf16_t, 64>(a, st);
    return fwd::dispatch<bf16_t>(a, st);
}
}  // namespace slapo
