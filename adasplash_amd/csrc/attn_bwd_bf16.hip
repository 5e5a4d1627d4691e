// attn_bwd_dq_kernel / attn_bwd_dkdv_kernel instantiations for element type bf16_t.
#include "attn_bwd_kernel.h"
namespace adsp {
int launch_attn_bwd_bf16(const AttnBwdParams& p, int D, int am, hipStream_t s) { return launch_attn_bwd<bf16_t>(p, D, am, s); }
}  // namespace adsp
