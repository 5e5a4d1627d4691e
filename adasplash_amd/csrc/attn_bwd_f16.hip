// attn_bwd_dq_kernel / attn_bwd_dkdv_kernel instantiations for element type f16_t.
#include "attn_bwd_kernel.h"
namespace adsp {
int launch_attn_bwd_f16(const AttnBwdParams& p, int D, int am, hipStream_t s) { return launch_attn_bwd<f16_t>(p, D, am, s); }
}  // namespace adsp
