// attn_bwd_dq_kernel / attn_bwd_dkdv_kernel instantiations for element type float.
#include "attn_bwd_kernel.h"
namespace adsp {
int launch_attn_bwd_f32(const AttnBwdParams& p, int D, int am, hipStream_t s) { return launch_attn_bwd<float>(p, D, am, s); }
}  // namespace adsp
