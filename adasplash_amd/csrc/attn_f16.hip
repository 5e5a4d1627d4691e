// attn_fwd_kernel instantiations for element type f16_t: no or one solver step.
#include "attn_launch.h"
namespace adsp {
int launch_attn_multi_f16(const AttnParams& p, int D, int am, hipStream_t s);
int launch_attn_f16(const AttnParams& p, int D, int am, hipStream_t s) {
  return p.niter >= 2 ? launch_attn_multi_f16(p, D, am, s) : launch_attn<f16_t, false>(p, D, am, s);
}
}  // namespace adsp
