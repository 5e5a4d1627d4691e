// attn_fwd_kernel instantiations for element type f16_t: no solver step, or one behind the histogram.
#include "attn_launch.h"
namespace adsp {
int launch_attn_multi_f16(const AttnParams& p, int D, int am, hipStream_t s);
int launch_attn_f16(const AttnParams& p, int D, int am, hipStream_t s) {
  // one step without the histogram is the block-mask variant's: made for sparse supports, which the lists serve
  const bool multi = p.niter >= 2 || (p.niter == 1 && !p.use_hist);
  return multi ? launch_attn_multi_f16(p, D, am, s) : launch_attn<f16_t, false>(p, D, am, s);
}
}  // namespace adsp
