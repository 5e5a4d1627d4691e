// attn_fwd_kernel instantiations for element type float: two and more solver steps, or one without the histogram.
#include "attn_launch.h"
namespace adsp {
int launch_attn_multi_f32(const AttnParams& p, int D, int am, hipStream_t s) { return launch_attn<float, true>(p, D, am, s); }
}  // namespace adsp
