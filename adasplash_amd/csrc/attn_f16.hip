// attn_fwd_kernel instantiations for element type f16_t.
#include "attn_launch.h"
namespace adsp {
int launch_attn_f16(const AttnParams& p, int D, int am, hipStream_t s) { return launch_attn<f16_t>(p, D, am, s); }
}  // namespace adsp
