// attn_fwd_kernel instantiations for element type bf16_t.
#include "attn_launch.h"
namespace adsp {
int launch_attn_bf16(const AttnParams& p, int D, int am, hipStream_t s) { return launch_attn<bf16_t>(p, D, am, s); }
}  // namespace adsp
