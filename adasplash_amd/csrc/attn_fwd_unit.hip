// One translation unit per (element type, head dim, instance) of attn_fwd_kernel.  The build compiles this file
// once per combination with -DADSP_T=<bf16_t|f16_t|float> -DADSP_TAG=<bf16|f16|f32> -DADSP_D=<head dim>
// -DADSP_MULTI=<0|1>, so that the instantiations compile in parallel and a change to one of them recompiles little.
#include "attn_launch.h"

#define ADSP_CAT_(a, b, c, d) launch_attn_fwd_##a##_d##b##_m##c
#define ADSP_CAT(a, b, c) ADSP_CAT_(a, b, c, )

namespace adsp {
int ADSP_CAT(ADSP_TAG, ADSP_D, ADSP_MULTI)(const AttnParams& p, int am, hipStream_t s) {
  return launch_attn_am<ADSP_T, ADSP_D, (ADSP_MULTI != 0)>(p, am, s);
}
}  // namespace adsp
