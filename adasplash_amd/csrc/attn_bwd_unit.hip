// One translation unit per (element type, head dim) of attn_bwd_dq_kernel / attn_bwd_dkdv_kernel; compiled by the
// build once per combination with -DADSP_T=<bf16_t|f16_t|float> -DADSP_TAG=<bf16|f16|f32> -DADSP_D=<head dim>.
#include "attn_bwd_kernel.h"

#define ADSP_CAT_(a, b) launch_attn_bwd_##a##_d##b
#define ADSP_CAT(a, b) ADSP_CAT_(a, b)

namespace adsp {
int ADSP_CAT(ADSP_TAG, ADSP_D)(const AttnBwdParams& p, int am, int which, hipStream_t s) { return launch_attn_bwd_d<ADSP_T, ADSP_D>(p, am, which, s); }
}  // namespace adsp
