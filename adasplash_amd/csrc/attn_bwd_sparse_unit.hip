// One translation unit per (16-bit element type, head dim) of attn_bwd_dq_sparse_kernel and attn_bwd_dkdv_sparse_kernel; compiled by the build once
// per combination with -DADSP_T=<bf16_t|f16_t> -DADSP_TAG=<bf16|f16> -DADSP_D=<64|128>.
#include "attn_bwd_sparse_kernel.h"

#define ADSP_CAT_(a, b) launch_attn_bwd_sparse_##a##_d##b
#define ADSP_CAT(a, b) ADSP_CAT_(a, b)

namespace adsp {
int ADSP_CAT(ADSP_TAG, ADSP_D)(const AttnBwdParams& p, int am, int keys, int max_slots, hipStream_t s) {
  return launch_attn_bwd_sparse<ADSP_T, ADSP_D>(p, am, keys, max_slots, s);
}
}  // namespace adsp
