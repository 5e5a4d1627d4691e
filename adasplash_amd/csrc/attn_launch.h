// Host-side launch of attn_fwd_kernel for one (element type, head dim, instance) over the alpha modes; kMulti is the
// instance with candidate lists and block bits.  Each combination is a translation unit of its own (attn_fwd_unit.hip).
#pragma once
#include "attn_kernel.h"

namespace adsp {

template <typename T, int D, int AM, bool kMulti> static int launch_attn_one(const AttnParams& p, hipStream_t s) {
  using G = TileGeo<T, D>;
  auto kern = attn_fwd_kernel<T, D, AM, kMulti>;
  const long long group = p.Hq / p.Hkv;
  const long long n_mblk = (p.N + G::kBM - 1) / G::kBM;
  const long long total = (long long)p.B * p.Hkv * n_mblk * group;
  const long long per_xcd = (total + 7) / 8;
  // dynamic LDS: the tile masks, and in the instance with the candidate lists, up to 128K keys, the
  // per-wave block bits as well (beyond that they would cost occupancy)
  AttnParams q = p;
  q.fine_masks = (kMulti && p.mask_words <= 64) ? 1 : 0;
  const size_t words = (size_t)(q.fine_masks ? 4 + 4 * G::kNW : 4) * p.mask_words + G::kPoolTail;  // + the candidate lists' bookkeeping
  hipLaunchKernelGGL(kern, dim3((unsigned)(per_xcd * 8)), dim3(G::kThreads), words * sizeof(uint32_t), s, q);
  return 0;
}

template <typename T, int D, bool kMulti> static int launch_attn_am(const AttnParams& p, int am, hipStream_t s) {
  if (am == ATT_15) return launch_attn_one<T, D, ATT_15, kMulti>(p, s);
  if (am == ATT_2) return launch_attn_one<T, D, ATT_2, kMulti>(p, s);
  return launch_attn_one<T, D, ATT_GEN, kMulti>(p, s);
}

}  // namespace adsp
