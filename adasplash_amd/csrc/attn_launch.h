// Host-side dispatch of attn_fwd_kernel over (head dim, alpha mode) for one element type.
#pragma once
#include "attn_kernel.h"

namespace adsp {

template <typename T, int D, int AM> static int launch_attn_one(const AttnParams& p, hipStream_t s) {
  using G = TileGeo<T, D>;
  auto kern = attn_fwd_kernel<T, D, AM>;
  const long long group = p.Hq / p.Hkv;
  const long long n_mblk = (p.N + G::kBM - 1) / G::kBM;
  const long long total = (long long)p.B * p.Hkv * n_mblk * group;
  const long long per_xcd = (total + 7) / 8;
  hipLaunchKernelGGL(kern, dim3((unsigned)(per_xcd * 8)), dim3(G::kThreads), (size_t)4 * p.mask_words * sizeof(uint32_t), s, p);  // dynamic LDS: the tile masks
  return 0;
}

template <typename T, int D> static int launch_attn_am(const AttnParams& p, int am, hipStream_t s) {
  if (am == ATT_15) return launch_attn_one<T, D, ATT_15>(p, s);
  if (am == ATT_2) return launch_attn_one<T, D, ATT_2>(p, s);
  return launch_attn_one<T, D, ATT_GEN>(p, s);
}

template <typename T> static int launch_attn(const AttnParams& p, int D, int am, hipStream_t s) {
  switch (D) {
    case 16: return launch_attn_am<T, 16>(p, am, s);
    case 32: return launch_attn_am<T, 32>(p, am, s);
    case 64: return launch_attn_am<T, 64>(p, am, s);
    case 128: return launch_attn_am<T, 128>(p, am, s);
    case 256: return launch_attn_am<T, 256>(p, am, s);
  }
  return 2;
}

}  // namespace adsp
