// Fused sparse entmax attention forward for gfx950 (one kernel: threshold solver + output).
//
// Work decomposition
//   workgroup = 256 threads = 4 waves, owns kBM = 128 consecutive query rows of one (batch, head);
//   wave w owns rows [32w, 32w+32); inside a wave, lane l holds query row (l & 31) and, of every
//   32-key block, the 16 keys {8g + 4(l >> 5) + r : g, r in 0..3} -- the C layout of the 32x32 MFMA when
//   the product is taken as S^T = K Q^T.  All per-row quantities (max, histogram, Halley sums, tau,
//   sum of p) are therefore lane-local accumulators that need one cross-lane add (lane ^ 32) per pass.
//   K tiles (64 keys) and V tiles are staged through LDS, double-buffered, shared by the four waves.
//
// Passes over the K tiles of a row block (every pass recomputes S^T with MFMA, scores never leave
// registers):
//   A  row max m                                          -> tau in [m - 1, m - n^(1-alpha)]
//   B  (alpha = 1.5 / 2) 8-bin histogram of z - (m - 1)   -> bracket [lo, lo + 1/8]; tile mask {z > m-1}
//   C  x niter: sums of u^c0, u^(c0-1), u^(c0-2)          -> Halley / Newton / bisection step; tile mask
//                                                           refined to {z > lo}
//   D  p = [z - tau]_+^c0, out += P V over masked tiles, divided by sum p at the end.
// The accumulator of the S^T MFMA is initialised with -tau (resp. -(m-1)), so z - tau costs no VALU op.
//
// The 16-bit path consumes V through a key-major copy (see vt_layout_kernel) so that the PV product
// out^T = V^T P^T can take P^T straight from the S^T accumulators without an LDS round trip.
#pragma once
#include "common.h"
#include "solver.h"
#include "attn_params.h"

namespace adsp {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));

template <typename T> struct is16 { static constexpr bool value = true; };
template <> struct is16<float> { static constexpr bool value = false; };

template <typename T> __device__ __forceinline__ f32x16 mfma_16bit(u32x4 a, u32x4 b, f32x16 c);
template <> __device__ __forceinline__ f32x16 mfma_16bit<bf16_t>(u32x4 a, u32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}
template <> __device__ __forceinline__ f32x16 mfma_16bit<f16_t>(u32x4 a, u32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
}

// LDS geometry of one K tile and one V tile.
template <typename T, int D> struct TileGeo {
  static constexpr bool k16 = is16<T>::value;
  static constexpr int kEB = k16 ? 2 : 4;
  static constexpr int kKPitch = D * kEB + 16;  // bytes per key row (+16 B pad against bank conflicts)
  static constexpr int kKTile = kBN * kKPitch;
  static constexpr int kVPitch = k16 ? (kBN * 2 + 16) : (D * 4 + 16);
  static constexpr int kVRows = k16 ? D : kBN;
  static constexpr int kVTile = kVRows * kVPitch;
  static constexpr int kMaskBytes = 2 * kMaskWords * 4;
  static constexpr int kNBuf = (2 * (kKTile + kVTile) + kMaskBytes <= 150 * 1024) ? 2 : 1;
  static constexpr int kLdsBytes = kNBuf * (kKTile + kVTile) + kMaskBytes;
  static constexpr int kKChunksPerRow = D * kEB / 16;
  static constexpr int kKChunks = kBN * kKChunksPerRow;
  static constexpr int kKPerThread = (kKChunks + kThreads - 1) / kThreads;
  static constexpr int kVChunksPerRow = k16 ? 8 : (D * 4 / 16);
  static constexpr int kVChunks = kVRows * kVChunksPerRow;
  static constexpr int kVPerThread = (kVChunks + kThreads - 1) / kThreads;
  static constexpr int kQRegs = k16 ? (D / 16) * 4 : D / 2;  // dwords of Q held per lane
  static constexpr int kDB = D >= 32 ? D / 32 : 1;           // 32-wide d blocks of the output
};

template <int AM> __device__ __forceinline__ float attn_prob(float d, float c0) {
  if constexpr (AM == ATT_2) return fmaxf(d, 0.f);
  if constexpr (AM == ATT_15) {
    float r = fmaxf(d, 0.f);
    return r * r;
  }
  return d > 0.f ? fast_exp2(fast_log2(d) * c0) : 0.f;
}

template <typename T, int D, int AM>
__global__ __launch_bounds__(kThreads) void attn_fwd_kernel(AttnParams p) {
  using G = TileGeo<T, D>;
  constexpr bool k16 = G::k16;
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char* kbuf0 = smem;
  unsigned char* vbuf0 = smem + G::kNBuf * G::kKTile;
  uint32_t* maskA = reinterpret_cast<uint32_t*>(smem + G::kNBuf * (G::kKTile + G::kVTile));
  uint32_t* maskB = maskA + kMaskWords;

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, lq = lane & 31, lh = lane >> 5;

  // ---- XCD-aware block -> (batch, kv head, row block, head in group) mapping -------------------------
  // Hardware block ids are dealt round-robin to the 8 XCDs; give each XCD a contiguous range of logical
  // ids so the row blocks and grouped heads that share one K/V head hit the same L2.  Inside a K/V head
  // the longest (last) row blocks of a causal problem go first.
  const int group = p.Hq / p.Hkv;
  const long long total = (long long)p.B * p.Hkv * p.n_mblk * group;
  const long long per_xcd = (total + 7) / 8;
  const long long logical = (long long)(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if ((blockIdx.x >> 3) >= per_xcd || logical >= total) return;
  const int hg = (int)(logical % group);
  const int mi = (int)((logical / group) % p.n_mblk);
  const int bkv = (int)(logical / ((long long)group * p.n_mblk));
  const int b = bkv / p.Hkv, kvh = bkv % p.Hkv;
  const int h = kvh * group + hg;
  const int mblk = p.n_mblk - 1 - mi;
  const int m0 = mblk * kBM;

  const int N = p.N;
  int L = N;
  if (p.varlen) {
    long long l = p.varlen_bits == 64 ? ((const long long*)p.varlen)[b] : (long long)((const int*)p.varlen)[b];
    L = (int)(l < 0 ? 0 : (l > N ? N : l));
  }

  const size_t qo_base = ((size_t)(b * p.Hq + h) * N) * D;  // elements
  const size_t kv_base = ((size_t)(b * p.Hkv + kvh) * N) * D;
  int32_t* bmask_out = p.bmask ? p.bmask + ((size_t)(b * p.Hq + h) * p.n_mblk + mblk) * p.mask_words : nullptr;

  const int qi = m0 + wave * 32 + lq;  // this lane's query row

  // Row block entirely inside the padding: zero output rows, empty mask.
  if (m0 >= L) {
    if (bmask_out && tid < p.mask_words) bmask_out[tid] = 0;
    constexpr int kRowDw = D * G::kEB / 4;
    uint32_t* o32 = reinterpret_cast<uint32_t*>(p.out) + (qo_base + (size_t)m0 * D) * G::kEB / 4;
    const int rows = (N - m0) < kBM ? (N - m0) : kBM;
    for (int i = tid; i < rows * kRowDw; i += kThreads) o32[i] = 0u;
    return;
  }

  const int row_hi = (m0 + kBM < L ? m0 + kBM : L);          // keys needed by the causal block: [0, row_hi)
  const int nt = p.causal ? (row_hi + kBN - 1) / kBN : (L + kBN - 1) / kBN;
  const int lim = p.causal ? (qi < L - 1 ? qi : L - 1) : L - 1;  // last valid key of this lane's row
  const int wave_row0 = m0 + wave * 32;

  // ---- Q fragments, pre-scaled by (alpha-1)/sqrt(D) and rounded back to the input type ----------------
  uint32_t qf[G::kQRegs];
  {
    const bool ok = qi < N;
    if constexpr (k16) {
      const uint16_t* qrow = reinterpret_cast<const uint16_t*>(p.q) + qo_base + (size_t)(ok ? qi : 0) * D;
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) {
        u32x4 raw = *reinterpret_cast<const u32x4*>(qrow + ks * 16 + 8 * lh);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float lo = unpack_lo<T>(raw[e]) * p.qscale, hi = unpack_hi<T>(raw[e]) * p.qscale;
          qf[ks * 4 + e] = ok ? pack2<T>(lo, hi) : 0u;
        }
      }
    } else {
      const float* qrow = reinterpret_cast<const float*>(p.q) + qo_base + (size_t)(ok ? qi : 0) * D;
#pragma unroll
      for (int g = 0; g < D / 8; ++g) {
        f32x4 raw = *reinterpret_cast<const f32x4*>(qrow + 8 * g + 4 * lh);
#pragma unroll
        for (int e = 0; e < 4; ++e) qf[g * 4 + e] = ok ? __builtin_bit_cast(uint32_t, raw[e] * p.qscale) : 0u;
      }
    }
  }

  // ---- tile staging ---------------------------------------------------------------------------------
  const unsigned char* kglob = reinterpret_cast<const unsigned char*>(p.k) + kv_base * G::kEB;
  const unsigned char* vglob =
      k16 ? reinterpret_cast<const unsigned char*>(p.vt) + ((size_t)(b * p.Hkv + kvh) * D) * p.Npad * 2
          : reinterpret_cast<const unsigned char*>(p.v) + kv_base * G::kEB;
  u32x4 kreg[G::kKPerThread];
  u32x4 vreg[G::kVPerThread];

  auto load_k = [&](int kt) {
#pragma unroll
    for (int i = 0; i < G::kKPerThread; ++i) {
      int c = tid + i * kThreads;
      int key = c / G::kKChunksPerRow, seg = c % G::kKChunksPerRow;
      int gk = kt * kBN + key;
      u32x4 z = {0u, 0u, 0u, 0u};
      kreg[i] = (c < G::kKChunks && gk < N)
                    ? *reinterpret_cast<const u32x4*>(kglob + ((size_t)gk * D) * G::kEB + seg * 16)
                    : z;
    }
  };
  auto store_k = [&](unsigned char* kb) {
#pragma unroll
    for (int i = 0; i < G::kKPerThread; ++i) {
      int c = tid + i * kThreads;
      int key = c / G::kKChunksPerRow, seg = c % G::kKChunksPerRow;
      if (c < G::kKChunks) *reinterpret_cast<u32x4*>(kb + key * G::kKPitch + seg * 16) = kreg[i];
    }
  };
  auto load_v = [&](int kt) {
#pragma unroll
    for (int i = 0; i < G::kVPerThread; ++i) {
      int c = tid + i * kThreads;
      int row = c / G::kVChunksPerRow, seg = c % G::kVChunksPerRow;
      u32x4 z = {0u, 0u, 0u, 0u};
      if constexpr (k16) {
        vreg[i] = (c < G::kVChunks)
                      ? *reinterpret_cast<const u32x4*>(vglob + ((size_t)row * p.Npad + (size_t)kt * kBN) * 2 + seg * 16)
                      : z;
      } else {
        int gk = kt * kBN + row;
        vreg[i] = (c < G::kVChunks && gk < N)
                      ? *reinterpret_cast<const u32x4*>(vglob + ((size_t)gk * D) * 4 + seg * 16)
                      : z;
      }
    }
  };
  auto store_v = [&](unsigned char* vb) {
#pragma unroll
    for (int i = 0; i < G::kVPerThread; ++i) {
      int c = tid + i * kThreads;
      int row = c / G::kVChunksPerRow, seg = c % G::kVChunksPerRow;
      if (c < G::kVChunks) *reinterpret_cast<u32x4*>(vb + row * G::kVPitch + seg * 16) = vreg[i];
    }
  };

  // Next tile index > cur allowed by `mask` (nullptr = every tile), or -1.
  auto next_tile = [&](const uint32_t* mask, int cur) -> int {
    int t = cur + 1;
    if (!mask) return t < nt ? t : -1;
    while (t < nt) {
      uint32_t w = mask[t >> 5] >> (t & 31);
      if (w) {
        t += __builtin_ctz(w);
        return t < nt ? t : -1;
      }
      t = (t | 31) + 1;
    }
    return -1;
  };

  // Runs body(kt, kbuf, vbuf) over the selected tiles with the next tile's global loads in flight.
  auto tile_loop = [&](const uint32_t* mask, bool with_v, auto&& body) {
    __syncthreads();  // previous pass is done with the LDS tiles and the masks are visible
    int cur = next_tile(mask, -1);
    if (cur >= 0) {
      load_k(cur);
      if (with_v) load_v(cur);
      store_k(kbuf0);
      if (with_v) store_v(vbuf0);
    }
    __syncthreads();
    int it = 0;
    while (cur >= 0) {
      const int nxt = next_tile(mask, cur);
      if (nxt >= 0) {
        load_k(nxt);
        if (with_v) load_v(nxt);
      }
      const int bi = G::kNBuf == 2 ? (it & 1) : 0;
      body(cur, kbuf0 + bi * G::kKTile, vbuf0 + bi * G::kVTile);
      if constexpr (G::kNBuf == 1) __syncthreads();
      if (nxt >= 0) {
        const int bn = G::kNBuf == 2 ? ((it + 1) & 1) : 0;
        store_k(kbuf0 + bn * G::kKTile);
        if (with_v) store_v(vbuf0 + bn * G::kVTile);
      }
      __syncthreads();
      cur = nxt;
      ++it;
    }
  };

  // S^T block: 32 keys (kb-th half of the tile) x 32 query rows, accumulator pre-loaded with `init`.
  auto scores = [&](const unsigned char* kb_lds, int kb, float init) -> f32x16 {
    f32x16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = init;
    const unsigned char* krow = kb_lds + (kb * 32 + lq) * G::kKPitch;
    if constexpr (k16) {
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) {
        u32x4 a = *reinterpret_cast<const u32x4*>(krow + (ks * 16 + 8 * lh) * 2);
        u32x4 bq = {qf[ks * 4], qf[ks * 4 + 1], qf[ks * 4 + 2], qf[ks * 4 + 3]};
        acc = mfma_16bit<T>(a, bq, acc);
      }
    } else {
#pragma unroll
      for (int g = 0; g < D / 8; ++g) {
        f32x4 a = *reinterpret_cast<const f32x4*>(krow + (8 * g + 4 * lh) * 4);
#pragma unroll
        for (int e = 0; e < 4; ++e)
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], __builtin_bit_cast(float, qf[g * 4 + e]), acc, 0, 0, 0);
      }
    }
    return acc;
  };
  // -inf on keys past the row's last valid key (causal diagonal, sequence tail).
  auto mask_block = [&](f32x16& acc, int kt, int kb) {
    const int jb = kt * kBN + kb * 32 + 4 * lh;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = (jb + 8 * (i >> 2) + (i & 3) <= lim) ? acc[i] : -INFINITY;
  };
  // Calls f(acc, kb) for the (up to two) 32-key blocks of tile kt that this wave's rows can see.
  auto for_blocks = [&](int kt, const unsigned char* kb_lds, float init, auto&& f) {
    if (p.causal && kt * kBN > wave_row0 + 31) return;
    const bool need_mask = (kt * kBN + kBN - 1 > L - 1) || (p.causal && kt * kBN + kBN - 1 > wave_row0);
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      if (p.causal && kt * kBN + kb * 32 > wave_row0 + 31) continue;
      f32x16 acc = scores(kb_lds, kb, init);
      if (need_mask) mask_block(acc, kt, kb);
      f(acc, kb);
    }
  };

  for (int i = tid; i < 2 * kMaskWords; i += kThreads) maskA[i] = 0u;

  // ---- pass A: row max -------------------------------------------------------------------------------
  float m = -INFINITY;
  tile_loop(nullptr, false, [&](int kt, const unsigned char* kb_lds, const unsigned char*) {
    for_blocks(kt, kb_lds, 0.f, [&](const f32x16& acc, int) {
#pragma unroll
      for (int i = 0; i < 16; ++i) m = fmaxf(m, acc[i]);
    });
  });
  m = fmaxf(m, __shfl_xor(m, 32, 64));

  // Tightest a-priori bracket: tau in [m - 1, m - n^(1 - alpha)], n = number of valid keys of the row
  // (all n equal to the max is the extreme case; adasplash/adasplash_block_mask.py:167-175).
  const float n_keys = (float)(lim + 1);
  const float hi_cap = m - fast_exp2((1.f - p.alpha) * fast_log2(n_keys));
  Bracket br;
  br.lo = m - 1.f;
  br.hi = hi_cap;
  br.t = 0.5f * (br.lo + br.hi);

  uint32_t* mask_cur = nullptr;  // mask consumed by the next pass
  uint32_t* mask_new = maskA;    // mask produced by the running pass

  // ---- pass B: histogram bracket (alpha = 1.5 or 2) ----------------------------------------------------
  if (AM != ATT_GEN && p.use_hist) {
    const float t_shift = m - 1.f;
    float cnt[kAttnBins];
#pragma unroll
    for (int bI = 0; bI < kAttnBins; ++bI) cnt[bI] = 0.f;
    unsigned long long packed = 0ull;  // eight 8-bit counters, flushed before any can overflow
    int since_flush = 0;
    auto flush = [&]() {
#pragma unroll
      for (int bI = 0; bI < kAttnBins; ++bI) cnt[bI] += (float)((uint32_t)(packed >> (8 * bI)) & 0xffu);
      packed = 0ull;
      since_flush = 0;
    };
    tile_loop(nullptr, false, [&](int kt, const unsigned char* kb_lds, const unsigned char*) {
      bool any = false;
      for_blocks(kt, kb_lds, -t_shift, [&](const f32x16& acc, int) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const float d = acc[i];  // z - (m - 1), in (-inf, 1]
          const int bin = (int)fminf(fmaxf(d * (float)kAttnBins, 0.f), (float)(kAttnBins - 1));
          packed += d >= 0.f ? (1ull << (8 * bin)) : 0ull;
          any |= d >= 0.f;
        }
      });
      if (++since_flush == 7) flush();  // <= 32 increments per tile and lane: 7 tiles stay below 255
      if (__builtin_amdgcn_ballot_w64(any) != 0ull && lane == 0) atomicOr(&mask_new[kt >> 5], 1u << (kt & 31));
    });
    flush();
#pragma unroll
    for (int bI = 0; bI < kAttnBins; ++bI) cnt[bI] += __shfl_xor(cnt[bI], 32, 64);
    float lo = (AM == ATT_15) ? hist_bracket_alpha15<kAttnBins>(cnt, t_shift) : hist_bracket_alpha2<kAttnBins>(cnt, t_shift);
    br.lo = fmaxf(lo, t_shift);
    br.hi = fminf(br.lo + 1.f / (float)kAttnBins, hi_cap);
    br.hi = fmaxf(br.hi, br.lo);
    br.t = 0.5f * (br.lo + br.hi);
    mask_cur = mask_new;
    mask_new = maskB;
  }

  // ---- pass C: niter safeguarded Halley / Newton steps -------------------------------------------------
  {
    float t_prev = br.t, f_prev = 0.f;
    for (int it = 0; it < p.niter; ++it) {
      const float t = br.t;
      const float dl = br.lo - t;  // z > lo  <=>  (z - t) > dl
      float a0 = 0.f, a1 = 0.f, a2 = 0.f;
      tile_loop(mask_cur, false, [&](int kt, const unsigned char* kb_lds, const unsigned char*) {
        float dmax = -INFINITY;
        for_blocks(kt, kb_lds, -t, [&](const f32x16& acc, int) {
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const float d = acc[i];
            dmax = fmaxf(dmax, d);
            if constexpr (AM == ATT_15) {
              const float u = fmaxf(d, 0.f);
              a0 = fmaf(u, u, a0);
              a1 += u;
              a2 += d > 0.f ? 1.f : 0.f;
            } else if constexpr (AM == ATT_2) {
              a0 += fmaxf(d, 0.f);
              a1 += d > 0.f ? 1.f : 0.f;
            } else {
              if (d > 0.f) {
                const float e0 = fast_exp2(fast_log2(d) * p.c0);
                const float r = fast_rcp(d);
                const float e1 = e0 * r;
                a0 += e0;
                a1 += e1;
                a2 += e1 * r;
              }
            }
          }
        });
        if (__builtin_amdgcn_ballot_w64(dmax > dl) != 0ull && lane == 0) atomicOr(&mask_new[kt >> 5], 1u << (kt & 31));
      });
      a0 += __shfl_xor(a0, 32, 64);
      a1 += __shfl_xor(a1, 32, 64);
      a2 += __shfl_xor(a2, 32, 64);
      hybrid_step(br, a0, a1, a2, p.c0, AM != ATT_2 && p.alpha <= 1.5f, p.alpha <= 2.0f, it > 0, t_prev, f_prev);
      // the mask just written becomes the one to read; the other array is cleared for the next pass
      __syncthreads();
      uint32_t* old = mask_cur;
      mask_cur = mask_new;
      mask_new = (mask_cur == maskA) ? maskB : maskA;
      (void)old;
      for (int i = tid; i < kMaskWords; i += kThreads) mask_new[i] = 0u;
    }
  }
  const float tau = br.t;

  // ---- pass D: out = sum_j p_j v_j / sum_j p_j over the masked tiles ------------------------------------
  f32x16 o[G::kDB];
#pragma unroll
  for (int db = 0; db < G::kDB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
  float psum = 0.f;
  tile_loop(mask_cur, true, [&](int kt, const unsigned char* kb_lds, const unsigned char* vb_lds) {
    for_blocks(kt, kb_lds, -tau, [&](const f32x16& acc, int kb) {
      float pv[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        pv[i] = attn_prob<AM>(acc[i], p.c0);
        psum += pv[i];
      }
      if constexpr (k16) {
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          u32x4 bp = {pack2<T>(pv[8 * s], pv[8 * s + 1]), pack2<T>(pv[8 * s + 2], pv[8 * s + 3]),
                      pack2<T>(pv[8 * s + 4], pv[8 * s + 5]), pack2<T>(pv[8 * s + 6], pv[8 * s + 7])};
#pragma unroll
          for (int db = 0; db < G::kDB; ++db) {
            const int drow = db * 32 + lq;
            u32x4 a = {0u, 0u, 0u, 0u};
            if (D >= 32 || drow < D)
              a = *reinterpret_cast<const u32x4*>(vb_lds + drow * G::kVPitch + (kb * 32 + 16 * s + 8 * lh) * 2);
            o[db] = mfma_16bit<T>(a, bp, o[db]);
          }
        }
      } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = kb * 32 + 8 * (i >> 2) + 4 * lh + (i & 3);
#pragma unroll
          for (int db = 0; db < G::kDB; ++db) {
            const int dcol = db * 32 + lq;
            float a = 0.f;
            if (D >= 32 || dcol < D) a = *reinterpret_cast<const float*>(vb_lds + key * G::kVPitch + dcol * 4);
            o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, pv[i], o[db], 0, 0, 0);
          }
        }
      }
    });
  });
  psum += __shfl_xor(psum, 32, 64);
  const float inv = psum > 0.f ? 1.f / psum : 0.f;

  // ---- epilogue -------------------------------------------------------------------------------------
  if (qi < N) {
    const bool live = qi < L;
    if (live && lh == 0 && p.taus) p.taus[(size_t)(b * p.Hq + h) * N + qi] = tau;
    unsigned char* orow = reinterpret_cast<unsigned char*>(p.out) + (qo_base + (size_t)qi * D) * G::kEB;
#pragma unroll
    for (int db = 0; db < G::kDB; ++db) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int d0 = db * 32 + 8 * g + 4 * lh;
        if (D >= 32 || d0 < D) {
          float x0 = live ? o[db][4 * g] * inv : 0.f, x1 = live ? o[db][4 * g + 1] * inv : 0.f;
          float x2 = live ? o[db][4 * g + 2] * inv : 0.f, x3 = live ? o[db][4 * g + 3] * inv : 0.f;
          if constexpr (k16) {
            typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
            u32x2 w = {pack2<T>(x0, x1), pack2<T>(x2, x3)};
            *reinterpret_cast<u32x2*>(orow + d0 * 2) = w;
          } else {
            f32x4 w = {x0, x1, x2, x3};
            *reinterpret_cast<f32x4*>(orow + d0 * 4) = w;
          }
        }
      }
    }
  }
  __syncthreads();
  if (bmask_out && tid < p.mask_words) {
    uint32_t w;
    if (mask_cur) {
      w = tid < kMaskWords ? mask_cur[tid] : 0u;
    } else {  // no mask was built (niter = 0 without histogram): every tile of the domain was visited
      int first = tid * 32;
      int cntb = nt - first;
      w = cntb >= 32 ? 0xffffffffu : (cntb > 0 ? ((1u << cntb) - 1u) : 0u);
    }
    bmask_out[tid] = (int32_t)w;
  }
}

}  // namespace adsp
