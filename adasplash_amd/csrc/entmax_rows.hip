// Row-wise alpha-entmax forward / backward for gfx950.
//
// Forward: y[r, j] = [(alpha-1) x[r, j] - tau_r]_+^(1/(alpha-1)).  The kernel is HBM-bound: a row is read
// from HBM exactly once (16-byte loads, the whole row then lives in registers), every solver pass
// (max, histogram bracket, refinement) runs on the register copy with wave64 butterflies (plus one LDS
// exchange when a row spans four waves), and the result is written once.  Rows that do not fit in
// registers, or whose base is not 16-byte aligned, take a streaming variant that re-reads the row
// (from L2) per pass.  Semantics follow adasplash/triton_entmax_v2.py:363-536.
#include "common.h"
#include "solver.h"
#include "../../include/adasplash_hip.h"

namespace adsp {

constexpr int kRowBins = 4;  // histogram bins of the standalone rows kernel (triton_entmax_v2.py:386)

enum AlphaMode { AM_15 = 0, AM_2 = 1, AM_GEN = 2 };

struct RowsParams {
  const void* x;
  void* y;
  long long rows, cols;
  float scale;  // alpha - 1
  float c0;     // 1 / (alpha - 1)
  int n_iter;
  int use_hist;
  int allow_halley, allow_newton;
};

// ---- reductions across the TPR threads that share a row ---------------------------------------------
template <int TPR> __device__ __forceinline__ float row_max(float v, float* sm) {
  if constexpr (TPR == 16) return group16_max(v);
  v = wave_max(v);
  if constexpr (TPR > 64) {
    __syncthreads();
    if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = v;
    __syncthreads();
    v = sm[0];
#pragma unroll
    for (int w = 1; w < TPR / 64; ++w) v = fmaxf(v, sm[w]);
  }
  return v;
}
template <int TPR, int K> __device__ __forceinline__ void row_sum(float (&v)[K], float* sm) {
  if constexpr (TPR == 16) {
#pragma unroll
    for (int k = 0; k < K; ++k) v[k] = group16_sum(v[k]);
    return;
  }
#pragma unroll
  for (int k = 0; k < K; ++k) v[k] = wave_sum(v[k]);
  if constexpr (TPR > 64) {
    __syncthreads();
    if ((threadIdx.x & 63) == 0) {
#pragma unroll
      for (int k = 0; k < K; ++k) sm[(threadIdx.x >> 6) * K + k] = v[k];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < K; ++k) {
      float s = sm[k];
#pragma unroll
      for (int w = 1; w < TPR / 64; ++w) s += sm[w * K + k];
      v[k] = s;
    }
  }
}

template <int AM> __device__ __forceinline__ float prob(float u, float c0) {
  // u = z - tau (may be <= 0)
  if constexpr (AM == AM_2) return fmaxf(u, 0.f);
  if constexpr (AM == AM_15) {
    float r = fmaxf(u, 0.f);
    return r * r;
  }
  return u > 0.f ? fast_exp2(fast_log2(u) * c0) : 0.f;
}

template <int AM> __device__ __forceinline__ void accum_stats(float u, float c0, float (&a)[3]) {
  if constexpr (AM == AM_2) {
    a[0] += fmaxf(u, 0.f);
    a[1] += u > 0.f ? 1.f : 0.f;
  } else if constexpr (AM == AM_15) {
    float r = fmaxf(u, 0.f);
    a[0] = fmaf(r, r, a[0]);
    a[1] += r;
    a[2] += u > 0.f ? 1.f : 0.f;
  } else {
    if (u > 0.f) {
      float uc = fmaxf(u, 1e-6f);  // same clamp as the reference's masked power (triton_entmax_v2.py:35-39)
      float lg = fast_log2(uc);
      a[0] += fast_exp2(lg * c0);
      a[1] += fast_exp2(lg * (c0 - 1.f));
      a[2] += fast_exp2(lg * (c0 - 2.f));
    }
  }
}

// The whole per-row solve, generic over how the row's scaled elements z are visited.
// `Row::for_each(f)` calls f(z) for every element this thread owns (invalid slots yield -inf).
template <int AM, int TPR, typename Row>
__device__ __forceinline__ float solve_row(const Row& row, const RowsParams& p, float* sm) {
  float m = -INFINITY;
  row.for_each([&](float z) { m = fmaxf(m, z); });
  m = row_max<TPR>(m, sm);

  Bracket br;
  if (AM != AM_GEN && p.use_hist) {
    const float t_shift = m - 1.f;
    float cnt[kRowBins];
#pragma unroll
    for (int b = 0; b < kRowBins; ++b) cnt[b] = 0.f;
    row.for_each([&](float z) {
      float pr = (z - t_shift) * (float)kRowBins;
      if (pr >= 0.f) {
#pragma unroll
        for (int b = 0; b < kRowBins; ++b) {
          bool in = (b == kRowBins - 1) ? (pr >= (float)b) : (pr >= (float)b && pr < (float)(b + 1));
          cnt[b] += in ? 1.f : 0.f;
        }
      }
    });
    row_sum<TPR, kRowBins>(cnt, sm);
    br.lo = (AM == AM_15) ? hist_bracket_alpha15<kRowBins>(cnt, t_shift, 1.f / kRowBins, true, 1.f)
                          : hist_bracket_alpha2<kRowBins>(cnt, t_shift, 1.f / kRowBins, true, 1.f);
    br.lo = fmaxf(br.lo, t_shift);
    br.hi = fminf(br.lo + 1.f / (float)kRowBins, m);
    br.t = hist_start_point<kRowBins>(cnt, t_shift, br.lo, br.hi);
  } else {
    br.lo = m - 1.f;
    br.hi = m;
    br.t = 0.5f * (br.lo + br.hi);
  }

  // n_iter refinement steps as requested, then keep stepping (the row is in registers, so a step costs
  // no memory traffic) until |f| is at rounding level or the extra-step cap is reached.
  float t_prev = br.t, f_prev = 0.f;
  const int kExtra = 12;
  for (int it = 0; it < p.n_iter + kExtra; ++it) {
    float a[3] = {0.f, 0.f, 0.f};
    const float t = br.t;
    row.for_each([&](float z) { accum_stats<AM>(z - t, p.c0, a); });
    row_sum<TPR, 3>(a, sm);
    if (it >= p.n_iter && fabsf(a[0] - 1.f) <= 2e-6f) break;
    hybrid_step(br, a[0], a[1], a[2], p.c0, p.allow_halley, p.allow_newton, it > 0, t_prev, f_prev);
    // at large |tau| the spacing of floats keeps |f| above any fixed bound (alpha = 2, inputs of size 16:
    // f moves in steps of 2e-6 per support entry); a step that no longer moves tau ends the search as well
    if (it >= p.n_iter && fabsf(br.t - t) <= 2.4e-7f * fabsf(t)) break;
  }
  return br.t;
}

// ---- streaming rows (any length / alignment): one 256-thread block per row, scalar accesses --------
template <typename T> __device__ __forceinline__ float load_elem(const void* base, size_t i);
template <> __device__ __forceinline__ float load_elem<float>(const void* b, size_t i) { return ((const float*)b)[i]; }
template <> __device__ __forceinline__ float load_elem<bf16_t>(const void* b, size_t i) {
  return bf16_bits_to_float(((const uint16_t*)b)[i]);
}
template <> __device__ __forceinline__ float load_elem<f16_t>(const void* b, size_t i) {
  return f16_bits_to_float(((const uint16_t*)b)[i]);
}
template <typename T> __device__ __forceinline__ void store_elem(void* base, size_t i, float v);
template <> __device__ __forceinline__ void store_elem<float>(void* b, size_t i, float v) { ((float*)b)[i] = v; }
template <> __device__ __forceinline__ void store_elem<bf16_t>(void* b, size_t i, float v) {
  ((uint16_t*)b)[i] = (uint16_t)float_to_bf16_bits(v);
}
template <> __device__ __forceinline__ void store_elem<f16_t>(void* b, size_t i, float v) {
  ((uint16_t*)b)[i] = (uint16_t)float_to_f16_bits(v);
}

template <typename T, int TPR> struct StreamRow {
  const void* x;
  size_t base;
  long long cols;
  float scale;
  int t_in_row;
  template <typename F> __device__ __forceinline__ void for_each(F f) const {
    for (long long j = t_in_row; j < cols; j += TPR) f(load_elem<T>(x, base + j) * scale);
  }
};

// ---- register-resident rows ------------------------------------------------------------------------
// The row stays in registers as loaded (raw 16-byte chunks).  Only entries with z >= max - 1 can be in the
// support (tau >= max - 1 for every alpha), so after the max pass those candidates are compacted into a
// short LDS list and the whole threshold solve runs on that list inside one wave; the other entries are
// touched twice more at most: one compare against the candidate threshold and one against tau, both
// done per 16-byte chunk on the chunk's maximum.  Rows with more candidates than the list holds fall
// back to solving on the full register copy.
constexpr int kCandPerLane = 16;
constexpr int kCandCap = 64 * kCandPerLane;  // list capacity per row

template <typename T> __device__ __forceinline__ float chunk_elem(u32x4 raw, int e) {
  // the element is copied to a scalar first: bit-casting a vector-element expression directly makes this
  // compiler read element 0 whatever the index
  if constexpr (elem_traits<T>::kVec == 4) {
    const uint32_t w = raw[e];
    return __builtin_bit_cast(float, w);
  } else {
    const uint32_t w = raw[e >> 1];
    return (e & 1) ? unpack_hi<T>(w) : unpack_lo<T>(w);
  }
}

template <int K> struct ListRow {
  float z[K];
  template <typename F> __device__ __forceinline__ void for_each(F f) const {
#pragma unroll
    for (int i = 0; i < K; ++i) f(z[i]);
  }
  // thread t of the `stride` threads that solve the list takes entries t, t + stride, ...
  __device__ __forceinline__ void load(const float* list, int n, int t, int stride = 64) {
#pragma unroll
    for (int i = 0; i < K; ++i) {
      const int idx = i * stride + t;
      z[i] = idx < n ? list[idx] : -INFINITY;
    }
  }
};

// Register budget: rows of up to 16 chunks per lane are compiled for four waves per SIMD (128 registers),
// except fp16 whose unpacking needs more live values; longer rows get two waves (256 registers).
template <typename T, int NCHUNK> constexpr int rows_min_waves() {
  return (NCHUNK <= 8 || (NCHUNK <= 16 && (elem_traits<T>::kVec == 4 || elem_traits<T>::kIsBf16))) ? 4 : 2;
}

template <typename T, int AM, int NCHUNK, int TPR>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(rows_min_waves<T, NCHUNK>()))) void entmax_rows_reg_kernel(RowsParams p) {
  constexpr int kVec = elem_traits<T>::kVec;
  constexpr int kRowsPerBlock = 256 / TPR;
  __shared__ float sm[32];
  // Short rows (16 threads each, four to a wave): the row's own 16 lanes solve its list.
  constexpr int kCap = TPR == 16 ? (NCHUNK * TPR * kVec < 512 ? NCHUNK * TPR * kVec : 512) : kCandCap;
  __shared__ float cand[kRowsPerBlock][kCap];
  __shared__ int cand_n[kRowsPerBlock];
  const int tid = threadIdx.x;
  const int t_in_row = tid % TPR, r_in_blk = tid / TPR, lane = tid & 63;
  long long row = (long long)blockIdx.x * kRowsPerBlock + r_in_blk;
  // TPR == 256: one row per block, every thread is active.  TPR == 64: a wave owns a row, and a wave
  // past the last row simply leaves (no block-level barrier is used in that configuration).
  if (row >= p.rows) return;

  const long long nvec = p.cols / kVec;
  const u32x4* xrow = reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(p.x) +
                                                     (size_t)row * p.cols * elem_traits<T>::kBytes);
  u32x4* yrow = reinterpret_cast<u32x4*>(reinterpret_cast<char*>(p.y) + (size_t)row * p.cols * elem_traits<T>::kBytes);

  struct {
    u32x4 raw[NCHUNK];
    bool valid[NCHUNK];
  } r;
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    long long vi = (long long)c * TPR + t_in_row;
    r.valid[c] = vi < nvec;
    // a lane past the row end re-reads the row's last chunk and ignores it: no branch between the loads
    r.raw[c] = __builtin_nontemporal_load(xrow + (r.valid[c] ? vi : nvec - 1));
  }
  if (t_in_row == 0) cand_n[r_in_blk] = 0;

  // pass 1: per-chunk and row maxima, in the input's own units
  float cmax[NCHUNK];
  float xm = -INFINITY;
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    float cm = -INFINITY;
    if constexpr (kVec == 4) {
#pragma unroll
      for (int e = 0; e < 4; ++e) cm = fmaxf(cm, chunk_elem<T>(r.raw[c], e));
    } else if constexpr (sizeof(T) == 2 && elem_traits<T>::kIsBf16) {
      // bf16: the upper element of a dword is compared as the dword itself (the lower element only adds
      // mantissa bits below one bf16 ulp), so a chunk maximum may exceed the true one by less than an
      // ulp -- harmless for the two "can this chunk matter" tests, and removed from the row maximum below
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t w = r.raw[c][e];
        cm = fmaxf(cm, fmaxf(__builtin_bit_cast(float, w), __builtin_bit_cast(float, w << 16)));
      }
    } else {
#pragma unroll
      for (int e = 0; e < kVec; ++e) cm = fmaxf(cm, chunk_elem<T>(r.raw[c], e));
    }
    cmax[c] = r.valid[c] ? cm : -INFINITY;
    xm = fmaxf(xm, cmax[c]);
  }
  xm = row_max<TPR>(xm, sm);  // (TPR == 256: its barriers also publish cand_n = 0)
  if constexpr (elem_traits<T>::kIsBf16) xm = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, xm) & 0xffff0000u);

  // pass 2: compact the candidates z >= max - 1 into the row's LDS list
  const float x_thr = xm - p.c0;  // (alpha-1) x >= (alpha-1) xm - 1
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    if (cmax[c] >= x_thr) {
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        const float x = chunk_elem<T>(r.raw[c], e);
        if (x >= x_thr) {
          const int idx = atomicAdd(&cand_n[r_in_blk], 1);
          if (idx < kCap) cand[r_in_blk][idx] = x * p.scale;
        }
      }
    }
  }
  if constexpr (TPR > 64) __syncthreads();
  const int n_cand = cand_n[r_in_blk];

  float tau;
  if constexpr (TPR == 16) {
    if (n_cand <= 16) {
      ListRow<1> lr;
      lr.load(cand[r_in_blk], n_cand, t_in_row, 16);
      tau = solve_row<AM, 16>(lr, p, sm);
    } else if (n_cand <= kCap) {
      ListRow<kCap / 16> lr;
      lr.load(cand[r_in_blk], n_cand, t_in_row, 16);
      tau = solve_row<AM, 16>(lr, p, sm);
    } else {
      StreamRow<T, 16> sr{p.x, (size_t)row * p.cols, p.cols, p.scale, t_in_row};
      tau = solve_row<AM, 16>(sr, p, sm);
    }
  } else if (n_cand <= 64) {
    // every wave of the row solves the same short list redundantly: wave-level reductions only.  The
    // usual case (a peaked row) has at most one candidate per lane.
    ListRow<1> lr;
    lr.load(cand[r_in_blk], n_cand, lane);
    tau = solve_row<AM, 64>(lr, p, sm);
  } else if (n_cand <= kCandCap) {
    ListRow<kCandPerLane> lr;
    lr.load(cand[r_in_blk], n_cand, lane);
    tau = solve_row<AM, 64>(lr, p, sm);
  } else {
    // too many candidates for the list: solve on the whole row, re-read (from L2) pass by pass
    StreamRow<T, TPR> sr{p.x, (size_t)row * p.cols, p.cols, p.scale, t_in_row};
    tau = solve_row<AM, TPR>(sr, p, sm);
  }

  // pass 3: outputs; a chunk whose maximum is not above tau is all zeros
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    if (r.valid[c]) {
      long long vi = (long long)c * TPR + t_in_row;
      u32x4 o = {0u, 0u, 0u, 0u};
      if (cmax[c] * p.scale > tau) {
        if constexpr (kVec == 4) {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            o[e] = __builtin_bit_cast(uint32_t, prob<AM>(chunk_elem<T>(r.raw[c], e) * p.scale - tau, p.c0));
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            o[e] = pack2<T>(prob<AM>(chunk_elem<T>(r.raw[c], 2 * e) * p.scale - tau, p.c0),
                            prob<AM>(chunk_elem<T>(r.raw[c], 2 * e + 1) * p.scale - tau, p.c0));
        }
      }
      __builtin_nontemporal_store(o, yrow + vi);
    }
  }
}

template <typename T, int AM> __global__ __launch_bounds__(256) void entmax_rows_stream_kernel(RowsParams p) {
  __shared__ float sm[32];
  for (long long row = blockIdx.x; row < p.rows; row += gridDim.x) {
    StreamRow<T, 256> r{p.x, (size_t)row * p.cols, p.cols, p.scale, (int)threadIdx.x};
    const float tau = solve_row<AM, 256>(r, p, sm);
    for (long long j = threadIdx.x; j < p.cols; j += 256) {
      float z = load_elem<T>(p.x, r.base + j) * p.scale;
      store_elem<T>(p.y, r.base + j, prob<AM>(z - tau, p.c0));
    }
  }
}

// ---- backward: dx = u*dy - (sum u*dy / sum u) * u, u = y^(2-alpha) on y > 0 (triton_entmax_v2.py:541-617)
template <typename T, int AM> __global__ __launch_bounds__(256) void entmax_rows_bwd_kernel(
    const void* y, const void* dy, void* dx, long long rows, long long cols, float cf) {
  __shared__ float sm[32];
  for (long long row = blockIdx.x; row < rows; row += gridDim.x) {
    const size_t base = (size_t)row * cols;
    float s[2] = {0.f, 0.f};
    for (long long j = threadIdx.x; j < cols; j += 256) {
      float yy = load_elem<T>(y, base + j);
      float g = load_elem<T>(dy, base + j);
      float u = 0.f;
      if (yy > 0.f) u = (AM == AM_2) ? 1.f : (AM == AM_15 ? sqrtf(yy) : fast_exp2(fast_log2(fmaxf(yy, 1e-6f)) * cf));
      s[0] = fmaf(u, g, s[0]);
      s[1] += u;
    }
    row_sum<256, 2>(s, sm);
    const float q = s[1] > 0.f ? s[0] / s[1] : 0.f;
    for (long long j = threadIdx.x; j < cols; j += 256) {
      float yy = load_elem<T>(y, base + j);
      float g = load_elem<T>(dy, base + j);
      float u = 0.f;
      if (yy > 0.f) u = (AM == AM_2) ? 1.f : (AM == AM_15 ? sqrtf(yy) : fast_exp2(fast_log2(fmaxf(yy, 1e-6f)) * cf));
      store_elem<T>(dx, base + j, u * g - q * u);
    }
    __syncthreads();
  }
}

// Register-resident backward: y and dy are read from HBM once (16-byte non-temporal loads), dx is written
// once.  The support of an entmax row is small, so most 16-byte chunks of y are all zeros: their dy is never
// loaded and their dx is stored as zeros without arithmetic.
template <int AM> __device__ __forceinline__ float bwd_u(float yy, float cf) {
  if (!(yy > 0.f)) return 0.f;
  if constexpr (AM == AM_2) return 1.f;
  if constexpr (AM == AM_15) return __builtin_amdgcn_sqrtf(yy);  // one instruction, 1 ulp
  return fast_exp2(fast_log2(fmaxf(yy, 1e-6f)) * cf);
}

template <typename T, int AM, int NCHUNK, int TPR>
__global__ __launch_bounds__(256) void entmax_rows_bwd_reg_kernel(const void* y, const void* dy, void* dx,
                                                                     long long rows, long long cols, float cf) {
  constexpr int kVec = elem_traits<T>::kVec;
  constexpr int kRowsPerBlock = 256 / TPR;
  __shared__ float sm[32];
  const int tid = threadIdx.x;
  const int t_in_row = tid % TPR, r_in_blk = tid / TPR;
  const long long row = (long long)blockIdx.x * kRowsPerBlock + r_in_blk;
  if (row >= rows) return;  // TPR == 256: the whole block; TPR == 64: a wave, and no block barrier is used
  const long long nvec = cols / kVec;
  const size_t row_bytes = (size_t)row * cols * elem_traits<T>::kBytes;
  const u32x4* yrow = reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(y) + row_bytes);
  const u32x4* grow = reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(dy) + row_bytes);
  u32x4* xrow = reinterpret_cast<u32x4*>(reinterpret_cast<char*>(dx) + row_bytes);

  u32x4 yr[NCHUNK], gr[NCHUNK];
  bool valid[NCHUNK], live[NCHUNK];
  // every lane loads (a lane past the row end re-reads the row's last chunk and ignores it): no branches, so
  // all the loads of a row are in flight together
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    const long long vi = (long long)c * TPR + t_in_row;
    valid[c] = vi < nvec;
    yr[c] = __builtin_nontemporal_load(yrow + (valid[c] ? vi : nvec - 1));
  }
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) live[c] = valid[c] && (yr[c][0] | yr[c][1] | yr[c][2] | yr[c][3]) != 0u;
  // dy matters only where y has a non-zero element: the other lanes re-read the row's first chunk (one cached
  // line per wave instead of a kilobyte of HBM traffic) so that these loads need no branch either
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) gr[c] = __builtin_nontemporal_load(grow + (live[c] ? (long long)c * TPR + t_in_row : 0ll));
  float s[2] = {0.f, 0.f};
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    if (live[c]) {
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        const float u = bwd_u<AM>(chunk_elem<T>(yr[c], e), cf);
        s[0] = fmaf(u, chunk_elem<T>(gr[c], e), s[0]);
        s[1] += u;
      }
    }
  }
  row_sum<TPR, 2>(s, sm);
  const float q = s[1] > 0.f ? s[0] / s[1] : 0.f;
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    if (valid[c]) {
      u32x4 o = {0u, 0u, 0u, 0u};
      if (live[c]) {
        if constexpr (kVec == 4) {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            o[e] = __builtin_bit_cast(uint32_t, bwd_u<AM>(chunk_elem<T>(yr[c], e), cf) * (chunk_elem<T>(gr[c], e) - q));
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            o[e] = pack2<T>(bwd_u<AM>(chunk_elem<T>(yr[c], 2 * e), cf) * (chunk_elem<T>(gr[c], 2 * e) - q),
                            bwd_u<AM>(chunk_elem<T>(yr[c], 2 * e + 1), cf) * (chunk_elem<T>(gr[c], 2 * e + 1) - q));
        }
      }
      __builtin_nontemporal_store(o, xrow + (long long)c * TPR + t_in_row);
    }
  }
}

// ---- host dispatch ---------------------------------------------------------------------------------
template <typename T, int AM, int NCHUNK, int TPR> static void launch_reg(const RowsParams& p, hipStream_t s) {
  constexpr int rpb = 256 / TPR;
  long long blocks = (p.rows + rpb - 1) / rpb;
  hipLaunchKernelGGL((entmax_rows_reg_kernel<T, AM, NCHUNK, TPR>), dim3((unsigned)blocks), dim3(256), 0, s, p);
}

template <typename T, int AM> static void launch_fwd(const RowsParams& p, bool aligned, hipStream_t s) {
  constexpr int kVec = elem_traits<T>::kVec;
  const long long nvec = p.cols / kVec;
  const bool can_reg = aligned && (p.cols % kVec == 0) && p.rows < (1ll << 31);
  if (can_reg) {
    const long long c64 = (nvec + 63) / 64, c256 = (nvec + 255) / 256;
    // A wave per row (no block barriers) while the row fits in eight 16-byte chunks per lane; four waves per
    // row beyond that, where more loads in flight per row pay more than the barriers cost (measured on
    // 2^27-element problems: bf16 4096 columns 74 % of HBM peak with a wave per row against 42 %, 8192
    // columns 66 % against 74-77 %).
    const long long c16 = (nvec + 15) / 16;
    constexpr long long kShortRowChunks = 8;
    // Short rows: 16 threads per row, four rows to a wave, so that the per-row solve is shared out.
    if (c16 <= kShortRowChunks) {
      if (c16 <= 1) return launch_reg<T, AM, 1, 16>(p, s);
      if (c16 <= 2) return launch_reg<T, AM, 2, 16>(p, s);
      if (c16 <= 4) return launch_reg<T, AM, 4, 16>(p, s);
      if (c16 <= 8) return launch_reg<T, AM, 8, 16>(p, s);
    }
    const int tpr = c64 <= 8 ? 64 : 256;
    if (tpr == 64) {
      if (c64 <= 1) return launch_reg<T, AM, 1, 64>(p, s);
      if (c64 <= 2) return launch_reg<T, AM, 2, 64>(p, s);
      if (c64 <= 4) return launch_reg<T, AM, 4, 64>(p, s);
      if (c64 <= 8) return launch_reg<T, AM, 8, 64>(p, s);
      if (c64 <= 16) return launch_reg<T, AM, 16, 64>(p, s);
      if (c64 <= 32) return launch_reg<T, AM, 32, 64>(p, s);
    } else {
      if (c256 <= 1) return launch_reg<T, AM, 1, 256>(p, s);
      if (c256 <= 2) return launch_reg<T, AM, 2, 256>(p, s);
      if (c256 <= 4) return launch_reg<T, AM, 4, 256>(p, s);
      if (c256 <= 8) return launch_reg<T, AM, 8, 256>(p, s);
      if (c256 <= 16) return launch_reg<T, AM, 16, 256>(p, s);
      if (c256 <= 32) return launch_reg<T, AM, 32, 256>(p, s);
    }
  }
  long long blocks = p.rows < 65536 ? p.rows : 65536;
  hipLaunchKernelGGL((entmax_rows_stream_kernel<T, AM>), dim3((unsigned)blocks), dim3(256), 0, s, p);
}

template <typename T> static void launch_fwd_am(const RowsParams& p, int am, bool aligned, hipStream_t s) {
  if (am == AM_15) return launch_fwd<T, AM_15>(p, aligned, s);
  if (am == AM_2) return launch_fwd<T, AM_2>(p, aligned, s);
  return launch_fwd<T, AM_GEN>(p, aligned, s);
}

template <typename T, int AM, int NCHUNK, int TPR>
static void launch_bwd_reg(const void* y, const void* dy, void* dx, long long rows, long long cols, float cf, hipStream_t s) {
  constexpr int rpb = 256 / TPR;
  const long long blocks = (rows + rpb - 1) / rpb;
  hipLaunchKernelGGL((entmax_rows_bwd_reg_kernel<T, AM, NCHUNK, TPR>), dim3((unsigned)blocks), dim3(256), 0, s, y, dy, dx,
                     rows, cols, cf);
}

// true if a register-resident kernel took the row shape
template <typename T, int AM>
static bool launch_bwd_fast(const void* y, const void* dy, void* dx, long long rows, long long cols, float cf, hipStream_t s) {
  constexpr int kVec = elem_traits<T>::kVec;
  const bool aligned = (((uintptr_t)y | (uintptr_t)dy | (uintptr_t)dx) & 15) == 0;
  if (!aligned || cols % kVec != 0 || rows >= (1ll << 31)) return false;
  const long long nvec = cols / kVec;
  const long long c64 = (nvec + 63) / 64, c256 = (nvec + 255) / 256;
  const long long c16 = (nvec + 15) / 16;  // short rows: 16 threads per row, four rows to a wave
  if (c16 <= 1) return launch_bwd_reg<T, AM, 1, 16>(y, dy, dx, rows, cols, cf, s), true;
  if (c16 <= 2) return launch_bwd_reg<T, AM, 2, 16>(y, dy, dx, rows, cols, cf, s), true;
  if (c16 <= 4) return launch_bwd_reg<T, AM, 4, 16>(y, dy, dx, rows, cols, cf, s), true;
  if (c16 <= 8) return launch_bwd_reg<T, AM, 8, 16>(y, dy, dx, rows, cols, cf, s), true;
  if (c64 <= 1) return launch_bwd_reg<T, AM, 1, 64>(y, dy, dx, rows, cols, cf, s), true;
  if (c64 <= 2) return launch_bwd_reg<T, AM, 2, 64>(y, dy, dx, rows, cols, cf, s), true;
  if (c64 <= 4) return launch_bwd_reg<T, AM, 4, 64>(y, dy, dx, rows, cols, cf, s), true;
  if (c256 <= 2) return launch_bwd_reg<T, AM, 2, 256>(y, dy, dx, rows, cols, cf, s), true;
  if (c256 <= 4) return launch_bwd_reg<T, AM, 4, 256>(y, dy, dx, rows, cols, cf, s), true;
  if (c256 <= 8) return launch_bwd_reg<T, AM, 8, 256>(y, dy, dx, rows, cols, cf, s), true;
  if (c256 <= 16) return launch_bwd_reg<T, AM, 16, 256>(y, dy, dx, rows, cols, cf, s), true;
  return false;
}

template <typename T> static void launch_bwd_am(const void* y, const void* dy, void* dx, long long rows, long long cols,
                                                int am, float cf, hipStream_t s) {
  if (am == AM_15 && launch_bwd_fast<T, AM_15>(y, dy, dx, rows, cols, cf, s)) return;
  if (am == AM_2 && launch_bwd_fast<T, AM_2>(y, dy, dx, rows, cols, cf, s)) return;
  if (am == AM_GEN && launch_bwd_fast<T, AM_GEN>(y, dy, dx, rows, cols, cf, s)) return;
  long long blocks = rows < 65536 ? rows : 65536;
  if (am == AM_15)
    hipLaunchKernelGGL((entmax_rows_bwd_kernel<T, AM_15>), dim3((unsigned)blocks), dim3(256), 0, s, y, dy, dx, rows, cols, cf);
  else if (am == AM_2)
    hipLaunchKernelGGL((entmax_rows_bwd_kernel<T, AM_2>), dim3((unsigned)blocks), dim3(256), 0, s, y, dy, dx, rows, cols, cf);
  else
    hipLaunchKernelGGL((entmax_rows_bwd_kernel<T, AM_GEN>), dim3((unsigned)blocks), dim3(256), 0, s, y, dy, dx, rows, cols, cf);
}

static int alpha_mode(double alpha) { return alpha == 1.5 ? AM_15 : (alpha == 2.0 ? AM_2 : AM_GEN); }

}  // namespace adsp

extern "C" int adsp_entmax_rows_fwd(const void* x, void* y, int64_t rows, int64_t cols, int dtype, double alpha,
                                    int n_iter, int use_histogram, int fast_math, void* stream) {
  using namespace adsp;
  (void)fast_math;
  if (rows < 0 || cols < 0) return ADSP_ERR_SHAPE;
  if (rows == 0 || cols == 0) return ADSP_OK;
  if (!x || !y) return ADSP_ERR_NULL;
  if (!(alpha > 1.0) || n_iter < 0) return ADSP_ERR_UNSUPPORTED;
  if (dtype != ADSP_F32 && dtype != ADSP_BF16 && dtype != ADSP_F16) return ADSP_ERR_DTYPE;
  RowsParams p;
  p.x = x;
  p.y = y;
  p.rows = rows;
  p.cols = cols;
  p.scale = (float)(alpha - 1.0);
  p.c0 = (float)(1.0 / (alpha - 1.0));
  p.n_iter = n_iter;
  p.use_hist = use_histogram ? 1 : 0;
  p.allow_halley = alpha <= 1.5;
  p.allow_newton = alpha <= 2.0;
  const int am = alpha_mode(alpha);
  const bool aligned = (((uintptr_t)x | (uintptr_t)y) & 15) == 0;
  hipStream_t s = (hipStream_t)stream;
  (void)hipGetLastError();
  if (dtype == ADSP_F32) launch_fwd_am<float>(p, am, aligned, s);
  else if (dtype == ADSP_BF16) launch_fwd_am<bf16_t>(p, am, aligned, s);
  else launch_fwd_am<f16_t>(p, am, aligned, s);
  return hipGetLastError() == hipSuccess ? ADSP_OK : ADSP_ERR_LAUNCH;
}

extern "C" int adsp_entmax_rows_bwd(const void* y, const void* dy, void* dx, int64_t rows, int64_t cols, int dtype,
                                    double alpha, void* stream) {
  using namespace adsp;
  if (rows < 0 || cols < 0) return ADSP_ERR_SHAPE;
  if (rows == 0 || cols == 0) return ADSP_OK;
  if (!y || !dy || !dx) return ADSP_ERR_NULL;
  if (!(alpha > 1.0)) return ADSP_ERR_UNSUPPORTED;
  const int am = alpha_mode(alpha);
  const float cf = (float)(2.0 - alpha);
  hipStream_t s = (hipStream_t)stream;
  (void)hipGetLastError();
  if (dtype == ADSP_F32) launch_bwd_am<float>(y, dy, dx, rows, cols, am, cf, s);
  else if (dtype == ADSP_BF16) launch_bwd_am<bf16_t>(y, dy, dx, rows, cols, am, cf, s);
  else if (dtype == ADSP_F16) launch_bwd_am<f16_t>(y, dy, dx, rows, cols, am, cf, s);
  else return ADSP_ERR_DTYPE;
  return hipGetLastError() == hipSuccess ? ADSP_OK : ADSP_ERR_LAUNCH;
}
