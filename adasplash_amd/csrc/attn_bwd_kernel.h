// Backward of the sparse entmax attention for gfx950: dQ kernel and dK/dV kernel.
//
// With x_ij = q_i.k_j / sqrt(D), z = (alpha-1) x, p_ij = [z_ij - tau_i]_+^(1/(alpha-1)) and u = p^(2-alpha),
// the entmax Jacobian is diag(u) - u u^T / sum(u), hence for dP_ij = dO_i . v_j
//   delta_i = sum_j u_ij dP_ij / sum_j u_ij,   dX_ij = u_ij (dP_ij - delta_i),
//   dQ_i = sum_j dX_ij k_j / sqrt(D),  dK_j = sum_i dX_ij q_i / sqrt(D),  dV_j = sum_i p_ij dO_i
// (adasplash/adasplash_v2.py:839-1234 for alpha = 1.5, adasplash/adasplash_block_mask.py:493-919 for any alpha).
// The forward divides its output by sum_j p_ij, so dV uses p_ij / sum_j p_ij as well.
//
// Both kernels recompute the scores with MFMA in the forward's layout: the product is taken as
// (LDS tile rows) x (register fragments of the lane's own row), so a lane owns one query row in the dQ
// kernel and one key row in the dK/dV kernel, and the other index runs over its 16 accumulator registers.
//   dQ kernel, one workgroup per 128 query rows:  pass 1 accumulates sum p, sum u, sum u dP -> delta;
//                                                 pass 2 forms dX and dQ^T += K^T dX^T.
//   dK/dV kernel, one workgroup per 128 keys, all query heads of the K/V head in turn:
//                                                 pass 1 dV^T += dO^T P, pass 2 dK^T += Q^T dX.
// P / dX go from the accumulators straight into the next MFMA; the operands that run along the tile's rows (K^T, dO^T,
// Q^T) come out of row-major tiles through the transposing LDS read (16-bit types, see acc_block).
#pragma once
#include <type_traits>
#include "attn_kernel.h"
#include "attn_bwd_params.h"

namespace adsp {

constexpr int kBwdRows = 128;  // rows (queries resp. keys) per workgroup = 4 waves x 32

// p and u = p^(2-alpha) from r = z - tau.
template <int AM> __device__ __forceinline__ void bwd_prob(float r, float c0, float& pr, float& u) {
  if constexpr (AM == ATT_15) {
    u = __builtin_amdgcn_fmed3f(r, 0.f, INFINITY);
    pr = u * u;
  } else if constexpr (AM == ATT_2) {
    pr = __builtin_amdgcn_fmed3f(r, 0.f, INFINITY);
    u = r > 0.f ? 1.f : 0.f;
  } else {
    const bool pos = r > 0.f;
    const float rr = pos ? r : 1.f;
    const float e = fast_exp2(fast_log2(rr) * c0);
    pr = pos ? e : 0.f;
    u = pos ? e * fast_rcp(rr) : 0.f;
  }
}

template <typename T, int D> struct BwdTiles {
  using G = TileGeo<T, D>;
  using KS = Swz<G::kKRow>;
  static constexpr bool k16 = G::k16;
  // Swizzle of a 16-bit tile that acc_block reads with the transposing LDS read (see attn_fwd_kernel's V tile): the
  // four rows times two column blocks that two groups of 16 lanes address together fall into eight different eighths
  // of the banks.
  static __device__ __forceinline__ int tsw(int row) {
    constexpr int kC = KS::kC;
    if constexpr (kC >= 16) return (4 * row) & 15;
    else if constexpr (kC == 8) return (2 * row) & 7;
    else if constexpr (kC == 4) return row & 2;
    else return 0;
  }
  static constexpr int kTile = G::kKTile;  // bytes of a [64][D] tile, in either orientation
  static constexpr int kNW = kBwdRows / 32;
  static constexpr int kSlots = k16 ? 3 : 2;  // tiles per pipeline stage
  // Double-buffer only while two workgroups still fit a CU: a second resident workgroup hides a tile's
  // load latency better than a second stage does, and brings a second wave to every SIMD.
  static constexpr int kNBuf = (2 * kSlots * kTile <= 64 * 1024) ? 2 : 1;
  static constexpr int kMinWaves = G::kMinWaves < 2 ? G::kMinWaves : 2;
  static constexpr int kLoads = kTile / 1024;

  // DMA of rows [row0, row0 + 64) of a row-major [N][D] tensor into a swizzled tile; rows from `N` on (the tensor's end,
  // or the sequence's for a tile that meets a product unmasked) are replaced by the last one before it.  kT: the tile
  // is read by acc_block (transposing reads, their swizzle); else by dot_block.
  template <bool kT = false>
  static __device__ __forceinline__ void issue_rows(const unsigned char* g, int row0, int N, unsigned char* lds, int wave,
                                                    int lane) {
    // the address is a wave-uniform base plus a 32-bit lane offset; for a whole tile the offset does not depend on the
    // tile and the base is formed with scalar instructions
    if (row0 + kBN <= N) {
      const unsigned char* base = uniform_ptr(g + (size_t)row0 * G::kKRow);
#pragma unroll
      for (int j0 = 0; j0 < (kLoads + kNW - 1) / kNW; ++j0) {
        const int j = j0 * kNW + wave;
        if (kLoads % kNW == 0 || j < kLoads) {
          const int P = j * 64 + lane;
          const int row = P / KS::kC, c = (P % KS::kC) ^ (kT ? tsw(row) : KS::sw(row));
          dma16s(base, (uint32_t)(row * G::kKRow + c * 16), lds + j * 1024);
        }
      }
    } else {
      g = uniform_ptr(g);
#pragma unroll
      for (int j0 = 0; j0 < (kLoads + kNW - 1) / kNW; ++j0) {
        const int j = j0 * kNW + wave;
        if (kLoads % kNW == 0 || j < kLoads) {
          const int P = j * 64 + lane;
          const int row = P / KS::kC, c = (P % KS::kC) ^ (kT ? tsw(row) : KS::sw(row));
          int gr = row0 + row;
          gr = gr < N ? gr : N - 1;  // rows past the end are masked by the caller
          dma16s(g, (uint32_t)gr * (uint32_t)G::kKRow + (uint32_t)(c * 16), lds + j * 1024);
        }
      }
    }
  }
  // Fragments of the lane's own row (B operand of the score-like products).
  static __device__ __forceinline__ void load_row_frags(const void* base, size_t row, bool ok, int lh,
                                                        uint32_t (&f)[G::kQRegs]) {
    if constexpr (k16) {
      const uint16_t* r = reinterpret_cast<const uint16_t*>(base) + row * D;
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) {
        u32x4 raw = *reinterpret_cast<const u32x4*>(r + ks * 16 + 8 * lh);
#pragma unroll
        for (int e = 0; e < 4; ++e) f[ks * 4 + e] = ok ? raw[e] : 0u;
      }
    } else {
      const float* r = reinterpret_cast<const float*>(base) + row * D;
#pragma unroll
      for (int g = 0; g < D / 8; ++g) {
        u32x4 raw = *reinterpret_cast<const u32x4*>(r + 8 * g + 4 * lh);
#pragma unroll
        for (int e = 0; e < 4; ++e) f[g * 4 + e] = ok ? raw[e] : 0u;
      }
    }
  }
  // acc[i] = (tile row kb*32 + 8(i/4) + 4 lh + i%4) . (lane's row), for the 32 lane rows of the wave.
  // kLean: addresses by xor with immediates (fewer registers, a few more VALU instructions) -- see below.
  template <bool kLean = false>
  static __device__ __forceinline__ f32x16 dot_block(const unsigned char* tile, int kb, const uint32_t (&f)[G::kQRegs],
                                                     int lq, int lh) {
    f32x16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
    const int row = kb * 32 + lq;
    const unsigned char* trow = tile + row * G::kKRow;
    const int sw = KS::sw(row);
    if constexpr (k16 && !kLean) {
      u32x4 a[D / 16];
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) a[ks] = *reinterpret_cast<const u32x4*>(trow + (((2 * ks + lh) ^ sw) << 4));
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) {
        u32x4 b = {f[ks * 4], f[ks * 4 + 1], f[ks * 4 + 2], f[ks * 4 + 3]};
        acc = mfma_16bit<T>(a[ks], b, acc);
      }
    } else if constexpr (k16) {
      // chunk 2 ks + lh of row r sits at r * row_bytes + (((2 ks + lh) ^ sw(r)) << 4)
      //   = (r * row_bytes + ((lh ^ sw(r)) << 4)) ^ (ks << 5): one lane constant, an xor with an immediate per read
      // (rows r and r + 32 share sw, so the block is an offset); the empty asm keeps the xors here instead of a
      // register per fragment hoisted out of the walk
      uint32_t ta = (uint32_t)(uintptr_t)tile + (uint32_t)(lq * G::kKRow + ((lh ^ KS::sw(lq)) << 4));
      asm volatile("" : "+v"(ta));
      u32x4 a[D / 16];
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) a[ks] = lds_read16(ta ^ (ks << 5), kb * 32 * G::kKRow);
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) {
        u32x4 b = {f[ks * 4], f[ks * 4 + 1], f[ks * 4 + 2], f[ks * 4 + 3]};
        acc = mfma_16bit<T>(a[ks], b, acc);
      }
    } else {
#pragma unroll
      for (int g = 0; g < D / 8; ++g) {
        f32x4 a = *reinterpret_cast<const f32x4*>(trow + (((2 * g + lh) ^ sw) << 4));
#pragma unroll
        for (int e = 0; e < 4; ++e)
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], __builtin_bit_cast(float, f[g * 4 + e]), acc, 0, 0, 0);
      }
    }
    return acc;
  }
  // o^T[d][lane row] += sum over the 32 tile rows of block kb of  tile[row][d] * w[row][lane row], where
  // w holds the lane's 16 values in the accumulator order of dot_block.  `tile` is row-major; only its first
  // `rows_valid` rows count (padding rows of the caller's tensors may hold anything: fp32 zeroes the operand; the
  // 16-bit tiles carry a valid row in their place, see issue_rows, and the callers select, not multiply, a zero weight
  // for every pair outside the mask or the sequence, so such a row adds exactly nothing).  16-bit: the operand
  // that runs along the tile's rows comes from two transposing reads per 16 rows -- in a group of 16 lanes, lane
  // 4 r + c points at row (4 g + r [+ 8]) of the half block, g = lane / 32, and at columns 4 c .. 4 c + 3 of the group's
  // 16 (groups 0 / 2: columns 0 .. 15 of a block of 32, groups 1 / 3: 16 .. 31), and receives column lane % 16 of four rows.
  template <bool kLean = false>
  static __device__ __forceinline__ void acc_block(f32x16 (&o)[G::kDB], const unsigned char* tile, int kb,
                                                   const float (&w)[16], int lq, int lh, int rows_valid) {
    if constexpr (k16) {
      const int lane = lh * 32 + lq;
      const int a4 = lane & 15, grp = lane >> 4, r = a4 >> 2, c = a4 & 3, dl = grp & 1;
      uint32_t ta[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int x = 4 * lh + r + 8 * h;
        ta[h] = (uint32_t)(uintptr_t)tile + (uint32_t)(x * G::kKRow + (((2 * dl + (c >> 1)) ^ tsw(x)) << 4) + (c & 1) * 8);
        if (D < 32 && dl) ta[h] = (uint32_t)(uintptr_t)tile;  // (D = 16: these lanes' columns do not exist; their operand is zeroed)
      }
      asm volatile("" : "+v"(ta[0]), "+v"(ta[1]));
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        u32x4 b = {pack2<T>(w[8 * s], w[8 * s + 1]), pack2<T>(w[8 * s + 2], w[8 * s + 3]),
                   pack2<T>(w[8 * s + 4], w[8 * s + 5]), pack2<T>(w[8 * s + 6], w[8 * s + 7])};
#pragma unroll
        for (int db = 0; db < G::kDB; ++db) {
          const int drow = db * 32 + lq;
          const u32x2_t a0 = lds_read8_tr(ta[0] ^ (db << 6), (kb * 32 + 16 * s) * G::kKRow);
          const u32x2_t a1 = lds_read8_tr(ta[1] ^ (db << 6), (kb * 32 + 16 * s) * G::kKRow);
          u32x4 a = {a0[0], a0[1], a1[0], a1[1]};
          if (D < 32 && drow >= D) a = u32x4{0u, 0u, 0u, 0u};
          o[db] = mfma_16bit<T>(a, b, o[db]);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int row = kb * 32 + 8 * (i >> 2) + 4 * lh + (i & 3);
#pragma unroll
        for (int db = 0; db < G::kDB; ++db) {
          const int dcol = db * 32 + lq;
          float a = 0.f;
          if (D >= 32 || dcol < D) a = *reinterpret_cast<const float*>(tile + KS::off(row, dcol >> 2) + (dcol & 3) * 4);
          if (row >= rows_valid) a = 0.f;
          o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, w[i], o[db], 0, 0, 0);
        }
      }
    }
  }
  // Writes scale * o^T (32 rows of this wave x D) to rows [row0, row0 + 32) of a row-major tensor, through
  // an LDS transpose in `stage` (32 * kKRow bytes, private to the wave).
  static __device__ __forceinline__ void store_rows(const f32x16 (&o)[G::kDB], float scale, unsigned char* stage,
                                                    void* gbase, int row0, int N, int lane) {
    const int lq = lane & 31, lh = lane >> 5;
#pragma unroll
    for (int db = 0; db < G::kDB; ++db) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int d0 = db * 32 + 8 * g + 4 * lh;
        if (D >= 32 || d0 < D) {
          const float x0 = o[db][4 * g] * scale, x1 = o[db][4 * g + 1] * scale;
          const float x2 = o[db][4 * g + 2] * scale, x3 = o[db][4 * g + 3] * scale;
          if constexpr (k16) {
            u32x2 w = {pack2<T>(x0, x1), pack2<T>(x2, x3)};
            *reinterpret_cast<u32x2*>(stage + KS::off(lq, d0 >> 3) + (d0 & 7) * 2) = w;
          } else {
            f32x4 w = {x0, x1, x2, x3};
            *reinterpret_cast<f32x4*>(stage + KS::off(lq, d0 >> 2)) = w;
          }
        }
      }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the wave reads back what it wrote itself
    unsigned char* obase = reinterpret_cast<unsigned char*>(gbase) + (size_t)row0 * G::kKRow;
    constexpr int kChunks = 32 * KS::kC;
#pragma unroll
    for (int j = 0; j < (kChunks + 63) / 64; ++j) {
      const int id = j * 64 + lane;
      const int row = id / KS::kC, c = id % KS::kC;
      if ((kChunks % 64 == 0 || id < kChunks) && row0 + row < N) {
        u32x4 w = *reinterpret_cast<const u32x4*>(stage + KS::off(row, c));
        *reinterpret_cast<u32x4*>(obase + (size_t)row * G::kKRow + c * 16) = w;
      }
    }
  }
};

__device__ __forceinline__ int bwd_seq_len(const AttnBwdParams& p, int b) {
  int L = p.N;
  if (p.varlen) {
    long long l = p.varlen_bits == 64 ? ((const long long*)p.varlen)[b] : (long long)((const int*)p.varlen)[b];
    L = (int)(l < 0 ? 0 : (l > p.N ? p.N : l));
  }
  return L;
}


// ---------------------------------------------------------------------------------------------------------
// dQ kernel: one block per (K/V head, query head in its group, row block of 128 queries)
// ---------------------------------------------------------------------------------------------------------
constexpr int kDqPlainMaxD = 128;  // largest 16-bit head dim whose unmasked blocks take the predicate-free code
constexpr int kDqWaves64 = 3;      // waves per SIMD of the dQ kernel at 16-bit D <= 64
template <typename T, int D> constexpr int dq_waves() { return (TileGeo<T, D>::k16 && D <= 64) ? kDqWaves64 : BwdTiles<T, D>::kMinWaves; }

template <typename T, int D, int AM>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu((dq_waves<T, D>()), (dq_waves<T, D>() > 2 ? dq_waves<T, D>() : 2)))) void attn_bwd_dq_kernel(AttnBwdParams p) {
  using BT = BwdTiles<T, D>;
  using G = TileGeo<T, D>;
  constexpr bool k16 = G::k16;
  __shared__ __align__(1024) unsigned char a0[BT::kTile];  // K tile, row-major
  __shared__ __align__(1024) unsigned char b0[BT::kTile];  // V tile, row-major
  __shared__ __align__(1024) unsigned char c0[k16 ? BT::kTile : 16];  // K^T tile (16-bit)
  __shared__ __align__(1024) unsigned char a1[BT::kNBuf == 2 ? BT::kTile : 16];
  __shared__ __align__(1024) unsigned char b1[BT::kNBuf == 2 ? BT::kTile : 16];
  __shared__ __align__(1024) unsigned char c1[(k16 && BT::kNBuf == 2) ? BT::kTile : 16];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, lq = lane & 31, lh = lane >> 5;
  const int N = p.N;
  const int n_blk = (N + kBwdRows - 1) / kBwdRows;
  const int group = p.Hq / p.Hkv;
  int bkv, mi, hg;
  if (!xcd_block_map(p.B * p.Hkv, n_blk, group, p.causal != 0, 2ll * N * D * G::kEB, bkv, mi, hg)) return;  // (K and V of a head)
  const int mblk = n_blk - 1 - mi;  // the longest causal rows first; a group's heads side by side
  const int b = bkv / p.Hkv, kvh = bkv % p.Hkv;
  const int h = kvh * group + hg;
  const int bh = b * p.Hq + h;
  // behind the sparse-support dQ kernel: only the row blocks it flagged (all of them when it stepped aside)
  if (p.block_flags && p.queue[kCtrlAllDense] == 0u && (p.queue[kCtrlFlagged] == 0u || p.block_flags[(size_t)bh * n_blk + mblk] == 0)) return;
  const int L = bwd_seq_len(p, b);
  const int m0 = mblk * kBwdRows;
  const int wave_row0 = m0 + wave * 32;
  const int qi = wave_row0 + lq;
  const size_t q_base = (size_t)bh * N;                   // rows
  const size_t kv_base = (size_t)(b * p.Hkv + kvh) * N;  // rows
  unsigned char* dq_rows = reinterpret_cast<unsigned char*>(p.dq) + q_base * G::kKRow;

  if (m0 >= L) {  // padding rows: zero gradient
    constexpr int kRowDw = D * G::kEB / 4;
    uint32_t* o32 = reinterpret_cast<uint32_t*>(dq_rows) + (size_t)m0 * kRowDw;
    const int rows = (N - m0) < kBwdRows ? (N - m0) : kBwdRows;
    for (int i = tid; i < rows * kRowDw; i += 256) o32[i] = 0u;
    return;
  }

  uint32_t qf[G::kQRegs], dof[G::kQRegs];
  {
    const bool ok = qi < L;  // padding rows take no part
    BT::load_row_frags(p.q, q_base + (ok ? qi : 0), ok, lh, qf);
    BT::load_row_frags(p.dout, q_base + (ok ? qi : 0), ok, lh, dof);
  }
  const bool live = qi < L;
  const float tau = live ? p.taus[q_base + qi] : INFINITY;
  const int lim = p.causal ? (qi < L - 1 ? qi : L - 1) : L - 1;  // last valid key of the lane's row
  const int lim_all = p.causal ? (wave_row0 < L - 1 ? wave_row0 : L - 1) : L - 1;  // smallest `lim` of the wave (wave-uniform)
  const int row_hi = (m0 + kBwdRows < L ? m0 + kBwdRows : L);
  const int nt = p.causal ? (row_hi + kBN - 1) / kBN : (L + kBN - 1) / kBN;
  const int32_t* mrow = p.bmask ? p.bmask + ((size_t)bh * p.n_mblk + mblk) * p.mask_words : nullptr;

  const unsigned char* kg = reinterpret_cast<const unsigned char*>(p.k) + kv_base * G::kKRow;
  const unsigned char* vg = reinterpret_cast<const unsigned char*>(p.v) + kv_base * G::kKRow;

  auto next_tile = [&](int cur) -> int {
    int t = cur + 1;
    if (!mrow) return t < nt ? t : -1;
    while (t < nt) {
      uint32_t w = (uint32_t)mrow[t >> 5] >> (t & 31);
      if (w) {
        t += __builtin_ctz(w);
        return t < nt ? t : -1;
      }
      t = (t | 31) + 1;
    }
    return -1;
  };
  auto issue = [&](unsigned char* a, unsigned char* bb, unsigned char* c, int kt, bool with_t) {
    BT::issue_rows(kg, kt * kBN, N, a, wave, lane);
    BT::issue_rows(vg, kt * kBN, N, bb, wave, lane);
    if constexpr (k16) {
      if (with_t) BT::template issue_rows<true>(kg, kt * kBN, L, c, wave, lane);  // K again, for the transposing reads of dQ
    }
  };
  auto tile_loop = [&](bool with_t, auto&& body) {
    __syncthreads();
    int cur = next_tile(-1);
    if (cur >= 0) issue(a0, b0, c0, cur, with_t);
    while (cur >= 0) {
      __builtin_amdgcn_s_waitcnt(0x0f70);
      __syncthreads();
      int nxt = next_tile(cur);
      if constexpr (BT::kNBuf == 2) {
        if (nxt >= 0) issue(a1, b1, c1, nxt, with_t);
        __builtin_amdgcn_sched_barrier(0);
      }
      body(cur, a0, b0, c0);
      if constexpr (BT::kNBuf == 1) {
        __syncthreads();
        if (nxt >= 0) issue(a0, b0, c0, nxt, with_t);
        cur = nxt;
      } else {
        cur = nxt;
        if (cur < 0) break;
        __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
        nxt = next_tile(cur);
        if (nxt >= 0) issue(a0, b0, c0, nxt, with_t);
        __builtin_amdgcn_sched_barrier(0);
        body(cur, a1, b1, c1);
        cur = nxt;
      }
    }
  };
  // r = z - tau for the 16 keys of block kb (-inf where the row may not look), and dP.  A block that every row of
  // the wave sees in full (below the causal diagonal, inside the sequence) is "plain": no per-score predicate,
  // one fma per score instead of a compare and two selects more.  The choice is a template argument so that each
  // kind of block is one piece of straight-line code, products included.
  // (only where the second code path fits the register budget: at D = 128 it costs spills and more than it saves)
  constexpr bool kPlainBlocks = k16 && D <= kDqPlainMaxD;
  auto block_is_plain = [&](int kt, int kb) { return kPlainBlocks && kt * kBN + kb * 32 + 31 <= lim_all; };
  auto block_terms = [&](auto plain_c, int kt, int kb, const unsigned char* ka, const unsigned char* va, float (&r)[16],
                         f32x16& dp) {
    f32x16 s = BT::template dot_block<true>(ka, kb, qf, lq, lh);
    dp = BT::template dot_block<true>(va, kb, dof, lq, lh);
    if constexpr (decltype(plain_c)::value) {
#pragma unroll
      for (int i = 0; i < 16; ++i) r[i] = fmaf(s[i], p.qscale, -tau);
    } else {
      const int jb = kt * kBN + kb * 32 + 4 * lh;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const bool ok = jb + 8 * (i >> 2) + (i & 3) <= lim;
        r[i] = ok ? fmaf(s[i], p.qscale, -tau) : -INFINITY;
        dp[i] = ok ? dp[i] : 0.f;  // keys past the end may hold anything
      }
    }
  };

  // ---- pass 1: sum p, sum u, sum u dP ----
  float zsum = 0.f, usum = 0.f, udp = 0.f;
  tile_loop(false, [&](int kt, const unsigned char* ka, const unsigned char* va, const unsigned char*) {
    if (p.causal && kt * kBN > wave_row0 + 31) return;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      if (p.causal && kt * kBN + kb * 32 > wave_row0 + 31) continue;
      auto block = [&](auto plain_c) {
        float r[16];
        f32x16 dp;
        block_terms(plain_c, kt, kb, ka, va, r, dp);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          float pr, u;
          bwd_prob<AM>(r[i], p.c0, pr, u);
          zsum += pr;
          usum += u;
          udp = fmaf(u, dp[i], udp);
        }
      };
      if constexpr (!kPlainBlocks) {
        block(std::false_type{});
      } else if (block_is_plain(kt, kb)) {
        asm volatile("; plain block" ::: "memory");
        block(std::true_type{});
      } else {
        asm volatile("; masked block" ::: "memory");
        block(std::false_type{});
      }
    }
  });
  zsum += __shfl_xor(zsum, 32, 64);
  usum += __shfl_xor(usum, 32, 64);
  udp += __shfl_xor(udp, 32, 64);
  const float delta = usum > 0.f ? udp / usum : 0.f;
  if (live && lh == 0) {
    p.delta[q_base + qi] = delta;
    p.zinv[q_base + qi] = zsum > 0.f ? 1.f / zsum : 0.f;
  }

  // ---- pass 2: dX = u (dP - delta), dQ^T += K^T dX^T ----
  f32x16 acc[G::kDB];
#pragma unroll
  for (int db = 0; db < G::kDB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[db][i] = 0.f;
  tile_loop(true, [&](int kt, const unsigned char* ka, const unsigned char* va, const unsigned char* kta) {
    if (p.causal && kt * kBN > wave_row0 + 31) return;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      if (p.causal && kt * kBN + kb * 32 > wave_row0 + 31) continue;
      auto block = [&](auto plain_c) {
        float r[16];
        f32x16 dp;
        block_terms(plain_c, kt, kb, ka, va, r, dp);
        float dx[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          float pr, u;
          bwd_prob<AM>(r[i], p.c0, pr, u);
          dx[i] = u * (dp[i] - delta);
        }
        BT::template acc_block<true>(acc, k16 ? kta : ka, kb, dx, lq, lh, L - kt * kBN);
      };
      if constexpr (!kPlainBlocks) {
        block(std::false_type{});
      } else if (block_is_plain(kt, kb)) {
        asm volatile("; plain block" ::: "memory");
        block(std::true_type{});
      } else {
        asm volatile("; masked block" ::: "memory");
        block(std::false_type{});
      }
    }
  });

  __syncthreads();  // the tile buffers become the transpose scratch: a quarter of a0/b0 per wave pair
  unsigned char* stage = (wave < 2 ? a0 : b0) + (wave & 1) * (32 * G::kKRow);
  BT::store_rows(acc, p.sm_scale, stage, dq_rows, wave_row0, N, lane);
}

// ---------------------------------------------------------------------------------------------------------
// dK / dV kernel: one block per (K/V head, block of 128 keys)
// ---------------------------------------------------------------------------------------------------------
template <typename T, int D, int AM>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu((BwdTiles<T, D>::kMinWaves), 2))) void attn_bwd_dkdv_kernel(AttnBwdParams p) {
  using BT = BwdTiles<T, D>;
  using G = TileGeo<T, D>;
  constexpr bool k16 = G::k16;
  __shared__ __align__(1024) unsigned char a0[BT::kTile];  // Q tile, row-major
  __shared__ __align__(1024) unsigned char b0[BT::kTile];  // dO tile, row-major
  __shared__ __align__(1024) unsigned char c0[k16 ? BT::kTile : 16];  // dO^T (pass 1) or Q^T (pass 2) tile, 16-bit
  __shared__ __align__(1024) unsigned char a1[BT::kNBuf == 2 ? BT::kTile : 16];
  __shared__ __align__(1024) unsigned char b1[BT::kNBuf == 2 ? BT::kTile : 16];
  __shared__ __align__(1024) unsigned char c1[(k16 && BT::kNBuf == 2) ? BT::kTile : 16];
  // 16-bit types with D <= 64 make one walk over the query tiles and keep both accumulators (at D = 128
  // the two accumulators plus the K and V fragments no longer fit 256 registers); that needs dO^T and Q^T
  // at the same time
  constexpr bool kFused = k16 && D <= 64;
  __shared__ __align__(1024) unsigned char d0[kFused ? BT::kTile : 16];  // Q^T tile
  __shared__ __align__(1024) unsigned char d1[(kFused && BT::kNBuf == 2) ? BT::kTile : 16];
  __shared__ __align__(16) float scal0[3][kBN];  // tau, 1 / sum p, delta of the tile's queries
  __shared__ __align__(16) float scal1[3][kBN];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, lq = lane & 31, lh = lane >> 5;
  const int N = p.N;
  int bkv, nblk;  // early key blocks have the most causal work and come first
  int member_unused;
  // (the key blocks of a K/V head stream q and dout of all its query heads)
  if (!xcd_block_map(p.B * p.Hkv, (N + kBwdRows - 1) / kBwdRows, 1, p.causal != 0, 2ll * (p.Hq / p.Hkv) * N * D * G::kEB, bkv, nblk, member_unused)) return;
  const int b = bkv / p.Hkv, kvh = bkv % p.Hkv;
  const int group = p.Hq / p.Hkv;
  // behind the sparse-support dK/dV kernel: only the key blocks it flagged (all of them when it stepped aside)
  if (p.kv_flags && p.queue2[kCtrlAllDense] == 0u &&
      (p.queue2[kCtrlFlagged] == 0u || p.kv_flags[(size_t)bkv * ((N + kBwdRows - 1) / kBwdRows) + nblk] == 0))
    return;
  const int L = bwd_seq_len(p, b);
  const int n0 = nblk * kBwdRows;
  const int wave_key0 = n0 + wave * 32;
  const int kj = wave_key0 + lq;
  const size_t kv_base = (size_t)bkv * N;
  unsigned char* dk_rows = reinterpret_cast<unsigned char*>(p.dk) + kv_base * G::kKRow;
  unsigned char* dv_rows = reinterpret_cast<unsigned char*>(p.dv) + kv_base * G::kKRow;

  if (n0 >= L) {  // padding keys: zero gradient
    constexpr int kRowDw = D * G::kEB / 4;
    const int rows = (N - n0) < kBwdRows ? (N - n0) : kBwdRows;
    uint32_t* k32 = reinterpret_cast<uint32_t*>(dk_rows) + (size_t)n0 * kRowDw;
    uint32_t* v32 = reinterpret_cast<uint32_t*>(dv_rows) + (size_t)n0 * kRowDw;
    for (int i = tid; i < rows * kRowDw; i += 256) {
      k32[i] = 0u;
      v32[i] = 0u;
    }
    return;
  }

  uint32_t kf[G::kQRegs], vf[G::kQRegs];
  {
    const bool ok = kj < L;  // padding keys take no part
    BT::load_row_frags(p.k, kv_base + (ok ? kj : 0), ok, lh, kf);
    BT::load_row_frags(p.v, kv_base + (ok ? kj : 0), ok, lh, vf);
  }
  const bool key_live = kj < L;
  const int t_first = p.causal ? n0 / kBN : 0;  // query tiles below the key block see none of its keys
  const int nt = (L + kBN - 1) / kBN;

  // Runs body(qt, tiles, scalars) over every (query tile, query head of the group) pair.  The walk is tile
  // major and goes from the last tile down: all key blocks of a K/V head then sit on the same query tile at
  // about the same time, so the workgroups that run side by side on an XCD find the tile in its L2 (head
  // major, each would soon be streaming another head's tensors and the working set would be all of them).
  // A step is numbered c = tile * group + head.
  auto tile_loop = [&](int pass, auto&& body) {
    const int ktile0 = n0 / kBN;
    auto head_of = [&](int c) { return kvh * group + c % group; };
    auto next_step = [&](int cur) -> int {
      int c = cur - 1;
      if (!p.bmask) return c >= t_first * group ? c : -1;
      for (; c >= t_first * group; --c) {
        // column of the forward's tile mask for this key block: is any of its two 64-key tiles kept for
        // the 128-row block that holds the query tile?  (a 128-key block starts on an even tile, so both
        // bits sit in one word)
        const int t = c / group;
        const int32_t* mcol = p.bmask + (size_t)(b * p.Hq + head_of(c)) * p.n_mblk * p.mask_words;
        const uint32_t w = (uint32_t)mcol[(size_t)(t >> 1) * p.mask_words + (ktile0 >> 5)] >> (ktile0 & 31);
        if (w & 3u) return c;
      }
      return -1;
    };
    auto issue = [&](unsigned char* a, unsigned char* bb, unsigned char* c, unsigned char* d, float (*sc)[kBN], int step) {
      const int qt = step / group;
      const size_t bh = (size_t)(b * p.Hq + head_of(step));
      const size_t q_base = bh * N;
      const unsigned char* qg = reinterpret_cast<const unsigned char*>(p.q) + q_base * G::kKRow;
      const unsigned char* dog = reinterpret_cast<const unsigned char*>(p.dout) + q_base * G::kKRow;
      BT::issue_rows(qg, qt * kBN, N, a, wave, lane);
      if (pass >= 2 || !k16) BT::issue_rows(dog, qt * kBN, N, bb, wave, lane);
      if constexpr (k16) {
        // the operand of the pass that runs along the queries, in the format of the transposing reads: dO for dV
        // (pass 1 and the fused pass 3), q for dK (pass 2; the fused pass takes it as a second such tile)
        BT::template issue_rows<true>(pass == 2 ? qg : dog, qt * kBN, L, c, wave, lane);
        if constexpr (kFused) {
          if (pass == 3) BT::template issue_rows<true>(qg, qt * kBN, L, d, wave, lane);
        }
      }
      // tau, 1 / sum p and delta of the tile's 64 queries: one 4-byte DMA per lane, an array per wave.
      // Entries of queries past the sequence end are never used (block_r masks those queries).
      if (wave < 3) {
        const float* src = wave == 0 ? p.taus : (wave == 1 ? p.zinv : p.delta);
        int qrow = qt * kBN + lane;
        qrow = qrow < N ? qrow : N - 1;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + q_base + qrow),
                                         (__attribute__((address_space(3))) void*)&sc[wave][0], 4, 0, 0);
      }
    };
    __syncthreads();
    int cur = next_step(nt * group);
    if (cur >= 0) issue(a0, b0, c0, d0, scal0, cur);
    while (cur >= 0) {
      __builtin_amdgcn_s_waitcnt(0x0f70);
      __syncthreads();
      int nxt = next_step(cur);
      if constexpr (BT::kNBuf == 2) {
        if (nxt >= 0) issue(a1, b1, c1, d1, scal1, nxt);
        __builtin_amdgcn_sched_barrier(0);
      }
      body(cur / group, a0, b0, c0, d0, scal0);
      if constexpr (BT::kNBuf == 1) {
        __syncthreads();
        if (nxt >= 0) issue(a0, b0, c0, d0, scal0, nxt);
        cur = nxt;
      } else {
        cur = nxt;
        if (cur < 0) break;
        __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
        nxt = next_step(cur);
        if (nxt >= 0) issue(a0, b0, c0, d0, scal0, nxt);
        __builtin_amdgcn_sched_barrier(0);
        body(cur / group, a1, b1, c1, d1, scal1);
        cur = nxt;
      }
    }
  };
  // r = z - tau_i for the 16 queries of block qb against the lane's key (-inf where query i may not see it)
  // Returns true for a plain block: every key of the wave is seen by every query of the block (all inside the
  // sequence, the block below the causal diagonal).  Such a block needs no per-score predicate, and the selects
  // that keep 0 x (anything in a padding row) out of the gradients can go too.
  auto block_r = [&](int qt, int qb, const unsigned char* qa, const float (*sc)[kBN], float (&r)[16]) -> bool {
    f32x16 s = BT::dot_block(qa, qb, kf, lq, lh);
    const int q_first = qt * kBN + qb * 32;
    const bool plain = wave_key0 + 31 < L && q_first + 31 < L && (!p.causal || wave_key0 + 31 <= q_first);
    if (plain) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x4 tq = *reinterpret_cast<const f32x4*>(&sc[0][qb * 32 + 8 * g + 4 * lh]);
#pragma unroll
        for (int e = 0; e < 4; ++e) r[4 * g + e] = fmaf(s[4 * g + e], p.qscale, -tq[e]);
      }
    } else {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x4 tq = *reinterpret_cast<const f32x4*>(&sc[0][qb * 32 + 8 * g + 4 * lh]);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int i = 4 * g + e;
          const int qrow = q_first + 8 * g + 4 * lh + e;
          const bool ok = key_live && qrow < L && (!p.causal || kj <= qrow);
          r[i] = ok ? fmaf(s[i], p.qscale, -tq[e]) : -INFINITY;
        }
      }
    }
    return plain;
  };
  // MFMA operands of the two gradient products from r: p / sum p for dV, u (dP - delta) for dK.  Outside plain
  // blocks a zero weight is selected, not multiplied: its partner may sit in a padding row and hold anything.
  auto weights_p = [&](bool plain, int qb, const float (&r)[16], const float (*sc)[kBN], float (&w)[16]) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const f32x4 zi = *reinterpret_cast<const f32x4*>(&sc[1][qb * 32 + 8 * g + 4 * lh]);
      if (plain) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float pr, u;
          bwd_prob<AM>(r[4 * g + e], p.c0, pr, u);
          w[4 * g + e] = pr * zi[e];
        }
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float pr, u;
          bwd_prob<AM>(r[4 * g + e], p.c0, pr, u);
          w[4 * g + e] = pr > 0.f ? pr * zi[e] : 0.f;
        }
      }
    }
  };
  auto weights_x = [&](bool plain, int qb, const float (&r)[16], const f32x16& dp, const float (*sc)[kBN], float (&w)[16]) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const f32x4 di = *reinterpret_cast<const f32x4*>(&sc[2][qb * 32 + 8 * g + 4 * lh]);
      if (plain) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float pr, u;
          bwd_prob<AM>(r[4 * g + e], p.c0, pr, u);
          w[4 * g + e] = u * (dp[4 * g + e] - di[e]);
        }
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float pr, u;
          bwd_prob<AM>(r[4 * g + e], p.c0, pr, u);
          w[4 * g + e] = u > 0.f ? u * (dp[4 * g + e] - di[e]) : 0.f;
        }
      }
    }
  };
  auto block_visible = [&](int qt, int qb) {  // does any query of the block see any key of this wave?
    return !p.causal || qt * kBN + qb * 32 + 31 >= wave_key0;
  };

  f32x16 acc[G::kDB];
  unsigned char* stage = (wave < 2 ? a0 : b0) + (wave & 1) * (32 * G::kKRow);

  if constexpr (kFused) {
    // ---- one walk: dV^T += dO^T P and dK^T += Q^T dX ----
    f32x16 acc_k[G::kDB];
#pragma unroll
    for (int db = 0; db < G::kDB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        acc[db][i] = 0.f;
        acc_k[db][i] = 0.f;
      }
    {
      tile_loop(3,
                [&](int qt, const unsigned char* qa, const unsigned char* doa, const unsigned char* dota,
                    const unsigned char* qta, const float (*sc)[kBN]) {
#pragma unroll
                  for (int qb = 0; qb < 2; ++qb) {
                    if (!block_visible(qt, qb)) continue;
                    float r[16], w[16];
                    const bool plain = block_r(qt, qb, qa, sc, r);
                    // dV first: p / sum p
                    weights_p(plain, qb, r, sc, w);
                    BT::acc_block(acc, dota, qb, w, lq, lh, L - qt * kBN);
                    // then dK: u (dP - delta)
                    f32x16 dp = BT::dot_block(doa, qb, vf, lq, lh);
                    weights_x(plain, qb, r, dp, sc, w);
                    BT::acc_block(acc_k, qta, qb, w, lq, lh, L - qt * kBN);
                  }
                });
    }
    __syncthreads();
    BT::store_rows(acc, 1.f, stage, dv_rows, wave_key0, N, lane);
    __builtin_amdgcn_s_waitcnt(0xc07f);
    BT::store_rows(acc_k, p.sm_scale, stage, dk_rows, wave_key0, N, lane);
    return;
  }

  // ---- pass 1: dV^T += dO^T P ----
#pragma unroll
  for (int db = 0; db < G::kDB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[db][i] = 0.f;
  {
    tile_loop(1,
              [&](int qt, const unsigned char* qa, const unsigned char* doa, const unsigned char* ta, const unsigned char*,
                  const float (*sc)[kBN]) {
#pragma unroll
                for (int qb = 0; qb < 2; ++qb) {
                  if (!block_visible(qt, qb)) continue;
                  float r[16], w[16];
                  const bool plain = block_r(qt, qb, qa, sc, r);
                  weights_p(plain, qb, r, sc, w);
                  BT::acc_block(acc, k16 ? ta : doa, qb, w, lq, lh, L - qt * kBN);
                }
              });
  }
  __syncthreads();
  BT::store_rows(acc, 1.f, stage, dv_rows, wave_key0, N, lane);

  // ---- pass 2: dK^T += Q^T dX ----
#pragma unroll
  for (int db = 0; db < G::kDB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[db][i] = 0.f;
  {
    tile_loop(2,
              [&](int qt, const unsigned char* qa, const unsigned char* doa, const unsigned char* ta, const unsigned char*,
                  const float (*sc)[kBN]) {
#pragma unroll
                for (int qb = 0; qb < 2; ++qb) {
                  if (!block_visible(qt, qb)) continue;
                  float r[16], w[16];
                  const bool plain = block_r(qt, qb, qa, sc, r);
                  f32x16 dp = BT::dot_block(doa, qb, vf, lq, lh);
                  weights_x(plain, qb, r, dp, sc, w);
                  BT::acc_block(acc, k16 ? ta : qa, qb, w, lq, lh, L - qt * kBN);
                }
              });
  }
  __syncthreads();
  BT::store_rows(acc, p.sm_scale, stage, dk_rows, wave_key0, N, lane);
}

// which: 1 = the dQ kernel, 2 = the dK/dV kernel, 3 = both, in that order
template <typename T, int D> static int launch_attn_bwd_d(const AttnBwdParams& p, int am, int which, hipStream_t s) {
  const long long nq = (p.N + kBwdRows - 1) / kBwdRows;
  const dim3 gq((unsigned)(((long long)p.B * p.Hq * nq + 7) / 8 * 8)), gk((unsigned)(((long long)p.B * p.Hkv * nq + 7) / 8 * 8));
  if (am == ATT_15) {
    if (which & 1) hipLaunchKernelGGL((attn_bwd_dq_kernel<T, D, ATT_15>), gq, dim3(256), 0, s, p);
    if (which & 2) hipLaunchKernelGGL((attn_bwd_dkdv_kernel<T, D, ATT_15>), gk, dim3(256), 0, s, p);
  } else if (am == ATT_2) {
    if (which & 1) hipLaunchKernelGGL((attn_bwd_dq_kernel<T, D, ATT_2>), gq, dim3(256), 0, s, p);
    if (which & 2) hipLaunchKernelGGL((attn_bwd_dkdv_kernel<T, D, ATT_2>), gk, dim3(256), 0, s, p);
  } else {
    if (which & 1) hipLaunchKernelGGL((attn_bwd_dq_kernel<T, D, ATT_GEN>), gq, dim3(256), 0, s, p);
    if (which & 2) hipLaunchKernelGGL((attn_bwd_dkdv_kernel<T, D, ATT_GEN>), gk, dim3(256), 0, s, p);
  }
  return 0;
}

}  // namespace adsp
