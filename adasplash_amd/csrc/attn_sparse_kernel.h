// Sparse-support forward for 16-bit inputs, alpha = 1.5 / 2 (gfx950): two cheap score walks and no P V product.
//
// When a row's support is a few dozen keys out of thousands (unit-variance q and k at head dim 128: about 25 of
// 8192), every 128 x 64 tile still holds a member of some row's support, so a tile mask skips nothing, yet the
// output needs only those few keys.  This kernel finds them with two walks over K whose vector work per score is
// about one instruction, then solves the threshold and forms the output from the short candidate lists:
//
//   walk 1  S^T = K Q^T per tile on the fp8 MFMA (twice the 16-bit rate, half the tile bytes) from an e4m3 copy of K
//           and Q fragments rounded the same way; a lane keeps the four largest block maxima of its half of the row's
//           keys together with the keys they belong to.  Both operands are first put on a grid of 1/16, so every
//           product is a multiple of 2^-8 and the sums are exact in fp32; the accumulators start at 1536 + i 2^-13 for
//           the lane's i-th value of a block, which leaves i in the four lowest mantissa bits of every score: the
//           maximum of a block knows its key without an instruction per score.  These scores are approximate and only
//           choose keys (a wrong position, should the exactness ever fail, is a poor choice and no more): the scores
//           of the eight chosen keys of a row are then recomputed from the 16-bit inputs.  The threshold of any subset
//           of a row's scores is a lower bound of the row's threshold (f only grows when entries are added), so a few
//           Newton steps from the left on those eight values give a lower bound `lo` that lies within a few
//           hundredths (in z) of the threshold for such rows, whichever keys were chosen.
//   walk 2  the same products with the accumulators preloaded with -lo; a lane whose eight scores of a 16-key half
//           block have a positive maximum writes those eight values and the half block's index to its event list in
//           global memory (a per-workgroup slot of the workspace; the events are a few per cent of the scores).
//   lists   every lane turns its events into (score - lo, key) pairs in LDS (the K tile buffers, idle by then), the
//           two lanes of a row run Newton's iteration on them to convergence (from the left: monotone, never past
//           the root), and the output is the weighted sum of the V rows of the support, read from the row-major V.
//
// A row block whose lanes run out of event slots or list room (a dense support) is left to the dense kernel: the
// kernel writes one flag per row block, and attn_fwd_kernel, launched behind it, serves the flagged ones.
//
// The kernel is persistent: a fixed number of workgroups (one event slot each) draw row blocks from per-XCD
// counters in the same XCD-aware order as the dense kernel, longest causal row blocks first, and help the other
// XCDs when their own counter runs out.
#pragma once
#include <type_traits>

#include "attn_kernel.h"

namespace adsp {

#ifndef ADSP_GATHER_DEPTH
#define ADSP_GATHER_DEPTH 8
#endif
#ifndef ADSP_SPARSE_WAVES
#define ADSP_SPARSE_WAVES 4
#endif
// Profiling builds only (-DADSP_SPARSE_STOP=n in the build's extra flags): a row block ends behind its first walk (1),
// the lower bound (2), the second walk (3) or the thresholds (4), so that the stages can be timed by difference.  Such
// a build computes no output.
#ifndef ADSP_SPARSE_STOP
#define ADSP_SPARSE_STOP 0
#endif
constexpr int kSparseStreamCap = 1616;  // candidates per wave the workspace slot holds (SparseGeo::kListCap is at most this)
constexpr int kSparseMaxKeys = 65536;   // the lists hold 16-bit key indices

// acc[2 i] += v[i].lo * p, acc[2 i + 1] += v[i].hi * p for the eight elements of a 16-byte chunk, with the weight given
// as the pairs plo = (p, 0) and phi = (0, p) of the element type: eight two-term dot products with fp32 accumulation.
// They are issued as one block that ends in idle cycles: on this part the instruction that follows a v_dot2c must
// not overwrite one of its source registers (a conversion placed there by the compiler did, and the last of eight
// sums came out wrong), and the compiler does not keep such writes away by itself.
template <typename T> __device__ __forceinline__ void dot2_chunk(float (&acc)[8], u32x4 v, uint32_t plo, uint32_t phi);
#define ADSP_DOT2_CHUNK(OP)                                                                                          \
  asm volatile(OP " %0, %8, %12\n\t" OP " %1, %8, %13\n\t" OP " %2, %9, %12\n\t" OP " %3, %9, %13\n\t"           \
               OP " %4, %10, %12\n\t" OP " %5, %10, %13\n\t" OP " %6, %11, %12\n\t" OP " %7, %11, %13\n\ts_nop 3" \
               : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]), "+v"(acc[4]), "+v"(acc[5]), "+v"(acc[6]),   \
                 "+v"(acc[7])                                                                                        \
               : "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]), "v"(plo), "v"(phi))
template <> __device__ __forceinline__ void dot2_chunk<bf16_t>(float (&acc)[8], u32x4 v, uint32_t plo, uint32_t phi) {
  ADSP_DOT2_CHUNK("v_dot2c_f32_bf16");
}
template <> __device__ __forceinline__ void dot2_chunk<f16_t>(float (&acc)[8], u32x4 v, uint32_t plo, uint32_t phi) {
  ADSP_DOT2_CHUNK("v_dot2c_f32_f16");
}
#undef ADSP_DOT2_CHUNK

// two 16-byte chunks of e4m3 values as one operand of the fp8 MFMA (64 values of k per lane pair)
typedef int i32x8 __attribute__((ext_vector_type(8)));
__device__ __forceinline__ f32x16 mfma_fp8(u32x4 a_lo, u32x4 a_hi, const uint32_t* b, f32x16 c) {
  const i32x8 a = {(int)a_lo[0], (int)a_lo[1], (int)a_lo[2], (int)a_lo[3], (int)a_hi[0], (int)a_hi[1], (int)a_hi[2], (int)a_hi[3]};
  const i32x8 bb = {(int)b[0], (int)b[1], (int)b[2], (int)b[3], (int)b[4], (int)b[5], (int)b[6], (int)b[7]};
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, bb, c, 0, 0, 0, 0, 0, 0);  // both operands e4m3, no block scales
}

// median of three unsigned values
__device__ __forceinline__ uint32_t umed3(uint32_t a, uint32_t b, uint32_t c) {
  uint32_t r;
  asm("v_med3_u32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
// First walk: a score past a row's last valid key (0 lies below every real one, which start at 1024), and the
// rounding of an operand to a multiple of 1/16 (the sum with 1.5 * 2^19 has its last place there).
constexpr float kW1Masked = 0.f;
__device__ __forceinline__ float grid16(float x) {
  const float c = 786432.f;
  return (x + c) - c;
}

// inclusive prefix sum over the wave on the DPP network; all 64 lanes active
__device__ __forceinline__ int wave_scan_i(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);  // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);  // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);  // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);  // row_shr:8: a scan inside each row of 16
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1 and 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2 and 3
  return v;
}

// Should a sparse-support kernel leave the whole launch to the dense kernel?  The K/V heads the probe left unmarked
// (`hints[2 u] < 1 << 20`) must hold at least half of the launch's work (sequence length squared), else the kernel steps
// aside altogether: a launch split between the two kernels pays both kernels' tails, and with little to gain that
// costs more than it saves.  Integer sums: the same decision in every workgroup and on every call.  All threads of the
// workgroup call it together.
__device__ __forceinline__ bool sparse_steps_aside(const uint32_t* hints, const void* varlen, int varlen_bits, int B, int Hkv, int N) {
  __shared__ unsigned long long s_work[2];
  if (threadIdx.x < 2) s_work[threadIdx.x] = 0ull;
  __syncthreads();
  const int units = B * Hkv;
  unsigned long long mine = 0ull, all = 0ull;
  for (int u = threadIdx.x; u < units; u += blockDim.x) {
    long long l = N;
    if (varlen) {
      l = varlen_bits == 64 ? ((const long long*)varlen)[u / Hkv] : (long long)((const int*)varlen)[u / Hkv];
      l = l < 0 ? 0 : (l > N ? N : l);
    }
    all += (unsigned long long)(l * l);
    if (hints[2 * u] < (1u << 20)) mine += (unsigned long long)(l * l);
  }
  if (all) atomicAdd(&s_work[0], all);
  if (mine) atomicAdd(&s_work[1], mine);
  __syncthreads();
  return 2ull * s_work[1] < s_work[0] || s_work[1] == 0ull;
}

template <typename T, int D> struct SparseGeo {
  using G = TileGeo<T, D>;
  static constexpr int kNW = 4;
  static constexpr int kBM = 32 * kNW;
  static constexpr int kThreads = 64 * kNW;
  // K stages during the walks, with the waves' event rings behind them; afterwards the whole array holds the
  // candidate lists.  Two stages of 16-bit tiles: 39 KB, four workgroups per CU (one wave of each per SIMD); three
  // stages (52 KB at head dim 128, three workgroups per CU) measured slower.  The fp8 tiles of the first walk are
  // half as large and go through the same bytes in four stages.
  static constexpr int kStages = 2;
  static constexpr int kStages8 = 4;
  static constexpr int kK8Row = D;              // bytes per key row of the fp8 tile
  static constexpr int kK8Tile = kBN * kK8Row;
  static constexpr int kK8Loads = kK8Tile / 1024;
  static constexpr int kMinLds = 39 * 1024;  // (1 KB left for the small arrays)
  static constexpr int kLds = kStages * G::kKTile + 4608 > kMinLds ? kStages * G::kKTile + 4608 : kMinLds;  // rings of >= 32 events
  static constexpr int kWaveLds = kLds / kNW;
  // candidates per wave: scores (fp32) and keys (16 bits: the path serves up to 65536 keys) in two arrays, then the
  // rows' counters, offsets and 1 / sum
  static constexpr int kListCapRaw = (kWaveLds - 512) / 6 / 8 * 8;
  static constexpr int kListCap = kListCapRaw > kSparseStreamCap ? kSparseStreamCap : kListCapRaw;
  static constexpr int kRingBytes = (kLds - kStages * G::kKTile) / kNW;
  static constexpr int kRing = kRingBytes / 36 > 192 ? 192 : kRingBytes / 36;  // events: 8 scores and a tag
  static_assert(kRing >= 32, "half a wave can bring 32 events at once");
};

template <typename T, int D, int AM>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(ADSP_SPARSE_WAVES, ADSP_SPARSE_WAVES))) void attn_fwd_sparse_kernel(AttnParams p) {
  using G = TileGeo<T, D>;
  using SG = SparseGeo<T, D>;
  using KS = Swz<G::kKRow>;
  using KS8 = Swz<SG::kK8Row>;
  static_assert(G::k16, "16-bit element types only");
  static_assert(D % 64 == 0, "the fp8 products take 64 values of the head dim at a time");
  static_assert(AM == ATT_15 || AM == ATT_2 || AM == ATT_GEN, "alpha = 1.5, 2 or any other in (1, 2)");
  constexpr int NW = SG::kNW, BM = SG::kBM;
  __shared__ __align__(1024) unsigned char lds_all[SG::kLds];
  __shared__ int s_item;
  // a lane ran out of event slots, or a wave out of list room.  Two words: the walks write the one of the tile's
  // parity and read the other one behind the next barrier, so no wave can read a word another one is still setting
  __shared__ uint32_t s_giveup[2];
  extern __shared__ uint32_t mask_out[];  // p.mask_words words: key tiles that hold a non-zero probability

  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int N = p.N;
  const int n_mblk = (N + BM - 1) / BM;
  const int group = p.Hq / p.Hkv;
  const long long total = (long long)p.B * p.Hkv * n_mblk * group;
  const long long per_xcd = (total + 7) / 8;
  const float qs = p.qscale, inv_qs = 1.f / p.qscale;
  constexpr int kKPer = (G::kKLoads + NW - 1) / NW;
  constexpr int kK8Per = SG::kK8Loads / NW;
  static_assert(SG::kK8Loads % NW == 0 && (NW * 64 / KS8::kC) % 16 == 0, "every wave loads whole KBs of the fp8 tile, with one swizzle");
  static_assert(SG::kStages8 * SG::kK8Tile <= SG::kStages * G::kKTile, "the fp8 stages lie inside the 16-bit ones");
  constexpr bool kKStep = (NW * 64 / KS::kC) % 16 == 0 && (NW * 64) % KS::kC == 0;
  static_assert(kKStep && G::kKLoads % NW == 0, "head dims 32 .. 128");

  if (sparse_steps_aside(p.hints, p.varlen, p.varlen_bits, p.B, p.Hkv, p.N)) {
    if (blockIdx.x == 0 && threadIdx.x == 0) p.queue[kCtrlAllDense] = 1u;
    return;
  }
  int queues_tried = 0;  // thread 0: how many of the eight counters were found empty
  for (;;) {
    // The lane's constants are formed anew for every row block (the empty asm hides that they repeat): hoisted out
    // of this loop they would stay live through both walks, and the walks have no registers to spare.
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const int lane = tid & 63, lq = lane & 31, lh = lane >> 5;
    // tile DMA and fragment-read geometry (see attn_fwd_kernel)
    const uint32_t koff = (uint32_t)((wave * 64 + lane) / KS::kC * G::kKRow + ((((wave * 64 + lane) % KS::kC) ^ KS::sw((wave * 64 + lane) / KS::kC)) << 4));
    const uint32_t k_lane = (uint32_t)(lq * G::kKRow + ((lh ^ KS::sw(lq)) << 4));
    // the same for the fp8 tile: rows of D bytes, a lane's 32 values of a 64-value slice are two adjacent chunks
    const uint32_t koff8 = (uint32_t)((wave * 64 + lane) / KS8::kC * SG::kK8Row + ((((wave * 64 + lane) % KS8::kC) ^ KS8::sw((wave * 64 + lane) / KS8::kC)) << 4));
    const uint32_t k8_lane = (uint32_t)(lq * SG::kK8Row + (((2 * lh) ^ KS8::sw(lq)) << 4));

    __syncthreads();  // the previous row block is done with LDS and with s_item
    if (tid == 0) {
      int got = -1;
      while (queues_tried < 8) {
        const int x = ((int)(blockIdx.x & 7) + queues_tried) & 7;
        const long long i = (long long)atomicAdd(&p.queue[x], 1u);
        const long long logical = (long long)x * per_xcd + i;
        if (i < per_xcd && logical < total) {
          got = (int)logical;
          break;
        }
        ++queues_tried;
      }
      s_item = got;
      s_giveup[0] = 0u;
      s_giveup[1] = 0u;
    }
    for (int i = tid; i < p.mask_words; i += SG::kThreads) mask_out[i] = 0u;
    __syncthreads();
    const int logical = s_item;
    if (logical < 0) break;

    // ---- row block -> (batch, kv head, row block, head in group), as in attn_fwd_kernel ---------------------
    const int hg = logical % group;
    const int mi = (logical / group) % n_mblk;
    int bkv = logical / (group * n_mblk);
    {
      const int units = p.B * p.Hkv;
      if (units % 8 == 0) bkv = (bkv % (units / 8)) * 8 + bkv / (units / 8);
    }
    const int b = bkv / p.Hkv, kvh = bkv % p.Hkv;
    const int h = kvh * group + hg;
    const int mblk = n_mblk - 1 - mi;
    const int m0 = mblk * BM;
    int L = N;
    if (p.varlen) {
      long long l = p.varlen_bits == 64 ? ((const long long*)p.varlen)[b] : (long long)((const int*)p.varlen)[b];
      L = (int)(l < 0 ? 0 : (l > N ? N : l));
    }
    int32_t* const flag = p.block_flags + ((size_t)(b * p.Hq + h) * n_mblk + mblk);
    const size_t qo_base = ((size_t)(b * p.Hq + h) * N) * D;
    const size_t kv_base = ((size_t)(b * p.Hkv + kvh) * N) * D;
    int32_t* const bmask_out = p.bmask ? p.bmask + ((size_t)(b * p.Hq + h) * p.n_mblk + (size_t)mblk) * p.mask_words : nullptr;
    const int qi = m0 + wave * 32 + lq;

    if (m0 >= L) {  // row block entirely inside the padding: zero rows, empty mask
      if (bmask_out)
        for (int i = tid; i < p.mask_words; i += SG::kThreads) bmask_out[i] = 0;
      constexpr int kRowDw = D * 2 / 4;
      uint32_t* o32 = reinterpret_cast<uint32_t*>(p.out) + (qo_base + (size_t)m0 * D) * 2 / 4;
      const int rows = (N - m0) < BM ? (N - m0) : BM;
      for (int i = tid; i < rows * kRowDw; i += SG::kThreads) o32[i] = 0u;
      if (tid == 0) *flag = 0;
      continue;
    }

    const int row_hi = (m0 + BM < L ? m0 + BM : L);
    // The probe's verdict: with this K/V head's score spread, rows that see more keys than `w1_scales[...][2]` are
    // predicted to have supports beyond what the lists hold; such a row block goes to the dense kernel unseen.  (The
    // same inputs take the same way on every call: nothing here depends on what other workgroups do.)
    if ((float)(p.causal ? row_hi : L) > p.w1_scales[4 * (b * p.Hkv + kvh) + 2]) {
      if (tid == 0) {
        *flag = 1;
        atomicAdd(&p.queue[kCtrlFlagged], 1u);
      }
      continue;
    }
    const int nt = p.causal ? (row_hi + kBN - 1) / kBN : (L + kBN - 1) / kBN;
    const int lim = p.causal ? (qi < L - 1 ? qi : L - 1) : L - 1;
    const int wave_row0 = m0 + wave * 32;
    const bool live = qi < L;

    // ---- Q fragments of the first walk, rounded to e4m3: per 64-value slice of the head dim the lane holds the 32
    // values [32 lh, 32 lh + 32) of its row, in the order of the copy of K.  Rows past the valid length are zero
    // (their scores are never used). ------------------------------------------------------------------------------
    const uint16_t* const qrow = reinterpret_cast<const uint16_t*>(p.q) + qo_base + (size_t)(live ? qi : 0) * D;
    const float aq = p.w1_scales[4 * (b * p.Hkv + kvh)], aqk = aq * p.w1_scales[4 * (b * p.Hkv + kvh) + 1];
    uint32_t q8[D / 64 * 8];
    uint32_t qf[G::kQRegs];  // those of the 16-bit products: loaded behind the first walk
#pragma unroll
    for (int c = 0; c < D / 64; ++c) {
#pragma unroll
      for (int hq = 0; hq < 4; ++hq) {
        const u32x4 raw = *reinterpret_cast<const u32x4*>(qrow + c * 64 + lh * 32 + hq * 8);
#pragma unroll
        for (int e = 0; e < 4; e += 2) {
          uint32_t w = cvt_e4m3_pair(grid16(aq * unpack_lo<T>(raw[e])), grid16(aq * unpack_hi<T>(raw[e])), 0u, false);
          w = cvt_e4m3_pair(grid16(aq * unpack_lo<T>(raw[e + 1])), grid16(aq * unpack_hi<T>(raw[e + 1])), w, true);
          q8[c * 8 + hq * 2 + (e >> 1)] = live ? w : 0u;
        }
      }
    }

    const unsigned char* kglob = reinterpret_cast<const unsigned char*>(p.k) + kv_base * 2;
    const unsigned char* k8glob = p.k8 + (size_t)(b * p.Hkv + kvh) * (size_t)p.Npad * SG::kK8Row;
    // (the copy is padded to whole tiles, so no tile sticks out)
    auto issue_k8 = [&](unsigned char* lds, int kt) {
      const unsigned char* base = uniform_ptr(k8glob + (size_t)kt * SG::kK8Tile);
#pragma unroll
      for (int j0 = 0; j0 < kK8Per; ++j0) dma16s(base + j0 * (NW * 1024), koff8, lds + (j0 * NW + wave) * 1024);
    };
    auto issue_k = [&](unsigned char* lds, int kt) {
      const unsigned char* base = uniform_ptr(kglob + (size_t)kt * G::kKTile);
      if ((kt + 1) * kBN <= N) {
#pragma unroll
        for (int j0 = 0; j0 < kKPer; ++j0) dma16s(base + j0 * (NW * 1024), koff, lds + (j0 * NW + wave) * 1024);
      } else {  // the last tile sticks out of the tensor: rows past the end are masked later, any valid row will do
        const unsigned char* g = uniform_ptr(kglob);
        const int row0 = (int)(koff / G::kKRow);
        const uint32_t coff = koff % G::kKRow;
#pragma unroll
        for (int j0 = 0; j0 < kKPer; ++j0) {
          int gk = kt * kBN + row0 + j0 * (NW * 64 / KS::kC);
          gk = gk < N ? gk : N - 1;
          dma16s(g, (uint32_t)gk * (uint32_t)G::kKRow + coff, lds + (j0 * NW + wave) * 1024);
        }
      }
    };
    // body(kt, tile) over all key tiles of the row block; stops when a lane gave up.  The K tiles go through a ring of
    // kStages LDS buffers: the load of tile t + kStages - 1 is issued behind the barrier that opens tile t (every wave
    // is done with tile t - 1, whose buffer it takes) and has kStages - 1 tile times to arrive.
    // (stages_c, tile_c, per_c: the ring's depth, the bytes of a tile and the loads per wave and tile, as constants)
    auto walk = [&](auto stages_c, auto tile_c, auto per_c, auto&& issue, auto&& body) {
      constexpr int kStages = decltype(stages_c)::value, kTile = decltype(tile_c)::value, kPer = decltype(per_c)::value;
      __syncthreads();
#pragma unroll
      for (int s = 0; s < kStages - 1; ++s)
        if (s < nt) issue(lds_all + s * kTile, s);
      int stage = 0;  // buffer of tile cur
      for (int cur = 0; cur < nt; ++cur) {
        // this wave's share of tile cur has landed: everything but the loads issued after it (those of the tiles in
        // between; stores issued after it only make the wait longer than needed)
        if (cur + kStages - 1 <= nt) {
          if constexpr (kStages == 2) __builtin_amdgcn_s_waitcnt(0x0f70);
          else __builtin_amdgcn_s_waitcnt(0x0f70 | ((kStages - 2) * kPer));
        } else {
          __builtin_amdgcn_s_waitcnt(0x0f70);  // the last tiles: nothing was issued behind them
        }
        __syncthreads();
        if (s_giveup[(cur + 1) & 1]) break;  // set while the previous tile was worked on
        const int pre = cur + kStages - 1;
        if (pre < nt) issue(lds_all + (stage == 0 ? kStages - 1 : stage - 1) * kTile, pre);
        __builtin_amdgcn_sched_barrier(0);
        body(cur, lds_all + stage * kTile);
        stage = stage + 1 == kStages ? 0 : stage + 1;
      }
    };
    // accumulator start values of the first walk (opaque to the compiler: they must stay in registers)
    float ctag[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      ctag[i] = 1536.f + (float)i * (1.f / 8192.f);
      asm volatile("" : "+v"(ctag[i]));
    }
    // approximate S^T of one tile from the fp8 operands; f(s0, s1) unless no row of the wave sees the tile.  A score
    // is 1536 + (the sum of the products, a multiple of 2^-8 below 512 in size) + (its index among the lane's 16
    // values of the block) 2^-13: a float in [1024, 2048) whose mantissa holds the index in bits 0 .. 3 and the sum
    // from bit 5 on.  Scores past a row's last valid key are 0.
    auto for_tile8 = [&](int kt, const unsigned char* kt_lds, auto&& f) {
      if (p.causal && kt * kBN > wave_row0 + 31) return;
      const bool need_mask = (kt * kBN + kBN - 1 > L - 1) || (p.causal && kt * kBN + kBN - 1 > wave_row0);
      f32x16 s0, s1;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        s0[i] = ctag[i];
        s1[i] = ctag[i];
      }
      uint32_t ka = (uint32_t)(uintptr_t)kt_lds + k8_lane;
      asm volatile("" : "+v"(ka));
      u32x4 a0[D / 32], a1[D / 32];
#pragma unroll
      for (int c = 0; c < D / 32; ++c) a0[c] = lds_read16(ka ^ (((c >> 1) * 4 + (c & 1)) << 4));
#pragma unroll
      for (int c = 0; c < D / 32; ++c) a1[c] = lds_read16(ka ^ (((c >> 1) * 4 + (c & 1)) << 4), 32 * SG::kK8Row);
#pragma unroll
      for (int c = 0; c < D / 64; ++c) s0 = mfma_fp8(a0[2 * c], a0[2 * c + 1], q8 + c * 8, s0);
#pragma unroll
      for (int c = 0; c < D / 64; ++c) s1 = mfma_fp8(a1[2 * c], a1[2 * c + 1], q8 + c * 8, s1);
      if (need_mask) {
        const int jb = kt * kBN + 4 * lh;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          s0[i] = (jb + 8 * (i >> 2) + (i & 3) <= lim) ? s0[i] : kW1Masked;
          s1[i] = (jb + 32 + 8 * (i >> 2) + (i & 3) <= lim) ? s1[i] : kW1Masked;
        }
      }
      f(s0, s1);
    };
    // S^T of one tile (two 32-key blocks), accumulators preloaded with `init`; f(s0, s1) unless no row of the wave
    // sees the tile.  Scores past a row's last valid key are -inf.
    auto for_tile = [&](int kt, const unsigned char* kt_lds, float init, auto&& f) {
      if (p.causal && kt * kBN > wave_row0 + 31) return;
      const bool need_mask = (kt * kBN + kBN - 1 > L - 1) || (p.causal && kt * kBN + kBN - 1 > wave_row0);
      f32x16 s0, s1;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        s0[i] = init;
        s1[i] = init;
      }
      uint32_t ka = (uint32_t)(uintptr_t)kt_lds + k_lane;
      asm volatile("" : "+v"(ka));
      u32x4 a0[D / 16], a1[D / 16];
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) a0[ks] = lds_read16(ka ^ (ks << 5));
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) a1[ks] = lds_read16(ka ^ (ks << 5), 32 * G::kKRow);
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) {
        u32x4 bq = {qf[ks * 4], qf[ks * 4 + 1], qf[ks * 4 + 2], qf[ks * 4 + 3]};
        s0 = mfma_16bit<T>(a0[ks], bq, s0);
      }
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) {
        u32x4 bq = {qf[ks * 4], qf[ks * 4 + 1], qf[ks * 4 + 2], qf[ks * 4 + 3]};
        s1 = mfma_16bit<T>(a1[ks], bq, s1);
      }
      // the order of issue: four fragment reads ahead of the first product, then one read behind every product
      __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
      for (int i = 0; i < 2 * (D / 16) - 4; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
      if (need_mask) {
        const int jb = kt * kBN + 4 * lh;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          s0[i] = (jb + 8 * (i >> 2) + (i & 3) <= lim) ? s0[i] : -INFINITY;
          s1[i] = (jb + 32 + 8 * (i >> 2) + (i & 3) <= lim) ? s1[i] : -INFINITY;
        }
      }
      f(s0, s1);
    };

    // ---- walk 1: the four largest block maxima of the lane's keys ---------------------------------------------
    // A block maximum becomes a 29-bit word: the sum in steps of 1/16 (14 bits), the 32-key block (11 bits), the
    // position in the block (4 bits); unsigned comparisons order the words by their sums.  Words whose sum field is
    // 0 (nothing seen, or only masked scores) stand for no key.
    // A flat score distribution (a support of hundreds of keys) shows early: most block maxima lie close to the
    // running maximum.  Tiles 6 .. 11 are counted; if more than half of their (lane, block) maxima lie within 1/4 (in
    // z) of the lane's running maximum, the row block is given up before the walk is over.  A heuristic that only
    // decides which kernel does the work.
    uint32_t t1 = 0u, t2 = 0u, t3 = 0u, t4 = 0u;
    auto keep_top = [&](uint32_t x) {
      const uint32_t n2 = umed3(t1, t2, x), n3 = umed3(t2, t3, x), n4 = umed3(t3, t4, x);
      t1 = t1 > x ? t1 : x;
      t2 = n2;
      t3 = n3;
      t4 = n4;
    };
    int near_cnt = 0;
    const uint32_t near_d = (uint32_t)fminf(0.25f * inv_qs * 16.f * aqk, 8191.f) << 15;
    walk(std::integral_constant<int, SG::kStages8>{}, std::integral_constant<int, SG::kK8Tile>{}, std::integral_constant<int, kK8Per>{}, issue_k8, [&](int kt, const unsigned char* kt_lds) {
      for_tile8(kt, kt_lds, [&](const f32x16& s0, const f32x16& s1) {
        float m0v = fmaxf(s0[0], s0[1]), m1v = fmaxf(s1[0], s1[1]);
#pragma unroll
        for (int i = 2; i < 16; i += 2) {
          m0v = fmaxf(fmaxf(m0v, s0[i]), s0[i + 1]);
          m1v = fmaxf(fmaxf(m1v, s1[i]), s1[i + 1]);
        }
        const uint32_t b0 = __builtin_bit_cast(uint32_t, m0v), b1 = __builtin_bit_cast(uint32_t, m1v);
        const uint32_t k0 = (((b0 >> 9) & 0x3fffu) << 15) | ((b0 & 15u) | ((uint32_t)(2 * kt) << 4));
        const uint32_t k1 = (((b1 >> 9) & 0x3fffu) << 15) | ((b1 & 15u) | ((uint32_t)(2 * kt + 1) << 4));
        keep_top(k0);
        keep_top(k1);
        if (kt >= 6 && kt < 12) {
          const uint32_t near = t1 > near_d ? t1 - near_d : 0u;
          near_cnt += __builtin_popcountll(__builtin_amdgcn_ballot_w64(live && k0 > near)) + __builtin_popcountll(__builtin_amdgcn_ballot_w64(live && k1 > near));
          if (kt == 11 && near_cnt > 6 * 128 / 2 && lane == 0) s_giveup[1] = 1u;
        }
      });
    });

    __syncthreads();
    if (s_giveup[0] | s_giveup[1]) {  // a flat score distribution: the dense kernel's case
      if (tid == 0) {
        *flag = 1;
        atomicAdd(&p.queue[kCtrlFlagged], 1u);
        atomicAdd(&p.queue[kCtrlGaveUp], 1u);
      }
      continue;
    }
#if ADSP_SPARSE_STOP == 1
    continue;
#endif
    // ---- lower bound of the row's threshold from its eight kept values (raw score units) --------------------
    // f(t) = qs^2 sum (r - t)_+^2 - 1 (alpha 1.5) or qs sum (r - t)_+ - 1 (alpha 2) is convex and decreasing and
    // f(max - 1 / qs) >= 0, so Newton from there approaches the subset's root from the left and never passes it.
    // ---- Q fragments of the 16-bit products ----------------------------------------------------------------------
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) {
      const u32x4 raw = *reinterpret_cast<const u32x4*>(qrow + ks * 16 + 8 * lh);
#pragma unroll
      for (int e = 0; e < 4; ++e) qf[ks * 4 + e] = live ? raw[e] : 0u;
    }
    // ---- the scores of the row's eight chosen keys from the 16-bit inputs, with the products of the second walk: in
    // product m the A operand's row i is the key that row i chose as its m-th (a lane fetches its slice of that key's
    // row from memory), so the diagonal of S^T holds the wanted scores, bit for bit those the second walk will see
    // ----------------------------------------------------------------------------------------------------------------
    float r[8];
    {
      // The rows of the chosen keys are gathered into LDS the way the walks' tiles get there: per product m the wave
      // loads a 32-row "tile" whose row i is the key that row i chose as its m-th, with 1 KB DMA instructions (a
      // group of kC lanes per key row: whole rows, coalesced), and reads the A fragments from it as from a K tile.
      const uint32_t u[4] = {t1, t2, t3, t4};
      constexpr int kRowsPer = 64 / KS::kC;   // key rows per 1 KB DMA instruction
      constexpr int kInstr = 32 / kRowsPer;   // instructions per gathered tile
      uint32_t* const ktab = reinterpret_cast<uint32_t*>(lds_all + SG::kStages * G::kKTile + wave * SG::kRingBytes);  // [8][kRowsPer][kInstr]
      unsigned char* const gtile = lds_all + wave * (32 * G::kKRow);
      bool okm[4], okp[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t w = u[i];
        okm[i] = (w >> 15) != 0u;
        uint32_t key = ((w >> 4) & 0x7ffu) * 32u + 8u * ((w & 15u) >> 2) + (w & 3u) + 4u * (uint32_t)lh;
        // (a position that did not survive -- sums beyond the tags' range -- may name a key the row does not see: only
        // scores of the row's own keys bound its threshold)
        okm[i] = okm[i] && (int)key <= lim;
        key = okm[i] ? key : 0u;
        ktab[(4 * lh + i) * 32 + (lq % kRowsPer) * kInstr + lq / kRowsPer] = key;
        okp[i] = __shfl_xor((int)okm[i], 32, 64) != 0;
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
      const int diag = ((lq >> 3) << 2) | (lq & 3);  // which of the lane's 16 values of a block belongs to key lq of the block,
      const bool diag_here = lh == ((lq >> 2) & 1);  // and which of the row's two lanes holds it
      const unsigned char* kg = uniform_ptr(kglob);
      const int grow = lane / KS::kC, gslot = lane % KS::kC;
#pragma unroll
      for (int m = 0; m < 8; ++m) {
        uint32_t keys[kInstr];
#pragma unroll
        for (int j = 0; j < kInstr; j += 4) {
          const u32x4 kk = *reinterpret_cast<const u32x4*>(&ktab[m * 32 + grow * kInstr + j]);
          keys[j] = kk[0];
          keys[j + 1] = kk[1];
          keys[j + 2] = kk[2];
          keys[j + 3] = kk[3];
        }
#pragma unroll
        for (int j = 0; j < kInstr; ++j) {
          const int rr = j * kRowsPer + grow;
          dma16s(kg, keys[j] * (uint32_t)G::kKRow + (uint32_t)((gslot ^ KS::sw(rr)) << 4), gtile + j * 1024);
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): the gathered tile is in LDS (this wave's own loads)
        f32x16 acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.f;
        uint32_t ka = (uint32_t)(uintptr_t)gtile + k_lane;
        asm volatile("" : "+v"(ka));
        u32x4 af[D / 16];
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) af[ks] = lds_read16(ka ^ (ks << 5));
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) acc = mfma_16bit<T>(af[ks], u32x4{qf[ks * 4], qf[ks * 4 + 1], qf[ks * 4 + 2], qf[ks * 4 + 3]}, acc);
        float d = acc[0];
#pragma unroll
        for (int i = 1; i < 16; ++i) d = diag == i ? acc[i] : d;
        const float other = __shfl_xor(d, 32, 64);
        d = diag_here ? d : other;
        const bool ok = ((m < 4) == (lh == 0)) ? okm[m & 3] : okp[m & 3];
        r[m] = ok ? d : -INFINITY;
      }
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the last fragment reads are done before the tiles of walk 2 arrive
    }
    float lo_raw;
    {
      const float rmax = fmaxf(r[0], r[4]);
      float t = rmax - inv_qs;
      const float target = (AM == ATT_15) ? inv_qs * inv_qs : inv_qs;
#pragma unroll 1
      for (int it = 0; it < 8; ++it) {
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float u = fmaxf(r[i] - t, 0.f);
          if constexpr (AM == ATT_15) {
            a0 = fmaf(u, u, a0);
            a1 += u;
          } else if constexpr (AM == ATT_2) {
            a0 += u;
            a1 += u > 0.f ? 1.f : 0.f;
          } else {  // any alpha: sums of (qs u)^c0 and (qs u)^(c0 - 1), in z units
            const float uz = u * qs;
            const float pw = u > 0.f ? fast_exp2(p.c0 * fast_log2(uz)) : 0.f;
            a0 += pw;
            a1 += u > 0.f ? pw * fast_rcp(uz) : 0.f;
          }
        }
        // (any alpha: f = a0 - 1, f' = -c0 qs a1 per raw unit; the steps of a convex decreasing f from the left never
        // pass its root, converged or not: what the eight rounds leave is a valid bound)
        const float step = (AM == ATT_15) ? (a0 - target) / (2.f * a1) : (AM == ATT_2) ? (a0 - target) / a1 : (a0 - 1.f) * inv_qs / (p.c0 * a1);
        t += (a1 > 0.f && step > 0.f) ? step : 0.f;
      }
      // the margin covers the rounding of the iteration; rows past the valid length take no part in walk 2
      lo_raw = t - (1e-5f * inv_qs + 1e-6f * fabsf(rmax));
      // (a row none of whose chosen keys could be used -- its first walk's sums left the tags' range -- has no bound:
      // the row block goes to the dense kernel; the second walk stops at its first tile)
      if (live && !(rmax > -INFINITY)) s_giveup[1] = 1u;
      lo_raw = (live && rmax > -INFINITY) ? lo_raw : INFINITY;
    }

#if ADSP_SPARSE_STOP == 2
    if (lo_raw == 12345.f) p.taus[qi] = lo_raw;  // (keeps the bound alive)
    continue;
#endif
    // ---- walk 2: collect the scores above the bound -------------------------------------------------------------
    // A lane whose eight scores of a 16-key half block have a positive maximum puts them, with a tag, into the wave's
    // ring in LDS (slots are handed out with a ballot: no atomics).  When the ring is full the wave empties it, one
    // event per lane: the positive entries go to the wave's candidate stream in global memory as (score - lo, key and
    // row) pairs, compact and in bursts, so the tile loop rarely waits for a store.
    float* const ring = reinterpret_cast<float*>(lds_all + SG::kStages * G::kKTile + wave * SG::kRingBytes);
    uint32_t* const ring_tag = reinterpret_cast<uint32_t*>(ring + SG::kRing * 8);
    // (kept for the backward, the stream has a place of its own per row block and wave)
    const size_t stream_id = ((size_t)(b * p.Hq + h) * n_mblk + mblk) * NW + wave;
    uint2* const stream = p.save_streams ? reinterpret_cast<uint2*>(p.save_streams) + stream_id * (size_t)kSparseStreamCap
                                         : reinterpret_cast<uint2*>(p.events) + ((size_t)blockIdx.x * NW + wave) * (size_t)kSparseStreamCap;
    int ring_n = 0, stream_n = 0;  // wave-uniform
    // (kt: the tile being worked on; a stream that fills faster than the tiles go by will not last: give up early)
    auto flush = [&](int parity, int kt) {
      for (int e0 = 0; e0 < ring_n; e0 += 64) {
        const int e = e0 + lane;
        const bool has = e < ring_n;
        f32x4 w0 = {0.f, 0.f, 0.f, 0.f}, w1 = {0.f, 0.f, 0.f, 0.f};
        uint32_t tag = 0u;
        if (has) {
          w0 = *reinterpret_cast<const f32x4*>(ring + e * 8);
          w1 = *reinterpret_cast<const f32x4*>(ring + e * 8 + 4);
          tag = ring_tag[e];
        }
        int c = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) c += (w0[i] > 0.f ? 1 : 0) + (w1[i] > 0.f ? 1 : 0);
        const int incl = wave_scan_i(c);
        const int total_c = __builtin_amdgcn_readlane(incl, 63);
        if (stream_n + total_c > SG::kListCap || (long long)(stream_n + total_c) * nt > (long long)SG::kListCap * (kt + 16)) {
          if (lane == 0) s_giveup[parity] = 1u;
        } else {
          // producer lane = tag & 63: row (tag & 31), key half (tag >> 5) & 1; half block (tag >> 6) & 3 of tile tag >> 8
          const uint32_t key0 = (tag >> 8) * kBN + ((tag >> 6) & 3u) * 16 + 4 * ((tag >> 5) & 1u);
          const uint32_t rowbits = (tag & 31u) << 20;
          uint2* dst = stream + stream_n + (incl - c);
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const float x = i < 4 ? w0[i & 3] : w1[i & 3];
            if (x > 0.f) {
              *dst = uint2{__builtin_bit_cast(uint32_t, x), (key0 + 8 * (i >> 2) + (i & 3)) | rowbits};
              ++dst;
            }
          }
          stream_n += total_c;
        }
      }
      ring_n = 0;
    };
    // the lanes of `m` (those of them for which `mine` holds put their half block) take consecutive ring slots
    auto put = [&](unsigned long long m, bool mine, const f32x16& s, int first, uint32_t tag, int kt) {
      const int c = __builtin_popcountll(m);
      if (ring_n + c > SG::kRing) flush(kt & 1, kt);
      if (mine) {
        const int slot = ring_n + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
        f32x4 w0 = {s[first], s[first + 1], s[first + 2], s[first + 3]};
        f32x4 w1 = {s[first + 4], s[first + 5], s[first + 6], s[first + 7]};
        *reinterpret_cast<f32x4*>(ring + slot * 8) = w0;
        *reinterpret_cast<f32x4*>(ring + slot * 8 + 4) = w1;
        ring_tag[slot] = (tag << 6) | (uint32_t)lane;
      }
      ring_n += c;
    };
    auto collect = [&](const f32x16& s, int first, float hmax, uint32_t tag, int kt) {
      const unsigned long long m = __builtin_amdgcn_ballot_w64(hmax > 0.f);
      if (m != 0ull) {
        if (__builtin_popcountll(m) <= SG::kRing) {
          put(m, hmax > 0.f, s, first, tag, kt);
        } else {  // more events than the ring holds at once (the first tiles of a sequence): in two halves
          put(m & 0xffffffffull, hmax > 0.f && lane < 32, s, first, tag, kt);
          put(m & ~0xffffffffull, hmax > 0.f && lane >= 32, s, first, tag, kt);
        }
      }
    };
    // One decision per tile: the four half blocks' events are counted together; when they fit the ring (after a flush
    // if need be) every lane writes its events at slots known from the four ballots, without further tests.  A tile
    // with more events than the ring holds (the first tiles of a sequence) goes through in eight parts.
    auto put_at = [&](unsigned long long m, bool mine, const f32x16& s, int first, uint32_t tag, int base) {
      if (mine) {
        const int slot = base + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
        f32x4 w0 = {s[first], s[first + 1], s[first + 2], s[first + 3]};
        f32x4 w1 = {s[first + 4], s[first + 5], s[first + 6], s[first + 7]};
        *reinterpret_cast<f32x4*>(ring + slot * 8) = w0;
        *reinterpret_cast<f32x4*>(ring + slot * 8 + 4) = w1;
        ring_tag[slot] = (tag << 6) | (uint32_t)lane;
      }
    };
    walk(std::integral_constant<int, SG::kStages>{}, std::integral_constant<int, G::kKTile>{}, std::integral_constant<int, kKPer>{}, issue_k, [&](int kt, const unsigned char* kt_lds) {
      for_tile(kt, kt_lds, -lo_raw, [&](const f32x16& s0, const f32x16& s1) {
        float h00 = s0[0], h01 = s0[8], h10 = s1[0], h11 = s1[8];
#pragma unroll
        for (int i = 1; i < 8; ++i) {
          h00 = fmaxf(h00, s0[i]);
          h01 = fmaxf(h01, s0[8 + i]);
          h10 = fmaxf(h10, s1[i]);
          h11 = fmaxf(h11, s1[8 + i]);
        }
        const unsigned long long m0 = __builtin_amdgcn_ballot_w64(h00 > 0.f), m1 = __builtin_amdgcn_ballot_w64(h01 > 0.f);
        const unsigned long long m2 = __builtin_amdgcn_ballot_w64(h10 > 0.f), m3 = __builtin_amdgcn_ballot_w64(h11 > 0.f);
        const int c0 = __builtin_popcountll(m0), c1 = __builtin_popcountll(m1), c2 = __builtin_popcountll(m2), c3 = __builtin_popcountll(m3);
        const int E = c0 + c1 + c2 + c3;
        if (E != 0) {
          int step = E <= SG::kRing ? -1 : 0;
          do {
            unsigned long long sub = 0ull;
            int need = E;
            if (step >= 0) {
              const int hb = step >> 1;
              sub = hb == 0 ? m0 : hb == 1 ? m1 : hb == 2 ? m2 : m3;
              sub &= (step & 1) ? ~0xffffffffull : 0xffffffffull;
              need = __builtin_popcountll(sub);
            }
            if (ring_n + need > SG::kRing) flush(kt & 1, kt);
            if (step < 0) {
              put_at(m0, h00 > 0.f, s0, 0, (uint32_t)(kt * 4 + 0), ring_n);
              put_at(m1, h01 > 0.f, s0, 8, (uint32_t)(kt * 4 + 1), ring_n + c0);
              put_at(m2, h10 > 0.f, s1, 0, (uint32_t)(kt * 4 + 2), ring_n + c0 + c1);
              put_at(m3, h11 > 0.f, s1, 8, (uint32_t)(kt * 4 + 3), ring_n + c0 + c1 + c2);
              step = 8;
            } else {
              const int hb = step >> 1;
              if ((sub >> lane) & 1ull) {
                f32x4 w0, w1;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                  w0[i] = hb == 0 ? s0[i] : hb == 1 ? s0[8 + i] : hb == 2 ? s1[i] : s1[8 + i];
                  w1[i] = hb == 0 ? s0[4 + i] : hb == 1 ? s0[12 + i] : hb == 2 ? s1[4 + i] : s1[12 + i];
                }
                const int slot = ring_n + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(sub >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)sub, 0u));
                *reinterpret_cast<f32x4*>(ring + slot * 8) = w0;
                *reinterpret_cast<f32x4*>(ring + slot * 8 + 4) = w1;
                ring_tag[slot] = ((uint32_t)(kt * 4 + hb) << 6) | (uint32_t)lane;
              }
              ++step;
            }
            ring_n += need;
          } while (step < 8);
        }
      });
    });
    flush(0, nt);
    __builtin_amdgcn_s_waitcnt(0x0f70);  // the wave's stream is in memory before it reads it back
    __syncthreads();                      // every wave has left the K tiles: LDS becomes the lists
    if (s_giveup[0] | s_giveup[1]) {
      if (tid == 0) {
        *flag = 1;
        atomicAdd(&p.queue[kCtrlFlagged], 1u);
        atomicAdd(&p.queue[kCtrlGaveUp], 1u);
      }
      continue;
    }

#if ADSP_SPARSE_STOP == 3
    continue;
#endif
    // ---- the wave's stream -> per-row lists in its share of LDS (a counting sort by row) ----------------------------
    unsigned char* const wave_lds = lds_all + wave * SG::kWaveLds;
    float* const lval = reinterpret_cast<float*>(wave_lds);                                  // kListCap scores, later probabilities
    uint16_t* const lkey = reinterpret_cast<uint16_t*>(wave_lds + SG::kListCap * 4);         // their keys
    uint32_t* const row_cnt = reinterpret_cast<uint32_t*>(wave_lds + SG::kListCap * 6);     // 32 counters
    uint32_t* const row_start = row_cnt + 32;                                                // 33 offsets
    float* const row_inv = reinterpret_cast<float*>(row_start + 33);                         // 32 x 1 / sum p
    if (lane < 32) row_cnt[lane] = 0u;
    {
      constexpr int kPer = (SG::kListCap + 63) / 64;
      uint2 ent[kPer];
      uint32_t pos[kPer];
#pragma unroll
      for (int j = 0; j < kPer; ++j) {
        const int e = j * 64 + lane;
        ent[j] = uint2{0u, 0u};
        if (e < stream_n) ent[j] = stream[e];
      }
#pragma unroll
      for (int j = 0; j < kPer; ++j) {
        const int e = j * 64 + lane;
        pos[j] = 0u;
        if (e < stream_n) pos[j] = atomicAdd(&row_cnt[(ent[j].y >> 20) & 31u], 1u);
      }
      {
        const int c = lane < 32 ? (int)row_cnt[lane] : 0;
        const int incl = wave_scan_i(c);
        if (lane < 32) row_start[lane] = (uint32_t)(incl - c);
        if (lane == 31) row_start[32] = (uint32_t)incl;
      }
#pragma unroll
      for (int j = 0; j < kPer; ++j) {
        const int e = j * 64 + lane;
        if (e < stream_n) {
          const uint32_t at = row_start[(ent[j].y >> 20) & 31u] + pos[j];
          lval[at] = __builtin_bit_cast(float, ent[j].x);
          lkey[at] = (uint16_t)(ent[j].y & 0xffffu);
          // the tile mask takes every candidate's tile: a superset of the tiles with a non-zero probability by the few
          // candidates below the threshold, cheaper to mark here (one entry per lane) than in the output loop
          const uint32_t tile = (ent[j].y & 0xffffu) / kBN;
          atomicOr(&mask_out[tile >> 5], 1u << (tile & 31));
        }
      }
    }

    // ---- threshold: Newton from the left on the row's candidates (its two lanes take alternate entries) -----------
    const int row_lo = (int)row_start[lq], row_end = (int)row_start[lq + 1];
    float t = 0.f;  // threshold minus lo, raw units
    {
      const float target = (AM == ATT_15) ? inv_qs * inv_qs : inv_qs;
      // (any alpha: the steps shrink like 1 - 1 / c0 while f is large, so the rounds are more; the launch keeps alphas
      // whose c0 = 1 / (alpha - 1) exceeds 8 on the dense kernel)
      // (four of the lane's entries per turn, read together; the longest list of the wave sets the number of turns, and
      // a lane past its list's end reads on inside the wave's LDS and takes -inf)
      const int max_len = (int)wave_max((float)(row_end - row_lo));
      for (int it = 0; it < (AM == ATT_GEN ? 96 : 24); ++it) {
        float a0 = 0.f, a1 = 0.f;
        for (int o = 0; o < max_len; o += 8) {
          const int e0 = row_lo + lh + o;
          const int e0r = e0 < SG::kListCap ? e0 : SG::kListCap;
          float x[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float raw = lval[e0r + 2 * j];
            x[j] = e0 + 2 * j < row_end ? raw : -INFINITY;
          }
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float u = fmaxf(x[j] - t, 0.f);
            if constexpr (AM == ATT_15) {
              a0 = fmaf(u, u, a0);
              a1 += u;
            } else if constexpr (AM == ATT_2) {
              a0 += u;
              a1 += u > 0.f ? 1.f : 0.f;
            } else {
              const float uz = u * qs;
              const float pw = u > 0.f ? fast_exp2(p.c0 * fast_log2(uz)) : 0.f;
              a0 += pw;
              a1 += u > 0.f ? pw * fast_rcp(uz) : 0.f;
            }
          }
        }
        a0 += __shfl_xor(a0, 32, 64);
        a1 += __shfl_xor(a1, 32, 64);
        const float step = (AM == ATT_15) ? (a0 - target) / (2.f * a1) : (AM == ATT_2) ? (a0 - target) / a1 : (a0 - 1.f) * inv_qs / (p.c0 * a1);
        const bool move = a1 > 0.f && step > (AM == ATT_GEN ? 2e-6f : 1e-7f) * inv_qs;  // (any alpha: the powers carry a relative 1e-6)
        t += move ? step : 0.f;
        if (__builtin_amdgcn_ballot_w64(move) == 0ull) break;
      }
    }
    // scores -> probabilities (not yet normalised): the row's first lane rewrites its list in place, keeping only the
    // support; 1 / sum per row
    {
      float psum = 0.f;
      int w = row_lo;
      if (lh == 0) {
        for (int e = row_lo; e < row_end; ++e) {
          const float u = lval[e] - t;
          const uint16_t key = lkey[e];
          if (u > 0.f) {
            const float pv = (AM == ATT_15) ? u * u : (AM == ATT_2) ? u : fast_exp2(p.c0 * fast_log2(u * qs));
            lval[w] = __builtin_bit_cast(float, pack2<T>(pv, 0.f));  // the pair (p, 0) of the element type, as the output loop takes it
            lkey[w] = key;
            ++w;
            psum += pv;
          }
        }
        row_cnt[lq] = (uint32_t)(w - row_lo);
        row_inv[lq] = (live && psum > 0.f) ? 1.f / psum : 0.f;
        if (live && p.taus) p.taus[(size_t)(b * p.Hq + h) * N + qi] = (lo_raw + t) * qs;
        if (live && p.save_tshift) p.save_tshift[(size_t)(b * p.Hq + h) * N + qi] = t;
      }
    }

#if ADSP_SPARSE_STOP == 4
    continue;
#endif
    // ---- output: a group of D / 8 lanes per row, each lane 8 columns; the V rows of a row's support are fetched
    // kDepth at a time (all in flight together), weighted, summed, and the row is stored with 16-byte accesses.  The
    // weights enter the two-term dot product as (p, 0) and (0, p) pairs of the element type, i.e. rounded to it, as
    // the P operand of the dense kernel's MFMA is. ---------------------------------------------------------------------
    {
      constexpr int kLPR = D / 8;         // lanes per row
      constexpr int kGroups = 64 / kLPR;  // rows in progress per wave
      constexpr int kDepth = ADSP_GATHER_DEPTH;
      const int grp = lane / kLPR, col = lane % kLPR;
      const unsigned char* vrows = reinterpret_cast<const unsigned char*>(p.v) + kv_base * 2;
      const uint32_t col16 = (uint32_t)col * 16u;  // (32-bit offsets per lane: a head's rows span N * D * 2 <= 16 MB)
      unsigned char* obase = reinterpret_cast<unsigned char*>(p.out) + (qo_base + (size_t)wave_row0 * D) * 2 + col * 16;
      // The rows are served kGroups at a time and a round lasts as long as its longest support: rows in the order of
      // their supports' sizes, longest first, keep the rows of a round alike.
      uint8_t* const order = reinterpret_cast<uint8_t*>(row_inv + 32);
      {
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        int rank = 0;
        const int mine = lane < 32 ? (int)row_cnt[lane] : 0;
        for (int o = 0; o < 32; ++o) {
          const int c = (int)row_cnt[o];
          rank += (c > mine || (c == mine && o < lane)) ? 1 : 0;
        }
        if (lane < 32) order[rank] = (uint8_t)lane;
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
      }
      for (int r0 = 0; r0 < 32; r0 += kGroups) {
        const int r = (int)order[r0 + grp];
        const int e_lo = (int)row_start[r], e_hi = e_lo + (int)row_cnt[r];
        float acc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = 0.f;
        // (the rows of a round come longest support first: the first group's row sets the number of turns)
        const int n_turns = (__builtin_amdgcn_readfirstlane(e_hi - e_lo) + kDepth - 1) / kDepth;
        for (int turn = 0; turn < n_turns; ++turn) {
          const int eb = e_lo + turn * kDepth;
          // (a group whose list has ended reads on without a condition, at a place inside the wave's LDS)
          const int ebr = eb < SG::kListCap ? eb : SG::kListCap;
          u32x4 vv[kDepth];
          uint32_t pw[kDepth];
#pragma unroll
          for (int j = 0; j < kDepth; ++j) {
            // a slot without a member takes the first key's row (always valid) with a zero weight: no zeroing, no branch
            const bool has = eb + j < e_hi;
            const uint32_t kraw = (uint32_t)lkey[ebr + j];
            const uint32_t wraw = __builtin_bit_cast(uint32_t, lval[ebr + j]);
            const uint32_t key = has ? kraw : 0u;
            pw[j] = has ? wraw : 0u;
            vv[j] = *reinterpret_cast<const u32x4*>(vrows + (key * (uint32_t)(D * 2) + col16));
          }
#pragma unroll
          for (int j = 0; j < kDepth; ++j) {
            dot2_chunk<T>(acc, vv[j], pw[j], pw[j] << 16);
          }
        }
        const float inv = row_inv[r];
        if (wave_row0 + r < N) {
          u32x4 w = {pack2<T>(acc[0] * inv, acc[1] * inv), pack2<T>(acc[2] * inv, acc[3] * inv),
                     pack2<T>(acc[4] * inv, acc[5] * inv), pack2<T>(acc[6] * inv, acc[7] * inv)};
          *reinterpret_cast<u32x4*>(obase + (size_t)r * (D * 2)) = w;
        }
      }
    }
    __syncthreads();  // every wave's tile marks are in
    if (bmask_out)
      for (int i = tid; i < p.mask_words; i += SG::kThreads) bmask_out[i] = (int32_t)mask_out[i];
    if (p.save_lens && lane == 0) p.save_lens[stream_id] = (uint16_t)stream_n;
    if (tid == 0) {
      *flag = 0;
      if (p.save_flags) p.save_flags[(size_t)(b * p.Hq + h) * n_mblk + mblk] = 1;
    }
  }
}

// Workgroups to launch: as many as fit the device at once (each owns one event slot), at most `max_slots`.
template <typename T, int D, int AM> static int launch_attn_sparse_one(const AttnParams& p, int max_slots, hipStream_t s) {
  using SG = SparseGeo<T, D>;
  auto kern = attn_fwd_sparse_kernel<T, D, AM>;
  static int per_cu = 0, n_cu = 0;  // (one device family per process: gfx950)
  const size_t dyn = (size_t)p.mask_words * sizeof(uint32_t);
  if (per_cu == 0) {
    int dev = 0, blocks = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 2;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, kern, SG::kThreads, dyn) != hipSuccess || blocks <= 0) blocks = 1;
    n_cu = prop.multiProcessorCount;
    per_cu = blocks;
  }
  long long grid = (long long)per_cu * n_cu;
  if (grid > max_slots) grid = max_slots;
  grid = grid / 8 * 8;  // the same number of workgroups on every XCD
  if (grid < 8) grid = 8;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(SG::kThreads), dyn, s, p);
  return 0;
}

template <typename T, int D> static int launch_attn_sparse(const AttnParams& p, int am, int max_slots, hipStream_t s) {
  if (am == ATT_15) return launch_attn_sparse_one<T, D, ATT_15>(p, max_slots, s);
  if (am == ATT_2) return launch_attn_sparse_one<T, D, ATT_2>(p, max_slots, s);
  if (am == ATT_GEN) return launch_attn_sparse_one<T, D, ATT_GEN>(p, max_slots, s);
  return 2;
}

}  // namespace adsp
