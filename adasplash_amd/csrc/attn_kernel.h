// Fused sparse entmax attention forward for gfx950 (one kernel: threshold solver + output).
//
// Work decomposition
//   workgroup = 4 waves, owns 128 consecutive query rows of one (batch, head) and is sized so that two to four
//   workgroups fit a CU; wave w owns rows [32w, 32w+32); inside a wave, lane l holds query row (l & 31)
//   and, of every 32-key block, the 16 keys {8g + 4(l >> 5) + r : g, r in 0..3} -- the C layout of the
//   32x32 MFMA when the product is taken as S^T = K Q^T.  All per-row quantities (max, histogram,
//   Halley sums, tau, sum of p) are therefore lane-local accumulators that need one cross-lane add
//   (lane ^ 32) per pass.
//   K tiles (64 keys) and V tiles go HBM/L2 -> LDS with direct 16-byte loads (no staging registers),
//   double-buffered: the next tile is in flight while the current one is multiplied.  Rows are
//   XOR-swizzled in 16-byte chunks instead of padded, so the DMA can write contiguous kilobytes and the
//   ds_read_b128 of 16 consecutive rows still covers all 64 banks.
//
// Passes over the K tiles of a row block (every pass recomputes S^T with MFMA; scores never leave
// registers).  s = q.k is kept in raw units and the (alpha-1)/sqrt(D) scale is applied to per-row
// scalars only, so the MFMA operands are the caller's q and k bit for bit:
//   A+B (alpha = 1.5 / 2) row max m and, in the same walk, a histogram of z on an absolute grid of bins of width
//      1/8 under the running maximum -> bracket [lo, lo + 1/8] of tau; tile mask {z within 1 of the running max}
//   A  (other alpha) row max m                            -> tau in [m - 1, m - n^(1-alpha)]
//   C  x niter: sums of u^c0, u^(c0-1), u^(c0-2)          -> Halley / Newton / bisection step; every one
//                                                           refines the tile mask to {z > lower bound}
//   D  p = [z - tau]_+^c0, out += P V over masked tiles, divided by sum p at the end.
// In walks C and D the accumulator of the S^T MFMA is initialised with -tau, so z - tau costs no VALU op.
//
// The PV product is taken as out^T = V^T P^T, so that P^T goes straight from the S^T accumulators into the next MFMA
// without an LDS round trip; the 16-bit V tiles are row-major like K's and the operand V^T comes out of the
// transposing LDS read (ds_read_b64_tr_b16).
#pragma once
#include <type_traits>
#include "common.h"
#include "solver.h"
#include "attn_params.h"

namespace adsp {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 h2_t __attribute__((ext_vector_type(2)));

typedef uint16_t u16x2_t __attribute__((ext_vector_type(2)));
// per 16-bit half: v >> sh, v << sh
__device__ __forceinline__ uint32_t pk_shr16(uint32_t v, uint32_t sh2) {
  return __builtin_bit_cast(uint32_t, __builtin_bit_cast(u16x2_t, v) >> __builtin_bit_cast(u16x2_t, sh2));
}
__device__ __forceinline__ uint32_t pk_shl16(uint32_t v, uint32_t sh2) {
  return __builtin_bit_cast(uint32_t, __builtin_bit_cast(u16x2_t, v) << __builtin_bit_cast(u16x2_t, sh2));
}
// bitwise full adder: a + b + c = sum + 2 carry
__device__ __forceinline__ void full_add(uint32_t a, uint32_t b, uint32_t c, uint32_t& sum, uint32_t& carry) {
  // one three-input bit operation each (truth tables of xor3 and majority)
  const uint32_t x = __builtin_amdgcn_bitop3_b32(a, b, c, 0x96);
  carry = __builtin_amdgcn_bitop3_b32(a, b, c, 0xe8);
  sum = x;
}

// two floats -> packed f16, rounded towards zero (one instruction)
__device__ __forceinline__ h2_t pkrtz(float a, float b) { return __builtin_bit_cast(h2_t, __builtin_amdgcn_cvt_pkrtz(a, b)); }

template <typename T> struct is16 { static constexpr bool value = true; };
template <> struct is16<float> { static constexpr bool value = false; };

template <typename T> __device__ __forceinline__ f32x16 mfma_16bit(u32x4 a, u32x4 b, f32x16 c);
template <> __device__ __forceinline__ f32x16 mfma_16bit<bf16_t>(u32x4 a, u32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}
template <> __device__ __forceinline__ f32x16 mfma_16bit<f16_t>(u32x4 a, u32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
}

// Sum of four 16-bit values of every lane on the matrix pipe: a 4x4x4 product in 16 blocks of four lanes with A = 1
// gives each lane, in every register of its accumulator, c + (the sum of its own four B values).  Two passes
// against the four vector additions it replaces, on a pipe that the vector-bound walks leave idle.
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
template <typename T> __device__ __forceinline__ f32x4_t lane_sum4(u32x2_t b, f32x4_t c);
template <> __device__ __forceinline__ f32x4_t lane_sum4<bf16_t>(u32x2_t b, f32x4_t c) {
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  const u32x2_t ones = {0x3f803f80u, 0x3f803f80u};
  return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(s16x4, ones), __builtin_bit_cast(s16x4, b), c, 0, 0, 0);
}
template <> __device__ __forceinline__ f32x4_t lane_sum4<f16_t>(u32x2_t b, f32x4_t c) {
  typedef _Float16 h16x4 __attribute__((ext_vector_type(4)));
  const u32x2_t ones = {0x3c003c00u, 0x3c003c00u};
  return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(h16x4, ones), __builtin_bit_cast(h16x4, b), c, 0, 0, 0);
}
template <> __device__ __forceinline__ f32x4_t lane_sum4<float>(u32x2_t, f32x4_t c) { return c; }

// 16-byte global -> LDS copy per lane: lane i of the wave writes LDS bytes [16 i, 16 i + 16) after the
// wave-uniform base `lds`, from its own global address.
__device__ __forceinline__ void dma16(const void* gsrc, void* lds) {
  // Issued as inline assembly on purpose: the compiler treats the builtin form as an access that may touch both
  // memory and LDS, and while one is in flight it waits for *every* outstanding LDS read (lgkmcnt(0)) before the
  // first use of any of them.  The hardware does not count this load in lgkmcnt (measured), so the tile loop's
  // own vmcnt(0) + barrier is all the ordering it needs; the "memory" clobber keeps LDS accesses from moving
  // across it.
  const uint32_t base = (uint32_t)(uintptr_t)lds;  // wave-uniform LDS byte address
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :
               : "v"(gsrc), "s"(__builtin_amdgcn_readfirstlane(base))
               : "memory");  // (m0 is a reserved register: the compiler sets it itself before each of its own uses)
}

// The same with the global address split into a wave-uniform base (a scalar register pair) and a 32-bit byte offset per
// lane: the tile loops keep the lane offsets in registers and form only the tile's base, with scalar instructions.
// A pointer the caller knows to be the same in every lane, moved to scalar registers (free when the compiler can see
// that it is uniform, two v_readfirstlane otherwise).
__device__ __forceinline__ const unsigned char* uniform_ptr(const void* ptr) {
  const unsigned long long a = (unsigned long long)(uintptr_t)ptr;
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(a >> 32));
  return reinterpret_cast<const unsigned char*>((uintptr_t)(((unsigned long long)hi << 32) | lo));
}
__device__ __forceinline__ void dma16s(const void* gbase, uint32_t off, void* lds) {
  const uint32_t base = (uint32_t)(uintptr_t)lds;
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(off), "s"(gbase), "s"(__builtin_amdgcn_readfirstlane(base))
               : "memory");  // (m0 is a reserved register: the compiler sets it itself before each of its own uses)
}

// 16-byte LDS read at a byte address held as an integer (plus a constant that lands in the instruction's offset field)
__device__ __forceinline__ u32x4 lds_read16(uint32_t addr, int imm = 0) {
  return *(const __attribute__((address_space(3))) u32x4*)(addr + imm);
}

// 8-byte transposing LDS read (ds_read_b64_tr_b16): within every group of 16 lanes, lane 4 r + c gives the address of four
// consecutive 16-bit values, and lane j receives, as its element r, value j % 4 of the four that lane 4 r + j / 4
// addressed.  With lane 4 r + c pointing at columns 4 c .. 4 c + 3 of row r of a row-major tile, lane j ends up with
// column j of rows 0 .. 3: an MFMA operand that runs along the rows, from a tile stored along the columns.
__device__ __forceinline__ u32x2_t lds_read8_tr(uint32_t addr, int imm = 0) {
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  return __builtin_bit_cast(u32x2_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(addr + imm)));
}

// Tile geometry.  A tile row has kC 16-byte chunks; chunk c of row r is stored at chunk position
// c ^ sw(r), with sw chosen so that 16 consecutive rows reading the same logical chunk touch 16 different
// 16-byte bank groups.
template <int ROW_BYTES> struct Swz {
  static constexpr int kC = ROW_BYTES / 16;
  static constexpr int kShift = kC >= 16 ? 0 : (kC == 8 ? 1 : (kC == 4 ? 2 : (kC == 2 ? 3 : 4)));
  static constexpr int kMask = (kC >= 16 ? 16 : kC) - 1;
  __device__ static __forceinline__ int sw(int row) { return (row >> kShift) & kMask; }
  __device__ static __forceinline__ int off(int row, int c) { return row * ROW_BYTES + ((c ^ sw(row)) << 4); }
};

template <typename T, int D> struct TileGeo {
  static constexpr bool k16 = is16<T>::value;
  static constexpr int kEB = k16 ? 2 : 4;
  static constexpr int kKRow = D * kEB;                // bytes per key row of the K tile
  static constexpr int kKTile = kBN * kKRow;
  static constexpr int kVRow = kKRow;  // the V tile has the K tile's format: [64 keys][D], row-major
  static constexpr int kVRows = kBN;
  static constexpr int kVTile = kVRows * kVRow;
  static constexpr int kNBuf = (2 * (kKTile + kVTile) <= 144 * 1024) ? 2 : 1;
  // Workgroups of four waves; two to four of them share a CU (registers and LDS permitting), one wave of each
  // per SIMD.  Their barriers are independent, so one workgroup's wait for a tile overlaps the others' MFMAs.
  static constexpr int kNW = 4;
  static constexpr int kBM = 32 * kNW;
  static constexpr int kThreads = 64 * kNW;
  // words of dynamic LDS after the tile masks: the waves' chunk counters and two flags
  static constexpr int kPoolTail = kNW + 2;
  // Waves per SIMD the register allocation is held to.  The walks are bound by dependent latency, so more
  // resident waves pay even at the price of a few spills: four for 16-bit D <= 64 (C5 23.3 -> 16.3 ms), three
  // for 16-bit D = 128 (168 registers; 12 % fewer cycles than two, part of which the clock gives back), two for
  // fp32 D <= 64, one for the shapes that need more than 256 registers.
  // 16-bit D = 128: one V tile instead of two (48 KB of tiles) lets three workgroups share a CU; the output walk
  // then loads a tile's V while its scores are computed and waits for it before the first PV product.
  static constexpr bool kVSingle = k16 && D == 128;
  static constexpr int kMinWaves = (k16 && D <= 64) ? 4 : (kVSingle ? 3 : ((!k16 && D <= 64) ? 2 : 1));
  static constexpr int kQRegs = k16 ? (D / 16) * 4 : D / 2;  // dwords of Q held per lane
  static constexpr int kDB = D >= 32 ? D / 32 : 1;           // 32-wide d blocks of the output
  static constexpr int kKLoads = kKTile / 1024;              // wave-level 1 KB DMA instructions per K tile
  static constexpr int kVLoads = kVTile / 1024;
};

template <int AM> __device__ __forceinline__ float attn_prob(float r, float qs, float c0) {
  // r = s - tau_raw in raw score units; the result only needs to be proportional to the probability
  // (the output is normalised by the row sum), so alpha = 1.5 and 2 skip the scale.
  if constexpr (AM == ATT_2) return __builtin_amdgcn_fmed3f(r, 0.f, INFINITY);
  if constexpr (AM == ATT_15) {
    float u = __builtin_amdgcn_fmed3f(r, 0.f, INFINITY);
    return u * u;
  }
  return r > 0.f ? fast_exp2(fast_log2(r * qs) * c0) : 0.f;
}

// Waves per SIMD the kernel is compiled for.  The list-carrying instance does not fit the 168 registers of three
// waves at 16-bit D = 128 (its solver walk spilled a hundred of them): it gets two waves' worth there.
template <typename T, int D, bool kMulti> constexpr int fwd_min_waves() {
  return (kMulti && TileGeo<T, D>::kVSingle) ? 2 : TileGeo<T, D>::kMinWaves;
}

// kMulti: the instance that carries the candidate lists of the solver walks and the per-wave block bits; it serves
// two and more solver steps, and a single step without the histogram (the block-mask variant, made for sparse
// supports).  The other one (no step, or one step behind the histogram) does not pay for their registers.
template <typename T, int D, int AM, bool kMulti>
__global__ __launch_bounds__((TileGeo<T, D>::kThreads))
__attribute__((amdgpu_waves_per_eu(fwd_min_waves<T, D, kMulti>(), (fwd_min_waves<T, D, kMulti>() > 2 ? fwd_min_waves<T, D, kMulti>() : 2)))) void attn_fwd_kernel(AttnParams p) {
  using G = TileGeo<T, D>;
  using KS = Swz<G::kKRow>;
  using VS = Swz<G::kVRow>;
  constexpr bool k16 = G::k16;
  constexpr int NW = G::kNW;
  constexpr int BM = G::kBM;
  // one array per pipeline stage: distinct objects let the compiler see that the DMA into one stage
  // never aliases the ds_reads of the other
  __shared__ __align__(1024) unsigned char k_lds0[G::kKTile];
  __shared__ __align__(1024) unsigned char v_lds0[G::kVTile];
  __shared__ __align__(1024) unsigned char k_lds1[G::kNBuf == 2 ? G::kKTile : 16];
  __shared__ __align__(1024) unsigned char v_lds1[(G::kNBuf == 2 && !G::kVSingle) ? G::kVTile : 16];
  // tile masks, sized by the launch for this problem's number of key tiles (4 x mask_words words of dynamic LDS):
  // two that the walks read and write in turn, and one per 128-row half of the row block for the bmask output.
  // With p.fine_masks another 2 x kNW x 2 x mask_words words follow: for each of the two walk masks and each
  // wave, one bit per 32-key block (bit 2 kt + kb) saying whether that wave's 32 rows need the block.
  extern __shared__ uint32_t mask_pool[];
  uint32_t* const mask_a = mask_pool;
  uint32_t* const mask_b = mask_pool + p.mask_words;
  uint32_t* const mask_out0 = mask_pool + 2 * p.mask_words;
  constexpr bool kFine = kMulti;  // the walks of a single step gain too little from them
  uint32_t* const fine_pool = kFine && p.fine_masks ? mask_pool + 4 * p.mask_words : nullptr;
  // after the masks, the bookkeeping of the candidate lists (see the solver walks): a chunk counter per wave and
  // two flag words
  constexpr int kPoolTail = G::kPoolTail;
  static_assert(kPoolTail == NW + 2, "launch and kernel disagree on the LDS tail");
  const int mask_pool_words = (p.fine_masks ? 4 + 4 * G::kNW : 4) * p.mask_words;
  uint32_t* const chunk_ctr = mask_pool + mask_pool_words;
  uint32_t* const list_flag = chunk_ctr + NW;

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, lives in an SGPR
  const int lane = tid & 63, lq = lane & 31, lh = lane >> 5;

  // ---- block -> (batch, kv head, row block, head in group): xcd_block_map; causal: longest row blocks first ----
  const int n_mblk = (p.N + BM - 1) / BM;
  const int group = p.Hq / p.Hkv;
  int bkv, mi, hg;
  if (!xcd_block_map(p.B * p.Hkv, n_mblk, group, p.causal != 0, 2ll * p.N * D * G::kEB, bkv, mi, hg)) return;  // (K and V of a head)
  const int b = bkv / p.Hkv, kvh = bkv % p.Hkv;
  const int h = kvh * group + hg;
  const int mblk = n_mblk - 1 - mi;
  const int m0 = mblk * BM;
  // behind the sparse-support kernel: only the row blocks it left over (its flags are per 128 rows, BM here)
  if (p.block_flags && p.queue[kCtrlAllDense] == 0u &&
      (p.queue[kCtrlFlagged] == 0u || p.block_flags[(size_t)(b * p.Hq + h) * n_mblk + mblk] == 0))
    return;

  const int N = p.N;
  int L = N;
  if (p.varlen) {
    long long l = p.varlen_bits == 64 ? ((const long long*)p.varlen)[b] : (long long)((const int*)p.varlen)[b];
    L = (int)(l < 0 ? 0 : (l > N ? N : l));
  }

  const size_t qo_base = ((size_t)(b * p.Hq + h) * N) * D;  // elements
  const size_t kv_base = ((size_t)(b * p.Hkv + kvh) * N) * D;
  // bmask rows are 128 query rows each, whatever BM this instantiation uses
  constexpr int kHalves = BM / kMaskRows;
  int32_t* bmask_out =
      p.bmask ? p.bmask + ((size_t)(b * p.Hq + h) * p.n_mblk + (size_t)mblk * kHalves) * p.mask_words : nullptr;

  const int qi = m0 + wave * 32 + lq;  // this lane's query row

  // Row block entirely inside the padding: zero output rows, empty mask.
  if (m0 >= L) {
    if (bmask_out) {
      for (int i = tid; i < kHalves * p.mask_words; i += G::kThreads)
        if (m0 + (i / p.mask_words) * kMaskRows < N) bmask_out[i] = 0;
    }
    constexpr int kRowDw = D * G::kEB / 4;
    uint32_t* o32 = reinterpret_cast<uint32_t*>(p.out) + (qo_base + (size_t)m0 * D) * G::kEB / 4;
    const int rows = (N - m0) < BM ? (N - m0) : BM;
    for (int i = tid; i < rows * kRowDw; i += G::kThreads) o32[i] = 0u;
    return;
  }

  const int row_hi = (m0 + BM < L ? m0 + BM : L);  // keys needed by the causal block: [0, row_hi)
  const int nt = p.causal ? (row_hi + kBN - 1) / kBN : (L + kBN - 1) / kBN;
  const int lim = p.causal ? (qi < L - 1 ? qi : L - 1) : L - 1;  // last valid key of this lane's row
  const int wave_row0 = m0 + wave * 32;
  const float qs = p.qscale, inv_qs = 1.f / p.qscale;

  // ---- Q fragments (unscaled) --------------------------------------------------------------------------
  uint32_t qf[G::kQRegs];
  {
    const bool ok = qi < N;
    if constexpr (k16) {
      const uint16_t* qrow = reinterpret_cast<const uint16_t*>(p.q) + qo_base + (size_t)(ok ? qi : 0) * D;
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) {
        u32x4 raw = *reinterpret_cast<const u32x4*>(qrow + ks * 16 + 8 * lh);
#pragma unroll
        for (int e = 0; e < 4; ++e) qf[ks * 4 + e] = ok ? raw[e] : 0u;
      }
    } else {
      const float* qrow = reinterpret_cast<const float*>(p.q) + qo_base + (size_t)(ok ? qi : 0) * D;
#pragma unroll
      for (int g = 0; g < D / 8; ++g) {
        u32x4 raw = *reinterpret_cast<const u32x4*>(qrow + 8 * g + 4 * lh);
#pragma unroll
        for (int e = 0; e < 4; ++e) qf[g * 4 + e] = ok ? raw[e] : 0u;
      }
    }
  }

  // ---- tile DMA ---------------------------------------------------------------------------------------
  const unsigned char* kglob = reinterpret_cast<const unsigned char*>(p.k) + kv_base * G::kEB;
  const unsigned char* vglob = reinterpret_cast<const unsigned char*>(p.v) + kv_base * G::kEB;

  // Wave-level load j of a tile fills LDS bytes [1024 j, 1024 j + 1024): chunk position P = 64 j + lane
  // belongs to row P / kC, stored chunk P % kC, i.e. logical chunk (P % kC) ^ sw(row).
  // Byte offsets of this lane's pieces inside a tile do not depend on the tile: they are kept in registers
  // and the DMA address is the tile's (wave-uniform) base plus that offset.
  // A wave's successive loads of a tile lie NW KB apart and NW * 64 / kC rows further down; when that is a multiple of
  // the swizzle period (16 rows) the lane's offset of load j0 is that of load 0 plus j0 * NW KB, which goes into the
  // scalar base: one offset register per tile kind instead of one per load.
  constexpr int kKPer = (G::kKLoads + NW - 1) / NW;
  constexpr bool kKStep = (NW * 64 / KS::kC) % 16 == 0 && (NW * 64) % KS::kC == 0;
  constexpr int kKOffs = kKStep ? 1 : kKPer;
  uint32_t koff[kKOffs], voff[kKOffs];
  // The 16-bit V tile has a swizzle of its own, made for the transposing reads of the output product.  Two groups of 16
  // lanes are served together: four rows (keys x .. x + 3) times two 32-byte column blocks, which must fall into
  // eight different 32-byte eighths of the 256 bytes that the 64 banks serve per cycle.  Rows 256 bytes or more apart
  // start in the same bank, so there the swizzle moves row r by 4 r chunks; rows of 128 bytes alternate between the
  // halves of the banks by themselves and are moved by 2 r (measured: no conflict cycles either way, against a
  // fifth of the LDS cycles with 2 r at 256 bytes).  Its period (4 rows) divides that of the K tile's, so the
  // scalar-base stepping of the loads holds for both.
  auto vsw = [](int row) -> int {
    if constexpr (k16) {
      constexpr int kC = KS::kC;
      if constexpr (kC >= 16) return (4 * row) & 15;
      else if constexpr (kC == 8) return (2 * row) & 7;
      else if constexpr (kC == 4) return row & 2;
      else return 0;
    } else {
      return KS::sw(row);
    }
  };
#pragma unroll
  for (int j0 = 0; j0 < kKOffs; ++j0) {
    const int P = (j0 * NW + wave) * 64 + lane;
    const int row = P / KS::kC;
    koff[j0] = (uint32_t)(row * G::kKRow + (((P % KS::kC) ^ KS::sw(row)) << 4));
    voff[j0] = (uint32_t)(row * G::kKRow + (((P % KS::kC) ^ vsw(row)) << 4));
  }
  // Swizzled read addresses without a register per fragment (three or four waves per SIMD leave none to spare): chunk c
  // of row r sits at r * row_bytes + ((c ^ sw(r)) << 4), and with c = 2 ks + lh that is
  // (r * row_bytes + ((lh ^ sw(r)) << 4)) ^ (ks << 5) -- one lane constant and one xor with an immediate per
  // read.  Rows r and r + 32 share sw, so the second key block is an offset.
  const uint32_t k_lane = (uint32_t)(lq * G::kKRow + ((lh ^ KS::sw(lq)) << 4));
  // The V operand of the output product (16-bit): out^T = V^T P^T wants, per lane, one output column d and eight keys
  // of a 16-key half -- in the order the score registers hold them: keys 4 g .. 4 g + 3 and 8 + 4 g .. 8 + 4 g + 3 for the
  // lane's half g = lane / 32 -- out of the row-major tile.  Two transposing reads bring them: in a group of 16 lanes,
  // lane 4 r + c points at key (4 g + r [+ 8]) and columns 4 c .. 4 c + 3 of the group's 16 columns (groups 0 / 2: columns
  // 0 .. 15 of a block of 32, groups 1 / 3: 16 .. 31).  The swizzle of these keys does not depend on the 16-key half, so the
  // lane's offsets are constants; the block of 32 columns is an xor with an immediate.
  uint32_t v_lane[2];
  {
    const int a = lane & 15, grp = lane >> 4, r = a >> 2, c = a & 3, g = grp >> 1, dl = grp & 1;
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      const int x = 4 * g + r + 8 * w;
      v_lane[w] = (uint32_t)(x * G::kVRow + (((2 * dl + (c >> 1)) ^ vsw(x)) << 4) + (c & 1) * 8);
    }
    if (D < 32 && dl) v_lane[0] = v_lane[1] = 0u;  // (D = 16: these lanes' columns do not exist; their operand is zeroed)
  }
  auto issue_rows = [&](const unsigned char* g, const uint32_t (&off)[kKOffs], unsigned char* lds, int kt, int limit, auto&& sw_of) {
    // a row-major [64][D] tile out of a row-major tensor (K or V); the last tile may stick out of the rows [0, limit)
    const unsigned char* base = uniform_ptr(g + (size_t)kt * G::kKTile);
    if ((kt + 1) * kBN <= limit) {  // one branch per tile, then straight-line loads
#pragma unroll
      for (int j0 = 0; j0 < kKPer; ++j0) {
        const int j = j0 * NW + wave;
        if (G::kKLoads % NW == 0 || j < G::kKLoads) {
          if constexpr (kKStep) dma16s(base + j0 * (NW * 1024), off[0], lds + j * 1024);
          else dma16s(base, off[j0], lds + j * 1024);
        }
      }
    } else {
#pragma unroll
      for (int j0 = 0; j0 < kKPer; ++j0) {
        const int j = j0 * NW + wave;
        if (G::kKLoads % NW == 0 || j < G::kKLoads) {
          const int P = j * 64 + lane;
          const int row = P / KS::kC, c = (P % KS::kC) ^ sw_of(row);
          int gk = kt * kBN + row;
          gk = gk < limit ? gk : limit - 1;  // rows past the end are masked later; any valid row will do
          dma16(g + (size_t)gk * G::kKRow + c * 16, lds + j * 1024);
        }
      }
    }
  };
  auto issue_k = [&](unsigned char* kb, int kt) { issue_rows(kglob, koff, kb, kt, N, [](int row) { return KS::sw(row); }); };
  // V: the same geometry.  Rows of v past the sequence's length may hold anything, and a zero probability does not
  // silence a NaN in the product: the 16-bit tiles take the last valid row in their place (fp32 zeroes the operand).
  auto issue_v = [&](unsigned char* vb, int kt) { issue_rows(vglob, voff, vb, kt, k16 ? L : N, vsw); };

  // Next tile index > cur allowed by `mask` (nullptr = every tile), or -1.  The mask word in use is kept in
  // a register, so LDS is read once per 32 tiles.
  int mw_index = -1;
  uint32_t mw_bits = 0u;
  // this wave's block bits of a walk mask (null: every block), and the pair of bits of tile kt, cached 16 tiles a word
  auto fine_of = [&](const uint32_t* mask) -> uint32_t* {
    if (!fine_pool || !mask) return nullptr;
    return fine_pool + ((mask == mask_a ? 0 : G::kNW) + wave) * 2 * p.mask_words;
  };
  int fw_index = -1;
  uint32_t fw_bits = 0u;
  auto block_bits = [&](const uint32_t* fine, int kt) -> uint32_t {
    if (!fine) return 3u;
    if ((kt >> 4) != fw_index) {
      fw_index = kt >> 4;
      fw_bits = (uint32_t)__builtin_amdgcn_readfirstlane((int)fine[fw_index]);
    }
    return (fw_bits >> ((kt & 15) * 2)) & 3u;
  };
  auto next_tile = [&](const uint32_t* mask, int cur) -> int {
    int t = cur + 1;
    if (!mask) return t < nt ? t : -1;
    while (t < nt) {
      if ((t >> 5) != mw_index) {
        mw_index = t >> 5;
        mw_bits = mask[mw_index];
      }
      const uint32_t w = mw_bits >> (t & 31);
      if (w) {
        t += __builtin_ctz(w);
        return t < nt ? t : -1;
      }
      t = (t | 31) + 1;
    }
    return -1;
  };

  // Runs body(kt, k_tile, v_tile) over the selected tiles; the DMA of the next tile is issued right
  // after the barrier that publishes the current one and completes under the current tile's MFMAs.
  bool k_after_v = false;  // single V tile: a K tile's loads were issued after the current V tile's
  auto tile_loop = [&](const uint32_t* mask, bool with_v, auto&& body) {
    __syncthreads();  // the previous pass is done with the LDS tiles; its mask writes are visible
    mw_index = -1;
    fw_index = -1;
    if constexpr (G::kVSingle) {
      if (with_v) {
        // K double-buffered, V single: the barrier that publishes K(t) also says every wave is done with V(t-1);
        // V(t) is then loaded under the score product of tile t and the body waits for it (a second barrier)
        // before its first PV product.
        int cur = next_tile(mask, -1);
        if (cur >= 0) issue_k(k_lds0, cur);
        while (cur >= 0) {
          __builtin_amdgcn_s_waitcnt(0x0f70);
          __syncthreads();
          int nxt = next_tile(mask, cur);
          issue_v(v_lds0, cur);
          if (nxt >= 0) issue_k(k_lds1, nxt);
          k_after_v = nxt >= 0;
          __builtin_amdgcn_sched_barrier(0);
          body(cur, k_lds0, v_lds0);
          cur = nxt;
          if (cur < 0) break;
          __builtin_amdgcn_s_waitcnt(0x0f70);
          __syncthreads();
          nxt = next_tile(mask, cur);
          issue_v(v_lds0, cur);
          if (nxt >= 0) issue_k(k_lds0, nxt);
          k_after_v = nxt >= 0;
          __builtin_amdgcn_sched_barrier(0);
          body(cur, k_lds1, v_lds0);
          cur = nxt;
        }
        return;
      }
    }
    int cur = next_tile(mask, -1);
    if (cur >= 0) {
      issue_k(k_lds0, cur);
      if (with_v) issue_v(v_lds0, cur);
    }
    while (cur >= 0) {
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's share of the tile has landed
      __syncthreads();
      int nxt = next_tile(mask, cur);
      if constexpr (G::kNBuf == 2) {
        if (nxt >= 0) {
          issue_k(k_lds1, nxt);
          if (with_v) issue_v(v_lds1, nxt);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      body(cur, k_lds0, v_lds0);
      if constexpr (G::kNBuf == 1) {
        __syncthreads();
        if (nxt >= 0) {
          issue_k(k_lds0, nxt);
          if (with_v) issue_v(v_lds0, nxt);
        }
        cur = nxt;
      } else {
        cur = nxt;
        if (cur < 0) break;
        __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
        nxt = next_tile(mask, cur);
        if (nxt >= 0) {
          issue_k(k_lds0, nxt);
          if (with_v) issue_v(v_lds0, nxt);
        }
        __builtin_amdgcn_sched_barrier(0);
        body(cur, k_lds1, v_lds1);
        cur = nxt;
      }
    }
  };

  // S^T of one tile: two 32-key blocks x 32 query rows, accumulators pre-loaded with `init`.  The K
  // fragments of a block are fetched together so that its MFMA chain can run back to back, and the two
  // chains are independent, which lets the second one cover the first one's result latency.
  auto tile_scores = [&](const unsigned char* kt_lds, float init, f32x16& s0, f32x16& s1) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      s0[i] = init;
      s1[i] = init;
    }
    const unsigned char* krow0 = kt_lds + lq * G::kKRow;
    const unsigned char* krow1 = kt_lds + (32 + lq) * G::kKRow;
    const int sw0 = KS::sw(lq), sw1 = KS::sw(32 + lq);
    if constexpr (k16) {
      uint32_t ka = (uint32_t)(uintptr_t)kt_lds + k_lane;
      asm volatile("" : "+v"(ka));  // keeps the eight xors here instead of eight registers hoisted out of the walk
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
    } else {
#pragma unroll
      for (int g = 0; g < D / 8; ++g) {
        f32x4 a0 = *reinterpret_cast<const f32x4*>(krow0 + (((2 * g + lh) ^ sw0) << 4));
        f32x4 a1 = *reinterpret_cast<const f32x4*>(krow1 + (((2 * g + lh) ^ sw1) << 4));
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float bq = __builtin_bit_cast(float, qf[g * 4 + e]);
          s0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0[e], bq, s0, 0, 0, 0);
          s1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[e], bq, s1, 0, 0, 0);
        }
      }
    }
  };
  // S^T of one 32-key block of the tile (used where register pressure forbids holding both blocks).
  auto block_scores = [&](const unsigned char* kt_lds, int kb, float init) -> f32x16 {
    f32x16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = init;
    const int row = kb * 32 + lq;
    const unsigned char* krow = kt_lds + row * G::kKRow;
    const int sw = KS::sw(row);
    if constexpr (k16 && G::kVSingle) {
      // register budget of three waves per SIMD: the K fragments are fetched four at a time
      uint32_t ka = (uint32_t)(uintptr_t)kt_lds + k_lane;
      asm volatile("" : "+v"(ka));
#pragma unroll
      for (int k0 = 0; k0 < D / 16; k0 += 4) {
        u32x4 a[4];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) a[ks] = lds_read16(ka ^ ((k0 + ks) << 5), kb * 32 * G::kKRow);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          u32x4 bq = {qf[(k0 + ks) * 4], qf[(k0 + ks) * 4 + 1], qf[(k0 + ks) * 4 + 2], qf[(k0 + ks) * 4 + 3]};
          acc = mfma_16bit<T>(a[ks], bq, acc);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    } else if constexpr (k16) {
      uint32_t ka = (uint32_t)(uintptr_t)kt_lds + k_lane;
      asm volatile("" : "+v"(ka));
      u32x4 a[D / 16];
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) a[ks] = lds_read16(ka ^ (ks << 5), kb * 32 * G::kKRow);
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) {
        u32x4 bq = {qf[ks * 4], qf[ks * 4 + 1], qf[ks * 4 + 2], qf[ks * 4 + 3]};
        acc = mfma_16bit<T>(a[ks], bq, acc);
      }
    } else {
#pragma unroll
      for (int g = 0; g < D / 8; ++g) {
        f32x4 a = *reinterpret_cast<const f32x4*>(krow + (((2 * g + lh) ^ sw) << 4));
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
  // Calls f(s0, s1) with the two score blocks of tile kt unless no row of this wave can see the tile.
  // Tiles that touch the causal diagonal or the sequence tail take the masked instantiation; both are
  // straight-line code so MFMA, LDS and VALU work of the two blocks can be interleaved.
  auto for_tile = [&](int kt, const unsigned char* kt_lds, float init, auto&& f) {
    if (p.causal && kt * kBN > wave_row0 + 31) return;
    const bool need_mask = (kt * kBN + kBN - 1 > L - 1) || (p.causal && kt * kBN + kBN - 1 > wave_row0);
    f32x16 s0, s1;
    // The two arms start with distinct fences so that their common LDS reads are not hoisted above the branch:
    // reads and MFMAs then share a basic block and the reads are waited for one by one, not all at once.
    if (need_mask) {
      asm volatile("; masked tile" ::: "memory");
      tile_scores(kt_lds, init, s0, s1);
      mask_block(s0, kt, 0);
      mask_block(s1, kt, 1);
      f(s0, s1);
    } else {
      asm volatile("; plain tile" ::: "memory");
      tile_scores(kt_lds, init, s0, s1);
      f(s0, s1);
    }
  };
  // Block-by-block variant: f(s, kb) per visible 32-key block.
  auto for_tile_blocks = [&](int kt, const unsigned char* kt_lds, float init, uint32_t bits, auto&& f) {
    if (p.causal && kt * kBN > wave_row0 + 31) return;
    const bool need_mask = (kt * kBN + kBN - 1 > L - 1) || (p.causal && kt * kBN + kBN - 1 > wave_row0);
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      if (!((bits >> kb) & 1u) || (p.causal && kt * kBN + kb * 32 > wave_row0 + 31)) continue;
      f32x16 acc = block_scores(kt_lds, kb, init);
      if (need_mask) mask_block(acc, kt, kb);
      f(acc, kb);
    }
  };
  // Per-block variant for the walks that follow a mask: f(s, kb) for the blocks of tile kt named by `bits`
  // (bit kb).  Both blocks take the two-chain code of for_tile; a single block takes one chain.
  auto for_tile_sel = [&](int kt, const unsigned char* kt_lds, float init, uint32_t bits, auto&& f) {
    if (bits == 0u || (p.causal && kt * kBN > wave_row0 + 31)) return;
    const bool need_mask = (kt * kBN + kBN - 1 > L - 1) || (p.causal && kt * kBN + kBN - 1 > wave_row0);
    if (bits == 3u) {
      f32x16 s0, s1;
      if (need_mask) {
        asm volatile("; masked tile" ::: "memory");
        tile_scores(kt_lds, init, s0, s1);
        mask_block(s0, kt, 0);
        mask_block(s1, kt, 1);
        f(s0, 0);
        f(s1, 1);
      } else {
        asm volatile("; plain tile" ::: "memory");
        tile_scores(kt_lds, init, s0, s1);
        f(s0, 0);
        f(s1, 1);
      }
    } else if (bits == 1u) {
      asm volatile("; block 0" ::: "memory");
      f32x16 acc = block_scores(kt_lds, 0, init);
      if (need_mask) mask_block(acc, kt, 0);
      f(acc, 0);
    } else {
      asm volatile("; block 1" ::: "memory");
      f32x16 acc = block_scores(kt_lds, 1, init);
      if (need_mask) mask_block(acc, kt, 1);
      f(acc, 1);
    }
  };
  auto mark_tile = [&](uint32_t* mask, int kt) { atomicOr(&mask[kt >> 5], 1u << (kt & 31)); };
  // one lane of a wave: the tile for the row block, and the wave's own blocks `bits` of it
  auto mark_blocks = [&](uint32_t* mask, uint32_t* fine, int kt, uint32_t bits) {
    atomicOr(&mask[kt >> 5], 1u << (kt & 31));
    if (fine) atomicOr(&fine[kt >> 4], bits << ((kt & 15) * 2));
  };
  auto clear_mask = [&](uint32_t* mask) {  // by every thread of the block
    for (int i = tid; i < p.mask_words; i += G::kThreads) mask[i] = 0u;
    if (fine_pool) {
      uint32_t* f = fine_pool + (mask == mask_a ? 0 : G::kNW) * 2 * p.mask_words;
      for (int i = tid; i < G::kNW * 2 * p.mask_words; i += G::kThreads) f[i] = 0u;
    }
  };

  for (int i = tid; i < mask_pool_words + kPoolTail; i += G::kThreads) mask_pool[i] = 0u;

  // ---- pass A (+B): row max, and for alpha = 1.5 / 2 the histogram bracket in the same walk ----------------
  uint32_t* mask_cur = nullptr;  // mask consumed by the next pass
  uint32_t* mask_new = mask_a;   // mask produced by the running pass
  uint32_t* fine_new = fine_of(mask_new);
  const int half = (wave * 32) / kMaskRows;  // which 128-row half of the row block this wave belongs to
  const bool with_hist = AM != ATT_GEN && p.use_hist;
  float m_raw = -INFINITY;
  float hist_lo = 0.f;  // lower bound of tau from the histogram (valid when with_hist)
  float cand_est = 0.f;  // with the histogram: how many scores of this wave's rows may lie above that bound
  constexpr float kBinW = 1.f / (float)kAttnBins;  // bin width in z units
  if (!with_hist) {
    // the max walk already tells which blocks can matter later: those with an entry within 1 (in z) of the lane's
    // running maximum, a superset of the entries within 1 of the row maximum
    tile_loop(nullptr, false, [&](int kt, const unsigned char* kt_lds, const unsigned char*) {
      bool any0 = false, any1 = false;
      for_tile(kt, kt_lds, 0.f, [&](const f32x16& s0, const f32x16& s1) {
        float tm0 = s0[0], tm1 = s1[0];
#pragma unroll
        for (int i = 1; i < 16; ++i) {
          tm0 = fmaxf(tm0, s0[i]);
          tm1 = fmaxf(tm1, s1[i]);
        }
        m_raw = fmaxf(m_raw, fmaxf(tm0, tm1));
        const float keep = m_raw - inv_qs * 1.0001f - 1e-6f * fabsf(m_raw);  // (margin: rounding of the difference)
        any0 = tm0 > keep;
        any1 = tm1 > keep;
      });
      if constexpr (kFine) {
        const uint32_t nb = (__builtin_amdgcn_ballot_w64(any0) != 0ull ? 1u : 0u) | (__builtin_amdgcn_ballot_w64(any1) != 0ull ? 2u : 0u);
        if (nb && lane == 0) mark_blocks(mask_new, fine_new, kt, nb);
      } else {
        if (__builtin_amdgcn_ballot_w64(any0 || any1) != 0ull && lane == 0) mark_tile(mask_new, kt);
      }
    });
    m_raw = fmaxf(m_raw, __shfl_xor(m_raw, 32, 64));
    mask_cur = mask_new;
    mask_new = mask_b;
    fine_new = fine_of(mask_new);
  } else {
    // The histogram lives on the absolute grid of bins [g / 8, (g + 1) / 8) of z; the solver needs the nine bins
    // g_top - 8 .. g_top below the bin of the row maximum, which cover [max - 1, max] (everything lower is
    // below tau).  A lane counts the 15 bins g0 .. g0 + 14 and keeps the bin of its running maximum among the
    // upper seven of them: only when the maximum climbs past the window does the window move (up to the
    // point where the maximum sits in its ninth bin again), dropping the bins that fall off the lower end.
    //
    // Counting is bit-sliced.  Two scores become one 32-bit word of two one-hot 16-bit halves -- bit g - g0 + 1
    // for bin g, bit 0 for everything below the window -- in 2 instructions per score (an fma to window
    // coordinates, a saturating float -> u16 pair conversion, a packed shift).  The 16 words of a tile go
    // through a carry-save adder tree (3-input xor / majority, 1 instruction per score) into bit planes:
    // plane k holds bit k of every counter, so a lane keeps 2 x 15 counters of kPlanes bits in kPlanes
    // registers.  Moving the window is one packed shift per plane.
    // A counter takes at most 16 entries per key tile (one per word and half), so 12 planes serve walks of up to 255
    // tiles and 20 planes the longest ones (2^19 entries with the 1M-key mask); the short form keeps 8 registers
    // fewer alive, ripples its three upper planes without a test and reads out 12 planes instead of 20.
    auto hist_walk = [&](auto planes_c) {
      constexpr int kPlanes = decltype(planes_c)::value;
      constexpr int W = kAttnBins + 1;
      constexpr int kNoOrigin = -(1 << 29);
      constexpr int kRipple = 9;      // planes below this one take the tile's carry unconditionally
      constexpr int kTopLo = W, kTopHi = 15;      // bit positions the bin of the maximum may occupy
      constexpr uint32_t kBinBits = 0xfffefffeu;  // everything but the below-window bit of each half
      const float c8 = (float)kAttnBins * qs;
      const float c8n = c8 * (1.f / 65535.f);  // the conversion maps [0, 1] to [0, 65535] and rounds to nearest
      uint32_t pl[kPlanes];
#pragma unroll
      for (int k = 0; k < kPlanes; ++k) pl[k] = 0u;
      int g0 = kNoOrigin;
      // window coordinate y = s c8 - g0 + 1: [0, 1) below the window, [i, i + 1) at bit position i; the
      // conversion rounds, hence the half
      float offn = (0.5f - (float)g0) * (1.f / 65535.f);
      // moves the window up by sh bins (per lane, sh >= 0)
      auto shift_planes = [&](int sh) {
        const uint32_t s1 = (uint32_t)(sh < 15 ? sh : 15);
        const uint32_t s2 = s1 | (s1 << 16);
#pragma unroll
        for (int k = 0; k < kPlanes; ++k) pl[k] = pk_shr16(pl[k], s2);
      };
      tile_loop(nullptr, false, [&](int kt, const unsigned char* kt_lds, const unsigned char*) {
        bool any0 = false, any1 = false;
        for_tile(kt, kt_lds, 0.f, [&](const f32x16& s0, const f32x16& s1) {
          float tm0 = s0[0], tm1 = s1[0];
#pragma unroll
          for (int i = 1; i < 16; ++i) {
            tm0 = fmaxf(tm0, s0[i]);
            tm1 = fmaxf(tm1, s1[i]);
          }
          m_raw = fmaxf(m_raw, fmaxf(tm0, tm1));
          {
            // a block matters to the later walks when one of its entries lies within 1 (in z) of the running
            // maximum; the margin covers the rounding of the difference
            const float keep = m_raw - inv_qs * 1.0001f - 1e-6f * fabsf(m_raw);
            any0 = tm0 > keep;
            any1 = tm1 > keep;
          }
          // bin of the maximum; the entries use the same scale, so none lands more than a rounding error above it
          const int g_top = m_raw > -INFINITY ? (int)floorf(m_raw * c8) : g0 + kTopLo - 1;
          int p_top = g_top - g0 + 1;
          if (__builtin_amdgcn_ballot_w64(p_top > kTopHi) != 0ull) {
            const int sh = p_top > kTopHi ? p_top - kTopLo : 0;
            shift_planes(sh);
            g0 += sh;
            p_top -= sh;
            offn = (0.5f - (float)g0) * (1.f / 65535.f);
          }
          uint32_t w[16];
#pragma unroll
          for (int j = 0; j < 16; ++j) {
            const float sa = j < 8 ? s0[(2 * j) & 15] : s1[(2 * j) & 15];
            const float sb = j < 8 ? s0[(2 * j + 1) & 15] : s1[(2 * j + 1) & 15];
            w[j] = pk_shl16(0x00010001u, __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pknorm_u16(fmaf(sa, c8n, offn), fmaf(sb, c8n, offn))));
          }
          // adder tree: 16 words + plane 0 -> plane 0 and 8 carries, those + plane 1 -> plane 1 and 4 carries, ...
          uint32_t c2[8], c4[4], c8w[2], c16;
          uint32_t acc = pl[0];
#pragma unroll
          for (int j = 0; j < 8; ++j) full_add(acc, w[2 * j], w[2 * j + 1], acc, c2[j]);
          pl[0] = acc;
          acc = pl[1];
#pragma unroll
          for (int j = 0; j < 4; ++j) full_add(acc, c2[2 * j], c2[2 * j + 1], acc, c4[j]);
          pl[1] = acc;
          acc = pl[2];
#pragma unroll
          for (int j = 0; j < 2; ++j) full_add(acc, c4[2 * j], c4[2 * j + 1], acc, c8w[j]);
          pl[2] = acc;
          acc = pl[3];
          full_add(acc, c8w[0], c8w[1], acc, c16);
          pl[3] = acc;
          // the carry out of the tree ripples through the next planes; a carry into plane kRipple is rare enough
          // for a branch.  The below-window bit would carry on every tile and is dropped.
          uint32_t carry = c16 & kBinBits;
#pragma unroll
          for (int k = 4; k < kRipple; ++k) {
            const uint32_t t = pl[k] & carry;
            pl[k] ^= carry;
            carry = t;
          }
          if (kPlanes - kRipple <= 3 || __builtin_amdgcn_ballot_w64(carry != 0u) != 0ull) {
#pragma unroll
            for (int k = kRipple; k < kPlanes; ++k) {
              const uint32_t t = pl[k] & carry;
              pl[k] ^= carry;
              carry = t;
            }
          }
        });
        if constexpr (kFine) {
          const uint32_t nb = (__builtin_amdgcn_ballot_w64(any0) != 0ull ? 1u : 0u) | (__builtin_amdgcn_ballot_w64(any1) != 0ull ? 2u : 0u);
          if (nb && lane == 0) mark_blocks(mask_new, fine_new, kt, nb);
        } else {
          if (__builtin_amdgcn_ballot_w64(any0 || any1) != 0ull && lane == 0) mark_tile(mask_new, kt);
        }
      });
      // the two lanes of a row bring their windows to the row's nine bins, bin g_top - 8 at bit position 1; then
      // the counters are read out of the planes (both halves of a word belong to the lane's row) and added up
      m_raw = fmaxf(m_raw, __shfl_xor(m_raw, 32, 64));
      const int g0_row = (m_raw > -INFINITY ? (int)floorf(m_raw * c8) : kNoOrigin + kAttnBins) - kAttnBins;
      shift_planes(g0_row - g0);  // >= 0: a lane's window starts at or below its own maximum's ninth bin
      float cnt[W];
#pragma unroll
      for (int bin = 0; bin < W; ++bin) {
        uint32_t c = 0u;
#pragma unroll
        for (int k = 0; k < kPlanes; ++k) {
          uint32_t bits = ((pl[k] >> (bin + 1)) & 1u) + ((pl[k] >> (bin + 17)) & 1u);
          // an entry a rounding error above the top bin counts as sitting in it
          if (bin == W - 1) bits += ((pl[k] >> (bin + 2)) & 1u) + ((pl[k] >> (bin + 18)) & 1u);
          c += bits << k;
        }
        cnt[bin] = (float)c;
      }
#pragma unroll
      for (int k = 0; k < W; ++k) cnt[k] += __shfl_xor(cnt[k], 32, 64);
      // Every entry counts as sitting on the lower edge of its bin, which gives a lower bound of tau that is
      // less than one bin width off (the entries left out lie below max - 1).
      const float t_shift = (float)g0_row * kBinW;
      hist_lo = (AM == ATT_15) ? hist_bracket_alpha15<W>(cnt, t_shift, kBinW) : hist_bracket_alpha2<W>(cnt, t_shift, kBinW);
      {
        float n_cand = 0.f;  // the entries of the bins that reach above the bound
#pragma unroll
        for (int k = 0; k < W; ++k) n_cand += (t_shift + (float)(k + 1) * kBinW > hist_lo) ? cnt[k] : 0.f;
        cand_est = wave_sum(lh == 0 && qi < L ? n_cand : 0.f);
      }
    };
    if (nt <= 255) hist_walk(std::integral_constant<int, 12>{});
    else hist_walk(std::integral_constant<int, 20>{});
    mask_cur = mask_new;
    mask_new = mask_b;
    fine_new = fine_of(mask_new);
  }
  const float m = m_raw * qs;  // row max of z = (alpha-1) q.k / sqrt(D)

  // Tightest a-priori bracket: tau in [m - 1, m - n^(1 - alpha)], n = number of valid keys of the row
  // (all n equal to the max is the extreme case; adasplash/adasplash_block_mask.py:167-175).
  const float n_keys = (float)(lim + 1);
  const float hi_cap = m - fast_exp2((1.f - p.alpha) * fast_log2(n_keys));
  Bracket br;  // in z units
  br.lo = m - 1.f;
  br.hi = hi_cap;
  if (with_hist) {
    // The nominal upper end lo + bin width serves as the starting point only; pass C replaces it by the
    // unconditional bound as soon as a Newton step proves it wrong.
    // the margin covers the rounding of the window coordinates (relative 2^-23 of the score's magnitude)
    br.lo = fmaxf(hist_lo - (2e-6f + 5e-7f * fabsf(m)), m - 1.f);
    br.hi = fminf(br.lo + kBinW + 4e-6f, hi_cap);
  }
  br.t = 0.5f * (br.lo + br.hi);

  // ---- pass C: niter safeguarded Halley / Newton steps ----------------------------------------------------
  // A walk that is not the last one also writes down the scores above the bracket's lower end (the only ones
  // later steps can see: tau never drops below it).  They go to the V tile buffers, idle until the output walk:
  // every wave owns a share of them, cut into chunks of kChunk (score, key index) pairs.  A lane keeps its own
  // list -- the ids of up to eight chunks live in registers -- and draws a chunk from the wave's counter when the
  // last one is full, so a row with a flat top can take many while most take one.  When no lane of the block ran
  // out of chunks, the remaining steps run on these lists without touching K again, and so does the output (the
  // V rows of the listed keys are gathered); otherwise the block keeps walking, as it does when the histogram
  // already shows more candidates than the chunks could hold.
  constexpr int kChunk = 4;       // entries per chunk: four scores, then their four key indices
  constexpr int kLaneChunks = 8;
  constexpr bool kTwoV = (G::kNBuf == 2 && !G::kVSingle);
  constexpr int kWavePoolBytes = kTwoV ? G::kVTile / (NW / 2) : G::kVTile / NW;
  constexpr int kChunksRaw = kWavePoolBytes / (kChunk * 8);
  constexpr int kChunks = kChunksRaw > 128 ? 128 : kChunksRaw;  // chunk ids are bytes
  constexpr bool kLists = kChunks >= 96;                         // one chunk a lane and some to spare
  float* const my_pool = reinterpret_cast<float*>(
      (kTwoV && wave >= NW / 2 ? v_lds1 : v_lds0) + (kTwoV ? wave % (NW / 2) : wave) * kWavePoolBytes);
  bool list_mode = false;            // uniform over the block
  int my_n = 0;                      // this lane's list: its length,
  unsigned long long my_ids = 0ull;  // the ids of its chunks (a byte each, in drawing order)
  const bool live_row = qi < L;
  // entry e of the lane's list: the score and the key index sit kChunk words apart
  auto list_slot = [&](int e) -> float* {
    return my_pool + (uint32_t)((my_ids >> (8 * (e / kChunk))) & 0xffull) * (2 * kChunk) + e % kChunk;
  };
  {
    float t_prev = br.t, f_prev = 0.f;
    bool may_build = cand_est <= 0.5f * (float)(kChunks * kChunk);  // uniform over the wave; one attempt only
    uint32_t my_chunk = 0u;            // the chunk being filled
    for (int it = 0; it < p.niter; ++it) {
      constexpr bool kWithLists = kMulti && kLists;
      const float init = -br.t * inv_qs;
      const float dl = (br.lo - br.t) * inv_qs;  // z > lo  <=>  (s - t_raw) > dl
      float a0 = 0.f, a1 = 0.f, a2 = 0.f;
      int cnt_pos = 0, cnt_neg = 0, n_seen = 0;  // n_seen - cnt_neg: scores above the threshold (packed path)
      // one score's terms in fp32; r = raw score - raw threshold
      auto add_score = [&](float r) {
        if constexpr (AM == ATT_15) {
          const float u = __builtin_amdgcn_fmed3f(r, 0.f, INFINITY);
          a0 = fmaf(u, u, a0);
          a1 += u;
          cnt_pos += r > 0.f;
        } else if constexpr (AM == ATT_2) {
          a0 += __builtin_amdgcn_fmed3f(r, 0.f, INFINITY);
          cnt_pos += r > 0.f;
        } else {
          if (r > 0.f) {
            const float uz = r * qs;
            const float e0 = fast_exp2(fast_log2(uz) * p.c0);
            const float rc = fast_rcp(uz);
            const float e1 = e0 * rc;
            a0 += e0;
            a1 += e1;
            a2 += e1 * rc;
          }
        }
      };
      // lists serve the later steps and, unless tile statistics are asked for, the output
      const bool want_lists = it + 1 < p.niter || !p.tile_counts;
      bool build = kWithLists && !list_mode && may_build && want_lists;  // uniform over the wave
      bool lane_full = false;
      const bool collecting = build;
      // The block maxima serve the tile mask of the next walk (and the lists).  When the histogram has counted, over
      // the wave's 32 rows, several candidates per key tile, no tile will drop out for this wave and the maxima are
      // not worth their instructions (uniform over the wave).
      const bool track = build || !(with_hist && cand_est > 4.f * (float)nt);
      // the lane's candidates of a block join its list; the wave stops collecting once a lane is out of room
      auto append_block = [&](const f32x16& sc, int key0) {  // key0: the lane's first key of the block
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          if (sc[i] > dl && live_row && !lane_full) {
            if (my_n % kChunk == 0) {
              const uint32_t c = my_n < kChunk * kLaneChunks ? atomicAdd(&chunk_ctr[wave], 1u) : (uint32_t)kChunks;
              if (c < (uint32_t)kChunks) {
                my_chunk = c;
                my_ids |= (unsigned long long)c << (8 * (my_n / kChunk));
              } else {
                lane_full = true;
              }
            }
            if (!lane_full) {
              float* slot = my_pool + my_chunk * (2 * kChunk) + my_n % kChunk;
              slot[0] = sc[i] - init;
              slot[kChunk] = __builtin_bit_cast(float, (uint32_t)(key0 + 8 * (i >> 2) + (i & 3)));
              ++my_n;
            }
          }
        }
        if (__builtin_amdgcn_ballot_w64(lane_full) != 0ull) build = false;
      };
      if (kWithLists && list_mode) {
        for (int e = 0; __builtin_amdgcn_ballot_w64(e < my_n) != 0ull; ++e)
          if (e < my_n) add_score(*list_slot(e) + init);
      } else {
      if (build) {
        my_n = 0;
        my_ids = 0ull;
        if (lane == 0) chunk_ctr[wave] = 0u;
      }
      const uint32_t* fine_cur = fine_of(mask_cur);
      tile_loop(mask_cur, false, [&](int kt, const unsigned char* kt_lds, const unsigned char*) {
        const uint32_t bits = block_bits(fine_cur, kt);
        float dmax0 = -INFINITY, dmax1 = -INFINITY;  // per 32-key block
        if constexpr (k16 && AM == ATT_15) {
          // 16-bit inputs, alpha = 1.5: the sums run on pairs of scores rounded (towards zero) to f16 -- packed max,
          // packed f16 sums over the tile (at most 16 terms of at most (sqrt(D) / (alpha - 1))^2 <= 1024 per half, added
          // to the fp32 sums once per tile), and the sign bits for the support count: 3.5 VALU instructions per
          // score instead of 5.5.  The rounding moves f by a few 1e-4 relative, far inside the 16-bit output
          // tolerance, and keeps {score > lower bound} a superset (negative values round up).  (alpha = 2 takes the
          // fp32 sums below, which cost it no more: there a threshold that is 1e-4 off is harmless to the output but
          // moves keys in and out of supports, and the backward weighs every member of a support alike.)  The sums use
          // v_pk_fma_f16 / v_pk_add_f16 and not the two-term dot product with fp32 accumulation: on this part a
          // wave's v_dot2 instructions and another wave's MFMAs exclude each other completely, while the other
          // vector instructions give up less than half of an MFMA's duration.
          auto packed_tile = [&](auto track_c) {
            constexpr bool kTrack = decltype(track_c)::value;
            const h2_t ninf2 = {(_Float16)-INFINITY, (_Float16)-INFINITY};
            const h2_t pinf2 = {(_Float16)INFINITY, (_Float16)INFINITY};
            // (a wave that does not track the block maxima marks every tile it visits)
            h2_t dm2[2] = {kTrack ? ninf2 : pinf2, kTrack ? ninf2 : pinf2};
            const h2_t zero2 = {(_Float16)0.f, (_Float16)0.f};
            h2_t sq2 = zero2, su2 = zero2;
            for_tile_sel(kt, kt_lds, init, bits, [&](const f32x16& sc, int kb) {
              n_seen += 16;
#pragma unroll
              for (int j = 0; j < 8; ++j) {
                const float ra = sc[2 * j];
                const float rb = sc[2 * j + 1];
                const h2_t h = pkrtz(ra, rb);
                if constexpr (kTrack) dm2[kb] = __builtin_elementwise_max(dm2[kb], h);
                // population count with the running total as its addend: one instruction
                asm("v_bcnt_u32_b32 %0, %1, %0" : "+v"(cnt_neg) : "v"(__builtin_bit_cast(uint32_t, h) & 0x80008000u));
                const h2_t u = __builtin_elementwise_max(h, zero2);
                if constexpr (AM == ATT_15) sq2 = __builtin_elementwise_fma(u, u, sq2);
                su2 = su2 + u;
              }
              if constexpr (kTrack)
                if (build && __builtin_amdgcn_ballot_w64(live_row && fmaxf((float)dm2[kb][0], (float)dm2[kb][1]) > dl) != 0ull) append_block(sc, kt * kBN + kb * 32 + 4 * lh);
            });
            if constexpr (AM == ATT_15) {
              a0 += (float)sq2[0] + (float)sq2[1];
              a1 += (float)su2[0] + (float)su2[1];
            } else {
              a0 += (float)su2[0] + (float)su2[1];
            }
            dmax0 = fmaxf((float)dm2[0][0], (float)dm2[0][1]);
            dmax1 = fmaxf((float)dm2[1][0], (float)dm2[1][1]);
          };
          if (track) packed_tile(std::true_type{});
          else packed_tile(std::false_type{});
        } else {
          for_tile_sel(kt, kt_lds, init, bits, [&](const f32x16& sc, int kb) {
            float dm = -INFINITY;
#pragma unroll
            for (int i = 0; i < 16; ++i) dm = fmaxf(dm, sc[i]);
            if (kb == 0) dmax0 = dm;
            else dmax1 = dm;
            // a block without a score above the lower end (dl <= 0 up to rounding) has none above the threshold
            if (__builtin_amdgcn_ballot_w64(dm > fminf(dl, 0.f)) != 0ull) {
#pragma unroll
              for (int i = 0; i < 16; ++i) add_score(sc[i]);
              if (build && __builtin_amdgcn_ballot_w64(live_row && dm > dl) != 0ull) append_block(sc, kt * kBN + kb * 32 + 4 * lh);
            }
          });
        }
        // every step tightens the masks to {z > lower bound} for the next walk
        if constexpr (kFine) {
          const uint32_t nb = (__builtin_amdgcn_ballot_w64(dmax0 > dl) != 0ull ? 1u : 0u) | (__builtin_amdgcn_ballot_w64(dmax1 > dl) != 0ull ? 2u : 0u);
          if (nb && lane == 0) mark_blocks(mask_new, fine_new, kt, nb);
        } else {
          if (__builtin_amdgcn_ballot_w64(fmaxf(dmax0, dmax1) > dl) != 0ull && lane == 0) mark_tile(mask_new, kt);
        }
      });
      if constexpr (k16 && AM == ATT_15) cnt_pos = n_seen - cnt_neg;
      }
      if constexpr (AM == ATT_15) {
        a0 *= qs * qs;
        a1 *= qs;
        a2 = (float)cnt_pos;
      } else if constexpr (AM == ATT_2) {
        a0 *= qs;
        a1 = (float)cnt_pos;
      }
      a0 += __shfl_xor(a0, 32, 64);
      a1 += __shfl_xor(a1, 32, 64);
      a2 += __shfl_xor(a2, 32, 64);
      // f is convex and decreasing, so a Newton step from the left never passes the root: if it lands
      // beyond the upper end although f(t) > 0, that end (the histogram's lo + bin width) was not valid
      // for this row and the unconditional bound takes its place.
      if (a0 > 1.f && br.t + (a0 - 1.f) / (p.c0 * a1) > br.hi) br.hi = hi_cap;
      hybrid_step(br, a0, a1, a2, p.c0, AM != ATT_2 && p.alpha <= 1.5f, p.alpha <= 2.0f, it > 0, t_prev, f_prev);
      if (!(kWithLists && list_mode)) {
        if (kWithLists && want_lists) {
          // a wave that gave up, or did not try, keeps the whole block walking
          const bool ovf = !collecting || !build;
          if (ovf && lane == 0) list_flag[it & 1] = 1u;
          // the other flag word is the next step's; its last readers passed this walk's barriers already
          if (tid == 0) list_flag[(it + 1) & 1] = 0u;
        }
        // the mask just written becomes the one to read; the other array is cleared for a later pass
        __syncthreads();
        mask_cur = mask_new;
        mask_new = (mask_cur == mask_a) ? mask_b : mask_a;
        fine_new = fine_of(mask_new);
        clear_mask(mask_new);
        if (kWithLists && want_lists) {
          if (list_flag[it & 1] == 0u) list_mode = true;
          else may_build = false;
        }
      }
    }
  }
  const float tau = br.t;

  // ---- pass D: out = sum_j p_j v_j / sum_j p_j over the masked tiles --------------------------------------
  f32x16 o[G::kDB];
#pragma unroll
  for (int db = 0; db < G::kDB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
  float psum = 0.f;
  f32x4_t psum4 = {0.f, 0.f, 0.f, 0.f};  // 16-bit walks: every register holds the lane's sum
  unsigned active16 = 0;  // 16x16 score tiles with a non-zero probability (wave-uniform count)
  // With the lists in place (and no tile statistics asked for) there is nothing to walk: a lane turns its
  // listed scores into probabilities and adds up the V rows of their keys, read from the row-major V.
  const bool gather = kMulti && kLists && list_mode && !p.tile_counts;
  if (gather) {
    if constexpr (kMulti && kLists) {
      const float init = -tau * inv_qs;
      const unsigned char* vrows = reinterpret_cast<const unsigned char*>(p.v) + kv_base * G::kEB;
      // one sweep over the list per 32 output columns: 32 accumulators at a time keep the kernel within the
      // registers its walks are compiled for
#pragma unroll
      for (int db = 0; db < G::kDB; ++db) {
        float acc[32];
#pragma unroll
        for (int d = 0; d < 32; ++d) acc[d] = 0.f;
        for (int e = 0; __builtin_amdgcn_ballot_w64(e < my_n) != 0ull; ++e) {
          if (e < my_n) {
            const float* slot = list_slot(e);
            const float pv = attn_prob<AM>(slot[0] + init, qs, p.c0);
            if (pv > 0.f) {
              const uint32_t key = __builtin_bit_cast(uint32_t, slot[kChunk]);
              if (db == 0) {
                psum += pv;
                if (bmask_out) mark_tile(mask_out0 + half * p.mask_words, (int)(key / kBN));
              }
              const u32x4* vr = reinterpret_cast<const u32x4*>(vrows + ((size_t)key * D + db * 32) * G::kEB);
              if constexpr (k16) {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                  const u32x4 w = vr[c];
#pragma unroll
                  for (int j = 0; j < 4; ++j) {
                    const uint32_t ww = w[j];
                    acc[8 * c + 2 * j] = fmaf(pv, unpack_lo<T>(ww), acc[8 * c + 2 * j]);
                    acc[8 * c + 2 * j + 1] = fmaf(pv, unpack_hi<T>(ww), acc[8 * c + 2 * j + 1]);
                  }
                }
              } else {
#pragma unroll
                for (int c = 0; c < 8; ++c) {
                  const u32x4 w = vr[c];
#pragma unroll
                  for (int j = 0; j < 4; ++j) {
                    const uint32_t ww = w[j];
                    acc[4 * c + j] = fmaf(pv, __builtin_bit_cast(float, ww), acc[4 * c + j]);
                  }
                }
              }
            }
          }
        }
        // the two lanes of a row each hold half of its output columns (8 g + 4 lh + j of every 32): a lane
        // keeps its half of its own sums and receives the partner's sums for that half
#pragma unroll
        for (int g = 0; g < 4; ++g) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float lo_part = acc[8 * g + j], hi_part = acc[8 * g + 4 + j];
            const float own = lh ? hi_part : lo_part, send = lh ? lo_part : hi_part;
            o[db][4 * g + j] = own + __shfl_xor(send, 32, 64);
          }
        }
      }
    }
  } else {
    const float init = -tau * inv_qs;
    const uint32_t* fine_cur = fine_of(mask_cur);
    tile_loop(mask_cur, true, [&](int kt, const unsigned char* kt_lds, const unsigned char* vt_lds) {
      const uint32_t bits = block_bits(fine_cur, kt);
      bool tile_active = false;
      // single V tile: every wave joins one barrier per tile once its own share of V has landed (the K loads of
      // the next tile, issued after it, may still be in flight), whether or not it has work in the tile
      bool v_ready = !G::kVSingle;
      auto need_v = [&]() {
        if constexpr (G::kVSingle) {
          if (!v_ready) {
            if (k_after_v) __builtin_amdgcn_s_waitcnt(0x0f70 | kKPer);  // vmcnt(kKPer)
            else __builtin_amdgcn_s_waitcnt(0x0f70);
            __syncthreads();
            v_ready = true;
          }
        }
      };
      for_tile_blocks(kt, kt_lds, init, bits, [&](const f32x16& acc, int kb) {
        float pv[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) pv[i] = attn_prob<AM>(acc[i], qs, p.c0);
        // 16-bit types: the probabilities are rounded to the operand format first; their sum is taken from the
        // rounded values (what the product below really weighs V with) on the matrix pipe, and "is there anything in
        // this 16-key half" from the or of the packed words.  fp32: plain sums.
        u32x4 bp[2];
        bool half_live[2];  // over the lane's keys of each 16-key half of the block
        if constexpr (k16) {
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            bp[s] = u32x4{pack2<T>(pv[8 * s], pv[8 * s + 1]), pack2<T>(pv[8 * s + 2], pv[8 * s + 3]),
                          pack2<T>(pv[8 * s + 4], pv[8 * s + 5]), pack2<T>(pv[8 * s + 6], pv[8 * s + 7])};
            half_live[s] = ((bp[s][0] | bp[s][1]) | (bp[s][2] | bp[s][3])) != 0u;
            psum4 = lane_sum4<T>(u32x2_t{bp[s][0], bp[s][1]}, psum4);
            psum4 = lane_sum4<T>(u32x2_t{bp[s][2], bp[s][3]}, psum4);
          }
        } else {
          float hsum[2] = {0.f, 0.f};
#pragma unroll
          for (int i = 0; i < 16; ++i) hsum[i >> 3] += pv[i];
          psum += hsum[0] + hsum[1];
          half_live[0] = hsum[0] > 0.f;
          half_live[1] = hsum[1] > 0.f;
        }
        tile_active |= half_live[0] || half_live[1];
        if (p.tile_counts) {
          // lanes 0-15 / 32-47 hold query rows 0-15, lanes 16-31 / 48-63 rows 16-31; registers 0-7 hold
          // keys 0-15 of the block, registers 8-15 keys 16-31.
          bool lo = false, hi = false;
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            lo |= pv[i] > 0.f;
            hi |= pv[8 + i] > 0.f;
          }
          lo = lo && qi < L;  // padded query rows are outside the domain
          hi = hi && qi < L;
          const unsigned long long blo = __builtin_amdgcn_ballot_w64(lo), bhi = __builtin_amdgcn_ballot_w64(hi);
          const unsigned long long q0 = 0x0000ffff0000ffffull, q1 = 0xffff0000ffff0000ull;
          active16 += ((blo & q0) != 0) + ((blo & q1) != 0) + ((bhi & q0) != 0) + ((bhi & q1) != 0);
        }
        need_v();
        if constexpr (k16) {
          uint32_t va0 = (uint32_t)(uintptr_t)vt_lds + v_lane[0], va1 = (uint32_t)(uintptr_t)vt_lds + v_lane[1];
          asm volatile("" : "+v"(va0), "+v"(va1));
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            // a 16-key half in which no row of the wave has a non-zero probability adds nothing: with a
            // support of a few keys per row that is a large share of the halves
            if (__builtin_amdgcn_ballot_w64(half_live[s]) == 0ull) continue;
#pragma unroll
            for (int db = 0; db < G::kDB; ++db) {
              const int drow = db * 32 + lq;
              const u32x2_t a0 = lds_read8_tr(va0 ^ (db << 6), (kb * 32 + 16 * s) * G::kVRow);
              const u32x2_t a1 = lds_read8_tr(va1 ^ (db << 6), (kb * 32 + 16 * s) * G::kVRow);
              u32x4 a = {a0[0], a0[1], a1[0], a1[1]};
              if (D < 32 && drow >= D) a = u32x4{0u, 0u, 0u, 0u};
              o[db] = mfma_16bit<T>(a, bp[s], o[db]);
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
              if (D >= 32 || dcol < D)
                a = *reinterpret_cast<const float*>(vt_lds + VS::off(key, dcol >> 2) + (dcol & 3) * 4);
              if (kt * kBN + key >= L) a = 0.f;  // padding rows of v may hold anything
              o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, pv[i], o[db], 0, 0, 0);
            }
          }
        }
      });
      need_v();
      // final block mask: tiles in which this 128-row half really has a non-zero probability
      if (bmask_out && __builtin_amdgcn_ballot_w64(tile_active && qi < L) != 0ull && lane == 0)
        mark_tile(mask_out0 + half * p.mask_words, kt);
    });
  }
  psum += psum4[0];
  psum += __shfl_xor(psum, 32, 64);
  const float inv = psum > 0.f ? 1.f / psum : 0.f;

  // ---- epilogue: normalise, transpose through LDS, 16-byte row-contiguous stores --------------------------
  if (tid == 0 && p.tile_counts) {  // 16x16 tiles of this row block that hold at least one valid (row, key)
    unsigned long long dom = 0;
    for (int r0 = m0; r0 < m0 + BM && r0 < L; r0 += 16) {
      const int last_row = (r0 + 15 < L - 1) ? r0 + 15 : L - 1;
      dom += p.causal ? (unsigned long long)(last_row / 16 + 1) : (unsigned long long)((L + 15) / 16);
    }
    atomicAdd(&p.tile_counts[0], dom);
  }
  if (p.tile_counts && lane == 0 && active16) atomicAdd(&p.tile_counts[1], (unsigned long long)active16);
  if (qi < L && lh == 0 && p.taus) p.taus[(size_t)(b * p.Hq + h) * N + qi] = tau;

  __syncthreads();  // every wave is done reading the tile buffers; they become the transpose scratch
  {
    using OS = Swz<G::kKRow>;  // a wave's 32 x D output tile uses the K-tile row format
    unsigned char* stage_arr =
        (wave >> 1) == 0 ? k_lds0 : ((wave >> 1) == 1 ? v_lds0 : ((wave >> 1) == 2 ? k_lds1 : v_lds1));
    unsigned char* ot = stage_arr + (wave & 1) * (32 * G::kKRow);
    const bool live = qi < L;
#pragma unroll
    for (int db = 0; db < G::kDB; ++db) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int d0 = db * 32 + 8 * g + 4 * lh;
        if (D >= 32 || d0 < D) {
          float x0 = live ? o[db][4 * g] * inv : 0.f, x1 = live ? o[db][4 * g + 1] * inv : 0.f;
          float x2 = live ? o[db][4 * g + 2] * inv : 0.f, x3 = live ? o[db][4 * g + 3] * inv : 0.f;
          if constexpr (k16) {
            u32x2 w = {pack2<T>(x0, x1), pack2<T>(x2, x3)};
            *reinterpret_cast<u32x2*>(ot + OS::off(lq, d0 >> 3) + (d0 & 7) * 2) = w;
          } else {
            f32x4 w = {x0, x1, x2, x3};
            *reinterpret_cast<f32x4*>(ot + OS::off(lq, d0 >> 2)) = w;
          }
        }
      }
    }
    // the same wave reads back what it wrote: no block barrier needed, only the LDS counter
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    unsigned char* obase = reinterpret_cast<unsigned char*>(p.out) + (qo_base + (size_t)wave_row0 * D) * G::kEB;
    constexpr int kChunks = 32 * OS::kC;
#pragma unroll
    for (int j = 0; j < (kChunks + 63) / 64; ++j) {
      const int id = j * 64 + lane;
      const int row = id / OS::kC, c = id % OS::kC;
      if ((kChunks % 64 == 0 || id < kChunks) && wave_row0 + row < N) {
        u32x4 w = *reinterpret_cast<const u32x4*>(ot + OS::off(row, c));
        *reinterpret_cast<u32x4*>(obase + (size_t)row * G::kKRow + c * 16) = w;
      }
    }
  }
  if (bmask_out) {
    __syncthreads();
    for (int i = tid; i < kHalves * p.mask_words; i += G::kThreads) {
      const int hf = i / p.mask_words, w = i % p.mask_words;
      if (m0 + hf * kMaskRows < N) bmask_out[i] = (int32_t)mask_out0[hf * p.mask_words + w];
    }
  }
}

}  // namespace adsp
