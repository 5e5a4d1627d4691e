// dQ of the sparse entmax attention from the rows' supports (gfx950, 16-bit inputs, alpha = 1.5 / 2, head dims 64 / 128):
// the backward's counterpart of attn_fwd_sparse_kernel.
//
// The forward left every row's threshold tau.  With it the support needs no search: one 16-bit score walk with the
// accumulators preloaded with -tau collects exactly the keys with a non-zero probability (the forward's second walk,
// with the threshold itself in place of a lower bound), a counting sort turns the wave's stream into per-row lists, and
// the rest is row-wise arithmetic on those few keys:
//   dP_ij = dO_i . v_j,  delta_i = sum_j u_ij dP_ij / sum_j u_ij,  dQ_i = sum_j u_ij (dP_ij - delta_i) k_j / sqrt(D)
// with u = p^(2 - alpha).  A group of D / 8 lanes serves a row: each lane holds eight columns of dO_i, fetches its
// 16 bytes of v_j and k_j, the group adds up the partial dot products on the DPP network, and since delta_i is only
// known at the end the lanes keep two sums, A = sum u dP k and B = sum u k: dQ_i = (A - delta_i B) / sqrt(D).  Weights
// and sums are fp32.  delta_i and 1 / sum_j p_ij go to the arrays the dense dK/dV kernel reads.
//
// Hand-over to the dK/dV kernel (when the stream has a place of its own): the loop over a row's members leaves dP_ij
// (fp32) in place of each member's score and the score (half precision) in place of its key; behind the row's last
// member, delta_i and sum p are known and every member gets its pair of weights (p_ij / sum p, u_ij (dP_ij -
// delta_i)) in the element type; a last pass writes the pairs into the first words of the stream's entries, which
// held each entry's place in the lists since the sort.
//
// Row blocks whose supports outgrow the stream or the lists are flagged and left to attn_bwd_dq_kernel, launched
// behind, exactly as in the forward; the kernel is persistent and draws row blocks from the same per-XCD counters.
#pragma once
#include "attn_bwd_kernel.h"
#include "attn_sparse_kernel.h"

// The dK/dV kernel on the streams: waves per SIMD and sets of member rows in flight per wave (a set = four members of each
// of the keys in progress: 36 registers).  Two waves with three sets measured best on the benchmark shapes; three
// waves leave room for two sets only and were 5 % slower.
#ifndef ADSP_DKDV_WAVES
#define ADSP_DKDV_WAVES 2
#endif
#ifndef ADSP_DKDV_QUADS
#define ADSP_DKDV_QUADS 3
#endif
// Profiling builds only (-DADSP_DQ_STOP=1 .. 3 / -DADSP_DKDV_STOP=1 .. 3 in the build's extra flags): the dQ kernel skips
// its loop over the members (1), ends a row block in front of the sort (2) or right behind its set-up (3); the dK/dV
// kernel on the streams ends a part behind the table of its pieces (1) or behind the sort (2), or an item behind its
// set-up (3), so that the stages can be timed by difference.  Such a build computes no gradients.  (Items that do
// nothing are bound by the eight work counters, 2048 increments each at c4's size: the floor of such a build says
// little about the full kernels.)
#ifndef ADSP_DQ_STOP
#define ADSP_DQ_STOP 0
#endif
#ifndef ADSP_DKDV_STOP
#define ADSP_DKDV_STOP 0
#endif

namespace adsp {

// 4-byte global -> LDS copy per lane (lane i writes LDS bytes [4 i, 4 i + 4) after the wave-uniform base `lds`), the
// global address given as a scalar base and a 32-bit byte offset per lane: dma16s of attn_kernel.h for single words
__device__ __forceinline__ void dma4s(const void* gbase, uint32_t off, void* lds) {
  const uint32_t base = (uint32_t)(uintptr_t)lds;
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1"
               :
               : "v"(off), "s"(gbase), "s"(__builtin_amdgcn_readfirstlane(base))
               : "memory");  // (m0 is a reserved register: the compiler sets it itself before each of its own uses)
}

// sum over a group of LANES (8 or 16) adjacent lanes, left in every lane of the group
// p[j] += a . b[j] over the eight 16-bit elements of a 16-byte chunk, j = 0 .. 3: sixteen two-term dot products with fp32
// accumulation (the products of 16-bit values are exact in fp32, as with unpack + fma, at a quarter of the
// instructions).  One block that ends in idle cycles: the instruction behind a v_dot2c must not overwrite one of its
// sources (see dot2_chunk of the forward).
template <typename T> __device__ __forceinline__ void dot8x4(float (&p)[4], u32x4 a, const u32x4 (&b)[4]);
#define ADSP_DOT8X4(OP)                                                                                               \
  asm volatile(OP " %0, %4, %8\n\t" OP " %1, %4, %12\n\t" OP " %2, %4, %16\n\t" OP " %3, %4, %20\n\t"                  \
               OP " %0, %5, %9\n\t" OP " %1, %5, %13\n\t" OP " %2, %5, %17\n\t" OP " %3, %5, %21\n\t"                  \
               OP " %0, %6, %10\n\t" OP " %1, %6, %14\n\t" OP " %2, %6, %18\n\t" OP " %3, %6, %22\n\t"                 \
               OP " %0, %7, %11\n\t" OP " %1, %7, %15\n\t" OP " %2, %7, %19\n\t" OP " %3, %7, %23\n\ts_nop 3"           \
               : "+v"(p[0]), "+v"(p[1]), "+v"(p[2]), "+v"(p[3])                                                        \
               : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(b[0][0]), "v"(b[0][1]), "v"(b[0][2]), "v"(b[0][3]),   \
                 "v"(b[1][0]), "v"(b[1][1]), "v"(b[1][2]), "v"(b[1][3]), "v"(b[2][0]), "v"(b[2][1]), "v"(b[2][2]),     \
                 "v"(b[2][3]), "v"(b[3][0]), "v"(b[3][1]), "v"(b[3][2]), "v"(b[3][3]))
template <> __device__ __forceinline__ void dot8x4<bf16_t>(float (&p)[4], u32x4 a, const u32x4 (&b)[4]) { ADSP_DOT8X4("v_dot2c_f32_bf16"); }
template <> __device__ __forceinline__ void dot8x4<f16_t>(float (&p)[4], u32x4 a, const u32x4 (&b)[4]) { ADSP_DOT8X4("v_dot2c_f32_f16"); }
#undef ADSP_DOT8X4

// Sixteen independent 4 x 4 x 4 products on the matrix pipe (a block = four neighbouring lanes): lane 4 b + i holds row i
// of A_b (four values along k) and column i of B_b; its four result registers are column i of D_b = A_b B_b + C_b.
typedef short mfma4_s4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ f32x4_t mfma4_bf16(u32x2_t a, u32x2_t b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(mfma4_s4, a), __builtin_bit_cast(mfma4_s4, b), c, 0, 0, 0);
}
// x as the sum of two bf16 values (16 bits of x in all): the leading one, or what is left of x behind it
__device__ __forceinline__ uint32_t bf16_part(float x, bool rest) {
  const float hi = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, x) & 0xffff0000u);
  return __builtin_bit_cast(uint32_t, rest ? x - hi : hi) >> 16;
}

template <int LANES> __device__ __forceinline__ float group_sum(float x) {
  if constexpr (LANES == 16) {
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x140, 0xf, 0xf, false));  // row_mirror
  }
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x141, 0xf, 0xf, false));  // row_half_mirror
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0xB1, 0xf, 0xf, false));   // quad_perm [1,0,3,2]
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x4E, 0xf, 0xf, false));   // quad_perm [2,3,0,1]
  return x;
}

template <typename T, int D, int AM>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(ADSP_SPARSE_WAVES, ADSP_SPARSE_WAVES))) void attn_bwd_dq_sparse_kernel(AttnBwdParams p) {
  using G = TileGeo<T, D>;
  using SG = SparseGeo<T, D>;
  using KS = Swz<G::kKRow>;
  static_assert(G::k16, "16-bit element types only");
  static_assert(AM == ATT_15 || AM == ATT_2 || AM == ATT_GEN, "alpha = 1.5, 2 or any other in (1, 2)");
  constexpr int NW = SG::kNW, BM = SG::kBM;
  __shared__ __align__(1024) unsigned char lds_all[SG::kLds];
  __shared__ int s_item, s_skip;
  // a lane ran out of event slots, or a wave out of list room.  Two words: the walks write the one of the tile's
  // parity and read the other one behind the next barrier, so no wave can read a word another one is still setting
  __shared__ uint32_t s_giveup[2];

  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int N = p.N;
  const int n_mblk = (N + BM - 1) / BM;
  const int group = p.Hq / p.Hkv;
  const long long total = (long long)p.B * p.Hkv * n_mblk * group;
  const long long per_xcd = (total + 7) / 8;
  const float qs = p.qscale, inv_qs = 1.f / p.qscale;
  constexpr int kKPer = (G::kKLoads + NW - 1) / NW;
  constexpr bool kKStep = (NW * 64 / KS::kC) % 16 == 0 && (NW * 64) % KS::kC == 0;
  static_assert(kKStep && G::kKLoads % NW == 0, "head dims 32 .. 128");

  // (the probe left too little to this kernel: the dense kernel serves everything)
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
      s_skip = 0;
      if (got >= 0) {  // the K/V head of the row block, as decoded below
        int unit = got / (group * n_mblk);
        const int units = p.B * p.Hkv;
        if (units % 8 == 0) unit = (unit % (units / 8)) * 8 + unit / (units / 8);
        // (a K/V head the probe marked is left to the dense kernel; nothing else is consulted, so the same inputs take
        // the same way on every call)
        s_skip = __hip_atomic_load(p.hints + 2 * unit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= (1u << 20) ? 1 : 0;
      }
      s_giveup[0] = 0u;
      s_giveup[1] = 0u;
    }
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
    const int qi = m0 + wave * 32 + lq;

    if (m0 >= L) {  // row block entirely inside the padding: zero gradient
      constexpr int kRowDw = D * 2 / 4;
      uint32_t* o32 = reinterpret_cast<uint32_t*>(p.dq) + (qo_base + (size_t)m0 * D) * 2 / 4;
      const int rows = (N - m0) < BM ? (N - m0) : BM;
      for (int i = tid; i < rows * kRowDw; i += SG::kThreads) o32[i] = 0u;
      if (tid == 0) *flag = 0;
      continue;
    }

    // (where the forward kept its candidate stream for this row block there is no walk: see below; a row block the
    // forward's sparse-support kernel did not serve -- its supports outgrew that kernel's lists, which are this one's --
    // goes to the dense kernel without a walk)
    const bool fwd_kept = p.fwd_streams != nullptr;
    const bool from_fwd = fwd_kept && p.fwd_flags[(size_t)(b * p.Hq + h) * n_mblk + mblk] == 1;
    if (s_skip || (fwd_kept && !from_fwd)) {
      if (tid == 0) {
        *flag = 1;
        atomicAdd(&p.queue[kCtrlFlagged], 1u);
      }
      continue;
    }
    const int row_hi = (m0 + BM < L ? m0 + BM : L);
    const int nt = p.causal ? (row_hi + kBN - 1) / kBN : (L + kBN - 1) / kBN;
    const int lim = p.causal ? (qi < L - 1 ? qi : L - 1) : L - 1;
    const int wave_row0 = m0 + wave * 32;
    const bool live = qi < L;

    // ---- Q fragments; rows past the valid length are zero (their scores are never used).  The forward's threshold
    // in raw score units: the walk's accumulators start at its negative, so a positive result is a member of the
    // support ----------------------------------------------------------------------------------------------------
    const uint16_t* const qrow = reinterpret_cast<const uint16_t*>(p.q) + qo_base + (size_t)(live ? qi : 0) * D;
    uint32_t qf[G::kQRegs];
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) {
      u32x4 raw = {0u, 0u, 0u, 0u};
      if (!from_fwd) raw = *reinterpret_cast<const u32x4*>(qrow + ks * 16 + 8 * lh);
#pragma unroll
      for (int e = 0; e < 4; ++e) qf[ks * 4 + e] = live ? raw[e] : 0u;
    }
    const float lo_raw = live ? p.taus[(size_t)(b * p.Hq + h) * N + qi] * inv_qs : INFINITY;

    const unsigned char* kglob = reinterpret_cast<const unsigned char*>(p.k) + kv_base * 2;
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

    // ---- the walk: collect the scores above the threshold ---------------------------------------------------------
    // A lane whose eight scores of a 16-key half block have a positive maximum puts them, with a tag, into the wave's
    // ring in LDS (slots are handed out with a ballot: no atomics).  When the ring is full the wave empties it, one
    // event per lane: the positive entries go to the wave's candidate stream in global memory as (score - threshold, key
    // and row) pairs, compact and in bursts, so the tile loop rarely waits for a store.
    float* const ring = reinterpret_cast<float*>(lds_all + SG::kStages * G::kKTile + wave * SG::kRingBytes);
    uint32_t* const ring_tag = reinterpret_cast<uint32_t*>(ring + SG::kRing * 8);
    // (with the hand-over to the dK/dV kernel the stream has a place of its own per row block and wave, and stays)
    const size_t stream_id = ((size_t)(b * p.Hq + h) * n_mblk + mblk) * NW + wave;
    uint2* const stream = p.streams ? reinterpret_cast<uint2*>(p.streams) + stream_id * (size_t)kSparseStreamCap
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
#if ADSP_DQ_STOP == 3
    continue;
#endif
    if (from_fwd) {
      // The forward's stream of this row block and wave holds every score above a lower bound of the rows' thresholds,
      // as (score - bound, key | row) pairs in the order of its walk, and the forward left every row's threshold minus
      // bound: the entries above it are the members, and their order stays (the table below relies on it).
      const int n_fwd = (int)p.fwd_lens[stream_id] < SG::kListCap ? (int)p.fwd_lens[stream_id] : SG::kListCap;
      const uint2* const src = reinterpret_cast<const uint2*>(p.fwd_streams) + stream_id * (size_t)kSparseStreamCap;
      const float t_mine = live ? p.fwd_tshift[(size_t)(b * p.Hq + h) * N + qi] : INFINITY;  // lanes r and r + 32: row r
      constexpr int kPerF = (SG::kListCap + 63) / 64;
      uint2 fe[kPerF];  // (all loads under way together: one trip to memory, not one per 64 entries)
#pragma unroll
      for (int j = 0; j < kPerF; ++j) {
        const int e = j * 64 + lane;
        fe[j] = uint2{0u, 0u};
        if (e < n_fwd) fe[j] = src[e];
      }
#pragma unroll
      for (int j = 0; j < kPerF; ++j) {
        if (j * 64 < n_fwd) {
          const int e = j * 64 + lane;
          const uint2 ent = fe[j];
          const float x = __builtin_bit_cast(float, ent.x) - __shfl(t_mine, (int)((ent.y >> 20) & 31u), 64);
          const bool keep = e < n_fwd && x > 0.f;
          const unsigned long long m = __builtin_amdgcn_ballot_w64(keep);
          if (keep) {
            const int at = stream_n + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
            stream[at] = uint2{__builtin_bit_cast(uint32_t, x), ent.y};
          }
          stream_n += __builtin_popcountll(m);
        }
      }
    } else {
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
        collect(s0, 0, h00, (uint32_t)(kt * 4 + 0), kt);
        collect(s0, 8, h01, (uint32_t)(kt * 4 + 1), kt);
        collect(s1, 0, h10, (uint32_t)(kt * 4 + 2), kt);
        collect(s1, 8, h11, (uint32_t)(kt * 4 + 3), kt);
      });
    });
    flush(0, nt);
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);  // the wave's stream is in memory before it reads it back
    __syncthreads();                      // every wave has left the K tiles: LDS becomes the lists
    if (s_giveup[0] | s_giveup[1]) {
      if (tid == 0) {
        *flag = 1;
        atomicAdd(&p.queue[kCtrlFlagged], 1u);
      }
      continue;
    }
#if ADSP_DQ_STOP == 2
    continue;
#endif

    // ---- the wave's stream -> per-row lists in its share of LDS (a counting sort by row) ----------------------------
    unsigned char* const wave_lds = lds_all + wave * SG::kWaveLds;
    float* const lval = reinterpret_cast<float*>(wave_lds);                                  // kListCap scores minus the threshold
    uint16_t* const lkey = reinterpret_cast<uint16_t*>(wave_lds + SG::kListCap * 4);         // their keys
    uint32_t* const row_cnt = reinterpret_cast<uint32_t*>(wave_lds + SG::kListCap * 6);     // 32 counters
    uint32_t* const row_start = row_cnt + 32;                                                // 33 offsets
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
      if (p.stream_dir) {
        // The walk went through the key tiles in order and the ring keeps the order of its events, so the stream is
        // sorted by 16-key half block.  dir[k] = index of the first entry whose key is >= 32 k (k = 0 .. 4 n_mblk; the last
        // one is the stream's length): the entry that opens a new 32-key block writes the offsets of the blocks it
        // skipped and its own, and the position behind the last entry closes the table.
        static_assert(kPer * 64 > SG::kListCap, "the position behind the last entry belongs to one of the groups");
        uint16_t* const dir = p.stream_dir + stream_id * (size_t)p.dir_stride;
        const int n32 = n_mblk * (BM / 32);
        int carry = -1;  // 32-key block of the entry before this group of 64
#pragma unroll
        for (int j = 0; j < kPer; ++j) {
          if (j * 64 <= stream_n) {
            const int e = j * 64 + lane;
            const int kb = e < stream_n ? (int)((ent[j].y & 0xffffu) >> 5) : n32;
            int prev = __shfl_up(kb, 1, 64);
            prev = lane == 0 ? carry : prev;
            if (e <= stream_n)
              for (int k = prev + 1; k <= kb; ++k) dir[k] = (uint16_t)e;
            carry = __builtin_amdgcn_readlane(kb, 63);
          }
        }
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
          // (hand-over: the entry's first word becomes its place in the lists until the weights are known)
          if (p.stream_dir) reinterpret_cast<uint32_t*>(stream + e)[0] = at;
        }
      }
    }

    // ---- per row: dP over the support, delta, dQ.  A group of D / 8 lanes per row, each lane 8 columns; the V and K
    // rows of kDepth members of the support are in flight together.  delta is only known behind the last member, so
    // the lanes keep A = sum u dP k and B = sum u k and form (A - delta B) / sqrt(D) at the end. ---------------------
    {
      constexpr int kLPR = D / 8;         // lanes per row
      constexpr int kGroups = 64 / kLPR;  // rows in progress per wave
      constexpr int kDepth = 4;
      const int grp = lane / kLPR, col = lane % kLPR;
      const bool hand_over = p.stream_dir != nullptr;  // the stream stays for the dK/dV kernel
      const unsigned char* vrows = reinterpret_cast<const unsigned char*>(p.v) + kv_base * 2;
      const unsigned char* krows = kglob;
      const uint32_t col16 = (uint32_t)col * 16u;  // (32-bit offsets per lane: a head's rows span N * D * 2 <= 16 MB)
      const unsigned char* dorows = reinterpret_cast<const unsigned char*>(p.dout) + (qo_base + (size_t)wave_row0 * D) * 2 + col * 16;
      unsigned char* dqrows = reinterpret_cast<unsigned char*>(p.dq) + (qo_base + (size_t)wave_row0 * D) * 2 + col * 16;
      // The rows are served kGroups at a time and a round lasts as long as its longest list: rows in the order of their
      // list lengths, longest first, keep the rows of a round alike.  row_cnt (free since the sort) becomes that order.
      {
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        int rank = 0;
        const int mine = lane < 32 ? (int)(row_start[lane + 1] - row_start[lane]) : 0;
        for (int o = 0; o < 32; ++o) {
          const int c = (int)(row_start[o + 1] - row_start[o]);
          rank += (c > mine || (c == mine && o < lane)) ? 1 : 0;
        }
        __builtin_amdgcn_wave_barrier();
        if (lane < 32) row_cnt[rank] = (uint32_t)lane;
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
      }
#if ADSP_DQ_STOP == 1
      for (int r0 = 0; r0 < 0; r0 += kGroups) {
#else
      for (int r0 = 0; r0 < 32; r0 += kGroups) {
#endif
        const int r = (int)row_cnt[r0 + grp];
        const bool row_live = wave_row0 + r < L;
        const int e_lo = (int)row_start[r], e_hi = (int)row_start[r + 1];
        u32x4 dov = {0u, 0u, 0u, 0u};  // the lane's eight columns of dO_i (rows past the valid length may hold anything: not read)
        if (row_live) dov = *reinterpret_cast<const u32x4*>(dorows + (size_t)r * (D * 2));
        // A = sum u dP k and B = sum u k.  bf16: on the matrix pipe, idle in this kernel -- per column of the lane a
        // 4 x 4 x 4 product whose k runs over the four members in flight, whose A rows are the weights u dP and u, each
        // split into two bf16 values (lane 4 b + i of a block supplies row i: the weights lose nothing that a 16-bit
        // result could show), and whose B column is the members' K values at that column; register i of the result adds
        // up weight i times K.  f16 (whose exponent range the weights can leave): fp32 multiply-adds.
        constexpr bool kOnMatrixPipe = std::is_same<T, bf16_t>::value;
        float acc_a[8], acc_b[8];
        f32x4_t acc4[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          acc_a[i] = 0.f;
          acc_b[i] = 0.f;
          acc4[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        }
        const bool kind_u = (lane & 2) != 0, kind_rest = (lane & 1) != 0;
        float zsum = 0.f, usum = 0.f, udp = 0.f;
        // (the rows of a round come longest list first: the first group's row sets the number of turns)
        const int n_turns = (__builtin_amdgcn_readfirstlane(e_hi - e_lo) + kDepth - 1) / kDepth;
        for (int turn = 0; turn < n_turns; ++turn) {
          const int eb = e_lo + turn * kDepth;
          // (a group whose list has ended reads on without a condition, at a place inside the wave's LDS)
          const int ebr = eb < SG::kListCap ? eb : SG::kListCap;
          u32x4 vv[kDepth], kk[kDepth];
          float val[kDepth];
#pragma unroll
          for (int j = 0; j < kDepth; ++j) {
            // a slot without a member takes the first key's rows (always valid) with a zero score: no weight, no branch
            const bool has = eb + j < e_hi;
            const uint32_t kraw = (uint32_t)lkey[ebr + j];
            const float vraw = lval[ebr + j];
            const uint32_t key = has ? kraw : 0u;
            val[j] = has ? vraw : 0.f;
            const uint32_t roff = key * (uint32_t)(D * 2) + col16;
            vv[j] = *reinterpret_cast<const u32x4*>(vrows + roff);
            kk[j] = *reinterpret_cast<const u32x4*>(krows + roff);
          }
          static_assert(kDepth == 4, "dot8x4 and the 4 x 4 x 4 products take four members");
          float part[kDepth] = {0.f, 0.f, 0.f, 0.f};
          dot8x4<T>(part, dov, vv);
          float dp[kDepth], uu[kDepth];
#pragma unroll
          for (int j = 0; j < kDepth; ++j) dp[j] = group_sum<kLPR>(part[j]);  // dO_i . v_j, in every lane of the group
#pragma unroll
          for (int j = 0; j < kDepth; ++j) {
            float pr;
            bwd_prob<AM>(val[j] * qs, p.c0, pr, uu[j]);  // (an absent member has val = 0: p = u = 0)
            zsum += pr;
            usum += uu[j];
            udp = fmaf(uu[j], dp[j], udp);
          }
          // (hand-over: dP takes the place of the member's score, and the score, as a half-precision value, the place of its
          // key; neither is needed again by this loop.  dP stays in fp32: dP - delta cancels most of it.)
          if (hand_over && col == 0) {
#pragma unroll
            for (int j = 0; j < kDepth; ++j) {
              if (eb + j < e_hi) {
                lval[eb + j] = dp[j];
                lkey[eb + j] = __builtin_bit_cast(uint16_t, (_Float16)val[j]);  // (11 bits: p and u are powers of it)
              }
            }
          }
          if constexpr (kOnMatrixPipe) {
            uint32_t w16[kDepth];
#pragma unroll
            for (int j = 0; j < kDepth; ++j) w16[j] = bf16_part(kind_u ? uu[j] : uu[j] * dp[j], kind_rest);
            const u32x2_t aw = {w16[0] | (w16[1] << 16), w16[2] | (w16[3] << 16)};
#pragma unroll
            for (int i = 0; i < 4; ++i) {  // (the members' values at an even and at an odd column: the low and the high halves)
              const u32x2_t b_even = {__builtin_amdgcn_perm(kk[1][i], kk[0][i], 0x05040100u), __builtin_amdgcn_perm(kk[3][i], kk[2][i], 0x05040100u)};
              const u32x2_t b_odd = {__builtin_amdgcn_perm(kk[1][i], kk[0][i], 0x07060302u), __builtin_amdgcn_perm(kk[3][i], kk[2][i], 0x07060302u)};
              acc4[2 * i] = mfma4_bf16(aw, b_even, acc4[2 * i]);
              acc4[2 * i + 1] = mfma4_bf16(aw, b_odd, acc4[2 * i + 1]);
            }
          } else {
#pragma unroll
            for (int j = 0; j < kDepth; ++j) {
              const float wa = uu[j] * dp[j];
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                const float klo = unpack_lo<T>(kk[j][i]), khi = unpack_hi<T>(kk[j][i]);
                acc_a[2 * i] = fmaf(wa, klo, acc_a[2 * i]);
                acc_a[2 * i + 1] = fmaf(wa, khi, acc_a[2 * i + 1]);
                acc_b[2 * i] = fmaf(uu[j], klo, acc_b[2 * i]);
                acc_b[2 * i + 1] = fmaf(uu[j], khi, acc_b[2 * i + 1]);
              }
            }
          }
        }
        if constexpr (kOnMatrixPipe) {
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            acc_a[i] = acc4[i][0] + acc4[i][1];
            acc_b[i] = acc4[i][2] + acc4[i][3];
          }
        }
        const float delta = usum > 0.f ? udp / usum : 0.f;
        if (hand_over) {
          // what the dK/dV kernel needs of a member: p / sum p (weight of dO_i in dV_j) and u (dP - delta) (weight of q_i
          // in dK_j), as a pair of the element type in place of the member's score
          const float zinv_r = zsum > 0.f ? 1.f / zsum : 0.f;
          __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
          __builtin_amdgcn_wave_barrier();
          for (int e = e_lo + col; e < e_hi; e += kLPR) {
            float pr, u;
            bwd_prob<AM>((float)__builtin_bit_cast(_Float16, lkey[e]) * qs, p.c0, pr, u);
            reinterpret_cast<uint32_t*>(lval)[e] = pack2<T>(pr * zinv_r, u * (lval[e] - delta));
          }
        }
        if (wave_row0 + r < N) {
          float g[8];
#pragma unroll
          for (int i = 0; i < 8; ++i) g[i] = row_live ? p.sm_scale * (acc_a[i] - delta * acc_b[i]) : 0.f;
          u32x4 w = {pack2<T>(g[0], g[1]), pack2<T>(g[2], g[3]), pack2<T>(g[4], g[5]), pack2<T>(g[6], g[7])};
          *reinterpret_cast<u32x4*>(dqrows + (size_t)r * (D * 2)) = w;
        }
        if (row_live && col == 0) {
          const size_t at = (size_t)(b * p.Hq + h) * N + wave_row0 + r;
          p.delta[at] = delta;
          p.zinv[at] = zsum > 0.f ? 1.f / zsum : 0.f;
        }
      }
      if (hand_over) {
        // every stream entry takes its member's pair of weights from the lists (its first word held the place)
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_s_waitcnt(0x0f70);
        constexpr int kPer = (SG::kListCap + 63) / 64;
        uint32_t at[kPer];  // (all loads under way together: one trip to memory, not one per 64 entries)
#pragma unroll
        for (int j = 0; j < kPer; ++j) {
          const int e = j * 64 + lane;
          at[j] = 0u;
          if (e < stream_n)  // (written by this wave: not from its L1)
            at[j] = __hip_atomic_load(reinterpret_cast<uint32_t*>(stream + e), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int j = 0; j < kPer; ++j) {
          const int e = j * 64 + lane;
          if (e < stream_n) reinterpret_cast<uint32_t*>(stream + e)[0] = reinterpret_cast<const uint32_t*>(lval)[at[j] < (uint32_t)SG::kListCap ? at[j] : 0u];
        }
      }
    }
    if (tid == 0) {
      *flag = 0;
    }
  }
}


// dK and dV from the keys' side of the same lists: the lane's "row" is a key, the tiles are rows of q of one query
// head, and a score minus the *query's* threshold is positive exactly when the key lies in that query's support (the
// thresholds of a tile's 64 queries arrive in LDS with the tile and are subtracted after the products).  The walk,
// the ring, the stream and the counting sort are those of the dQ kernel with the roles swapped; the lists then hold,
// per key, the queries that weight it.  A workgroup serves one (key block, query head).  The results are fp32
// partial rows per query head that dkdv_reduce_kernel adds up over the heads of a K/V head.  The first key blocks of a
// causal sequence lie in the supports of hundreds of queries each: when a wave's stream is half full the walk pauses,
// the lists made so far are worked off into the partial rows, and the walk goes on.  A key block that any of its query
// heads gives up all the same is flagged and computed, all heads, by attn_bwd_dkdv_kernel.
template <typename T, int D, int AM>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(ADSP_SPARSE_WAVES, ADSP_SPARSE_WAVES))) void attn_bwd_dkdv_sparse_kernel(AttnBwdParams p) {
  using G = TileGeo<T, D>;
  using SG = SparseGeo<T, D>;
  using KS = Swz<G::kKRow>;
  static_assert(G::k16, "16-bit element types only");
  static_assert(AM == ATT_15 || AM == ATT_2 || AM == ATT_GEN, "alpha = 1.5, 2 or any other in (1, 2)");
  constexpr int NW = SG::kNW, BM = SG::kBM;
  __shared__ __align__(1024) unsigned char lds_all[SG::kLds];
  __shared__ int s_item, s_skip;
  // a lane ran out of event slots, or a wave out of list room.  Two words: the walks write the one of the tile's
  // parity and read the other one behind the next barrier, so no wave can read a word another one is still setting
  __shared__ uint32_t s_giveup[2];
  __shared__ float s_tau[SG::kStages][kBN];  // thresholds of the tile's queries

  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int N = p.N;
  const int n_mblk = (N + BM - 1) / BM;
  const int group = p.Hq / p.Hkv;
  const long long total = (long long)p.B * p.Hkv * n_mblk * group;
  const long long per_xcd = (total + 7) / 8;
  const float qs = p.qscale, inv_qs = 1.f / p.qscale;
  constexpr int kKPer = (G::kKLoads + NW - 1) / NW;
  constexpr bool kKStep = (NW * 64 / KS::kC) % 16 == 0 && (NW * 64) % KS::kC == 0;
  static_assert(kKStep && G::kKLoads % NW == 0, "head dims 32 .. 128");

  // (the probe left too little to this kernel: the dense kernel serves everything)
  if (sparse_steps_aside(p.hints2, p.varlen, p.varlen_bits, p.B, p.Hkv, p.N)) {
    if (blockIdx.x == 0 && threadIdx.x == 0) p.queue2[kCtrlAllDense] = 1u;
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

    __syncthreads();  // the previous row block is done with LDS and with s_item
    if (tid == 0) {
      int got = -1;
      while (queues_tried < 8) {
        const int x = ((int)(blockIdx.x & 7) + queues_tried) & 7;
        const long long i = (long long)atomicAdd(&p.queue2[x], 1u);
        const long long logical = (long long)x * per_xcd + i;
        if (i < per_xcd && logical < total) {
          got = (int)logical;
          break;
        }
        ++queues_tried;
      }
      s_item = got;
      s_skip = 0;
      if (got >= 0) {  // the K/V head of the row block, as decoded below
        int unit = got / (group * n_mblk);
        const int units = p.B * p.Hkv;
        if (units % 8 == 0) unit = (unit % (units / 8)) * 8 + unit / (units / 8);
        s_skip = __hip_atomic_load(p.hints2 + 2 * unit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= (1u << 20) ? 1 : 0;
      }
      s_giveup[0] = 0u;
      s_giveup[1] = 0u;
    }
    __syncthreads();
    const int logical = s_item;
    if (logical < 0) break;

    // ---- item -> (batch, kv head, key block, head in group), in the order of the dQ kernel's row blocks ---------
    const int hg = logical % group;
    const int mi = (logical / group) % n_mblk;
    int bkv = logical / (group * n_mblk);
    {
      const int units = p.B * p.Hkv;
      if (units % 8 == 0) bkv = (bkv % (units / 8)) * 8 + bkv / (units / 8);
    }
    const int b = bkv / p.Hkv, kvh = bkv % p.Hkv;
    const int h = kvh * group + hg;
    const int mblk = mi;  // key block: with a causal mask the first ones see the most queries
    const int m0 = mblk * BM;
    int L = N;
    if (p.varlen) {
      long long l = p.varlen_bits == 64 ? ((const long long*)p.varlen)[b] : (long long)((const int*)p.varlen)[b];
      L = (int)(l < 0 ? 0 : (l > N ? N : l));
    }
    // a key block that any query head gives up goes to attn_bwd_dkdv_kernel with all its heads
    int32_t* const flag = p.kv_flags + ((size_t)(b * p.Hkv + kvh) * n_mblk + mblk);
    const size_t qo_base = ((size_t)(b * p.Hq + h) * N) * D;
    const size_t kv_base = ((size_t)(b * p.Hkv + kvh) * N) * D;
    const int qi = m0 + wave * 32 + lq;

    if (m0 >= L) continue;  // key block entirely inside the padding: dkdv_reduce_kernel writes its zeros without reading partial rows

    if (s_skip) {
      if (tid == 0) {
        *flag = 1;
        atomicAdd(&p.queue2[kCtrlFlagged], 1u);
      }
      continue;
    }
    // here the lane's "row" is a key (qi: its index) and the tiles hold queries: with a causal mask the tiles from the
    // key block's first key on, else all of them
    const int kt_first = p.causal ? m0 / kBN : 0;
    const int nt = (L + kBN - 1) / kBN - kt_first;
    const int lo_lim = p.causal ? qi : 0;  // first query that sees the lane's key
    const int wave_row0 = m0 + wave * 32;
    const bool live = qi < L;

    // ---- K fragments of the lane's key; keys past the valid length are zero and collect nothing ------------------
    const uint16_t* const qrow = reinterpret_cast<const uint16_t*>(p.k) + kv_base + (size_t)(live ? qi : 0) * D;
    uint32_t qf[G::kQRegs];  // (loaded at the start of every part of the walk: not kept through the list phases)
    const float* const tau_rows = p.taus + (size_t)(b * p.Hq + h) * N;

    // the tiles are rows of q of the item's query head; wave 0 also brings the thresholds of the tile's 64 queries
    const unsigned char* kglob = reinterpret_cast<const unsigned char*>(p.q) + qo_base * 2;
    auto issue_k = [&](unsigned char* lds, int cur) {
      const int kt = kt_first + cur;
      if (wave == 0) {
        const int stage_i = (int)((lds - lds_all) / G::kKTile);
        int gi = kt * kBN + lane;
        gi = gi < N ? gi : N - 1;
        dma4s(uniform_ptr(tau_rows), (uint32_t)gi * 4u, &s_tau[stage_i][0]);
      }
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
    // body(tile index, tile) over the query tiles of the item; stops when a lane gave up or asked for a break.  The tiles go through a ring of
    // kStages LDS buffers: the load of tile t + kStages - 1 is issued behind the barrier that opens tile t (every wave
    // is done with tile t - 1, whose buffer it takes) and has kStages - 1 tile times to arrive.
    // (stages_c, tile_c, per_c: the ring's depth, the bytes of a tile and the loads per wave and tile, as constants)
    // Here the walk starts at tile `first` and returns the tile it stopped in front of (nt: all done): a wave whose stream
    // is half full asks for a break, the lists made so far are worked off, and the walk goes on from there.
    auto walk = [&](int first, auto stages_c, auto tile_c, auto per_c, auto&& issue, auto&& body) -> int {
      constexpr int kStages = decltype(stages_c)::value, kTile = decltype(tile_c)::value, kPer = decltype(per_c)::value;
      __syncthreads();
#pragma unroll
      for (int s = 0; s < kStages - 1; ++s)
        if (first + s < nt) issue(lds_all + s * kTile, first + s);
      int stage = 0;  // buffer of tile cur
      int cur = first;
      for (; cur < nt; ++cur) {
        // this wave's share of tile cur has landed: everything but the loads issued after it (those of the tiles in
        // between; stores issued after it only make the wait longer than needed)
        if (cur + kStages - 1 <= nt) {
          if constexpr (kStages == 2) __builtin_amdgcn_s_waitcnt(0x0f70);
          else __builtin_amdgcn_s_waitcnt(0x0f70 | ((kStages - 2) * kPer));
        } else {
          __builtin_amdgcn_s_waitcnt(0x0f70);  // the last tiles: nothing was issued behind them
        }
        __syncthreads();
        if (cur > first && s_giveup[(cur + 1) & 1]) break;  // set while the previous tile was worked on
        const int pre = cur + kStages - 1;
        if (pre < nt) issue(lds_all + (stage == 0 ? kStages - 1 : stage - 1) * kTile, pre);
        __builtin_amdgcn_sched_barrier(0);
        body(cur, lds_all + stage * kTile);
        stage = stage + 1 == kStages ? 0 : stage + 1;
      }
      return cur;
    };
    // scores of one tile (two blocks of 32 queries) against the lanes' keys, minus the queries' thresholds; f(s0, s1)
    // unless no key of the wave is seen by the tile.  Pairs outside the mask or the sequence are -inf.
    auto for_tile = [&](int kt, const unsigned char* kt_lds, auto&& f) {
      if (p.causal && kt * kBN + kBN - 1 < wave_row0) return;  // every query of the tile lies before the wave's keys
      const bool need_mask = (kt * kBN + kBN - 1 > L - 1) || (p.causal && kt * kBN < wave_row0 + 31);
      f32x16 s0, s1;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        s0[i] = 0.f;
        s1[i] = 0.f;
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
      {  // minus the queries' thresholds (raw units): what is left positive is a member of that query's support
        const float* tq = &s_tau[(int)((kt_lds - lds_all) / G::kKTile)][4 * lh];
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const f32x4 t0 = *reinterpret_cast<const f32x4*>(tq + 8 * g4), t1 = *reinterpret_cast<const f32x4*>(tq + 32 + 8 * g4);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            s0[4 * g4 + e] = fmaf(t0[e], -inv_qs, s0[4 * g4 + e]);
            s1[4 * g4 + e] = fmaf(t1[e], -inv_qs, s1[4 * g4 + e]);
          }
        }
      }
      if (need_mask) {  // queries past the sequence's end (their thresholds may hold anything) or before the lane's key
        const int jb = kt * kBN + 4 * lh;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int i0 = jb + 8 * (i >> 2) + (i & 3), i1 = i0 + 32;
          s0[i] = (i0 < L && i0 >= lo_lim) ? s0[i] : -INFINITY;
          s1[i] = (i1 < L && i1 >= lo_lim) ? s1[i] : -INFINITY;
        }
      }
      f(s0, s1);
    };

    // ---- the walk: collect the scores above the threshold ---------------------------------------------------------
    // A lane whose eight scores of a 16-key half block have a positive maximum puts them, with a tag, into the wave's
    // ring in LDS (slots are handed out with a ballot: no atomics).  When the ring is full the wave empties it, one
    // event per lane: the positive entries go to the wave's candidate stream in global memory as (score - threshold, key
    // and row) pairs, compact and in bursts, so the tile loop rarely waits for a store.
    float* const ring = reinterpret_cast<float*>(lds_all + SG::kStages * G::kKTile + wave * SG::kRingBytes);
    uint32_t* const ring_tag = reinterpret_cast<uint32_t*>(ring + SG::kRing * 8);
    uint2* const stream = reinterpret_cast<uint2*>(p.events) + ((size_t)blockIdx.x * NW + wave) * (size_t)kSparseStreamCap;
    int ring_n = 0, stream_n = 0;  // wave-uniform
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
        // (no projection here: a key's queries thin out along the walk, the first tiles bring most of its members)
        if (stream_n + total_c > SG::kListCap) {
          if (lane == 0) atomicOr(&s_giveup[parity], 1u);  // bit 0: give the key block up
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
          if (stream_n > SG::kListCap / 2 && lane == 0) atomicOr(&s_giveup[parity], 2u);  // bit 1: break the walk here
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
      const bool mine = hmax > 0.f && live;
      const unsigned long long m = __builtin_amdgcn_ballot_w64(mine);
      if (m != 0ull) {
        if (__builtin_popcountll(m) <= SG::kRing) {
          put(m, mine, s, first, tag, kt);
        } else {  // more events than the ring holds at once: in two halves
          put(m & 0xffffffffull, mine && lane < 32, s, first, tag, kt);
          put(m & ~0xffffffffull, mine && lane >= 32, s, first, tag, kt);
        }
      }
    };
    int done = 0;           // tiles of the item walked so far
    bool gave_up = false;
    for (int seg = 0;; ++seg) {
    ring_n = 0;
    stream_n = 0;
    {
      const uint16_t* krow = qrow;
      asm volatile("" : "+v"(krow));  // (keeps the loads inside the loop)
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) {
        const u32x4 raw = *reinterpret_cast<const u32x4*>(krow + ks * 16 + 8 * lh);
#pragma unroll
        for (int e = 0; e < 4; ++e) qf[ks * 4 + e] = live ? raw[e] : 0u;
      }
    }
    done = walk(done, std::integral_constant<int, SG::kStages>{}, std::integral_constant<int, G::kKTile>{}, std::integral_constant<int, kKPer>{}, issue_k, [&](int cur, const unsigned char* kt_lds) {
      const int kt = kt_first + cur;
      for_tile(kt, kt_lds, [&](const f32x16& s0, const f32x16& s1) {
        float h00 = s0[0], h01 = s0[8], h10 = s1[0], h11 = s1[8];
#pragma unroll
        for (int i = 1; i < 8; ++i) {
          h00 = fmaxf(h00, s0[i]);
          h01 = fmaxf(h01, s0[8 + i]);
          h10 = fmaxf(h10, s1[i]);
          h11 = fmaxf(h11, s1[8 + i]);
        }
        collect(s0, 0, h00, (uint32_t)(kt * 4 + 0), kt);
        collect(s0, 8, h01, (uint32_t)(kt * 4 + 1), kt);
        collect(s1, 0, h10, (uint32_t)(kt * 4 + 2), kt);
        collect(s1, 8, h11, (uint32_t)(kt * 4 + 3), kt);
      });
    });
    flush(0, kt_first + done);
    __builtin_amdgcn_s_waitcnt(0x0f70);  // the wave's stream is in memory before it reads it back
    __syncthreads();                      // every wave has left the K tiles: LDS becomes the lists
    if ((s_giveup[0] | s_giveup[1]) & 1u) {
      gave_up = true;
      break;
    }

    // ---- the wave's stream -> per-row lists in its share of LDS (a counting sort by row) ----------------------------
    unsigned char* const wave_lds = lds_all + wave * SG::kWaveLds;
    float* const lval = reinterpret_cast<float*>(wave_lds);                                  // kListCap scores minus the threshold
    uint16_t* const lkey = reinterpret_cast<uint16_t*>(wave_lds + SG::kListCap * 4);         // their keys
    uint32_t* const row_cnt = reinterpret_cast<uint32_t*>(wave_lds + SG::kListCap * 6);     // 32 counters
    uint32_t* const row_start = row_cnt + 32;                                                // 33 offsets
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
        }
      }
    }

    // ---- per key: its list holds the queries (of this head) in whose support it lies, with score minus threshold.
    // A group of D / 8 lanes per key, each lane 8 columns of v_j; per member it fetches its 16 bytes of dO_i and q_i and
    // the row's delta_i and 1 / sum p (written by the dQ kernels), forms dP_ij = dO_i . v_j across the group and adds
    // p_ij / sum p * dO_i to dV_j and u_ij (dP_ij - delta_i) * q_i to dK_j. ---------------------------------------------
    {
      constexpr int kLPR = D / 8;         // lanes per key
      constexpr int kGroups = 64 / kLPR;  // keys in progress per wave
      constexpr int kDepth = 4;
      const int grp = lane / kLPR, col = lane % kLPR;
      const unsigned char* vrows = reinterpret_cast<const unsigned char*>(p.v) + kv_base * 2 + col * 16;
      const unsigned char* qrows = kglob + col * 16;
      const unsigned char* dorows = reinterpret_cast<const unsigned char*>(p.dout) + qo_base * 2 + col * 16;
      const float* const delta_rows = p.delta + (size_t)(b * p.Hq + h) * N;
      const float* const zinv_rows = p.zinv + (size_t)(b * p.Hq + h) * N;
      for (int r0 = 0; r0 < 32; r0 += kGroups) {
        const int r = r0 + grp;
        const int key = wave_row0 + r;
        const int e_lo = (int)row_start[r], e_hi = (int)row_start[r + 1];
        u32x4 vj = {0u, 0u, 0u, 0u};  // the lane's eight columns of v_j
        if (key < L) vj = *reinterpret_cast<const u32x4*>(vrows + (size_t)key * (D * 2));
        float acc_v[8], acc_k[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          acc_v[i] = 0.f;
          acc_k[i] = 0.f;
        }
        for (int eb = e_lo; __builtin_amdgcn_ballot_w64(eb < e_hi) != 0ull; eb += kDepth) {
          u32x4 dd[kDepth], qq[kDepth];
          float val[kDepth], dl[kDepth], zi[kDepth];
#pragma unroll
          for (int j = 0; j < kDepth; ++j) {
            val[j] = 0.f;
            dl[j] = 0.f;
            zi[j] = 0.f;
            dd[j] = u32x4{0u, 0u, 0u, 0u};
            qq[j] = u32x4{0u, 0u, 0u, 0u};
            if (eb + j < e_hi) {
              const uint32_t qidx = lkey[eb + j];
              val[j] = lval[eb + j];
              dd[j] = *reinterpret_cast<const u32x4*>(dorows + (size_t)qidx * (D * 2));
              qq[j] = *reinterpret_cast<const u32x4*>(qrows + (size_t)qidx * (D * 2));
              dl[j] = delta_rows[qidx];
              zi[j] = zinv_rows[qidx];
            }
          }
          static_assert(kDepth == 4, "dot8x4 takes four members");
          float part[kDepth] = {0.f, 0.f, 0.f, 0.f};
          dot8x4<T>(part, vj, dd);
#pragma unroll
          for (int j = 0; j < kDepth; ++j) {
            float dof[8];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              dof[2 * i] = unpack_lo<T>(dd[j][i]);
              dof[2 * i + 1] = unpack_hi<T>(dd[j][i]);
            }
            const float dp = group_sum<kLPR>(part[j]);  // dO_i . v_j, in every lane of the group
            float pr, u;
            bwd_prob<AM>(val[j] * qs, p.c0, pr, u);  // (an absent member has val = 0: p = u = 0)
            const float ph = pr * zi[j], dx = u * (dp - dl[j]);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              acc_v[2 * i] = fmaf(ph, dof[2 * i], acc_v[2 * i]);
              acc_v[2 * i + 1] = fmaf(ph, dof[2 * i + 1], acc_v[2 * i + 1]);
              acc_k[2 * i] = fmaf(dx, unpack_lo<T>(qq[j][i]), acc_k[2 * i]);
              acc_k[2 * i + 1] = fmaf(dx, unpack_hi<T>(qq[j][i]), acc_k[2 * i + 1]);
            }
          }
        }
        if (key < N) {
#pragma unroll
          for (int i = 0; i < 8; ++i) acc_k[i] *= p.sm_scale;
          // fp32 partial rows of this query head (dkdv_reduce_kernel adds up the heads of a K/V head).  While parts of the
          // walk are still to come the sums stay in the wave's rows of the workgroup's scratch slot, and the next part
          // adds to them.
          float* const sc = p.part_scratch + (((size_t)blockIdx.x * NW + wave) * 32 + r) * (2 * D) + col * 8;
          if (seg > 0) {
            const f32x4 k0 = *reinterpret_cast<const f32x4*>(sc), k1 = *reinterpret_cast<const f32x4*>(sc + 4);
            const f32x4 v0 = *reinterpret_cast<const f32x4*>(sc + D), v1 = *reinterpret_cast<const f32x4*>(sc + D + 4);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              acc_k[i] += k0[i];
              acc_k[4 + i] += k1[i];
              acc_v[i] += v0[i];
              acc_v[4 + i] += v1[i];
            }
          }
          if (done < nt) {
            *reinterpret_cast<f32x4*>(sc) = f32x4{acc_k[0], acc_k[1], acc_k[2], acc_k[3]};
            *reinterpret_cast<f32x4*>(sc + 4) = f32x4{acc_k[4], acc_k[5], acc_k[6], acc_k[7]};
            *reinterpret_cast<f32x4*>(sc + D) = f32x4{acc_v[0], acc_v[1], acc_v[2], acc_v[3]};
            *reinterpret_cast<f32x4*>(sc + D + 4) = f32x4{acc_v[4], acc_v[5], acc_v[6], acc_v[7]};
          } else {
            const size_t part_at = ((size_t)(b * p.Hq + h) * p.part_rows + key) * D + col * 8;
            float* const o0 = p.dk_part + part_at;
            float* const o1 = p.dv_part + part_at;
            __builtin_nontemporal_store(f32x4{acc_k[0], acc_k[1], acc_k[2], acc_k[3]}, reinterpret_cast<f32x4*>(o0));
            __builtin_nontemporal_store(f32x4{acc_k[4], acc_k[5], acc_k[6], acc_k[7]}, reinterpret_cast<f32x4*>(o0 + 4));
            __builtin_nontemporal_store(f32x4{acc_v[0], acc_v[1], acc_v[2], acc_v[3]}, reinterpret_cast<f32x4*>(o1));
            __builtin_nontemporal_store(f32x4{acc_v[4], acc_v[5], acc_v[6], acc_v[7]}, reinterpret_cast<f32x4*>(o1 + 4));
          }
        }
      }
    }
    if (done >= nt) break;
    __syncthreads();  // every wave is done with its lists: the walk takes the tiles' room back
    if (tid == 0) {
      s_giveup[0] = 0u;
      s_giveup[1] = 0u;
    }
    }  // (parts of the walk)
    if (gave_up) {
      if (tid == 0) {
        *flag = 1;
        atomicAdd(&p.queue2[kCtrlFlagged], 1u);
      }
      continue;
    }
    if (tid == 0) {
    }
  }
}



// dK and dV from the supports the dQ kernel found (16-bit inputs, alpha = 1.5 / 2, head dims 64 / 128): the same sums as
// attn_bwd_dkdv_sparse_kernel without its score walk and without its arithmetic per member.  The dQ kernel leaves the
// stream of every (row block, wave) in place -- per member the pair of weights (p_ij / sum_j p_ij, u_ij (dP_ij -
// delta_i)) in the element type and key | row, sorted by 16-key half block -- with a table of where each 32-key block
// starts.  A workgroup serves one (key block, query head); each of its waves owns 32 keys, looks up the pieces of all
// streams of the head that hold its keys (row blocks from its own on with a causal mask), fetches their entries -- all
// loads under way together, an entry finds its piece by a binary search in a table of the pieces in LDS -- sorts them
// by key into lists in LDS (a counting sort of (weights, query) pairs) and adds up, per key,
// weight times dO_i into dV_j and weight times q_i into dK_j: two-term dot products with the weight in one half of the
// pair, as the dense kernel's matrix products take the weights in the element type.  A wave that has more members than
// its lists hold works them off in parts (the sums wait in fp32 in the workgroup's scratch slot); the waves of a
// workgroup share nothing and do not wait for each other.  The sums are fp32 partial rows per query head for
// dkdv_reduce_kernel; where a K/V head has a single query head the last part writes dK and dV in the element type and
// there is no reduction.  With a causal mask the later key blocks of a sequence (dkdv_block_merged) are short: there
// one item serves all query heads of the K/V head and writes dK and dV itself.  A key block one of whose row blocks the
// dQ kernel gave up (no stream) is flagged for attn_bwd_dkdv_kernel with all its heads.
template <typename T, int D, int AM>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(ADSP_DKDV_WAVES, ADSP_DKDV_WAVES))) void attn_bwd_dkdv_stream_kernel(AttnBwdParams p) {
  constexpr int kQuads = ADSP_DKDV_QUADS;
  using G = TileGeo<T, D>;
  using SG = SparseGeo<T, D>;
  static_assert(G::k16, "16-bit element types only");
  static_assert(AM == ATT_15 || AM == ATT_2 || AM == ATT_GEN, "alpha = 1.5, 2 or any other in (1, 2)");
  constexpr int NW = SG::kNW, BM = SG::kBM;
  __shared__ __align__(16) unsigned char lds_all[NW * SG::kWaveLds];
  __shared__ int s_item, s_skip;

  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int tid = threadIdx.x, lane = tid & 63;
  const int N = p.N;
  const int n_mblk = (N + BM - 1) / BM;
  const int group = p.Hq / p.Hkv;
  const long long total = (long long)p.B * p.Hkv * n_mblk * group;
  const long long per_xcd = (total + 7) / 8;
  const float qs = p.qscale;

  // (the probe left too little to this kernel: the dense kernel serves everything)
  if (sparse_steps_aside(p.hints2, p.varlen, p.varlen_bits, p.B, p.Hkv, p.N)) {
    if (blockIdx.x == 0 && threadIdx.x == 0) p.queue2[kCtrlAllDense] = 1u;
    return;
  }
  int queues_tried = 0;  // thread 0: how many of the eight counters were found empty
  for (;;) {
    __syncthreads();  // the previous item is done with s_item
    if (tid == 0) {
      int got = -1;
      while (queues_tried < 8) {
        const int x = ((int)(blockIdx.x & 7) + queues_tried) & 7;
        const long long i = (long long)atomicAdd(&p.queue2[x], 1u);
        const long long logical = (long long)x * per_xcd + i;
        if (i < per_xcd && logical < total) {
          got = (int)logical;
          break;
        }
        ++queues_tried;
      }
      s_item = got;
      s_skip = 0;
      if (got >= 0) {  // the K/V head of the key block, as decoded below: marked dense by the probe?
        int unit = got / (group * n_mblk);
        const int units = p.B * p.Hkv;
        if (units % 8 == 0) unit = (unit % (units / 8)) * 8 + unit / (units / 8);
        s_skip = __hip_atomic_load(p.hints2 + 2 * unit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= (1u << 20) ? 1 : 0;
      }
    }
    __syncthreads();
    const int logical = s_item;
    if (logical < 0) break;

    // ---- item -> (batch, kv head, key block, head in group), in the order of the dQ kernel's row blocks ---------
    // query head after query head, and per head key block after key block (with a causal mask the first ones see the
    // most queries): the key blocks in flight on an XCD then gather rows of q and dO of one or two heads, some of
    // which stay in its L2
    const int mblk = logical % n_mblk;
    const int hg = (logical / n_mblk) % group;
    int bkv = logical / (group * n_mblk);
    {
      const int units = p.B * p.Hkv;
      if (units % 8 == 0) bkv = (bkv % (units / 8)) * 8 + bkv / (units / 8);
    }
    const int b = bkv / p.Hkv, kvh = bkv % p.Hkv;
    const int h = kvh * group + hg;
    const int m0 = mblk * BM;
    int L = N;
    if (p.varlen) {
      long long l = p.varlen_bits == 64 ? ((const long long*)p.varlen)[b] : (long long)((const int*)p.varlen)[b];
      L = (int)(l < 0 ? 0 : (l > N ? N : l));
    }
    // The late key blocks of a causal sequence are short items: there one item serves all query heads of the K/V head,
    // head after head with the sums waiting in the scratch slot, and writes dK and dV itself -- no partial rows, nothing
    // for dkdv_reduce_kernel to add (which applies the same test).  The items of the other heads end here.
    const bool merged = dkdv_block_merged(p.causal, group, m0, L, p.merge256);
    if (merged && hg != 0) continue;
    const int nh = merged ? group : 1;  // query heads of this item
    const bool direct = group == 1 || merged;  // no sums over heads left to do: dK and dV are written here
    if (m0 >= L) {  // key block entirely inside the padding: zero gradient (dkdv_reduce_kernel writes it unless `direct`)
      if (direct) {
        constexpr int kRowDw = D * 2 / 4;
        const size_t at = (((size_t)(b * p.Hkv + kvh) * N + m0) * D) * 2 / 4;
        uint32_t* const k32o = reinterpret_cast<uint32_t*>(p.dk) + at;
        uint32_t* const v32o = reinterpret_cast<uint32_t*>(p.dv) + at;
        const int rows = (N - m0) < BM ? (N - m0) : BM;
        for (int i = tid; i < rows * kRowDw; i += SG::kThreads) {
          k32o[i] = 0u;
          v32o[i] = 0u;
        }
      }
      continue;
    }
    // a key block that any query head gives up goes to attn_bwd_dkdv_kernel with all its heads
    int32_t* const flag = p.kv_flags + ((size_t)(b * p.Hkv + kvh) * n_mblk + mblk);
    const size_t kv_base = ((size_t)(b * p.Hkv + kvh) * N) * D;
    // the row blocks whose queries can hold the block's keys in their supports
    const int rb_lo = p.causal ? mblk : 0, rb_hi = (L - 1) / BM;
    {  // no stream where the dQ kernel gave a row block up
      int any = s_skip;
      for (int hh = 0; hh < nh; ++hh) {
        const int32_t* const dq_flags = p.block_flags + (size_t)(b * p.Hq + h + hh) * n_mblk;
        for (int rb = rb_lo + tid; rb <= rb_hi; rb += SG::kThreads) any |= dq_flags[rb] != 0 ? 1 : 0;
      }
      if (__syncthreads_or(any)) {
        if (tid == 0) {
          *flag = 1;
          atomicAdd(&p.queue2[kCtrlFlagged], 1u);
        }
        continue;
      }
    }
#if ADSP_DKDV_STOP == 3
    continue;
#endif
    const int wave_row0 = m0 + wave * 32;
    const int k32 = wave_row0 / 32;
    // (row block, wave of the dQ kernel) in order.  Where a 16-bit list entry can name a query of any head of the
    // item (heads x N <= 65536), a merged item takes the pieces of all its heads as one sequence -- query i of head g is
    // row g N + i from the first head's rows on -- and the sums of a part cover all heads; otherwise head follows head.
    const int np1 = (rb_hi - rb_lo + 1) * NW;
    const bool joint = merged && (long long)group * N <= 65536;
    const int n_pairs = joint ? np1 * group : np1;
    const int nh_turns = joint ? 1 : nh;
    int part = 0;  // parts of the item so far, over all its heads
    for (int hh = 0; hh < nh_turns; ++hh) {
    const size_t qo_base = ((size_t)(b * p.Hq + h + hh) * N) * D;
    const size_t head_stream0 = (size_t)(b * p.Hq + h + hh) * n_mblk * NW;  // first stream of the head
    const uint2* const src_streams = reinterpret_cast<const uint2*>(p.streams) + head_stream0 * (size_t)kSparseStreamCap;
    const uint16_t* const src_dir = p.stream_dir + head_stream0 * (size_t)p.dir_stride + k32;

    unsigned char* const wave_lds = lds_all + wave * SG::kWaveLds;
    float* const lval = reinterpret_cast<float*>(wave_lds);                                  // kListCap pairs of weights
    uint16_t* const lkey = reinterpret_cast<uint16_t*>(wave_lds + SG::kListCap * 4);         // their queries
    uint32_t* const row_cnt = reinterpret_cast<uint32_t*>(wave_lds + SG::kListCap * 6);     // 32 counters
    uint32_t* const row_start = row_cnt + 32;                                                // 33 offsets
    // while a part's entries are fetched the lists' room holds a table of its pieces: entries up to and including the
    // piece, and where the piece starts in its stream (which stream, and its first query row, follow from the piece's
    // number)
    constexpr int kTab = 1024;
    uint16_t* const pc_incl = reinterpret_cast<uint16_t*>(wave_lds);
    uint16_t* const pc_lo = pc_incl + kTab;
    static_assert(SG::kListCap * 4 >= 2 * kTab * 2 && SG::kListCap < 65536, "room for the table of pieces, 16-bit counts");

    int cursor = 0;  // next piece (wave-uniform)
    for (;; ++part) {
      // ---- the pieces of this part: as many as the lists and the table hold ----------------------------------------
      int stream_n = 0, n_tab = 0;  // wave-uniform
      const int cursor0 = cursor;   // first piece of the part
      while (cursor < n_pairs && n_tab < kTab) {
        const int pi = cursor + lane;
        uint32_t len = 0u, lo = 0u;
        if (pi < n_pairs) {
          // from the last row block down: a key block holds about as many members in a row block as any other key block
          // of its head does, so the key blocks of a head that run side by side ask for the same rows of q and dO at
          // about the same time, whichever key block they are (a tenth fewer L2 misses than from the first one up)
          int hj = 0, pj = pi;  // head within the item, piece within the head
          for (int g = 1; g < group && pj >= np1; ++g) {
            ++hj;
            pj -= np1;
          }
          const int rb = rb_hi - pj / NW, w = pj % NW;
          const size_t sid = ((size_t)hj * n_mblk + rb) * NW + w;
          uint32_t hi = src_dir[sid * (size_t)p.dir_stride + 1];
          lo = src_dir[sid * (size_t)p.dir_stride];
          hi = hi < (uint32_t)SG::kListCap ? hi : (uint32_t)SG::kListCap;  // (what the dQ kernel wrote lies within these bounds)
          lo = lo < hi ? lo : hi;
          len = hi - lo;
        }
        const int incl = wave_scan_i((int)len);
        // the pieces of this batch that still fit (the sums grow with the lane: a run of lanes from 0 on)
        const unsigned long long fm = __builtin_amdgcn_ballot_w64(pi < n_pairs && n_tab + lane < kTab && stream_n + incl <= SG::kListCap);
        const int m = __builtin_popcountll(fm);
        if (m == 0) break;  // (the part is not empty then: a single piece is no longer than a list)
        const int batch = __builtin_amdgcn_readlane(incl, m - 1);
        if (lane < m) {
          pc_incl[n_tab + lane] = (uint16_t)(stream_n + incl);
          pc_lo[n_tab + lane] = (uint16_t)lo;
        }
        stream_n += batch;
        n_tab += m;
        cursor += m;
        if (m < 64) break;  // the next piece does not fit, or there is none
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
#if ADSP_DKDV_STOP == 1
      if (cursor >= n_pairs) break;
      continue;
#endif

      // ---- the part's entries, all fetches under way together, -> per-key lists in the wave's share of LDS (a counting
      // sort by key).  Entry e of the part lies in the first piece whose running sum exceeds e. ------------------------
      if (lane < 32) row_cnt[lane] = 0u;
      {
        constexpr int kPer = (SG::kListCap + 63) / 64;
        uint2 ent[kPer];
        uint32_t rowv[kPer];
        uint32_t pos[kPer];
#pragma unroll
        for (int j = 0; j < kPer; ++j) {
          const int e = j * 64 + lane;
          ent[j] = uint2{0u, 0u};
          rowv[j] = 0u;
          if (e < stream_n) {
            int a = 0;  // pieces whose running sum is <= e
#pragma unroll
            for (int step = kTab / 2; step >= 1; step >>= 1) {
              const int t = a + step;
              if (t <= n_tab && (int)pc_incl[t - 1] <= e) a = t;
            }
            const int before = a ? (int)pc_incl[a - 1] : 0;
            int hj = 0, pj = cursor0 + a;
            for (int g = 1; g < group && pj >= np1; ++g) {
              ++hj;
              pj -= np1;
            }
            const int rb = rb_hi - pj / NW, w = pj % NW;
            ent[j] = src_streams[(uint32_t)((hj * n_mblk + rb) * NW + w) * (uint32_t)kSparseStreamCap + (uint32_t)pc_lo[a] + (uint32_t)(e - before)];
            rowv[j] = (uint32_t)(hj * N + rb * BM + w * 32);
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();  // (the table is read: its room becomes the lists)
#pragma unroll
        for (int j = 0; j < kPer; ++j) {  // (weights, query | key << 20)
          const uint32_t key = ent[j].y & 0xffffu, row = (ent[j].y >> 20) & 31u;
          ent[j].y = (rowv[j] + row) | ((key - (uint32_t)wave_row0) << 20);
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
          }
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
#if ADSP_DKDV_STOP == 2
      if (cursor >= n_pairs) break;
      continue;
#endif
      // The keys are served four at a time (a group of lanes each) and a round lasts as long as its longest list: keys
      // in the order of their list lengths, longest first, keep the four of a round alike.  row_cnt becomes that order.
      {
        int rank = 0;
        const int mine = lane < 32 ? (int)(row_start[lane + 1] - row_start[lane]) : 0;
        for (int o = 0; o < 32; ++o) {
          const int c = (int)(row_start[o + 1] - row_start[o]);
          rank += (c > mine || (c == mine && o < lane)) ? 1 : 0;
        }
        __builtin_amdgcn_wave_barrier();
        if (lane < 32) row_cnt[rank] = (uint32_t)lane;
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
      }

      // ---- per key: its list holds the queries (of this head) in whose support it lies, each with the pair of weights
      // the dQ kernel left.  A group of D / 8 lanes per key, each lane 8 columns; per member it fetches its 16 bytes of
      // dO_i and q_i and adds p_ij / sum p * dO_i to dV_j and u_ij (dP_ij - delta_i) * q_i to dK_j. ----------------------
      {
        constexpr int kLPR = D / 8;         // lanes per key
        constexpr int kGroups = 64 / kLPR;  // keys in progress per wave
        constexpr int kDepth = 4;
        const int grp = lane / kLPR, col = lane % kLPR;
        const unsigned char* const qrows = reinterpret_cast<const unsigned char*>(p.q) + qo_base * 2;
        const unsigned char* const dorows = reinterpret_cast<const unsigned char*>(p.dout) + qo_base * 2;
        const uint32_t col16 = (uint32_t)col * 16u;  // (32-bit offsets per lane: a head's rows span N * D * 2 <= 16 MB)
        constexpr int kRounds = 32 / kGroups;
        // The rounds (kGroups keys each, in the order of their list lengths) run as one sequence of member sets: the
        // fetches stay kQuads - 1 sets ahead across the rounds' borders, so the loads drain once per part and not once
        // per round.  A round lasts as long as its longest list, the one of its first key; a round without members still
        // takes one (empty) set, behind which its zero sums are stored.
        int nq_mine = 1;  // lane i < kRounds: sets of round i
        if (lane < kRounds) {
          const int r = (int)row_cnt[lane * kGroups];
          const int len = (int)(row_start[r + 1] - row_start[r]);
          nq_mine = len > 0 ? (len + kDepth - 1) / kDepth : 1;
        }
        int total = 0;
#pragma unroll
        for (int i = 0; i < kRounds; ++i) total += __builtin_amdgcn_readlane(nq_mine, i);
        float acc_v[8], acc_k[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          acc_v[i] = 0.f;
          acc_k[i] = 0.f;
        }
        struct Quad {
          u32x4 dd[kDepth], qq[kDepth];
          uint32_t w[kDepth];  // (p / sum p, u (dP - delta)) in the element type, from the dQ kernel
        };
        // the fetching side: round rf, set qf of nqf, the lane's list bounds and a valid query for slots without a member
        int rf = 0, qf = 0, nqf = __builtin_amdgcn_readlane(nq_mine, 0), fetched = 0;
        int e_f = 0, e_hi_f = 0;
        uint32_t safe_q = 0u;
        auto open_round = [&](int rr) {
          const int r = (int)row_cnt[rr * kGroups + grp];
          const int key = wave_row0 + r;
          e_f = (int)row_start[r];
          e_hi_f = (int)row_start[r + 1];
          safe_q = (uint32_t)(key < L ? key : L - 1);
        };
        open_round(0);
        auto fetch_next = [&](Quad& m) {
#pragma unroll
          for (int j = 0; j < kDepth; ++j) {
            const bool has = e_f + j < e_hi_f;
            const uint32_t qidx = has ? (uint32_t)lkey[e_f + j] : safe_q;  // (the list arrays end well inside the wave's LDS)
            m.w[j] = has ? reinterpret_cast<const uint32_t*>(lval)[e_f + j] : 0u;  // (no member: zero weights, no branch)
            const uint32_t roff = qidx * (uint32_t)(D * 2) + col16;
            m.dd[j] = *reinterpret_cast<const u32x4*>(dorows + roff);
            m.qq[j] = *reinterpret_cast<const u32x4*>(qrows + roff);
          }
          e_f += kDepth;
          ++fetched;
          if (++qf == nqf) {
            qf = 0;
            ++rf;
            if (rf < kRounds) {
              nqf = __builtin_amdgcn_readlane(nq_mine, rf);
              open_round(rf);
            }
          }
        };
        // the consuming side: round rc, set qc of nqc
        int rc = 0, qc = 0, nqc = __builtin_amdgcn_readlane(nq_mine, 0), consumed = 0;
        auto store_round = [&](int rr) {
          const int key = wave_row0 + (int)row_cnt[rr * kGroups + grp];
          if (key < N) {
#pragma unroll
            for (int i = 0; i < 8; ++i) acc_k[i] *= p.sm_scale;
            // While parts are still to come the sums stay in fp32, in the wave's rows of the workgroup's scratch slot, and
            // the next part adds to them.  The last part writes an fp32 partial row of this query head (dkdv_reduce_kernel
            // adds up the heads of a K/V head), or dK and dV themselves where the head is the only one.
            float* const sc = p.part_scratch + (((size_t)blockIdx.x * NW + wave) * 32 + (key - wave_row0)) * (2 * D) + col * 8;
            if (part > 0) {
              const f32x4 k0 = *reinterpret_cast<const f32x4*>(sc), k1 = *reinterpret_cast<const f32x4*>(sc + 4);
              const f32x4 v0 = *reinterpret_cast<const f32x4*>(sc + D), v1 = *reinterpret_cast<const f32x4*>(sc + D + 4);
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                acc_k[i] += k0[i];
                acc_k[4 + i] += k1[i];
                acc_v[i] += v0[i];
                acc_v[4 + i] += v1[i];
              }
            }
            if (cursor < n_pairs || hh + 1 < nh_turns) {
              *reinterpret_cast<f32x4*>(sc) = f32x4{acc_k[0], acc_k[1], acc_k[2], acc_k[3]};
              *reinterpret_cast<f32x4*>(sc + 4) = f32x4{acc_k[4], acc_k[5], acc_k[6], acc_k[7]};
              *reinterpret_cast<f32x4*>(sc + D) = f32x4{acc_v[0], acc_v[1], acc_v[2], acc_v[3]};
              *reinterpret_cast<f32x4*>(sc + D + 4) = f32x4{acc_v[4], acc_v[5], acc_v[6], acc_v[7]};
            } else if (direct) {
              const u32x4 wk = {pack2<T>(acc_k[0], acc_k[1]), pack2<T>(acc_k[2], acc_k[3]), pack2<T>(acc_k[4], acc_k[5]), pack2<T>(acc_k[6], acc_k[7])};
              const u32x4 wv = {pack2<T>(acc_v[0], acc_v[1]), pack2<T>(acc_v[2], acc_v[3]), pack2<T>(acc_v[4], acc_v[5]), pack2<T>(acc_v[6], acc_v[7])};
              *reinterpret_cast<u32x4*>(reinterpret_cast<uint16_t*>(p.dk) + kv_base + (size_t)key * D + col * 8) = wk;
              *reinterpret_cast<u32x4*>(reinterpret_cast<uint16_t*>(p.dv) + kv_base + (size_t)key * D + col * 8) = wv;
            } else {
              // (streamed past the caches: the rows of q and dO that the other key blocks of the head gather stay in L2)
              const size_t part_at = ((size_t)(b * p.Hq + h + hh) * p.part_rows + key) * D + col * 8;
              float* const o0 = p.dk_part + part_at;
              float* const o1 = p.dv_part + part_at;
              __builtin_nontemporal_store(f32x4{acc_k[0], acc_k[1], acc_k[2], acc_k[3]}, reinterpret_cast<f32x4*>(o0));
              __builtin_nontemporal_store(f32x4{acc_k[4], acc_k[5], acc_k[6], acc_k[7]}, reinterpret_cast<f32x4*>(o0 + 4));
              __builtin_nontemporal_store(f32x4{acc_v[0], acc_v[1], acc_v[2], acc_v[3]}, reinterpret_cast<f32x4*>(o1));
              __builtin_nontemporal_store(f32x4{acc_v[4], acc_v[5], acc_v[6], acc_v[7]}, reinterpret_cast<f32x4*>(o1 + 4));
            }
          }
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            acc_v[i] = 0.f;
            acc_k[i] = 0.f;
          }
        };
        // dV_j += p_ij / sum p * dO_i and dK_j += u_ij (dP_ij - delta_i) * q_i as two-term dot products with the weight
        // in one half of the pair
        auto consume_next = [&](const Quad& m) {
#pragma unroll
          for (int j = 0; j < kDepth; ++j) {
            dot2_chunk<T>(acc_v, m.dd[j], m.w[j] & 0xffffu, m.w[j] << 16);
            dot2_chunk<T>(acc_k, m.qq[j], m.w[j] >> 16, m.w[j] & 0xffff0000u);
          }
          ++consumed;
          if (++qc == nqc) {
            store_round(rc);
            qc = 0;
            ++rc;
            if (rc < kRounds) nqc = __builtin_amdgcn_readlane(nq_mine, rc);
          }
        };
        {
          Quad ring_q[kQuads];
#pragma unroll
          for (int k = 0; k < kQuads - 1; ++k)
            if (fetched < total) fetch_next(ring_q[k]);
          while (consumed < total) {
#pragma unroll
            for (int k = 0; k < kQuads; ++k) {
              if (consumed < total) {
                if (fetched < total) fetch_next(ring_q[(k + kQuads - 1) % kQuads]);
                consume_next(ring_q[k]);
              }
            }
          }
        }
      }
      if (cursor >= n_pairs && hh + 1 == nh_turns) break;
      // (the sums just written to the scratch slot are read back by the next part, by this wave: its stores have landed
      // before the next part begins; every lane is done with the lists)
      __builtin_amdgcn_s_waitcnt(0x0f70);
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
      if (cursor >= n_pairs) {
        ++part;
        break;
      }
    }
    }  // (heads of the item)
  }
}

// Workgroups to launch: as many as fit the device at once (each owns one stream slot), at most `max_slots`.
template <typename T, int D, int AM, int kKind> static int launch_attn_bwd_sparse_one(const AttnBwdParams& p, int max_slots, hipStream_t s) {
  using SG = SparseGeo<T, D>;
  auto kern = kKind == 2 ? attn_bwd_dkdv_stream_kernel<T, D, AM> : (kKind == 1 ? attn_bwd_dkdv_sparse_kernel<T, D, AM> : attn_bwd_dq_sparse_kernel<T, D, AM>);
  static int per_cu = 0, n_cu = 0;  // (one device family per process: gfx950; one pair per instantiation)
  if (per_cu == 0) {
    int dev = 0, blocks = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 2;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, kern, SG::kThreads, 0) != hipSuccess || blocks <= 0) blocks = 1;
    n_cu = prop.multiProcessorCount;
    per_cu = blocks;
  }
  long long grid = (long long)per_cu * n_cu;
  if (grid > max_slots) grid = max_slots;
  grid = grid / 8 * 8;  // the same number of workgroups on every XCD
  if (grid < 8) grid = 8;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(SG::kThreads), 0, s, p);
  return 0;
}

// keys = 0: the dQ kernel, 1: the dK/dV kernel that walks for itself, 2: the dK/dV kernel that takes the dQ kernel's streams
template <typename T, int D, int AM> static int launch_attn_bwd_sparse_am(const AttnBwdParams& p, int keys, int max_slots, hipStream_t s) {
  if (keys == 2) return launch_attn_bwd_sparse_one<T, D, AM, 2>(p, max_slots, s);
  if (keys == 1) return launch_attn_bwd_sparse_one<T, D, AM, 1>(p, max_slots, s);
  return launch_attn_bwd_sparse_one<T, D, AM, 0>(p, max_slots, s);
}
template <typename T, int D> static int launch_attn_bwd_sparse(const AttnBwdParams& p, int am, int keys, int max_slots, hipStream_t s) {
  if (am == ATT_15) return launch_attn_bwd_sparse_am<T, D, ATT_15>(p, keys, max_slots, s);
  if (am == ATT_2) return launch_attn_bwd_sparse_am<T, D, ATT_2>(p, keys, max_slots, s);
  if (am == ATT_GEN) return launch_attn_bwd_sparse_am<T, D, ATT_GEN>(p, keys, max_slots, s);
  return 2;
}

}  // namespace adsp
