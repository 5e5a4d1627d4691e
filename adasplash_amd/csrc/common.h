// Shared device helpers for the gfx950 kernels: element types, wave64 reductions, conversions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace adsp {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));  // a 16-byte global/LDS access

struct bf16_t { uint16_t bits; };  // storage-only tags; arithmetic is always fp32
struct f16_t { uint16_t bits; };

template <typename T> struct elem_traits;
template <> struct elem_traits<float> { static constexpr int kBytes = 4; static constexpr int kVec = 4; static constexpr bool kIsBf16 = false; };
template <> struct elem_traits<bf16_t> { static constexpr int kBytes = 2; static constexpr int kVec = 8; static constexpr bool kIsBf16 = true; };
template <> struct elem_traits<f16_t> { static constexpr int kBytes = 2; static constexpr int kVec = 8; static constexpr bool kIsBf16 = false; };

__device__ __forceinline__ float bf16_bits_to_float(uint32_t b) { return __builtin_bit_cast(float, b << 16); }
__device__ __forceinline__ uint32_t float_to_bf16_bits(float f) {
  return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)f);  // v_cvt_pk_bf16_f32, round to nearest even
}
__device__ __forceinline__ float f16_bits_to_float(uint32_t b) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)b);
}
__device__ __forceinline__ uint32_t float_to_f16_bits(float f) {
  return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);
}

// Two fp32 -> one dword of packed 16-bit elements (low half = a).
template <typename T> __device__ __forceinline__ uint32_t pack2(float a, float b);
template <> __device__ __forceinline__ uint32_t pack2<bf16_t>(float a, float b) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  f32x2 f = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}
template <> __device__ __forceinline__ uint32_t pack2<f16_t>(float a, float b) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
  f32x2 f = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2));
}
// two floats -> two e4m3 bytes in the low (hi = false) or high half of `old`; saturating at the format's largest value
__device__ __forceinline__ uint32_t cvt_e4m3_pair(float a, float b, uint32_t old, bool hi) {
  a = __builtin_amdgcn_fmed3f(a, -448.f, 448.f);
  b = __builtin_amdgcn_fmed3f(b, -448.f, 448.f);
  return hi ? (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, true) : (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, false);
}

template <typename T> __device__ __forceinline__ float unpack_lo(uint32_t w);
template <typename T> __device__ __forceinline__ float unpack_hi(uint32_t w);
template <> __device__ __forceinline__ float unpack_lo<bf16_t>(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
template <> __device__ __forceinline__ float unpack_hi<bf16_t>(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }
template <> __device__ __forceinline__ float unpack_lo<f16_t>(uint32_t w) { return f16_bits_to_float(w & 0xffffu); }
template <> __device__ __forceinline__ float unpack_hi<f16_t>(uint32_t w) { return f16_bits_to_float(w >> 16); }

// ---- wave64 butterflies ---------------------------------------------------------------------------
// Wave-wide reductions on the DPP network (row shifts, then the two row broadcasts of this ISA family); the
// result is read from lane 63 into a scalar register, so every lane gets it.  All 64 lanes must be active.
// Six VALU instructions, against six LDS-crossbar round trips for the same reduction written with shuffles.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_move(float old, float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, v), CTRL,
                                                               ROW_MASK, 0xf, false));
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_move<0x111, 0xf>(-INFINITY, v));  // row_shr:1
  v = fmaxf(v, dpp_move<0x112, 0xf>(-INFINITY, v));  // row_shr:2
  v = fmaxf(v, dpp_move<0x114, 0xf>(-INFINITY, v));  // row_shr:4
  v = fmaxf(v, dpp_move<0x118, 0xf>(-INFINITY, v));  // row_shr:8: lane 15 of a row holds the row's result
  v = fmaxf(v, dpp_move<0x142, 0xa>(-INFINITY, v));  // row_bcast:15 into rows 1 and 3
  v = fmaxf(v, dpp_move<0x143, 0xc>(-INFINITY, v));  // row_bcast:31 into rows 2 and 3
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_move<0x111, 0xf>(0.f, v);
  v += dpp_move<0x112, 0xf>(0.f, v);
  v += dpp_move<0x114, 0xf>(0.f, v);
  v += dpp_move<0x118, 0xf>(0.f, v);
  v += dpp_move<0x142, 0xa>(0.f, v);
  v += dpp_move<0x143, 0xc>(0.f, v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
// The same within every aligned group of 16 lanes (a DPP row): xor-butterflies over the quad, then the two
// mirrors; every lane of the group ends with the group's result.  Lanes of a group must be active together.
__device__ __forceinline__ float group16_max(float v) {
  v = fmaxf(v, dpp_move<0xb1, 0xf>(v, v));   // quad_perm [1, 0, 3, 2]
  v = fmaxf(v, dpp_move<0x4e, 0xf>(v, v));   // quad_perm [2, 3, 0, 1]
  v = fmaxf(v, dpp_move<0x141, 0xf>(v, v));  // row_half_mirror
  v = fmaxf(v, dpp_move<0x140, 0xf>(v, v));  // row_mirror
  return v;
}
__device__ __forceinline__ float group16_sum(float v) {
  v += dpp_move<0xb1, 0xf>(v, v);
  v += dpp_move<0x4e, 0xf>(v, v);
  v += dpp_move<0x141, 0xf>(v, v);
  v += dpp_move<0x140, 0xf>(v, v);
  return v;
}
__device__ __forceinline__ int wave_sum_i(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// ---- block numbering of the dense attention kernels -------------------------------------------------------
// Hardware block ids are dealt round-robin to the 8 XCDs (one L2 each): XCD x runs the blocks x, x + 8, ... in
// that order, a new one whenever a slot of its 32 CUs falls free.  The K/V heads (`units`) are dealt round-robin
// to the XCDs -- with right-padded batches a contiguous run of heads is one batch item, and the XCD that drew
// the longest sequence would finish last -- and an XCD works through its heads in sets.  A set is one head when
// the blocks cost the same (`balance` false) or a head alone has several blocks per slot; its K and V then stay
// in that L2.  When the blocks of a head differ in cost (causal: block index 0 is the longest) and a head has
// few of them, a set takes as many heads as give about two blocks per slot and runs them longest block first
// over all its heads: started in that order, the short blocks fill the slots the long ones leave, where head
// after head the last head's longest block would start when the others are almost through.
// `blocks` = blocks per (head, member of its group), `group` = query heads per K/V head, `unit_bytes` = what the
// blocks of one K/V head stream through L2 (they share it while they run side by side): a set never takes more heads
// than bring 8 MB of that, twice an XCD's L2 -- with more, the blocks of a head that are in flight together become
// too few to share their tiles, and on long sequences that costs more than the balance gains (dK/dV kernel on
// B=8, Hkv=8, group 4, N=8192, D=128: 10.1 ms with sets of four heads, 7.5 ms head after head).  Returns false for
// the padding blocks of the grid, else the K/V head, the block index and the member.
__device__ __forceinline__ bool xcd_block_map(int units, int blocks, int group, bool balance, long long unit_bytes, int& unit, int& blk,
                                              int& member) {
  const int inner = blocks * group;
  const int x = (int)(blockIdx.x & 7);
  const long long seq = (long long)(blockIdx.x >> 3);
  if (units % 8 != 0) {
    const long long total = (long long)units * inner;
    const long long per_xcd = (total + 7) / 8;
    const long long logical = x * per_xcd + seq;
    if (seq >= per_xcd || logical >= total) return false;
    unit = (int)(logical / inner);
    blk = (int)(logical % inner) / group;
    member = (int)(logical % inner) % group;
    return true;
  }
  const int upx = units / 8;  // heads of this XCD
  if (seq >= (long long)upx * inner) return false;
  constexpr int kSetBlocks = 256;  // two blocks for each of 32 CUs x 4 resident blocks
  constexpr long long kSetBytes = 8ll << 20;
  int g = balance ? (kSetBlocks + inner - 1) / inner : 1;
  const long long by_bytes = unit_bytes > 0 ? kSetBytes / unit_bytes : (long long)upx;
  g = g < by_bytes ? g : (int)by_bytes;
  g = g < 1 ? 1 : g;
  g = g < upx ? g : upx;
  const int set = (int)(seq / ((long long)g * inner));
  const int s = (int)(seq - (long long)set * g * inner);
  const int gsize = (upx - set * g) < g ? (upx - set * g) : g;
  const int span = gsize * group;
  blk = s / span;
  const int r = s % span;
  unit = (set * g + r / group) * 8 + x;
  member = r % group;
  return true;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

}  // namespace adsp
