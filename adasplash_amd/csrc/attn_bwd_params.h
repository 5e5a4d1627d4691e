// Launch parameters of the attention backward kernels.
#pragma once
#include <stdint.h>

namespace adsp {

struct AttnBwdParams {
  const void *q, *k, *v, *dout;
  void *dq, *dk, *dv;
  const float* taus;  // [B, Hq, N] thresholds of the forward, in z units
  float* delta;       // [B, Hq, N] written by the dQ kernel, read by the dK/dV kernel
  float* zinv;        // [B, Hq, N] 1 / sum_j p_ij, likewise
  const int32_t* bmask;  // [B, Hq, n_mblk, mask_words] tile mask of the forward, or null
  const void* varlen;
  int varlen_bits;
  int B, Hq, Hkv, N, Npad;
  int n_mblk, mask_words;
  int causal;
  float qscale;    // (alpha - 1) / sqrt(D)
  float sm_scale;  // 1 / sqrt(D)
  float c0;        // 1 / (alpha - 1)
  // the sparse-support dQ kernel and its hand-over to the dense one (null: dense kernels only), as in AttnParams
  int32_t* block_flags;   // [B, Hq, n_mblk] 1 = row block left to attn_bwd_dq_kernel
  uint32_t* queue;        // control words: work counters, flagged count, "every head dense"
  uint32_t* hints;        // two words per K/V head: word 0 is 1 << 20 where the probe left the head to the dense kernels
  unsigned char* events;  // candidate streams, one slot per workgroup of the sparse kernel
  // the sparse-support dK/dV kernel: a control block of its own, one flag per (K/V head, key block), fp32 partial rows
  // [B, Hq, part_rows, D] when a K/V head serves several query heads (null otherwise), and per workgroup and wave 32 fp32
  // rows of dK | dV for the sums of an item that is worked off in parts; the streams are shared
  uint32_t* queue2;
  uint32_t* hints2;
  int32_t* kv_flags;  // [B, Hkv, n_mblk] 1 = key block left to attn_bwd_dkdv_kernel
  float* dk_part;
  float* dv_part;
  int part_rows;  // rows per query head in dk_part / dv_part: N, or as many as the key blocks that are not merged can need
  float* part_scratch;  // [slots, waves, 32, 2 D]
  int merge256;         // key blocks from this share (in 256ths) of a causal sequence on are served all heads in one item; 0: none
  // hand-over of the supports from the dQ kernel to the dK/dV kernel (null: the dK/dV kernel walks for itself): the dQ
  // kernel's streams kept per (row block, wave) instead of per workgroup, and per stream the offsets of the 32-key blocks
  unsigned char* streams;  // [B, Hq, n_mblk, waves, stream capacity] per member (weights, key | row << 20): the pair p / sum p, u (dP - delta) in the element type
  uint16_t* stream_dir;    // [B, Hq, n_mblk, waves, dir_stride]: entry k = first stream entry with key >= 32 k
  int dir_stride;          // 4 n_mblk + 1 offsets, rounded up to an even count
  // supports the forward kept (null: none; see AttnParams): where the flag of a row block is 1 the dQ kernel takes
  // the forward's candidate stream and keeps the entries above the row's threshold instead of walking the scores
  const int32_t* fwd_flags;
  const uint16_t* fwd_lens;
  const float* fwd_tshift;
  const unsigned char* fwd_streams;
};

// Whether the kernel on the streams serves the key block starting at key m0 of a sequence of L keys with one item for all
// query heads of its K/V head (then it writes dK and dV itself and the reduction over the heads leaves the block alone).
__host__ __device__ inline bool dkdv_block_merged(int causal, int group, int m0, int L, int merge256) {
  return merge256 > 0 && causal && group > 1 && m0 < L && (long long)m0 * 256 >= (long long)L * merge256;
}

}  // namespace adsp
