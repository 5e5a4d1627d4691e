// Launch parameters and tile constants shared by the attention kernel and its C-ABI front end.
#pragma once
#include <stdint.h>

namespace adsp {

constexpr int kMaskRows = 128;   // query rows per row block of the bmask output
constexpr int kBN = 64;          // keys per tile
constexpr int kAttnBins = 8;     // histogram bins of the attention solver
constexpr int kMaskWords = 512;  // tile-mask capacity per row block: 512 * 32 tiles * 64 keys = 1M keys

enum AttnAlphaMode { ATT_15 = 0, ATT_2 = 1, ATT_GEN = 2 };
// control words of the sparse-support forward behind the eight work counters (AttnParams::queue)
constexpr int kCtrlFlagged = 8;     // row blocks left to the dense kernel
constexpr int kCtrlAllDense = 9;    // set by the sparse kernel when every K/V head was predicted dense: it served nothing
constexpr int kCtrlGaveUp = 10;     // of the row blocks left to the dense kernel, those the sparse kernel had started on

struct AttnParams {
  const void* q;
  const void* k;
  const void* v;   // row-major V: the fp32 path walks it; every path gathers rows of it for the list-based output
  void* out;
  float* taus;
  int32_t* bmask;
  const void* varlen;
  int varlen_bits;
  unsigned long long* tile_counts;
  int B, Hq, Hkv, N, Npad;
  int n_mblk;      // 128-row blocks per (b, h) in bmask
  int mask_words;  // int32 words per row block in bmask
  int fine_masks;  // set by the launch: the kernel keeps per-wave 32-key block bits beside the tile masks
  int niter;
  int causal;
  int use_hist;
  float qscale;  // (alpha - 1) / sqrt(D)
  float alpha;
  float c0;  // 1 / (alpha - 1)
  // Sparse-support path (16-bit types): attn_fwd_sparse_kernel runs first and writes one flag per 128-row block,
  // 1 = left to attn_fwd_kernel, which skips the others when block_flags is set.
  int32_t* block_flags;   // [B, Hq, n_mblk], or null: attn_fwd_kernel serves every row block
  uint32_t* queue;        // eight work counters, one per XCD, then the two control words above; zero at launch
  uint32_t* hints;        // [B * Hkv + 1][2]: word 0 of a K/V head is 1 << 20 when the probe leaves all of it to the dense kernel, else 0
  unsigned char* events;  // candidate streams, one slot per workgroup of the sparse kernel
  const unsigned char* k8;  // fp8 (e4m3) copy of K, [B * Hkv][Npad][D] bytes, rows past N zero: the operand of the first walk
  // Four floats per K/V head, set by the probe: powers of two for q and for k (they are multiplied by them before
  // they are rounded for the first walk, so that its scores stay inside the range its position tags need), the largest
  // number of keys a row may see for the head's score spread to predict a support that fits the lists (infinity when the
  // probe did not look: short sequences), and a spare word
  float* w1_scales;
  float probe_max_support;  // the support the probe lets a row have before it leaves the row to the dense kernel
  // Supports kept for the backward (null: none kept).  The sparse-support kernel then writes its candidate streams to a
  // place of their own per (row block, wave) and leaves them there, with their lengths, every row's threshold minus
  // lower bound (raw score units: an entry is a member of the support when its value exceeds it), and a flag per row
  // block, 1 = streams valid (the probe clears the flags; row blocks the dense kernel serves keep 0).
  int32_t* save_flags;          // [B, Hq, n_mblk]
  uint16_t* save_lens;          // [B, Hq, n_mblk, waves]
  float* save_tshift;           // [B, Hq, N]
  unsigned char* save_streams;  // [B, Hq, n_mblk, waves, stream capacity] (score - bound, key | row << 20) pairs
};

}  // namespace adsp
