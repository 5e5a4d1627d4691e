/*
 * adasplash_hip.h -- C ABI of the MI355X (gfx950) sparse entmax attention library.
 *
 * Every entry point takes raw device pointers, sizes and scalars, enqueues its kernels on the
 * HIP stream it is given (a hipStream_t passed as void*; NULL = the default stream), never
 * synchronises and never allocates.  The caller owns every buffer, including the workspace; what a call
 * computes depends on its arguments alone.  The return value is an adsp_status; nothing is thrown across
 * the ABI.
 *
 * State the library does hold, none of which carries results from one call to the next:
 *   - per process, the number of workgroups of the persistent kernels that fit the device, looked up on
 *     the first launch of each kernel (one device family per process is assumed: gfx950);
 *   - per device, the address of the 64 MiB scratch array behind adsp_attn_v2_fwd_noalloc, looked up on
 *     that entry point's first call on the device (calls through it share the array: see there);
 *   - the environment, read on every call (comparisons, tests and profiling; unset in normal use):
 *       ADSP_SPARSE=0               every row block on the dense kernels (no sparse-support kernels)
 *       ADSP_BWD_STREAMS=0          the sparse-support dK/dV kernel walks the scores itself instead of taking
 *                                   the dQ kernel's candidate streams
 *       ADSP_PROBE_MAX_SUPPORT=n    the support the probe lets a K/V head's longest rows have before it
 *                                   leaves the head to the dense kernels (default 28; 0: every head)
 *       ADSP_DKDV_MERGE256=n        the share of a causal sequence, in 256ths, from which on the dK/dV kernel serves
 *                                   a key block for all query heads of a K/V head at once (default 80; 0: never).
 *                                   Sizes the backward workspace too: the same value for the size query and the call.
 *
 * The entry points replace the Triton launches inside the reference's autograd wrappers (the
 * reference has no FFI of its own; these are the calls a binding would make in their place):
 *
 *   adsp_entmax_rows_fwd  <- _entmax_triton.forward -> _fwd_entmax
 *                            (adasplash/triton_entmax_v2.py:624-664, kernel :363-536)
 *   adsp_entmax_rows_bwd  <- _entmax_triton.backward -> _bwd_entmax
 *                            (adasplash/triton_entmax_v2.py:667-687, kernel :541-617)
 *   adsp_attn_v2_fwd      <- _sparse_attention.forward -> _get_tau, _get_tau_v2, _get_tau_v3,
 *                            _get_output (adasplash/adasplash_v2.py:1243-1438)
 *   adsp_attn_bwd         <- _sparse_attention.backward -> _bwd_preprocess, _bwd_q_kernel,
 *                            transpose_bmask, _bwd_kv_kernel (adasplash/adasplash_v2.py:1441-1564) and its
 *                            generic-alpha twin (adasplash/adasplash_block_mask.py:1079-1210)
 *   adsp_attn_v1_fwd      <- _sparse_attention.forward -> _get_tau,
 *                            compute_bidxs_and_cubcounts, _get_output
 *                            (adasplash/adasplash_block_mask.py:941-1076)
 */
#ifndef ADASPLASH_HIP_H
#define ADASPLASH_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  ADSP_OK = 0,
  ADSP_ERR_NULL = 1,        /* a required pointer is NULL */
  ADSP_ERR_SHAPE = 2,       /* a dimension is out of the supported range */
  ADSP_ERR_DTYPE = 3,       /* unknown element type */
  ADSP_ERR_ALIGN = 4,       /* a tensor base pointer is not 16-byte aligned */
  ADSP_ERR_UNSUPPORTED = 5, /* parameter combination the kernels do not implement */
  ADSP_ERR_WORKSPACE = 6,   /* workspace missing or smaller than adsp_attn_workspace_bytes() */
  ADSP_ERR_LAUNCH = 7,      /* the HIP runtime refused a launch (hipGetLastError() != success) */
  ADSP_ERR_TOO_LARGE = 8    /* adsp_attn_v2_fwd_noalloc: the problem needs more scratch than the library holds */
} adsp_status;

/* Element types of q/k/v/out and x/y. */
typedef enum { ADSP_F32 = 0, ADSP_BF16 = 1, ADSP_F16 = 2 } adsp_dtype;

/* Library ABI version (bumped when a signature changes). */
int adsp_version(void);

/*
 * Identity of the sources this library was built from: the first 16 hex digits of a SHA-256 over the
 * kernel sources, headers and compiler flags, baked in at build time ("unknown" for a build that did not
 * pass it).  No counterpart in the reference (pure Python, nothing to go stale); the Python loader compares
 * it with the tree it sits in so that a library older than its sources cannot be tested or benchmarked.
 */
const char* adsp_build_id(void);
/* The extra compiler flags of a profiling build (empty for a regular one); they enter adsp_build_id(). */
const char* adsp_build_flags(void);

/* Static, NUL-terminated description of a status code. */
const char* adsp_status_string(int status);

/*
 * Row-wise alpha-entmax over the last dimension: y[r, :] = [(alpha-1) x[r, :] - tau_r]_+^(1/(alpha-1)).
 *   x, y      : contiguous [rows, cols] arrays of `dtype`; y is fully overwritten (zeros included).
 *   alpha     : > 1.  n_iter : refinement steps after initialisation (>= 0).
 *   use_histogram : non-zero = histogram initialisation of tau (honoured for alpha in {1.5, 2}).
 *   fast_math : accepted for signature parity; the generic-alpha power always uses exp2/log2.
 * Replaces the launch at adasplash/triton_entmax_v2.py:650-658.
 */
int adsp_entmax_rows_fwd(const void* x, void* y, int64_t rows, int64_t cols, int dtype, double alpha,
                         int n_iter, int use_histogram, int fast_math, void* stream);

/*
 * Backward of the above: dx = u*dy - (sum(u*dy)/sum(u)) * u with u = y^(2-alpha) on the support.
 * Replaces the launch at adasplash/triton_entmax_v2.py:678-685.
 */
int adsp_entmax_rows_bwd(const void* y, const void* dy, void* dx, int64_t rows, int64_t cols, int dtype,
                         double alpha, void* stream);

/*
 * Bytes of scratch the forward entry points need for these dimensions; 0 for fp32 and for the head dims the
 * sparse-support kernel does not serve (then `workspace` may be NULL).  For the 16-bit types at head dims 64 and 128:
 * the work counters, row-block flags and candidate streams of the sparse-support kernel (up to 1024 slots of 51 KiB;
 * sequences of up to 65536 keys) and a one-byte (fp8 e4m3) copy of K.  The buffer must be 16-byte aligned device
 * memory; its contents need not survive between calls, and two calls that run at the same time need a buffer each.
 * For the block-mask variant pass Hq = Hkv = H.
 */
size_t adsp_attn_workspace_bytes(int B, int Hq, int Hkv, int N, int D, int dtype);

/* Number of int32 words per (batch, head) the block mask needs: n_row_blocks * words_per_row. */
size_t adsp_attn_bmask_words(int N);

/*
 * AdaSplash-2 forward: causal entmax-1.5 attention with GQA and right-padded variable lengths.
 *   q, out : [B, Hq, N, D]; k, v : [B, Hkv, N, D], contiguous, Hq % Hkv == 0, D in {16,32,64,128,256}.
 *   taus   : [B, Hq, N] fp32, receives the per-row threshold (rows past the valid length untouched).
 *   bmask  : [B, Hq, adsp_attn_bmask_words(N)] int32, receives the per-(128-row, 64-key) tile mask,
 *            bit (c % 32) of word c / 32 of a row block = key tile c holds a non-zero probability.
 *   varlen : NULL, or [B] valid lengths as int32 (varlen_bits = 32) or int64 (varlen_bits = 64);
 *            keys >= length are masked, output rows >= length are written as zeros.
 *   niter  : Halley/bisection refinement passes after the histogram bracket (>= 0).  fp32 takes niter + 1 of them,
 *            as the reference does (adasplash/adasplash_v2.py:567-611 and :617-681); the 16-bit types take niter on
 *            the dense kernel, and the sparse-support kernel (head dims 64 / 128) iterates to convergence.
 * Replaces the four launches at adasplash/adasplash_v2.py:1288-1419.
 */
int adsp_attn_v2_fwd(const void* q, const void* k, const void* v, void* out, float* taus, int32_t* bmask,
                     const void* varlen, int varlen_bits, int B, int Hq, int Hkv, int N, int D, int dtype,
                     int niter, void* workspace, size_t workspace_bytes, void* stream);

/*
 * adsp_attn_v2_fwd without a workspace argument, for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The
 * scratch memory (control words, flags, candidate streams and fp8 copy of K of the sparse-support kernel)
 * lives in a device array inside the library, 64 MiB on every GPU the library runs on, held until the process ends;
 * problems whose adsp_attn_workspace_bytes() exceeds adsp_attn_v2_fwd_noalloc_max_bytes() are rejected with
 * ADSP_ERR_TOO_LARGE.  The call allocates and frees nothing and records no memset (the kernels clear what must start
 * at zero).  All calls on one GPU share that array: calls that overlap on one GPU (two streams, two threads) race
 * and must be serialised by the caller.  Other arguments, results and status codes as adsp_attn_v2_fwd.
 */
size_t adsp_attn_v2_fwd_noalloc_max_bytes(void);
int adsp_attn_v2_fwd_noalloc(const void* q, const void* k, const void* v, void* out, float* taus, int32_t* bmask,
                             const void* varlen, int varlen_bits, int B, int Hq, int Hkv, int N, int D, int dtype,
                             int niter, void* stream);

/*
 * AdaSplash-1 (block-mask) forward: alpha-entmax attention for any alpha in (1, 2], causal or not,
 * right-padded variable lengths, no GQA (q, k, v share [B, H, N, D]).
 *   tile_counts : NULL, or 2 device uint64 that are incremented by {16x16 score tiles inside the
 *                 causal/valid domain, those that hold a non-zero probability} (for sparsity reports).
 * Other arguments as in adsp_attn_v2_fwd.  Replaces the launches at
 * adasplash/adasplash_block_mask.py:978-1003 and :1024-1054 plus the torch-side list building
 * (:298-320).
 */
int adsp_attn_v1_fwd(const void* q, const void* k, const void* v, void* out, float* taus, int32_t* bmask,
                     const void* varlen, int varlen_bits, int B, int H, int N, int D, int dtype, double alpha,
                     int is_causal, int niter, void* workspace, size_t workspace_bytes,
                     unsigned long long* tile_counts, void* stream);

/*
 * Supports kept for the backward.  No counterpart in the reference (its backward recomputes the scores of every tile of
 * the mask).  The sparse-support forward kernel finds, for every row, the few keys with a non-zero probability; the
 * _keep variants of the two forward entry points leave what they found in `supports` -- per 128-row block of a query
 * head its streams of (score, key) pairs, their lengths, every row's threshold relative to the streams' scores and a
 * flag -- and adsp_attn_bwd_kept, given the same buffer untouched, takes the supports from there instead of walking
 * the scores again.  adsp_attn_supports_bytes() is the size of that buffer (51 KiB per 128 query rows and head plus
 * 4 bytes per row; 0 where nothing is kept: fp32, head dims other than 64 and 128, N > 65536; `supports` may then be
 * NULL).  16-byte aligned device memory owned by the caller; it must hold what the forward wrote for the same
 * q, k, v, varlen until the backward has run.  Row blocks the forward served with its dense kernel keep no supports
 * and the backward walks them as adsp_attn_bwd does; with supports == NULL the three calls are adsp_attn_v2_fwd,
 * adsp_attn_v1_fwd (without tile statistics) and adsp_attn_bwd.
 */
size_t adsp_attn_supports_bytes(int B, int Hq, int Hkv, int N, int D, int dtype);
int adsp_attn_v2_fwd_keep(const void* q, const void* k, const void* v, void* out, float* taus, int32_t* bmask,
                          const void* varlen, int varlen_bits, int B, int Hq, int Hkv, int N, int D, int dtype,
                          int niter, void* workspace, size_t workspace_bytes, void* supports, size_t supports_bytes,
                          void* stream);
int adsp_attn_v1_fwd_keep(const void* q, const void* k, const void* v, void* out, float* taus, int32_t* bmask,
                          const void* varlen, int varlen_bits, int B, int H, int N, int D, int dtype, double alpha,
                          int is_causal, int niter, void* workspace, size_t workspace_bytes, void* supports,
                          size_t supports_bytes, void* stream);
int adsp_attn_bwd_kept(const void* q, const void* k, const void* v, const void* dout, const float* taus,
                       const int32_t* bmask, const void* varlen, int varlen_bits, void* dq, void* dk, void* dv,
                       float* delta, float* zinv, int B, int Hq, int Hkv, int N, int D, int dtype, double alpha,
                       int is_causal, void* workspace, size_t workspace_bytes, const void* supports,
                       size_t supports_bytes, void* stream);

/*
 * Workspace of adsp_attn_bwd in bytes; 0 for fp32 and for the head dims the sparse-support kernels do not serve (then
 * `workspace` may be NULL).  For the 16-bit element types at head dims 64 and 128 (sequences of up to 65536 keys): the
 * counters, flags and candidate streams of the sparse-support backward kernels, 1024 * D bytes of fp32 sums per
 * workgroup (items that are worked off in parts), fp32 partial rows of dk and dv per query head (2 * B * Hq * N * D * 4 bytes;
 * none where Hq == Hkv), and the supports the dq kernel hands to the dk/dv kernel: per query row block of 128 rows
 * 51 KiB of (weights, key) pairs and a table of 4 * ceil(N / 128) + 2 16-bit offsets per wave.
 * 16-byte aligned device memory; contents need not survive between calls; concurrent calls need a buffer each.
 * This is the size that serves any call with these dimensions.
 */
size_t adsp_attn_bwd_workspace_bytes(int B, int Hq, int Hkv, int N, int D, int dtype);

/*
 * The same for a call whose is_causal is known: with a causal mask the dk/dv kernel serves the later key blocks of a
 * sequence (from 5/16 of its length on) for all query heads of a K/V head at once and needs partial rows for the first
 * ones only (about 5/16 of the bytes above), so the workspace is smaller.  adsp_attn_bwd and adsp_attn_bwd_kept accept a
 * workspace of either size.  (No counterpart in the reference, which allocates inside its backward.)
 */
size_t adsp_attn_bwd_workspace_bytes_causal(int B, int Hq, int Hkv, int N, int D, int dtype, int is_causal);

/*
 * Backward of both attention variants: dq, dk, dv for the upstream gradient dout.
 *   q, dout, dq : [B, Hq, N, D]; k, v, dk, dv : [B, Hkv, N, D] (Hq == Hkv for the block-mask variant).
 *   taus, bmask : what the forward wrote for the same inputs (bmask may be NULL: every tile is visited).
 *   delta, zinv : [B, Hq, N] fp32 scratch owned by the caller; receive sum_j u_ij dP_ij / sum_j u_ij and
 *                 1 / sum_j p_ij per query row.
 *   alpha, is_causal : 1.5 / 1 for the AdaSplash-2 path, any alpha in (1, 2] for the block-mask path.
 * Rows of q, k, v and dout past a sequence's valid length are never used, whatever they hold; gradient rows
 * past the valid length are written as zeros.  Replaces the four launches at
 * adasplash/adasplash_v2.py:1456-1562 (delta from out2, dq, mask transpose, dk/dv with the GQA group loop)
 * and adasplash/adasplash_block_mask.py:1079-1210.
 */
int adsp_attn_bwd(const void* q, const void* k, const void* v, const void* dout, const float* taus,
                  const int32_t* bmask, const void* varlen, int varlen_bits, void* dq, void* dk, void* dv,
                  float* delta, float* zinv, int B, int Hq, int Hkv, int N, int D, int dtype, double alpha,
                  int is_causal, void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* ADASPLASH_HIP_H */
