// C ABI of the attention forward and backward: argument checks, re-layout launches, kernel dispatch.
#include "common.h"
#include "attn_params.h"
#include "attn_bwd_params.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>
#include "../../include/adasplash_hip.h"

namespace adsp {
// The kernels live in one translation unit per (element type, head dim, instance): attn_fwd_unit.hip and
// attn_bwd_unit.hip, compiled once per combination.
#define ADSP_DECL_D(tag, d)                                                      \
  int launch_attn_fwd_##tag##_d##d##_m0(const AttnParams&, int, hipStream_t);   \
  int launch_attn_fwd_##tag##_d##d##_m1(const AttnParams&, int, hipStream_t);   \
  int launch_attn_bwd_##tag##_d##d(const AttnBwdParams&, int, int, hipStream_t);
#define ADSP_DECL_TAG(tag) ADSP_DECL_D(tag, 16) ADSP_DECL_D(tag, 32) ADSP_DECL_D(tag, 64) ADSP_DECL_D(tag, 128) ADSP_DECL_D(tag, 256)
ADSP_DECL_TAG(f32)
ADSP_DECL_TAG(bf16)
ADSP_DECL_TAG(f16)
// attn_fwd_sparse_kernel (attn_sparse_unit.hip): 16-bit types, head dims 64 and 128
int launch_attn_sparse_bf16_d64(const AttnParams&, int, int, hipStream_t);
int launch_attn_sparse_bf16_d128(const AttnParams&, int, int, hipStream_t);
int launch_attn_sparse_f16_d64(const AttnParams&, int, int, hipStream_t);
int launch_attn_sparse_f16_d128(const AttnParams&, int, int, hipStream_t);
// attn_bwd_dq_sparse_kernel (attn_bwd_sparse_unit.hip): likewise
int launch_attn_bwd_sparse_bf16_d64(const AttnBwdParams&, int, int, int, hipStream_t);
int launch_attn_bwd_sparse_bf16_d128(const AttnBwdParams&, int, int, int, hipStream_t);
int launch_attn_bwd_sparse_f16_d64(const AttnBwdParams&, int, int, int, hipStream_t);
int launch_attn_bwd_sparse_f16_d128(const AttnBwdParams&, int, int, int, hipStream_t);

typedef int (*attn_fwd_fn)(const AttnParams&, int, hipStream_t);
typedef int (*attn_bwd_fn)(const AttnBwdParams&, int, int, hipStream_t);
#define ADSP_FWD_ROW(tag, d) {launch_attn_fwd_##tag##_d##d##_m0, launch_attn_fwd_##tag##_d##d##_m1}
#define ADSP_FWD_TAG(tag) {ADSP_FWD_ROW(tag, 16), ADSP_FWD_ROW(tag, 32), ADSP_FWD_ROW(tag, 64), ADSP_FWD_ROW(tag, 128), ADSP_FWD_ROW(tag, 256)}
#define ADSP_BWD_TAG(tag) {launch_attn_bwd_##tag##_d16, launch_attn_bwd_##tag##_d32, launch_attn_bwd_##tag##_d64, launch_attn_bwd_##tag##_d128, launch_attn_bwd_##tag##_d256}
// indexed by adsp_dtype (ADSP_F32 = 0, ADSP_BF16 = 1, ADSP_F16 = 2), head dim slot, instance
static const attn_fwd_fn kFwdTable[3][5][2] = {ADSP_FWD_TAG(f32), ADSP_FWD_TAG(bf16), ADSP_FWD_TAG(f16)};
static const attn_bwd_fn kBwdTable[3][5] = {ADSP_BWD_TAG(f32), ADSP_BWD_TAG(bf16), ADSP_BWD_TAG(f16)};
static int head_dim_slot(int D) { return D == 16 ? 0 : (D == 32 ? 1 : (D == 64 ? 2 : (D == 128 ? 3 : (D == 256 ? 4 : -1)))); }

// e4m3 copy of K for the first walk of the sparse-support forward: [B * Hkv][Npad][D] bytes in the order of K, values
// beyond the format's range saturated, rows from N on zero.  A thread converts 16 values.  Heads the probe has marked
// as dense are skipped (`hints`: two words per head).  The values are multiplied by the head's power of two first
// (`w1_scales`, from the probe).
// (the first walk's operands lie on a grid of 1/16, see attn_sparse_kernel.h)
#define G16(x) (((x) * ak + 786432.f) - 786432.f)
template <typename T>
__global__ __launch_bounds__(256) void k8_layout_kernel(const uint16_t* __restrict__ k, unsigned char* __restrict__ k8, int N,
                                                       int Npad, int D, const uint32_t* hints, const float* w1_scales) {
  const size_t head = blockIdx.y;
  if (hints[2 * head] >= (1u << 20)) return;
  const float ak = w1_scales[4 * head + 1];
  const int per_row = D / 16;
  const long long id = (long long)blockIdx.x * 256 + threadIdx.x;
  if (id >= (long long)Npad * per_row) return;
  const int row = (int)(id / per_row), c = (int)(id % per_row);
  u32x4 out = {0u, 0u, 0u, 0u};
  if (row < N) {
    const uint16_t* src = k + (head * (size_t)N + row) * D + c * 16;
    const u32x4 lo = *reinterpret_cast<const u32x4*>(src), hi = *reinterpret_cast<const u32x4*>(src + 8);
#pragma unroll
    for (int e = 0; e < 4; e += 2) {
      out[e >> 1] = cvt_e4m3_pair(G16(unpack_lo<T>(lo[e + 1])), G16(unpack_hi<T>(lo[e + 1])), cvt_e4m3_pair(G16(unpack_lo<T>(lo[e])), G16(unpack_hi<T>(lo[e])), 0u, false), true);
      out[2 + (e >> 1)] = cvt_e4m3_pair(G16(unpack_lo<T>(hi[e + 1])), G16(unpack_hi<T>(hi[e + 1])), cvt_e4m3_pair(G16(unpack_lo<T>(hi[e])), G16(unpack_hi<T>(hi[e])), 0u, false), true);
    }
  }
  *reinterpret_cast<u32x4*>(k8 + (head * (size_t)Npad + row) * D + c * 16) = out;
}

static int npad_of(int N) { return (N + kBN - 1) / kBN * kBN; }
static int mblocks_of(int N) { return (N + kMaskRows - 1) / kMaskRows; }
static int mask_words_of(int N) { return ((N + kBN - 1) / kBN + 31) / 32; }

// Control words of the sparse-support forward (the `queue` pointer of AttnParams): eight work counters, the number
// of row blocks it left to the dense kernel, a word saying that the probe below leaves every K/V head to the dense
// kernel; from word 64 on two words per K/V head and two more (the first of a head's pair is 1 << 20 when the probe
// leaves the whole head to the dense kernel; the backward's kernels keep row-block counters in the others), then four
// floats per K/V head (AttnParams::w1_scales).
//
// attn_probe_kernel clears them and looks at a sample of each K/V head's scores (one workgroup per head: four long
// query rows of the group's first head against 256 evenly spaced keys): from the sample's variance the support a
// Gaussian score distribution would have for a row that sees n keys follows in closed form (n s^2 g(a) = 1 with
// g(a) = (1 + a^2) Q(a) - a phi(a) for alpha = 1.5, n s h(a) = 1 with h(a) = phi(a) - a Q(a) for alpha = 2; support
// n Q(a)).  It grows with n: the probe stores the largest n whose predicted support the candidate lists hold, and the
// sparse-support kernels leave the row blocks that see more keys to the dense kernels without spending a walk on
// them.  The prediction only decides which kernel does the work (a row block it gets wrong is caught by the kernel's
// own checks), and it depends on the inputs alone: the same call takes the same way every time.
template <typename T>
__global__ __launch_bounds__(256) void attn_probe_kernel(AttnParams p, int D, int am) {
  __shared__ float qrows[4][256];
  __shared__ float red[4][2][4];
  __shared__ float ksum[4];
  const int u = blockIdx.x, tid = threadIdx.x;
  const int units = p.B * p.Hkv;
  uint32_t* const ctrl = p.queue;
  if (u == 0 && tid < 11) ctrl[tid] = 0u;
  if (u == 0 && tid < 2) ctrl[64 + 2 * units + tid] = 0u;
  if (tid < 2) ctrl[64 + 2 * u + tid] = 0u;
  const int b = u / p.Hkv, kvh = u % p.Hkv, group = p.Hq / p.Hkv;
  if (p.save_flags)  // supports kept for the backward: no row block of this K/V head has a valid stream yet
    for (int i = tid; i < group * p.n_mblk; i += 256) p.save_flags[(size_t)(b * p.Hq + kvh * group) * p.n_mblk + i] = 0;
  int L = p.N;
  if (p.varlen) {
    long long l = p.varlen_bits == 64 ? ((const long long*)p.varlen)[b] : (long long)((const int*)p.varlen)[b];
    L = (int)(l < 0 ? 0 : (l > p.N ? p.N : l));
  }
  if (p.w1_scales && tid < 4) p.w1_scales[4 * u + tid] = tid < 2 ? 1.f : (tid == 2 ? INFINITY : 0.f);
  if (L < 256) return;  // short sequences: finding out in the kernel costs little
  int rows[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) rows[j] = L - 1 - j * (L / 16);
  const uint16_t* qbase = reinterpret_cast<const uint16_t*>(p.q) + ((size_t)(b * p.Hq + kvh * group) * p.N) * D;
  for (int i = tid; i < 4 * D; i += 256) {
    const uint32_t w = qbase[(size_t)rows[i / D] * D + i % D];
    qrows[i / D][i % D] = elem_traits<T>::kIsBf16 ? bf16_bits_to_float(w) : f16_bits_to_float(w);
  }
  __syncthreads();
  const int span = (p.causal ? rows[3] + 1 : L);
  const int key = (int)(((long long)tid * span) / 256);
  const uint16_t* krow = reinterpret_cast<const uint16_t*>(p.k) + ((size_t)(b * p.Hkv + kvh) * p.N + key) * D;
  float dot[4] = {0.f, 0.f, 0.f, 0.f};
  float ksq = 0.f;
  for (int d = 0; d < D; d += 8) {
    const u32x4 w = *reinterpret_cast<const u32x4*>(krow + d);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float lo = unpack_lo<T>(w[e]), hi = unpack_hi<T>(w[e]);
      ksq = fmaf(lo, lo, fmaf(hi, hi, ksq));
#pragma unroll
      for (int j = 0; j < 4; ++j) dot[j] = fmaf(lo, qrows[j][d + 2 * e], fmaf(hi, qrows[j][d + 2 * e + 1], dot[j]));
    }
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float z = dot[j] * p.qscale;
    const float s1 = wave_sum(z), s2 = wave_sum(z * z);
    if ((tid & 63) == 0) {
      red[tid >> 6][0][j] = s1;
      red[tid >> 6][1][j] = s2;
    }
  }
  {
    const float ks = wave_sum(ksq);
    if ((tid & 63) == 0) ksum[tid >> 6] = ks;
  }
  __syncthreads();
  if (tid == 0 && p.w1_scales) {
    // Scales of the first walk's operands: the sampled raw scores' root mean square goes to about 8 (the walk's
    // tags hold scores up to 512), shared between q and k so that k's own root mean square comes near 8 / sqrt(D).
    float raw2 = 0.f;
    for (int j = 0; j < 4; ++j) raw2 += red[0][1][j] + red[1][1][j] + red[2][1][j] + red[3][1][j];
    const float s_rms = sqrtf(raw2 / 1024.f) / p.qscale;
    const float k_rms = sqrtf((ksum[0] + ksum[1] + ksum[2] + ksum[3]) / (256.f * (float)D));
    if (s_rms > 0.f && k_rms > 0.f && s_rms < INFINITY && k_rms < INFINITY) {
      const float a = exp2f(rintf(log2f(8.f / s_rms)));
      float ak = exp2f(rintf(log2f(8.f / (sqrtf((float)D) * k_rms))));
      ak = fminf(fmaxf(ak, 0x1p-40f), 0x1p40f);
      float aq = fminf(fmaxf(a / ak, 0x1p-40f), 0x1p40f);
      p.w1_scales[4 * u] = aq;
      p.w1_scales[4 * u + 1] = ak;
    }
  }
  if (tid >= 64) return;
  // The first wave: the score spread pooled over the four sampled rows, and for 64 row lengths n (a geometric grid from
  // 64 to a million keys, one per lane) the support a Gaussian score distribution of that spread would have.  The
  // prediction grows with n; the largest n whose support still fits is what the sparse-support kernels compare a row
  // block's keys with.
  float var = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float s1 = red[0][0][j] + red[1][0][j] + red[2][0][j] + red[3][0][j];
    const float s2 = red[0][1][j] + red[1][1][j] + red[2][1][j] + red[3][1][j];
    const float mean = s1 / 256.f;
    var += 0.25f * fmaxf(s2 / 256.f - mean * mean, 0.f);
  }
  const float sd = sqrtf(var);
  const float n = 64.f * exp2f((float)tid * (14.f / 63.f));
  float lo = -2.f, hi = 7.f;
  for (int it = 0; it < 14; ++it) {
    const float a = 0.5f * (lo + hi);
    const float Q = 0.5f * erfcf(a * 0.70710678f), phi = 0.39894228f * __expf(-0.5f * a * a);
    float f;
    if (am == ATT_2) f = n * sd * (phi - a * Q);
    else if (am == ATT_15) f = n * var * ((1.f + a * a) * Q - a * phi);
    else {  // any alpha: n E[(sd (Z - a))_+^c0] by the midpoint rule over [a, a + 8]
      float acc = 0.f;
      for (int i = 0; i < 32; ++i) {
        const float x = 0.25f * ((float)i + 0.5f);
        acc += __expf(p.c0 * __logf(sd * x)) * 0.39894228f * __expf(-0.5f * (a + x) * (a + x));
      }
      f = n * acc * 0.25f;
    }
    if (f > 1.f) lo = a;
    else hi = a;
  }
  const float support = n * 0.5f * erfcf(0.5f * (lo + hi) * 0.70710678f);
  const unsigned long long fits = __builtin_amdgcn_ballot_w64(support <= p.probe_max_support);
  // (a spread of zero or a NaN predicts nothing: every length fits, and the kernels find out for themselves)
  const int top = fits == 0ull ? -1 : 63 - __builtin_clzll(fits);
  const float n_fit = top < 0 ? 0.f : (top == 63 ? INFINITY : 64.f * exp2f((float)top * (14.f / 63.f)));
  if (tid != 0) return;
  // A head goes one way as a whole: by its longest rows, which see all L keys and hold most of the work.  (Serving only
  // its shorter row blocks from their supports was measured and loses: for a row block of few tiles the fixed cost of the
  // lists outweighs the walks saved, and a launch split between the two kernels took 15 % longer than the dense kernel
  // alone.)  A marked head: the copy of K skips it and the sparse-support kernels leave its row blocks to the dense ones.
  const bool fits_all = n_fit >= (float)L;
  if (p.w1_scales) p.w1_scales[4 * u + 2] = fits_all ? INFINITY : 0.f;
  if (!fits_all) ctrl[64 + 2 * u] = 1u << 20;
}

// Workspace of the forward for the 16-bit types, for the head dims the sparse-support kernel serves: its work
// counters, its per-row-block flags, its candidate streams and the e4m3 copy of K that its first walk reads.  (The
// dense kernel needs none: it reads V row-major and transposes in the LDS read.)
constexpr int kSparseMaxSlots = 1024;                       // workgroups of the persistent kernel
constexpr size_t kSparseSlotBytes = (size_t)4 * 1616 * 8;   // four waves x 1616 candidates x (score, key)
struct FwdWorkspace {
  size_t vt_bytes, queue_off, scales_off, flags_off, events_off, k8_off, total;
  int slots;  // 0: no sparse-support kernel for these dimensions
};
static size_t align256(size_t x) { return (x + 255) / 256 * 256; }
static FwdWorkspace fwd_workspace(int B, int Hq, int Hkv, int N, int D, int dtype) {
  FwdWorkspace w = {};
  if (dtype == ADSP_F32) return w;
  w.vt_bytes = 0;
  w.total = 0;
  if ((D == 64 || D == 128) && N <= 65536) {  // (the candidate lists hold 16-bit key indices)
    const long long items = (long long)B * Hq * mblocks_of(N);
    long long slots = (items + 7) / 8 * 8;
    if (slots > kSparseMaxSlots) slots = kSparseMaxSlots;
    w.slots = (int)slots;
    w.queue_off = align256(w.vt_bytes);
    // eight counters, then two hint words per K/V head and two more, then four floats per K/V head
    w.scales_off = w.queue_off + 256 + ((size_t)B * Hkv + 1) * 8;
    w.flags_off = align256(w.scales_off + (size_t)B * Hkv * 16);
    w.events_off = align256(w.flags_off + (size_t)items * 4);
    w.k8_off = align256(w.events_off + (size_t)slots * kSparseSlotBytes);
    w.total = w.k8_off + (size_t)B * Hkv * npad_of(N) * D;  // the e4m3 copy of K
  }
  return w;
}

// Supports the forward keeps for the backward (adsp_attn_supports_bytes): a flag per row block, the length of every
// (row block, wave) stream, every row's threshold minus lower bound, and the streams.
struct SupportsLayout {
  size_t flags_off, lens_off, tshift_off, streams_off, total;  // total = 0: nothing to keep for these dimensions
};
static SupportsLayout supports_layout(int B, int Hq, int Hkv, int N, int D, int dtype) {
  SupportsLayout l = {};
  if (dtype == ADSP_F32 || fwd_workspace(B, Hq, Hkv, N, D, dtype).slots == 0) return l;
  const size_t items = (size_t)B * Hq * mblocks_of(N);
  l.flags_off = 0;
  l.lens_off = align256(items * 4);
  l.tshift_off = align256(l.lens_off + items * 4 * 2);
  l.streams_off = align256(l.tshift_off + (size_t)B * Hq * N * 4);
  l.total = l.streams_off + items * kSparseSlotBytes;
  return l;
}
__global__ __launch_bounds__(256) void fill_zero_kernel(int32_t* x, long long n) {
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256) x[i] = 0;
}

// ADSP_SPARSE=0 in the environment keeps every row block on the dense kernel (for comparisons and tests).
static bool sparse_enabled() {
  const char* e = getenv("ADSP_SPARSE");
  return !(e && strcmp(e, "0") == 0);
}
// The probe leaves a K/V head to the dense kernel when the support its Gaussian model predicts exceeds this many keys.
// ADSP_PROBE_MAX_SUPPORT in the environment overrides it (0: every head is left to the dense kernel, which then runs
// behind the sparse-support kernel as it does for the row blocks that kernel gives up; for comparisons).
static float probe_max_support() {
  const char* e = getenv("ADSP_PROBE_MAX_SUPPORT");
  return e ? (float)atof(e) : 28.f;
}

// ADSP_BWD_STREAMS=0 in the environment makes the sparse-support dK/dV kernel walk for itself instead of taking the
// dQ kernel's streams (for comparisons and tests).
static bool bwd_streams_enabled() {
  const char* e = getenv("ADSP_BWD_STREAMS");
  return !(e && strcmp(e, "0") == 0);
}

// With a causal mask the kernel on the dQ kernel's streams serves the key blocks from this share (in 256ths) of a
// sequence on with one item for all query heads of a K/V head (attn_bwd_dkdv_stream_kernel).  ADSP_DKDV_MERGE256 in the
// environment overrides it (0: every key block per query head, with partial rows; for comparisons and tests).
static int dkdv_merge256() {
  const char* e = getenv("ADSP_DKDV_MERGE256");
  int v = e ? atoi(e) : 80;
  return v < 0 ? 0 : (v > 256 ? 256 : v);
}

static int attn_common(const void* q, const void* k, const void* v, void* out, float* taus, int32_t* bmask,
                       const void* varlen, int varlen_bits, int B, int Hq, int Hkv, int N, int D, int dtype,
                       double alpha, int is_causal, int niter, int use_hist, void* workspace, size_t workspace_bytes,
                       unsigned long long* tile_counts, hipStream_t s, void* supports = nullptr, size_t supports_bytes = 0) {
  if (!q || !k || !v || !out) return ADSP_ERR_NULL;
  if (dtype != ADSP_F32 && dtype != ADSP_BF16 && dtype != ADSP_F16) return ADSP_ERR_DTYPE;
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || N <= 0 || Hq % Hkv != 0) return ADSP_ERR_SHAPE;
  if (D != 16 && D != 32 && D != 64 && D != 128 && D != 256) return ADSP_ERR_SHAPE;
  if (mask_words_of(N) > kMaskWords) return ADSP_ERR_SHAPE;
  if (!(alpha > 1.0) || niter < 0) return ADSP_ERR_UNSUPPORTED;
  if (varlen && varlen_bits != 32 && varlen_bits != 64) return ADSP_ERR_UNSUPPORTED;
  if ((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15) != 0) return ADSP_ERR_ALIGN;

  AttnParams p;
  p.q = q;
  p.k = k;
  p.v = v;
  p.out = out;
  p.taus = taus;
  p.bmask = bmask;
  p.varlen = varlen;
  p.varlen_bits = varlen_bits;
  p.tile_counts = tile_counts;
  p.B = B;
  p.Hq = Hq;
  p.Hkv = Hkv;
  p.N = N;
  p.Npad = npad_of(N);
  p.n_mblk = mblocks_of(N);
  p.mask_words = mask_words_of(N);
  // The dense kernel takes the reference's extra update when it serves the call alone: the reference's solver makes
  // `niter` refinements and one more behind the mask pass (adasplash/adasplash_v2.py:567-611 and :617-681), which is
  // what brings the default niter = 1 to 1e-4 in fp32 and keeps the thresholds the backward reads within 1e-5 for the
  // 16-bit types.  The second and later steps run on the candidate lists of the list-carrying instance when they fit,
  // without another K walk.  Behind the sparse-support kernel (which converges fully) the dense kernel serves the
  // row blocks whose supports did not fit that kernel's lists, longer than its own: there it walks `niter` steps.
  const int am = alpha == 1.5 ? ATT_15 : (alpha == 2.0 ? ATT_2 : ATT_GEN);
  const FwdWorkspace w = dtype == ADSP_F32 ? FwdWorkspace{} : fwd_workspace(B, Hq, Hkv, N, D, dtype);
  // Sparse-support kernel first (16-bit types, alpha 1.5 / 2 or any other in [1.125, 2): below that its solver on the
  // lists would need too many rounds; either entry point, no tile statistics asked for): it serves the row blocks
  // whose supports are short and flags the others for the dense kernel.
  const bool sparse = w.slots > 0 && (am == ATT_15 || am == ATT_2 || (alpha >= 1.125 && alpha < 2.0)) &&
                      !tile_counts && (long long)B * Hq * mblocks_of(N) < (1ll << 31) && sparse_enabled();
  if (!sparse) niter += 1;
  p.niter = niter;
  p.causal = is_causal ? 1 : 0;
  p.use_hist = use_hist;
  p.alpha = (float)alpha;
  p.c0 = (float)(1.0 / (alpha - 1.0));
  p.qscale = (float)((alpha - 1.0) / sqrt((double)D));

  p.block_flags = nullptr;
  p.queue = nullptr;
  p.hints = nullptr;
  p.events = nullptr;
  p.k8 = nullptr;
  p.w1_scales = nullptr;
  p.probe_max_support = 0.f;
  p.save_flags = nullptr;
  p.save_lens = nullptr;
  p.save_tshift = nullptr;
  p.save_streams = nullptr;

  (void)hipGetLastError();
  if (dtype != ADSP_F32) {
    const SupportsLayout sl = supports ? supports_layout(B, Hq, Hkv, N, D, dtype) : SupportsLayout{};
    if (sl.total && (supports_bytes < sl.total || ((uintptr_t)supports & 15) != 0)) return ADSP_ERR_WORKSPACE;
    if (w.total && (!workspace || workspace_bytes < w.total || ((uintptr_t)workspace & 15) != 0)) return ADSP_ERR_WORKSPACE;
    unsigned char* ws = (unsigned char*)workspace;
    if (sparse) {
      p.queue = (uint32_t*)(ws + w.queue_off);
      p.hints = p.queue + 64;
      p.block_flags = (int32_t*)(ws + w.flags_off);
      p.events = ws + w.events_off;
      p.k8 = ws + w.k8_off;
      p.w1_scales = (float*)(ws + w.scales_off);
      p.probe_max_support = probe_max_support();
      if (sl.total) {
        unsigned char* sp = (unsigned char*)supports;
        p.save_flags = (int32_t*)(sp + sl.flags_off);
        p.save_lens = (uint16_t*)(sp + sl.lens_off);
        p.save_tshift = (float*)(sp + sl.tshift_off);
        p.save_streams = sp + sl.streams_off;
      }
      const dim3 k8_grid((unsigned)(((long long)p.Npad * (D / 16) + 255) / 256), (unsigned)(B * Hkv));
      if (dtype == ADSP_BF16) {
        hipLaunchKernelGGL(attn_probe_kernel<bf16_t>, dim3((unsigned)(B * Hkv)), dim3(256), 0, s, p, D, am);
        hipLaunchKernelGGL(k8_layout_kernel<bf16_t>, k8_grid, dim3(256), 0, s, (const uint16_t*)k, ws + w.k8_off, N, p.Npad, D, (const uint32_t*)p.hints, (const float*)p.w1_scales);
      } else {
        hipLaunchKernelGGL(attn_probe_kernel<f16_t>, dim3((unsigned)(B * Hkv)), dim3(256), 0, s, p, D, am);
        hipLaunchKernelGGL(k8_layout_kernel<f16_t>, k8_grid, dim3(256), 0, s, (const uint16_t*)k, ws + w.k8_off, N, p.Npad, D, (const uint32_t*)p.hints, (const float*)p.w1_scales);
      }
      int rc = dtype == ADSP_BF16 ? (D == 64 ? launch_attn_sparse_bf16_d64(p, am, w.slots, s) : launch_attn_sparse_bf16_d128(p, am, w.slots, s))
                                  : (D == 64 ? launch_attn_sparse_f16_d64(p, am, w.slots, s) : launch_attn_sparse_f16_d128(p, am, w.slots, s));
      if (rc != 0) return ADSP_ERR_LAUNCH;
    } else if (sl.total) {  // nothing is kept by this call: the backward must not take what the buffer happens to hold
      const long long items = (long long)B * Hq * mblocks_of(N);
      hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((items + 255) / 256 > 1024 ? 1024 : (items + 255) / 256)), dim3(256), 0, s,
                         (int32_t*)((unsigned char*)supports + sl.flags_off), items);
    }
  }
  // The list-carrying instance serves two and more solver steps, and a single step without the histogram (the
  // block-mask variant's, made for sparse supports); the other one no step, or one behind the histogram -- and
  // whatever the sparse-support kernel leaves over: those row blocks did not fit its lists, which are longer than
  // this kernel's, so they are walked step by step, and the walk-only instance does that with fewer registers.
  const bool multi = (niter >= 2 || (niter == 1 && !use_hist)) && p.queue == nullptr;
  int rc = kFwdTable[dtype][head_dim_slot(D)][multi ? 1 : 0](p, am, s);
  if (rc != 0) return ADSP_ERR_LAUNCH;
  return hipGetLastError() == hipSuccess ? ADSP_OK : ADSP_ERR_LAUNCH;
}
}  // namespace adsp

extern "C" size_t adsp_attn_workspace_bytes(int B, int Hq, int Hkv, int N, int D, int dtype) {
  if (dtype == ADSP_F32 || B <= 0 || Hq <= 0 || Hkv <= 0 || N <= 0 || D <= 0) return 0;
  return adsp::fwd_workspace(B, Hq, Hkv, N, D, dtype).total;
}

extern "C" size_t adsp_attn_supports_bytes(int B, int Hq, int Hkv, int N, int D, int dtype) {
  if (dtype == ADSP_F32 || B <= 0 || Hq <= 0 || Hkv <= 0 || N <= 0 || D <= 0) return 0;
  return adsp::supports_layout(B, Hq, Hkv, N, D, dtype).total;
}

extern "C" size_t adsp_attn_bmask_words(int N) {
  if (N <= 0) return 0;
  return (size_t)adsp::mblocks_of(N) * adsp::mask_words_of(N);
}

extern "C" int adsp_attn_v2_fwd(const void* q, const void* k, const void* v, void* out, float* taus, int32_t* bmask,
                                const void* varlen, int varlen_bits, int B, int Hq, int Hkv, int N, int D, int dtype,
                                int niter, void* workspace, size_t workspace_bytes, void* stream) {
  return adsp::attn_common(q, k, v, out, taus, bmask, varlen, varlen_bits, B, Hq, Hkv, N, D, dtype, 1.5, 1, niter, 1,
                           workspace, workspace_bytes, nullptr, (hipStream_t)stream);
}

// ---- the entry point that allocates nothing -------------------------------------------------------------------
namespace adsp {
// Same work as adsp_attn_v2_fwd with the workspace taken from a file-scope device array instead of the caller.
// `noalloc_scratch` is a host-side stand-in for the symbol here: the address the kernels can use is looked up once
// per device with hipGetSymbolAddress (every GPU holds its own copy of the array) and only that pointer is passed on.
constexpr size_t kNoAllocScratchBytes = (size_t)64 << 20;
static __device__ __align__(256) unsigned char noalloc_scratch[kNoAllocScratchBytes];
constexpr int kMaxDevices = 64;
static void* g_noalloc_ptr[kMaxDevices] = {};

static int noalloc_scratch_ptr(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return ADSP_ERR_LAUNCH;
  void* ptr = __atomic_load_n(&g_noalloc_ptr[dev], __ATOMIC_ACQUIRE);
  if (!ptr) {
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(noalloc_scratch)) != hipSuccess || !ptr) return ADSP_ERR_LAUNCH;
    __atomic_store_n(&g_noalloc_ptr[dev], ptr, __ATOMIC_RELEASE);  // (two threads racing here store the same address)
  }
  *out = ptr;
  return ADSP_OK;
}
}  // namespace adsp

extern "C" size_t adsp_attn_v2_fwd_noalloc_max_bytes(void) { return adsp::kNoAllocScratchBytes; }

extern "C" int adsp_attn_v2_fwd_noalloc(const void* q, const void* k, const void* v, void* out, float* taus,
                                        int32_t* bmask, const void* varlen, int varlen_bits, int B, int Hq, int Hkv,
                                        int N, int D, int dtype, int niter, void* stream) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || N <= 0) return ADSP_ERR_SHAPE;
  if (D != 16 && D != 32 && D != 64 && D != 128 && D != 256) return ADSP_ERR_SHAPE;
  if (dtype != ADSP_F32 && dtype != ADSP_BF16 && dtype != ADSP_F16) return ADSP_ERR_DTYPE;
  const size_t need = adsp_attn_workspace_bytes(B, Hq, Hkv, N, D, dtype);
  if (need > adsp::kNoAllocScratchBytes) return ADSP_ERR_TOO_LARGE;
  void* ws = nullptr;
  if (need > 0) {
    const int rc = adsp::noalloc_scratch_ptr(&ws);
    if (rc != ADSP_OK) return rc;
  }
  return adsp::attn_common(q, k, v, out, taus, bmask, varlen, varlen_bits, B, Hq, Hkv, N, D, dtype, 1.5, 1, niter, 1, ws,
                           need, nullptr, (hipStream_t)stream);
}

extern "C" int adsp_attn_v1_fwd(const void* q, const void* k, const void* v, void* out, float* taus, int32_t* bmask,
                                const void* varlen, int varlen_bits, int B, int H, int N, int D, int dtype, double alpha,
                                int is_causal, int niter, void* workspace, size_t workspace_bytes,
                                unsigned long long* tile_counts, void* stream) {
  if (alpha > 2.0) return ADSP_ERR_UNSUPPORTED;
  return adsp::attn_common(q, k, v, out, taus, bmask, varlen, varlen_bits, B, H, H, N, D, dtype, alpha, is_causal, niter,
                           0, workspace, workspace_bytes, tile_counts, (hipStream_t)stream);
}

extern "C" int adsp_attn_v2_fwd_keep(const void* q, const void* k, const void* v, void* out, float* taus, int32_t* bmask,
                                     const void* varlen, int varlen_bits, int B, int Hq, int Hkv, int N, int D, int dtype,
                                     int niter, void* workspace, size_t workspace_bytes, void* supports,
                                     size_t supports_bytes, void* stream) {
  return adsp::attn_common(q, k, v, out, taus, bmask, varlen, varlen_bits, B, Hq, Hkv, N, D, dtype, 1.5, 1, niter, 1,
                           workspace, workspace_bytes, nullptr, (hipStream_t)stream, supports, supports_bytes);
}

extern "C" int adsp_attn_v1_fwd_keep(const void* q, const void* k, const void* v, void* out, float* taus, int32_t* bmask,
                                     const void* varlen, int varlen_bits, int B, int H, int N, int D, int dtype,
                                     double alpha, int is_causal, int niter, void* workspace, size_t workspace_bytes,
                                     void* supports, size_t supports_bytes, void* stream) {
  if (alpha > 2.0) return ADSP_ERR_UNSUPPORTED;
  return adsp::attn_common(q, k, v, out, taus, bmask, varlen, varlen_bits, B, H, H, N, D, dtype, alpha, is_causal, niter,
                           0, workspace, workspace_bytes, nullptr, (hipStream_t)stream, supports, supports_bytes);
}

namespace adsp {
// Workspace of the backward for the 16-bit types, for the head dims the sparse-support kernels serve: their work
// counters, per-row-block flags and candidate streams (the forward's layout without the copy of K).  (The dense
// kernels need none: they read k, q and dout row-major and transpose in the LDS read.)
struct BwdWorkspace {
  size_t copies_bytes, queue_off, flags_off, events_off, queue2_off, kvflags_off, scratch_off, part_off, part_bytes, streams_off, dir_off, total;
  int slots;       // 0: no sparse-support kernels for these dimensions
  int dir_stride;  // offsets per stream of the hand-over table
  int part_rows;   // rows per query head of the partial rows
  int merge256;    // what the dK/dV kernel on the streams is launched with
};
static BwdWorkspace bwd_workspace(int B, int Hq, int Hkv, int N, int D, int dtype, int causal) {
  BwdWorkspace w = {};
  if (dtype == ADSP_F32) return w;
  w.copies_bytes = 0;
  w.total = 0;
  if ((D == 64 || D == 128) && N <= 65536) {
    const long long items = (long long)B * Hq * mblocks_of(N);
    long long slots = (items + 7) / 8 * 8;
    if (slots > kSparseMaxSlots) slots = kSparseMaxSlots;
    w.slots = (int)slots;
    w.queue_off = align256(w.copies_bytes);
    w.flags_off = align256(w.queue_off + 256 + ((size_t)B * Hkv + 1) * 8);
    w.events_off = align256(w.flags_off + (size_t)items * 4);
    // the dK/dV kernel: control words and the probe's verdict per K/V head once more, a flag per (K/V head, key
    // block), fp32 sums per workgroup and fp32 partial rows of dK and dV per query head
    w.queue2_off = align256(w.events_off + (size_t)slots * kSparseSlotBytes);
    w.kvflags_off = align256(w.queue2_off + 256 + ((size_t)B * Hkv + 1) * 8);
    // (fp32 sums of an item worked off in parts: 32 rows of dK | dV per wave of every workgroup)
    w.scratch_off = align256(w.kvflags_off + (size_t)B * Hkv * mblocks_of(N) * 4);
    w.part_off = align256(w.scratch_off + (size_t)slots * 4 * 32 * 2 * D * 4);
    // (with one query head per K/V head the kernel on the streams writes dK and dV itself: no partial rows; with a
    // causal mask it does so for the key blocks it merges, and the others start in front of N * merge256 / 256)
    w.merge256 = (bwd_streams_enabled() && causal && Hq != Hkv) ? dkdv_merge256() : 0;
    w.part_rows = N;
    if (w.merge256 > 0) {
      const long long bound = ((long long)N * w.merge256 + 255) / 256;
      const long long rows = (bound + kMaskRows - 1) / kMaskRows * kMaskRows;
      if (rows < N) w.part_rows = (int)rows;
    }
    w.part_bytes = (Hq == Hkv && bwd_streams_enabled()) ? 0 : (size_t)B * Hq * w.part_rows * D * 4;
    // the dQ kernel's streams, kept per (row block, wave) for the dK/dV kernel, and where their 32-key blocks start
    w.streams_off = align256(w.part_off + 2 * w.part_bytes);
    w.dir_stride = (mblocks_of(N) * 4 + 2) / 2 * 2;
    w.dir_off = align256(w.streams_off + (size_t)items * kSparseSlotBytes);  // (a slot = the streams of four waves)
    w.total = w.dir_off + align256((size_t)items * 4 * w.dir_stride * 2);
  }
  return w;
}

// Clears the control words and key-block flags of the sparse-support dK/dV kernel and copies the probe's verdict per
// K/V head (the dQ kernel's words) into the kernel's own.
__global__ __launch_bounds__(256) void bwd_ctrl_clear_kernel(uint32_t* ctrl2, const uint32_t* hints1, int units, int32_t* kv_flags,
                                                            long long n_flags) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i < 10) ctrl2[i] = 0u;
  if (i < units) {
    ctrl2[64 + 2 * i] = hints1[2 * i] >= (1u << 20) ? (1u << 20) : 0u;
    ctrl2[64 + 2 * i + 1] = 0u;
  }
  if (i < 2) ctrl2[64 + 2 * units + i] = 0u;
  for (long long j = i; j < n_flags; j += (long long)gridDim.x * 256) kv_flags[j] = 0;
}

// dK, dV = sum over the query heads of a K/V head of the sparse-support kernel's fp32 partial rows; key blocks left to
// attn_bwd_dkdv_kernel are skipped (that kernel writes them), and so are those the kernel on the streams served for all
// heads at once.  A thread adds up 8 columns of
// one key row.  Rows past the valid length are zeros and their partial rows are not read (the key blocks that lie
// wholly in the padding have none).
typedef float reduce_f32x4 __attribute__((ext_vector_type(4)));
template <typename T>
__global__ __launch_bounds__(256) void dkdv_reduce_kernel(const float* __restrict__ dk_part, const float* __restrict__ dv_part,
                                                         void* dk, void* dv, const int32_t* kv_flags, const uint32_t* ctrl2,
                                                         const void* varlen, int varlen_bits, int B, int Hq, int Hkv, int N, int D,
                                                         int causal, int merge256, int part_rows) {
  if (ctrl2[kCtrlAllDense] != 0u) return;
  const int per_row = D / 8;
  const long long id = (long long)blockIdx.x * 256 + threadIdx.x;
  if (id >= (long long)B * Hkv * N * per_row) return;
  const int c = (int)(id % per_row);
  const long long rg = id / per_row;
  const int row = (int)(rg % N), bkv = (int)(rg / N);
  if (kv_flags[(size_t)bkv * ((N + kMaskRows - 1) / kMaskRows) + row / kMaskRows] != 0) return;
  const int group = Hq / Hkv, b = bkv / Hkv, kvh = bkv % Hkv;
  long long L = N;
  if (varlen) {
    L = varlen_bits == 64 ? ((const long long*)varlen)[b] : (long long)((const int*)varlen)[b];
    L = L < 0 ? 0 : (L > N ? N : L);
  }
  if (dkdv_block_merged(causal, group, row / kMaskRows * kMaskRows, (int)L, merge256)) return;  // (written by the kernel on the streams)
  float sk[8], sv[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) sk[i] = sv[i] = 0.f;
  for (int g = 0; g < (row < L ? group : 0); ++g) {
    const size_t at = (((size_t)(b * Hq + kvh * group + g) * part_rows) + row) * D + c * 8;
    const reduce_f32x4 k0 = __builtin_nontemporal_load(reinterpret_cast<const reduce_f32x4*>(dk_part + at));
    const reduce_f32x4 k1 = __builtin_nontemporal_load(reinterpret_cast<const reduce_f32x4*>(dk_part + at + 4));
    const reduce_f32x4 v0 = __builtin_nontemporal_load(reinterpret_cast<const reduce_f32x4*>(dv_part + at));
    const reduce_f32x4 v1 = __builtin_nontemporal_load(reinterpret_cast<const reduce_f32x4*>(dv_part + at + 4));
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      sk[i] += k0[i];
      sk[4 + i] += k1[i];
      sv[i] += v0[i];
      sv[4 + i] += v1[i];
    }
  }
  const size_t out = (((size_t)bkv * N) + row) * D + c * 8;
  const u32x4 wk = {pack2<T>(sk[0], sk[1]), pack2<T>(sk[2], sk[3]), pack2<T>(sk[4], sk[5]), pack2<T>(sk[6], sk[7])};
  const u32x4 wv = {pack2<T>(sv[0], sv[1]), pack2<T>(sv[2], sv[3]), pack2<T>(sv[4], sv[5]), pack2<T>(sv[6], sv[7])};
  *reinterpret_cast<u32x4*>(reinterpret_cast<uint16_t*>(dk) + out) = wk;
  *reinterpret_cast<u32x4*>(reinterpret_cast<uint16_t*>(dv) + out) = wv;
}
}  // namespace adsp

extern "C" size_t adsp_attn_bwd_workspace_bytes(int B, int Hq, int Hkv, int N, int D, int dtype) {
  if (dtype == ADSP_F32 || B <= 0 || Hq <= 0 || Hkv <= 0 || N <= 0 || D <= 0) return 0;
  return adsp::bwd_workspace(B, Hq, Hkv, N, D, dtype, 0).total;
}

extern "C" size_t adsp_attn_bwd_workspace_bytes_causal(int B, int Hq, int Hkv, int N, int D, int dtype, int is_causal) {
  if (dtype == ADSP_F32 || B <= 0 || Hq <= 0 || Hkv <= 0 || N <= 0 || D <= 0) return 0;
  return adsp::bwd_workspace(B, Hq, Hkv, N, D, dtype, is_causal ? 1 : 0).total;
}

static int attn_bwd_impl(const void* q, const void* k, const void* v, const void* dout, const float* taus,
                         const int32_t* bmask, const void* varlen, int varlen_bits, void* dq, void* dk, void* dv,
                         float* delta, float* zinv, int B, int Hq, int Hkv, int N, int D, int dtype, double alpha,
                         int is_causal, void* workspace, size_t workspace_bytes, const void* supports, size_t supports_bytes,
                         void* stream) {
  using namespace adsp;
  hipStream_t s = (hipStream_t)stream;
  if (!q || !k || !v || !dout || !taus || !dq || !dk || !dv || !delta || !zinv) return ADSP_ERR_NULL;
  if (dtype != ADSP_F32 && dtype != ADSP_BF16 && dtype != ADSP_F16) return ADSP_ERR_DTYPE;
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || N <= 0 || Hq % Hkv != 0) return ADSP_ERR_SHAPE;
  if (D != 16 && D != 32 && D != 64 && D != 128 && D != 256) return ADSP_ERR_SHAPE;
  if (mask_words_of(N) > kMaskWords) return ADSP_ERR_SHAPE;
  if (!(alpha > 1.0) || alpha > 2.0) return ADSP_ERR_UNSUPPORTED;
  if (varlen && varlen_bits != 32 && varlen_bits != 64) return ADSP_ERR_UNSUPPORTED;
  if ((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)dout | (uintptr_t)dq | (uintptr_t)dk | (uintptr_t)dv) & 15) != 0)
    return ADSP_ERR_ALIGN;

  AttnBwdParams p;
  p.q = q;
  p.k = k;
  p.v = v;
  p.dout = dout;
  p.dq = dq;
  p.dk = dk;
  p.dv = dv;
  p.taus = taus;
  p.delta = delta;
  p.zinv = zinv;
  p.bmask = bmask;
  p.varlen = varlen;
  p.varlen_bits = varlen_bits;
  p.B = B;
  p.Hq = Hq;
  p.Hkv = Hkv;
  p.N = N;
  p.Npad = npad_of(N);
  p.n_mblk = mblocks_of(N);
  p.mask_words = mask_words_of(N);
  p.causal = is_causal ? 1 : 0;
  p.qscale = (float)((alpha - 1.0) / sqrt((double)D));
  p.sm_scale = (float)(1.0 / sqrt((double)D));
  p.c0 = (float)(1.0 / (alpha - 1.0));
  p.block_flags = nullptr;
  p.queue = nullptr;
  p.hints = nullptr;
  p.events = nullptr;
  p.queue2 = nullptr;
  p.hints2 = nullptr;
  p.kv_flags = nullptr;
  p.dk_part = nullptr;
  p.dv_part = nullptr;
  p.part_scratch = nullptr;
  p.merge256 = 0;
  p.part_rows = N;
  p.streams = nullptr;
  p.stream_dir = nullptr;
  p.dir_stride = 0;
  p.fwd_flags = nullptr;
  p.fwd_lens = nullptr;
  p.fwd_tshift = nullptr;
  p.fwd_streams = nullptr;
  const int am = alpha == 1.5 ? ATT_15 : (alpha == 2.0 ? ATT_2 : ATT_GEN);
  bool sparse = false;
  BwdWorkspace w = {};

  (void)hipGetLastError();
  if (dtype != ADSP_F32) {
    w = bwd_workspace(B, Hq, Hkv, N, D, dtype, is_causal ? 1 : 0);
    const size_t need = w.total;
    if (need && (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 15) != 0)) return ADSP_ERR_WORKSPACE;
    // Sparse-support dQ kernel first (alpha 1.5 / 2): it serves the row blocks whose supports are short and flags the
    // others for attn_bwd_dq_kernel below; the dK/dV kernel reads delta and 1 / sum p from whichever of the two wrote them.
    sparse = w.slots > 0 && (am == ATT_15 || am == ATT_2 || (alpha >= 1.125 && alpha < 2.0)) &&
             (long long)B * Hq * mblocks_of(N) < (1ll << 31) && sparse_enabled();
    if (sparse) {
      unsigned char* ws = (unsigned char*)workspace;
      p.queue = (uint32_t*)(ws + w.queue_off);
      p.hints = p.queue + 64;
      p.block_flags = (int32_t*)(ws + w.flags_off);
      p.events = ws + w.events_off;
      if (bwd_streams_enabled()) {
        p.streams = ws + w.streams_off;
        p.stream_dir = (uint16_t*)(ws + w.dir_off);
        p.dir_stride = w.dir_stride;
      }
      if (supports) {  // what the forward kept: its candidate streams stand in for the dQ kernel's walk
        const SupportsLayout sl = supports_layout(B, Hq, Hkv, N, D, dtype);
        if (sl.total && (supports_bytes < sl.total || ((uintptr_t)supports & 15) != 0)) return ADSP_ERR_WORKSPACE;
        if (sl.total) {
          const unsigned char* sp = (const unsigned char*)supports;
          p.fwd_flags = (const int32_t*)(sp + sl.flags_off);
          p.fwd_lens = (const uint16_t*)(sp + sl.lens_off);
          p.fwd_tshift = (const float*)(sp + sl.tshift_off);
          p.fwd_streams = sp + sl.streams_off;
        }
      }
      AttnParams pp = {};  // what the probe reads: q, k, lengths, dimensions, scale and the control words it clears
      pp.q = q;
      pp.k = k;
      pp.varlen = varlen;
      pp.varlen_bits = varlen_bits;
      pp.B = B;
      pp.Hq = Hq;
      pp.Hkv = Hkv;
      pp.N = N;
      pp.causal = p.causal;
      pp.qscale = p.qscale;
      pp.c0 = p.c0;
      pp.queue = p.queue;
      pp.hints = p.hints;
      pp.probe_max_support = probe_max_support();
      int rc;
      if (dtype == ADSP_BF16) {
        hipLaunchKernelGGL(attn_probe_kernel<bf16_t>, dim3((unsigned)(B * Hkv)), dim3(256), 0, s, pp, D, am);
        rc = D == 64 ? launch_attn_bwd_sparse_bf16_d64(p, am, 0, w.slots, s) : launch_attn_bwd_sparse_bf16_d128(p, am, 0, w.slots, s);
      } else {
        hipLaunchKernelGGL(attn_probe_kernel<f16_t>, dim3((unsigned)(B * Hkv)), dim3(256), 0, s, pp, D, am);
        rc = D == 64 ? launch_attn_bwd_sparse_f16_d64(p, am, 0, w.slots, s) : launch_attn_bwd_sparse_f16_d128(p, am, 0, w.slots, s);
      }
      if (rc != 0) return ADSP_ERR_LAUNCH;
    }
  }
  if (!sparse) {
    if (kBwdTable[dtype][head_dim_slot(D)](p, am, 3, s) != 0) return ADSP_ERR_LAUNCH;
    return hipGetLastError() == hipSuccess ? ADSP_OK : ADSP_ERR_LAUNCH;
  }
  // dense dQ kernel on the row blocks the sparse one flagged (delta and 1 / sum p are complete behind it), then dK and
  // dV: the sparse-support kernel per (key block, query head), the dense kernel on the key blocks it flagged, and the
  // sum of the partial rows over the query heads of each K/V head
  if (kBwdTable[dtype][head_dim_slot(D)](p, am, 1, s) != 0) return ADSP_ERR_LAUNCH;
  {
    unsigned char* ws = (unsigned char*)workspace;
    p.queue2 = (uint32_t*)(ws + w.queue2_off);
    p.hints2 = p.queue2 + 64;
    p.kv_flags = (int32_t*)(ws + w.kvflags_off);
    p.part_scratch = (float*)(ws + w.scratch_off);
    if (p.streams) p.merge256 = w.merge256;
    p.part_rows = w.part_rows;
    if (w.part_bytes) {
      p.dk_part = (float*)(ws + w.part_off);
      p.dv_part = (float*)(ws + w.part_off + w.part_bytes);
    }
    const long long n_flags = (long long)B * Hkv * mblocks_of(N);
    long long clear_items = n_flags > (long long)B * Hkv ? n_flags : (long long)B * Hkv;  // (at least one thread per K/V head and per control word)
    if (clear_items < 10) clear_items = 10;
    long long clear_blocks = (clear_items + 255) / 256;
    if (clear_blocks > 1024) clear_blocks = 1024;
    hipLaunchKernelGGL(bwd_ctrl_clear_kernel, dim3((unsigned)clear_blocks), dim3(256), 0, s, p.queue2, (const uint32_t*)p.hints, B * Hkv,
                       p.kv_flags, n_flags);
    int rc;
    const int kind = p.streams ? 2 : 1;  // from the dQ kernel's streams, or with a walk of its own
    if (dtype == ADSP_BF16) rc = D == 64 ? launch_attn_bwd_sparse_bf16_d64(p, am, kind, w.slots, s) : launch_attn_bwd_sparse_bf16_d128(p, am, kind, w.slots, s);
    else rc = D == 64 ? launch_attn_bwd_sparse_f16_d64(p, am, kind, w.slots, s) : launch_attn_bwd_sparse_f16_d128(p, am, kind, w.slots, s);
    if (rc != 0) return ADSP_ERR_LAUNCH;
    if (kBwdTable[dtype][head_dim_slot(D)](p, am, 2, s) != 0) return ADSP_ERR_LAUNCH;
    if (w.part_bytes && !(p.streams && Hq == Hkv)) {  // (with one query head per K/V head the kernel on the streams writes dK and dV itself)
      const long long threads = (long long)B * Hkv * N * (D / 8);
      const dim3 grid((unsigned)((threads + 255) / 256));
      if (dtype == ADSP_BF16)
        hipLaunchKernelGGL(dkdv_reduce_kernel<bf16_t>, grid, dim3(256), 0, s, (const float*)p.dk_part, (const float*)p.dv_part, dk, dv,
                           (const int32_t*)p.kv_flags, (const uint32_t*)p.queue2, varlen, varlen_bits, B, Hq, Hkv, N, D, p.causal, p.merge256, p.part_rows);
      else
        hipLaunchKernelGGL(dkdv_reduce_kernel<f16_t>, grid, dim3(256), 0, s, (const float*)p.dk_part, (const float*)p.dv_part, dk, dv,
                           (const int32_t*)p.kv_flags, (const uint32_t*)p.queue2, varlen, varlen_bits, B, Hq, Hkv, N, D, p.causal, p.merge256, p.part_rows);
    }
  }
  return hipGetLastError() == hipSuccess ? ADSP_OK : ADSP_ERR_LAUNCH;
}

extern "C" int adsp_attn_bwd(const void* q, const void* k, const void* v, const void* dout, const float* taus,
                             const int32_t* bmask, const void* varlen, int varlen_bits, void* dq, void* dk, void* dv,
                             float* delta, float* zinv, int B, int Hq, int Hkv, int N, int D, int dtype, double alpha,
                             int is_causal, void* workspace, size_t workspace_bytes, void* stream) {
  return attn_bwd_impl(q, k, v, dout, taus, bmask, varlen, varlen_bits, dq, dk, dv, delta, zinv, B, Hq, Hkv, N, D, dtype, alpha,
                       is_causal, workspace, workspace_bytes, nullptr, 0, stream);
}

extern "C" int adsp_attn_bwd_kept(const void* q, const void* k, const void* v, const void* dout, const float* taus,
                                  const int32_t* bmask, const void* varlen, int varlen_bits, void* dq, void* dk, void* dv,
                                  float* delta, float* zinv, int B, int Hq, int Hkv, int N, int D, int dtype, double alpha,
                                  int is_causal, void* workspace, size_t workspace_bytes, const void* supports,
                                  size_t supports_bytes, void* stream) {
  return attn_bwd_impl(q, k, v, dout, taus, bmask, varlen, varlen_bits, dq, dk, dv, delta, zinv, B, Hq, Hkv, N, D, dtype, alpha,
                       is_causal, workspace, workspace_bytes, supports, supports_bytes, stream);
}

extern "C" int adsp_version(void) { return 3; }

#ifndef ADSP_BUILD_ID
#define ADSP_BUILD_ID "unknown"
#endif
extern "C" const char* adsp_build_id(void) { return ADSP_BUILD_ID; }
#ifndef ADSP_BUILD_FLAGS
#define ADSP_BUILD_FLAGS ""
#endif
extern "C" const char* adsp_build_flags(void) { return ADSP_BUILD_FLAGS; }

extern "C" const char* adsp_status_string(int status) {
  switch (status) {
    case ADSP_OK: return "ok";
    case ADSP_ERR_NULL: return "a required pointer is NULL";
    case ADSP_ERR_SHAPE: return "a dimension is out of the supported range";
    case ADSP_ERR_DTYPE: return "unknown element type";
    case ADSP_ERR_ALIGN: return "a tensor base pointer is not 16-byte aligned";
    case ADSP_ERR_UNSUPPORTED: return "unsupported parameter combination";
    case ADSP_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
    case ADSP_ERR_LAUNCH: return "HIP launch failed";
    case ADSP_ERR_TOO_LARGE: return "problem needs more scratch than the allocation-free entry point holds";
  }
  return "unknown status";
}
