// Scalar pieces of the row-threshold solver: histogram bracket, Halley / Newton / secant / bisection.
// tau is the root of f(tau) = sum_j [z_j - tau]_+^(1/(alpha-1)) - 1 with z = (alpha-1) * score.
// Every function here works on per-row scalars that all lanes of a row hold redundantly.
#pragma once
#include "common.h"

namespace adsp {

// Lower bound of tau from a histogram of z - t_shift on BINS bins of width w starting at 0, alpha = 1.5.
// Every member of a bin is placed on the bin's lower edge e, the bins are taken greedily from the top
// while the quantised threshold stays below the bin edge (n e^2 - 2 e sum z + sum z^2 < 1), and the
// threshold of the accepted set has the closed form below.  Since quantising scores downwards by at most
// w moves tau downwards by at most w, the result lo satisfies lo <= tau <= lo + w.
// With `exact_max` the row maximum, known to sit at max_pos above t_shift, enters with its exact value
// instead of its bin edge (the reference's variant: adasplash/adasplash_v2.py:434-461,
// adasplash/triton_entmax_v2.py:135-155, where max_pos = 1 and w = 1 / BINS).
template <int BINS>
__device__ __forceinline__ float hist_bracket_alpha15(const float (&cnt)[BINS], float t_shift, float w = 1.f / (float)BINS,
                                                      bool exact_max = false, float max_pos = 1.f) {
  float sz = exact_max ? max_pos : 0.f, sk = exact_max ? 1.f : 0.f, szz = exact_max ? max_pos * max_pos : 0.f;
#pragma unroll
  for (int sj = BINS - 1; sj >= 0; --sj) {
    float c = cnt[sj] - ((exact_max && sj == BINS - 1) ? 1.f : 0.f);
    const float e = (float)sj * w;
    float nz = sz + c * e, nk = sk + c, nzz = szz + c * (e * e);
    bool good = nk * e * e - 2.f * nz * e + nzz < 1.f;
    sz = good ? nz : sz;
    sk = good ? nk : sk;
    szz = good ? nzz : szz;
  }
  sk = fmaxf(sk, 1.f);
  float disc = fmaxf(sz * sz - sk * (szz - 1.f), 0.f);
  return t_shift + (sz - sqrtf(disc)) / sk;
}

// Same for alpha = 2 (adasplash/triton_entmax_v2.py:114-131): accept while sum z - n e < 1.
template <int BINS>
__device__ __forceinline__ float hist_bracket_alpha2(const float (&cnt)[BINS], float t_shift, float w = 1.f / (float)BINS,
                                                     bool exact_max = false, float max_pos = 1.f) {
  float sz = exact_max ? max_pos : 0.f, sk = exact_max ? 1.f : 0.f;
#pragma unroll
  for (int sj = BINS - 1; sj >= 0; --sj) {
    float c = cnt[sj] - ((exact_max && sj == BINS - 1) ? 1.f : 0.f);
    const float e = (float)sj * w;
    float nz = sz + c * e, nk = sk + c;
    bool good = (nz - nk * e) < 1.f;
    sz = good ? nz : sz;
    sk = good ? nk : sk;
  }
  sk = fmaxf(sk, 1.f);
  return t_shift + (sz - 1.f) / sk;
}

// Bin-centre surrogate f_hist(tau) = sum_b c_b [centre_b - tau]_+^2 - 1 (triton_entmax_v2.py:165-204).
template <int BINS>
__device__ __forceinline__ float hist_surrogate(const float (&cnt)[BINS], float t_shift, float tau) {
  float acc = 0.f;
#pragma unroll
  for (int b = 0; b < BINS; ++b) {
    float d = fmaxf(t_shift + ((float)b + 0.5f) / (float)BINS - tau, 0.f);
    acc += cnt[b] * d * d;
  }
  return acc - 1.f;
}

// Starting point inside [a, c]: root (nearest c) of the parabola through the surrogate at a, mid, c
// (triton_entmax_v2.py:208-322).
template <int BINS>
__device__ __forceinline__ float hist_start_point(const float (&cnt)[BINS], float t_shift, float a, float c) {
  const float EPS = 1e-10f;
  float b = 0.5f * (a + c);
  float fa = hist_surrogate<BINS>(cnt, t_shift, a);
  float fb = hist_surrogate<BINS>(cnt, t_shift, b);
  float fc = hist_surrogate<BINS>(cnt, t_shift, c);
  float den = (a - b) * (a - c) * (b - c);
  float A = (fa * (b - c) + fb * (c - a) + fc * (a - b)) / den;
  float B = (fa * (c * c - b * b) + fb * (a * a - c * c) + fc * (b * b - a * a)) / den;
  float C = (fa * b * c * (b - c) + fb * a * c * (c - a) + fc * a * b * (a - b)) / den;
  float mid = 0.5f * (a + c);
  float x_lin = fabsf(B) > EPS ? -C / B : mid;
  float disc = B * B - 4.f * A * C;
  float sq = sqrtf(fmaxf(disc, 0.f));
  float r1 = (-B + sq) / (2.f * A), r2 = (-B - sq) / (2.f * A);
  bool v1 = r1 >= a && r1 <= c, v2 = r2 >= a && r2 <= c;
  float x_quad = (v1 && v2) ? (fabsf(c - r1) <= fabsf(c - r2) ? r1 : r2) : (v1 ? r1 : (v2 ? r2 : mid));
  float sden = fc - fa;
  float x_sec = fabsf(sden) > EPS ? c - fc * (c - a) / sden : mid;
  x_quad = disc >= 0.f ? x_quad : x_sec;
  float x = fabsf(A) < EPS ? x_lin : x_quad;
  x = fabsf(den) < EPS ? mid : x;
  x = (x == x) ? x : mid;  // NaN guard
  return fminf(fmaxf(x, a), c);
}

struct Bracket {
  float t, lo, hi;
};

// One safeguarded step from the statistics at br.t:
//   a0 = sum u^c0, a1 = sum u^(c0-1), a2 = sum u^(c0-2) over u = z - t > 0  (c0 = 1/(alpha-1)).
// Halley when allowed, else Newton, else secant, else bisection; a candidate is accepted only when it
// is finite and lies inside the current bracket (widened by eps).  Follows
// adasplash/triton_entmax_v2.py:43-110 (and adasplash/adasplash_v2.py:69-90 for alpha = 1.5).
__device__ __forceinline__ void hybrid_step(Bracket& br, float a0, float a1, float a2, float c0, bool allow_halley,
                                            bool allow_newton, bool allow_secant, float& t_prev, float& f_prev) {
  const float EPS = 1e-6f, EPS_DEN = 1e-12f;
  const float c1 = c0 - 1.f;
  float t = br.t;
  float ff = a0 - 1.f;
  float df = -c0 * a1;
  float ddf = c0 * c1 * a2;
  br.lo = ff > 0.f ? t : br.lo;
  br.hi = ff < 0.f ? t : br.hi;
  float lo = br.lo - EPS, hi = br.hi + EPS;

  float cand = 0.f;
  bool has = false;
  {
    float den = 2.f * df * df - ff * ddf;
    float th = t - (2.f * ff * df) / den;
    bool ok = allow_halley && th > lo && th < hi && fabsf(den) > EPS_DEN;  // (NaN/inf fail the range test)
    cand = ok ? th : cand;
    has = ok;
  }
  {
    // From the right of the root a Newton step of the convex f can land below the bracket, by a rounding error
    // when the root is the lower end itself (one entry carries all the mass) or by far when the support grows
    // quickly to the left.  The root is not down there: the lower end is the best point in that direction, and
    // from it every later Newton step approaches the root from the left without passing it.
    // The ends themselves are acceptable (eps is smaller than the spacing of floats at large scores, so a strict
    // test would turn the exact landing on the lower end into an endless bisection towards it).
    float tn = fmaxf(t - ff / df, br.lo);
    bool ok = allow_newton && !has && tn >= lo && tn <= hi && fabsf(df) > EPS_DEN;
    cand = ok ? tn : cand;
    has = has || ok;
  }
  if (allow_secant) {
    float den = ff - f_prev;
    float ts = t - ff * (t - t_prev) / den;
    bool ok = !has && ts > lo && ts < hi && fabsf(den) > EPS_DEN;
    cand = ok ? ts : cand;
    has = has || ok;
  }
  t_prev = t;
  f_prev = ff;
  br.t = has ? cand : 0.5f * (br.lo + br.hi);
}

}  // namespace adsp
