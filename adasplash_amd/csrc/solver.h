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

// Starting point inside [a, c]: one step of Muller's method on the surrogate, through a, the midpoint and c (the
// reference starts from the same parabola, triton_entmax_v2.py:208-322).  Written around c with divided differences:
// p(x) = fc + w (x - c) + q (x - c)^2, root x = c - 2 fc / (w +- sqrt(w^2 - 4 fc q)) with the sign that makes the
// denominator larger, i.e. the root nearer to c, which also covers a vanishing curvature (x = c - fc / w).  Without a
// real root: the secant through the two ends; the midpoint when that fails too.  The result is clamped to [a, c]; it
// only seeds the iteration.
template <int BINS>
__device__ __forceinline__ float hist_start_point(const float (&cnt)[BINS], float t_shift, float a, float c) {
  const float b = 0.5f * (a + c), h = c - b;
  if (!(h > 0.f)) return b;
  const float fa = hist_surrogate<BINS>(cnt, t_shift, a);
  const float fb = hist_surrogate<BINS>(cnt, t_shift, b);
  const float fc = hist_surrogate<BINS>(cnt, t_shift, c);
  const float d1 = (fb - fa) / h, d2 = (fc - fb) / h;  // slopes of the two halves
  const float q = (d2 - d1) / (2.f * h);               // half the curvature
  const float w = d2 + q * h;                          // slope of the parabola at c
  const float disc = w * w - 4.f * fc * q;
  float x = b;
  if (disc >= 0.f) {
    const float root = sqrtf(disc);
    const float den = w >= 0.f ? w + root : w - root;
    if (den != 0.f) x = c - 2.f * fc / den;
  } else if (fc != fa) {
    x = c - fc * (c - a) / (fc - fa);
  }
  x = (x == x) ? x : b;  // (0 / 0 and inf - inf end here)
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
