// Special functions of the reference's unary table that the device libm does not supply: digamma, trigamma
// (src/libknet8/ops.jl:37-38, src/libknet8/gamma.jl) and the Bessel functions of integer order (src/libknet8/ops.jl:139-140,
// src/libknet8/cuda1.jl:49-79).  Everything is evaluated in fp64 and rounded once to T, which is what the CPU path does for
// Float32 arguments (SpecialFunctions.jl widens them), so the fp32 entry points are correctly rounded in all but rare cases.
//
// The routines are plain functions of doubles (KNET8_HD marks them for both host and device) so that a host compiler can
// build them for tests on the CPU.
#pragma once
#include <math.h>
#include <float.h>

#ifndef KNET8_HD
#define KNET8_HD __host__ __device__
#endif

namespace knet8 {

constexpr double kPi = 3.14159265358979323846;

// psi(x) for x >= 10 by the asymptotic series  ln x - 1/(2x) - sum_k B_2k / (2k x^2k)  (B_2k: Bernoulli numbers;
// the first omitted term, 3617/(8160 x^16), is below 5e-18 there).
KNET8_HD inline double digamma_large(double x) {
  const double z = 1.0 / (x * x);
  const double series = z * (1.0 / 12 - z * (1.0 / 120 - z * (1.0 / 252 - z * (1.0 / 240 - z * (1.0 / 132 - z * (691.0 / 32760 - z * (1.0 / 12)))))));
  return log(x) - 0.5 / x - series;
}

// digamma: the recurrence psi(x) = psi(x+1) - 1/x lifts the argument to >= 10; arguments <= 0 go through the reflection
// psi(x) = psi(1-x) - pi/tan(pi x), the tangent taken of the distance r to the nearest integer (|r| <= 1/2) so that it keeps
// its accuracy for large |x|.  At the poles 0, -1, -2, ... the result is the largest finite value of `big`'s type, as
// src/libknet8/gamma.jl:86-88 returns it.
KNET8_HD inline double digamma_f64(double x, double big) {
  double refl = 0.0;
  if (x != x) return x;
  if (x <= 0.0) {
    const double near = rint(x);
    if (near == x) return big;
    const double r = x - near;  // exact
    refl = (fabs(r) == 0.5) ? 0.0 : kPi / tan(kPi * r);
    x = 1.0 - x;
  }
  double w = 0.0;
  while (x < 10.0) {
    w += 1.0 / x;
    x += 1.0;
  }
  return digamma_large(x) - w - refl;
}

// trigamma = zeta(2, x) (src/libknet8/gamma.jl:237-239): psi1(x) = psi1(x+1) + 1/x^2 up to x >= 10, then
// 1/x + 1/(2x^2) + sum_k B_2k / x^(2k+1); for x <= 0 the reflection psi1(x) = pi^2/sin^2(pi x) - psi1(1-x).
// Poles give `big`, as the reference's zeta routine does for a non-positive integer argument.
KNET8_HD inline double trigamma_f64(double x, double big) {
  if (x != x) return x;
  double refl = 0.0, sign = 1.0;
  if (x <= 0.0) {
    const double near = rint(x);
    if (near == x) return big;
    const double r = x - near;  // exact
    const double s = sin(kPi * r);
    refl = (kPi / s) * (kPi / s);
    sign = -1.0;
    x = 1.0 - x;
  }
  double w = 0.0;
  while (x < 10.0) {
    w += 1.0 / (x * x);
    x += 1.0;
  }
  const double ix = 1.0 / x, z = ix * ix;
  const double tail = ix + 0.5 * z +
                      ix * z * (1.0 / 6 - z * (1.0 / 30 - z * (1.0 / 42 - z * (1.0 / 30 - z * (5.0 / 66 - z * (691.0 / 2730 - z * (7.0 / 6)))))));
  return refl + sign * (tail + w);
}

// J_n(x), n >= 2, x > 0.  Above the turning point (x > n) the upward recurrence J_{k+1} = (2k/x) J_k - J_{k-1} is stable.
// Below it the recurrence is run downwards from an order well above n, where any start vector converges to the minimal
// solution, and normalised with 1 = J_0 + 2 (J_2 + J_4 + ...).
KNET8_HD inline double besselj_pos(int n, double x) {
  if (x > (double)n) {
    double a = j0(x), b = j1(x);
    for (int k = 1; k < n; k++) {
      const double c = (2.0 * k / x) * b - a;
      a = b;
      b = c;
    }
    return b;
  }
  // J_n(x) underflows long before x^n/(2^n n!) does in exponent terms: nothing to resolve below that
  if (n > 4 && n * (log(0.5 * x) + 1.0 - log((double)n)) < -745.0) return 0.0;
  // start order: even, beyond n by enough that the error of the arbitrary start has decayed below 1 ulp at n
  int m = n + (int)sqrt(60.0 * n) + 8;
  if (m < (int)x + 24) m = (int)x + 24;
  m += m & 1;
  double hi = 0.0, cur = 1.0, sum = 0.0, ans = 0.0;
  for (int k = m; k > 0; k--) {
    const double lo = (2.0 * k / x) * cur - hi;
    hi = cur;
    cur = lo;
    if (fabs(cur) > 1e200) {  // rescale everything: only ratios matter
      cur *= 1e-200;
      hi *= 1e-200;
      sum *= 1e-200;
      ans *= 1e-200;
    }
    // cur is now J_{k-1} up to the common factor
    if (((k - 1) & 1) == 0 && k - 1 > 0) sum += cur;
    if (k - 1 == n) ans = cur;
  }
  const double norm = 2.0 * sum + cur;  // cur = J_0
  return ans / norm;
}

// besselj(d, x) for any integer d and real x: J_{-n} = (-1)^n J_n and J_n(-x) = (-1)^n J_n(x)
// (the sign rule of src/libknet8/ops.jl:139).
KNET8_HD inline double besselj_f64(int d, double x) {
  if (x != x) return x;
  int n = d < 0 ? -d : d;
  double sign = (d < 0 && (n & 1)) ? -1.0 : 1.0;
  if (x < 0.0) {
    x = -x;
    if (n & 1) sign = -sign;
  }
  if (n == 0) return j0(x);
  if (n == 1) return sign * j1(x);
  if (x == 0.0) return 0.0;
  if (isinf(x)) return 0.0;
  return sign * besselj_pos(n, x);
}

// bessely(d, x): the upward recurrence is stable for Y at every x > 0; Y_{-n} = (-1)^n Y_n (src/libknet8/ops.jl:140).
// x < 0 has no real value: NaN.  x == 0: -Inf.
KNET8_HD inline double bessely_f64(int d, double x) {
  if (x != x) return x;
  const int n = d < 0 ? -d : d;
  const double sign = (d < 0 && (n & 1)) ? -1.0 : 1.0;
  if (x < 0.0) return NAN;
  if (n == 0) return y0(x);
  if (n == 1) return sign * y1(x);
  if (x == 0.0) return -sign * INFINITY;
  if (isinf(x)) return 0.0;
  double a = y0(x), b = y1(x);
  for (int k = 1; k < n && b != -INFINITY; k++) {
    const double c = (2.0 * k / x) * b - a;
    a = b;
    b = c;
  }
  return sign * b;
}

template <typename T> KNET8_HD inline T kdigamma(T x) { return (T)digamma_f64((double)x, sizeof(T) == 4 ? (double)FLT_MAX : DBL_MAX); }
template <typename T> KNET8_HD inline T ktrigamma(T x) { return (T)trigamma_f64((double)x, sizeof(T) == 4 ? (double)FLT_MAX : DBL_MAX); }
template <typename T> KNET8_HD inline T kbesselj(int d, T x) { return (T)besselj_f64(d, (double)x); }
template <typename T> KNET8_HD inline T kbessely(int d, T x) { return (T)bessely_f64(d, (double)x); }

}  // namespace knet8
