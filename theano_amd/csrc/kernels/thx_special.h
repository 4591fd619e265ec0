// Complex numbers and Bessel functions of real order for the generated per-element code.
// Compiled by hipRTC after thx_common.h; nothing here is host code.
#pragma once

// ---- complex numbers -------------------------------------------------------------------------
// Storage is NumPy's: (real, imaginary) pairs of float32 or float64.  The generated code converts
// every operand to the result type before an operation (as NumPy's loops do), so only same-type
// operators exist.  The reference defines the same struct with +, -, *, / and == in C
// (theano/scalar/basic.py:498-641); division here is Smith's scaled form, which is NumPy's.
template <class T>
struct __attribute__((aligned(2 * sizeof(T)))) thx_cplx {
  T re, im;
  thx_cplx() = default;
  __device__ __forceinline__ thx_cplx(T r, T i) : re(r), im(i) {}
  template <class U> __device__ __forceinline__ thx_cplx(const thx_cplx<U>& o) : re((T)o.re), im((T)o.im) {}
  template <class U> __device__ __forceinline__ thx_cplx(U r) : re((T)r), im((T)0) {}

  // operators are friends found through their complex operand, so that a real on the other side converts
  friend THX_DEV thx_cplx operator+(thx_cplx a, thx_cplx b) { return thx_cplx(a.re + b.re, a.im + b.im); }
  friend THX_DEV thx_cplx operator-(thx_cplx a, thx_cplx b) { return thx_cplx(a.re - b.re, a.im - b.im); }
  friend THX_DEV thx_cplx operator-(thx_cplx a) { return thx_cplx(-a.re, -a.im); }
  friend THX_DEV thx_cplx operator*(thx_cplx a, thx_cplx b) {
    return thx_cplx(a.re * b.re - a.im * b.im, a.re * b.im + a.im * b.re);
  }
  friend THX_DEV thx_cplx operator/(thx_cplx a, thx_cplx b) {
    const T abr = b.re < 0 ? -b.re : b.re, abi = b.im < 0 ? -b.im : b.im;
    if (abr >= abi) {
      if (abr == 0 && abi == 0) return thx_cplx(a.re / abr, a.im / abi);   // x / 0: infinities and NaNs as IEEE gives them
      const T rat = b.im / b.re, scl = (T)1 / (b.re + b.im * rat);
      return thx_cplx((a.re + a.im * rat) * scl, (a.im - a.re * rat) * scl);
    }
    const T rat = b.re / b.im, scl = (T)1 / (b.im + b.re * rat);
    return thx_cplx((a.re * rat + a.im) * scl, (a.im * rat - a.re) * scl);
  }
  friend THX_DEV bool operator==(thx_cplx a, thx_cplx b) { return a.re == b.re && a.im == b.im; }
  friend THX_DEV bool operator!=(thx_cplx a, thx_cplx b) { return a.re != b.re || a.im != b.im; }
};
typedef thx_cplx<float> thx_c64;
typedef thx_cplx<double> thx_c128;

namespace thx {
THX_DEV thx_c64 shfl_xor_t(thx_c64 v, int m) { return thx_c64(shfl_xor_t(v.re, m), shfl_xor_t(v.im, m)); }
THX_DEV thx_c128 shfl_xor_t(thx_c128 v, int m) { return thx_c128(shfl_xor_t(v.re, m), shfl_xor_t(v.im, m)); }
}  // namespace thx

// libm by precision, so that one template serves both complex types
THX_DEV float thx_m_hypot(float a, float b) { return hypotf(a, b); }
THX_DEV double thx_m_hypot(double a, double b) { return hypot(a, b); }
THX_DEV float thx_m_atan2(float a, float b) { return atan2f(a, b); }
THX_DEV double thx_m_atan2(double a, double b) { return atan2(a, b); }
THX_DEV float thx_m_exp(float a) { return expf(a); }
THX_DEV double thx_m_exp(double a) { return exp(a); }
THX_DEV float thx_m_expm1(float a) { return expm1f(a); }
THX_DEV double thx_m_expm1(double a) { return expm1(a); }
THX_DEV float thx_m_log(float a) { return logf(a); }
THX_DEV double thx_m_log(double a) { return log(a); }
THX_DEV float thx_m_log1p(float a) { return log1pf(a); }
THX_DEV double thx_m_log1p(double a) { return log1p(a); }
THX_DEV float thx_m_sqrt(float a) { return sqrtf(a); }
THX_DEV double thx_m_sqrt(double a) { return sqrt(a); }
THX_DEV void thx_m_sincos(float a, float& s, float& c) { sincosf(a, &s, &c); }
THX_DEV void thx_m_sincos(double a, double& s, double& c) { sincos(a, &s, &c); }
THX_DEV float thx_m_sinh(float a) { return sinhf(a); }
THX_DEV double thx_m_sinh(double a) { return sinh(a); }
THX_DEV float thx_m_cosh(float a) { return coshf(a); }
THX_DEV double thx_m_cosh(double a) { return cosh(a); }
THX_DEV float thx_m_copysign(float a, float b) { return copysignf(a, b); }
THX_DEV double thx_m_copysign(double a, double b) { return copysign(a, b); }

template <class T> THX_DEV T thx_cabs(thx_cplx<T> z) { return thx_m_hypot(z.re, z.im); }
template <class T> THX_DEV T thx_cangle(thx_cplx<T> z) { return thx_m_atan2(z.im, z.re); }
template <class T> THX_DEV thx_cplx<T> thx_cconj(thx_cplx<T> z) { return thx_cplx<T>(z.re, -z.im); }
template <class T> THX_DEV thx_cplx<T> thx_cpolar(T r, T theta) {
  T s, c;
  thx_m_sincos(theta, s, c);
  return thx_cplx<T>(r * c, r * s);
}
template <class T> THX_DEV thx_cplx<T> thx_cexp(thx_cplx<T> z) {
  const T e = thx_m_exp(z.re);
  if (z.im == 0) return thx_cplx<T>(e, z.im);
  T s, c;
  thx_m_sincos(z.im, s, c);
  return thx_cplx<T>(e * c, e * s);
}
// exp(z) - 1 without the cancellation near 0: Re = expm1(x) cos y - 2 sin^2(y / 2)
template <class T> THX_DEV thx_cplx<T> thx_cexpm1(thx_cplx<T> z) {
  T s, c, sh, ch;
  thx_m_sincos(z.im, s, c);
  thx_m_sincos(z.im * (T)0.5, sh, ch);
  const T em = thx_m_expm1(z.re);
  return thx_cplx<T>(em * c - (T)2 * sh * sh, (em + (T)1) * s);
}
template <class T> THX_DEV thx_cplx<T> thx_clog(thx_cplx<T> z) {
  const T ax = z.re < 0 ? -z.re : z.re, ay = z.im < 0 ? -z.im : z.im;
  const T big = ax > ay ? ax : ay, small = ax > ay ? ay : ax;
  T lr;
  if (big > (T)0.5 && big < (T)2) {
    // |z| near 1: log|z| = log1p((big - 1)(big + 1) + small^2) / 2 keeps the leading digits
    lr = (T)0.5 * thx_m_log1p((big - (T)1) * (big + (T)1) + small * small);
  } else {
    lr = thx_m_log(thx_m_hypot(z.re, z.im));
  }
  return thx_cplx<T>(lr, thx_m_atan2(z.im, z.re));
}
template <class T> THX_DEV thx_cplx<T> thx_clog2(thx_cplx<T> z) {
  const thx_cplx<T> l = thx_clog(z);
  return thx_cplx<T>(l.re * (T)1.44269504088896340736, l.im * (T)1.44269504088896340736);
}
template <class T> THX_DEV thx_cplx<T> thx_clog10(thx_cplx<T> z) {
  const thx_cplx<T> l = thx_clog(z);
  return thx_cplx<T>(l.re * (T)0.43429448190325182765, l.im * (T)0.43429448190325182765);
}
template <class T> THX_DEV thx_cplx<T> thx_clog1p(thx_cplx<T> z) {
  // |1 + z|^2 - 1 = 2x + x^2 + y^2; left of x = -1/2 the sum 1 + x is exact and the plain form loses nothing
  const T lr = z.re < (T)-0.5 ? thx_m_log(thx_m_hypot((T)1 + z.re, z.im))
                              : (T)0.5 * thx_m_log1p(z.re * ((T)2 + z.re) + z.im * z.im);
  return thx_cplx<T>(lr, thx_m_atan2(z.im, (T)1 + z.re));
}
template <class T> THX_DEV thx_cplx<T> thx_csqrt(thx_cplx<T> z) {
  if (z.re == 0 && z.im == 0) return thx_cplx<T>((T)0, z.im);
  const T ax = z.re < 0 ? -z.re : z.re;
  const T t = thx_m_sqrt((T)0.5 * (ax + thx_m_hypot(z.re, z.im)));
  if (z.re >= 0) return thx_cplx<T>(t, z.im / ((T)2 * t));
  const T ay = z.im < 0 ? -z.im : z.im;
  return thx_cplx<T>(ay / ((T)2 * t), thx_m_copysign(t, z.im));
}
template <class T> THX_DEV thx_cplx<T> thx_csin(thx_cplx<T> z) {
  T s, c;
  thx_m_sincos(z.re, s, c);
  return thx_cplx<T>(s * thx_m_cosh(z.im), c * thx_m_sinh(z.im));
}
template <class T> THX_DEV thx_cplx<T> thx_ccos(thx_cplx<T> z) {
  T s, c;
  thx_m_sincos(z.re, s, c);
  return thx_cplx<T>(c * thx_m_cosh(z.im), -(s * thx_m_sinh(z.im)));
}
template <class T> THX_DEV thx_cplx<T> thx_csinh(thx_cplx<T> z) {
  T s, c;
  thx_m_sincos(z.im, s, c);
  return thx_cplx<T>(thx_m_sinh(z.re) * c, thx_m_cosh(z.re) * s);
}
template <class T> THX_DEV thx_cplx<T> thx_ccosh(thx_cplx<T> z) {
  T s, c;
  thx_m_sincos(z.im, s, c);
  return thx_cplx<T>(thx_m_cosh(z.re) * c, thx_m_sinh(z.re) * s);
}
// tanh(x + iy) = (sinh x cosh x + i sin y cos y) / (sinh^2 x + cos^2 y): the denominator is a sum of
// squares, so nothing cancels next to the poles.  Beyond |x| = 22 the real part is +-1 to the last
// place and the imaginary part 4 sin y cos y exp(-2|x|) (the squares would overflow).
template <class T> THX_DEV thx_cplx<T> thx_ctanh(thx_cplx<T> z) {
  T s, c;
  thx_m_sincos(z.im, s, c);
  const T ax = z.re < 0 ? -z.re : z.re;
  if (ax > (T)22) return thx_cplx<T>(thx_m_copysign((T)1, z.re), (T)4 * s * c * thx_m_exp(-(T)2 * ax));
  const T sh = thx_m_sinh(z.re), ch = thx_m_cosh(z.re);
  const T d = sh * sh + c * c;
  return thx_cplx<T>(sh * ch / d, s * c / d);
}
// tan z = -i tanh(iz)
template <class T> THX_DEV thx_cplx<T> thx_ctan(thx_cplx<T> z) {
  const thx_cplx<T> t = thx_ctanh(thx_cplx<T>(-z.im, z.re));
  return thx_cplx<T>(t.im, -t.re);
}
// z ** w = exp(w log z); 0 ** w is 0 for Re w > 0, 1 for w = 0 and NaN otherwise (NumPy's rule);
// small whole real exponents multiply out, as NumPy does, so that they are exact where it is
template <class T> THX_DEV thx_cplx<T> thx_cpow(thx_cplx<T> z, thx_cplx<T> w) {
  if (w.re == 0 && w.im == 0) return thx_cplx<T>((T)1, (T)0);
  if (z.re == 0 && z.im == 0) {
    if (w.re > 0 && w.im == 0) return thx_cplx<T>((T)0, (T)0);
    return thx_cplx<T>((T)NAN, (T)NAN);
  }
  if (w.im == 0 && w.re == (T)(int)w.re && w.re > -100 && w.re < 100) {
    int n = (int)w.re;
    const bool invert = n < 0;
    if (invert) n = -n;
    thx_cplx<T> r((T)1, (T)0), p = z;
    while (n) {
      if (n & 1) r = r * p;
      p = p * p;
      n >>= 1;
    }
    return invert ? thx_cplx<T>((T)1, (T)0) / r : r;
  }
  return thx_cexp(w * thx_clog(z));
}

// ---- Bessel functions of real order -----------------------------------------------------------
// J_v(x) and I_v(x) (scipy.special.jv / iv in the reference, theano/scalar/basic_scipy.py:698-857),
// in double precision.  For x > 0 and v >= 0 the classical route: the continued fraction of
// J'_v / J_v (respectively I'_v / I_v) evaluated with the modified Lentz method, a downward
// recurrence to an order mu in [-1/2, 1/2), and there either Temme's series (x < 2) or the second
// continued fraction p + iq (Steed's method; for I: the continued fraction of K_{mu+1} / K_mu with
// its sum), joined through the Wronskian.  Negative orders use the reflection formulas through
// Y_v and K_v, which the same evaluation provides; negative x is defined for whole orders only.
struct thx_bessel_pair { double first, second; };   // (J, Y) or (I, K)

// Temme's gamma-function auxiliaries for |mu| <= 1/2:
// gam1 = (1/Gamma(1-mu) - 1/Gamma(1+mu)) / (2 mu), gam2 = (1/Gamma(1-mu) + 1/Gamma(1+mu)) / 2.
// gam1 is summed from the odd coefficients of the power series of 1/Gamma(1+t) (Abramowitz & Stegun 6.1.34):
// the difference itself cancels to nothing as mu goes to 0.
__device__ inline void thx_bessel_gammas(double mu, double& gam1, double& gam2, double& gampl, double& gammi) {
  gampl = 1.0 / tgamma(1.0 + mu);
  gammi = 1.0 / tgamma(1.0 - mu);
  gam2 = 0.5 * (gammi + gampl);
  const double t = mu * mu;
  gam1 = -(0.5772156649015329 + t * (-0.0420026350340952 + t * (-0.0421977345555443 + t * (0.0072189432466630 +
           t * (-0.0002152416741149 + t * (-0.0000201348547807 + t * (0.0000011330272320 + t * (0.0000000061160950 +
           t * -0.0000000011812746))))))));
}

__device__ inline thx_bessel_pair thx_bessel_jy(double v, double x) {   // v >= 0, x > 0
  const double eps = 1e-16, fpmin = 1e-300, pi = 3.14159265358979323846;
  const int maxit = 100000;
  const int nl = x < 2.0 ? (int)(v + 0.5) : (int)fmax(0.0, v - x + 1.5);
  const double mu = v - nl, mu2 = mu * mu;
  const double xi = 1.0 / x, xi2 = 2.0 * xi, w = xi2 / pi;
  int isign = 1;
  double h = v * xi;
  if (h < fpmin) h = fpmin;
  double b = xi2 * v, d = 0.0, c = h;
  for (int i = 1; i <= maxit; ++i) {
    b += xi2;
    d = b - d;
    if (fabs(d) < fpmin) d = fpmin;
    c = b - 1.0 / c;
    if (fabs(c) < fpmin) c = fpmin;
    d = 1.0 / d;
    const double del = c * d;
    h = del * h;
    if (d < 0.0) isign = -isign;
    if (fabs(del - 1.0) < eps) break;
  }
  double rjl = isign * fpmin, rjpl = h * rjl;
  double rjl1 = rjl;
  double fact = v * xi;
  for (int l = nl; l >= 1; --l) {
    const double rjtemp = fact * rjl + rjpl;
    fact -= xi;
    rjpl = fact * rjtemp - rjl;
    rjl = rjtemp;
    if (fabs(rjl) > 1e250) {   // orders far above x: the ratio to the starting value leaves the exponent range
      rjl *= 1e-250;
      rjpl *= 1e-250;
      rjl1 *= 1e-250;
    }
  }
  if (rjl == 0.0) rjl = eps;
  const double f = rjpl / rjl;
  double rjmu, rymu, rymup, ry1;
  if (x < 2.0) {
    const double x2 = 0.5 * x, pimu = pi * mu;
    fact = fabs(pimu) < eps ? 1.0 : pimu / sin(pimu);
    d = -log(x2);
    double e = mu * d;
    const double fact2 = fabs(e) < eps ? 1.0 : sinh(e) / e;
    double gam1, gam2, gampl, gammi;
    thx_bessel_gammas(mu, gam1, gam2, gampl, gammi);
    double ff = 2.0 / pi * fact * (gam1 * cosh(e) + gam2 * fact2 * d);
    e = exp(e);
    double p = e / (gampl * pi), q = 1.0 / (e * pi * gammi);
    const double pimu2 = 0.5 * pimu;
    const double fact3 = fabs(pimu2) < eps ? 1.0 : sin(pimu2) / pimu2;
    const double r = pi * pimu2 * fact3 * fact3;
    c = 1.0;
    d = -x2 * x2;
    double sum = ff + r * q, sum1 = p;
    for (int i = 1; i <= maxit; ++i) {
      ff = (i * ff + p + q) / (i * i - mu2);
      c *= d / i;
      p /= i - mu;
      q /= i + mu;
      const double del = c * (ff + r * q);
      sum += del;
      sum1 += c * p - i * del;
      if (fabs(del) < (1.0 + fabs(sum)) * eps) break;
    }
    rymu = -sum;
    ry1 = -sum1 * xi2;
    rymup = mu * xi * rymu - ry1;
    rjmu = w / (rymup - f * rymu);
  } else {
    double a = 0.25 - mu2, p = -0.5 * xi, q = 1.0;
    const double br = 2.0 * x;
    double bi = 2.0, fct = a * xi / (p * p + q * q);
    double cr = br + q * fct, ci = bi + p * fct, den = br * br + bi * bi;
    double dr = br / den, di = -bi / den, dlr = cr * dr - ci * di, dli = cr * di + ci * dr;
    double temp = p * dlr - q * dli;
    q = p * dli + q * dlr;
    p = temp;
    for (int i = 2; i <= maxit; ++i) {
      a += 2 * (i - 1);
      bi += 2.0;
      dr = a * dr + br;
      di = a * di + bi;
      if (fabs(dr) + fabs(di) < fpmin) dr = fpmin;
      fct = a / (cr * cr + ci * ci);
      cr = br + cr * fct;
      ci = bi - ci * fct;
      if (fabs(cr) + fabs(ci) < fpmin) cr = fpmin;
      den = dr * dr + di * di;
      dr /= den;
      di /= -den;
      dlr = cr * dr - ci * di;
      dli = cr * di + ci * dr;
      temp = p * dlr - q * dli;
      q = p * dli + q * dlr;
      p = temp;
      if (fabs(dlr - 1.0) + fabs(dli) < eps) break;
    }
    const double gam = (p - f) / q;
    rjmu = sqrt(w / ((p - f) * gam + q));
    if (rjl < 0.0) rjmu = -rjmu;
    rymu = rjmu * gam;
    rymup = rymu * (p + q / gam);
    ry1 = mu * xi * rymu - rymup;
  }
  fact = rjmu / rjl;
  thx_bessel_pair out;
  out.first = rjl1 * fact;
  for (int i = 1; i <= nl; ++i) {
    const double rytemp = (mu + i) * xi2 * ry1 - rymu;
    rymu = ry1;
    ry1 = rytemp;
  }
  out.second = rymu;
  return out;
}

__device__ inline thx_bessel_pair thx_bessel_ik(double v, double x) {   // v >= 0, x > 0
  const double eps = 1e-16, fpmin = 1e-300, pi = 3.14159265358979323846;
  const int maxit = 100000;
  const int nl = (int)(v + 0.5);
  const double mu = v - nl, mu2 = mu * mu;
  const double xi = 1.0 / x, xi2 = 2.0 * xi;
  double h = v * xi;
  if (h < fpmin) h = fpmin;
  double b = xi2 * v, d = 0.0, c = h;
  for (int i = 1; i <= maxit; ++i) {
    b += xi2;
    d = 1.0 / (b + d);
    c = b + 1.0 / c;
    const double del = c * d;
    h = del * h;
    if (fabs(del - 1.0) < eps) break;
  }
  double ril = fpmin, ripl = h * ril;
  double ril1 = ril;
  double fact = v * xi;
  for (int l = nl; l >= 1; --l) {
    const double ritemp = fact * ril + ripl;
    fact -= xi;
    ripl = fact * ritemp + ril;
    ril = ritemp;
    if (ril > 1e250) {   // orders far above x: the ratio to the starting value leaves the exponent range
      ril *= 1e-250;
      ripl *= 1e-250;
      ril1 *= 1e-250;
    }
  }
  const double f = ripl / ril;
  double rkmu, rk1;
  if (x < 2.0) {
    const double x2 = 0.5 * x, pimu = pi * mu;
    fact = fabs(pimu) < eps ? 1.0 : pimu / sin(pimu);
    d = -log(x2);
    double e = mu * d;
    const double fact2 = fabs(e) < eps ? 1.0 : sinh(e) / e;
    double gam1, gam2, gampl, gammi;
    thx_bessel_gammas(mu, gam1, gam2, gampl, gammi);
    double ff = fact * (gam1 * cosh(e) + gam2 * fact2 * d);
    double sum = ff;
    e = exp(e);
    double p = 0.5 * e / gampl, q = 0.5 / (e * gammi);
    c = 1.0;
    d = x2 * x2;
    double sum1 = p;
    for (int i = 1; i <= maxit; ++i) {
      ff = (i * ff + p + q) / (i * i - mu2);
      c *= d / i;
      p /= i - mu;
      q /= i + mu;
      const double del = c * ff;
      sum += del;
      sum1 += c * (p - i * ff);
      if (fabs(del) < fabs(sum) * eps) break;
    }
    rkmu = sum;
    rk1 = sum1 * xi2;
  } else {
    b = 2.0 * (1.0 + x);
    d = 1.0 / b;
    h = d;
    double delh = d, q1 = 0.0, q2 = 1.0;
    const double a1 = 0.25 - mu2;
    double q = a1;
    c = a1;
    double a = -a1, s = 1.0 + q * delh;
    for (int i = 2; i <= maxit; ++i) {
      a -= 2 * (i - 1);
      c = -a * c / i;
      const double qnew = (q1 - b * q2) / a;
      q1 = q2;
      q2 = qnew;
      q += c * qnew;
      b += 2.0;
      d = 1.0 / (b + a * d);
      delh = (b * d - 1.0) * delh;
      h += delh;
      const double dels = q * delh;
      s += dels;
      if (fabs(dels / s) < eps) break;
    }
    h = a1 * h;
    rkmu = sqrt(pi / (2.0 * x)) * exp(-x) / s;
    rk1 = rkmu * (mu + x + 0.5 - h) * xi;
  }
  const double rkmup = mu * xi * rkmu - rk1;
  const double rimu = xi / (f * rkmu - rkmup);
  thx_bessel_pair out;
  out.first = (rimu * ril1) / ril;
  for (int i = 1; i <= nl; ++i) {
    const double rktemp = (mu + i) * xi2 * rk1 + rkmu;
    rkmu = rk1;
    rk1 = rktemp;
  }
  out.second = rkmu;
  return out;
}

// Hankel's asymptotic expansion, for x >= 30 and x >= v^2 (any real v): sqrt(2 / (pi x)) (P cos chi - Q sin chi),
// chi = x - (v / 2 + 1 / 4) pi, P and Q the even and odd terms of sum_k a_k(v) / x^k with
// a_k = (4 v^2 - 1)(4 v^2 - 9)...(4 v^2 - (2k - 1)^2) / (k! 8^k).  In that range the terms fall below 1e-17 of the
// sum long before they start to grow (at k ~ 2x).  cos and sin of chi come from those of x and of the order's part
// separately: forming chi first would lose the digits of the order's part in a large x.  The continued fraction
// of the general route takes about x iterations and loses accuracy with each, so it stops here.
__device__ inline double thx_jv_large_x(double v, double x) {
  const double pi = 3.14159265358979323846, mu = 4.0 * v * v;
  double term = 1.0, P = 1.0, Q = 0.0;
  for (int k = 1; k < 200; ++k) {
    const double odd = 2.0 * k - 1.0;
    const double next = term * (mu - odd * odd) / (8.0 * k * x);
    if (fabs(next) > fabs(term) && k > 1) break;
    term = next;
    // k = 1, 2, 3, 4, ...: Q +, P -, Q -, P +
    if (k & 1) Q += (k & 2) ? -term : term;
    else P += (k & 2) ? -term : term;
    if (fabs(term) < 1e-17 * (fabs(P) + fabs(Q))) break;
  }
  double sx, cx, sa, ca;
  sincos(x, &sx, &cx);
  // (v / 2 + 1 / 4) pi reduced by whole turns first: v / 2 + 1 / 4 = n + f with |f| <= 1 (two turns are 4 in these units)
  const double h = 0.5 * v + 0.25;
  const double f = h - 2.0 * floor(h * 0.5);       // in [0, 2): whole multiples of 2 pi dropped exactly
  sincos(f * pi, &sa, &ca);
  const double cchi = cx * ca + sx * sa, schi = sx * ca - cx * sa;
  return sqrt(2.0 / (pi * x)) * (P * cchi - Q * schi);
}

// J_v(x) for any real order and argument.
__device__ inline double thx_jv(double v, double x) {
  if (isnan(v) || isnan(x)) return NAN;
  const bool whole = v == floor(v);
  if (x < 0.0) {
    if (!whole) return NAN;
    const double r = thx_jv(v, -x);
    return fmod(fabs(v), 2.0) == 1.0 ? -r : r;     // J_n(-x) = (-1)^n J_n(x)
  }
  if (x == 0.0) {
    if (v == 0.0) return 1.0;
    if (v > 0.0 || whole) return 0.0;
    return copysign(INFINITY, tgamma(v + 1.0));   // (x / 2)^v / Gamma(v + 1) diverges for non-whole v < 0
  }
  if (isinf(x)) return 0.0;
  if (x >= 30.0 && x >= v * v) return thx_jv_large_x(v, x);
  if (v >= 0.0) return thx_bessel_jy(v, x).first;
  const double a = -v;
  const thx_bessel_pair p = thx_bessel_jy(a, x);
  if (whole) return fmod(a, 2.0) == 1.0 ? -p.first : p.first;
  // J_{-a} = cos(a pi) J_a - sin(a pi) Y_a
  const double pi = 3.14159265358979323846;
  return cos(a * pi) * p.first - sin(a * pi) * p.second;
}
__device__ inline float thx_jv(float v, float x) { return (float)thx_jv((double)v, (double)x); }

// I_v(x) for any real order and argument.
__device__ inline double thx_iv(double v, double x) {
  if (isnan(v) || isnan(x)) return NAN;
  const bool whole = v == floor(v);
  if (x < 0.0) {
    if (!whole) return NAN;
    const double r = thx_iv(v, -x);
    return fmod(fabs(v), 2.0) == 1.0 ? -r : r;     // I_n(-x) = (-1)^n I_n(x)
  }
  if (x == 0.0) {
    if (v == 0.0) return 1.0;
    if (v > 0.0 || whole) return 0.0;
    return INFINITY;
  }
  if (isinf(x)) return INFINITY;
  const double a = fabs(v);
  const thx_bessel_pair p = thx_bessel_ik(a, x);
  if (v >= 0.0 || whole) return p.first;
  // I_{-a} = I_a + (2 / pi) sin(a pi) K_a
  const double pi = 3.14159265358979323846;
  return p.first + 2.0 / pi * sin(a * pi) * p.second;
}
__device__ inline float thx_iv(float v, float x) { return (float)thx_iv((double)v, (double)x); }
