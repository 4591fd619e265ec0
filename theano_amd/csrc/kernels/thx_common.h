// Device-side helpers shared by every run-time compiled kernel (gfx950, wave64).
// This text is compiled by hipRTC together with a generated functor and one
// `extern "C"` entry point per launch plan; nothing here is host code.
#pragma once

typedef unsigned char thx_bool;  // numpy bool storage: one byte holding 0 or 1
typedef signed char thx_i8;
typedef unsigned char thx_u8;
typedef short thx_i16;
typedef unsigned short thx_u16;
typedef int thx_i32;
typedef unsigned int thx_u32;
typedef long long thx_i64;
typedef unsigned long long thx_u64;
typedef _Float16 thx_f16;
typedef float thx_f32;
typedef double thx_f64;

#ifndef INFINITY
#define INFINITY (__builtin_inff())
#endif
#ifndef NAN
#define NAN (__builtin_nanf(""))
#endif

#define THX_DEV __device__ __forceinline__
#define THX_WAVE 64

// Single-precision division as the generated per-element code spells it.  With THX_FAST_DIV: the
// divisor b = mb * 2^eb (mb in [0.5, 1)) becomes the factor r1 = rcp(mb) * 2^-eb (one v_rcp_f32, 1 ulp) and
// the quotient is a * r1, one rounding.  So that r1 stays a normal number for every b, the exponent it
// carries is eb clamped to [-120, 120] and what remains of it (nothing unless |b| is beyond 2^+-120) is a
// second, exact factor f2 = 2^(h - eb): the result is (a * r1) * f2, within 2.5 ulp of the quotient for
// every finite input including denormals, and 0, infinity and NaN come out as IEEE division gives them.
// The intermediate product equals the quotient in the common case; for |b| > 2^119 it is larger by at most
// 2^8 while the quotient cannot exceed 2^9, for |b| < 2^-121 it is smaller by at most 2^-28 while a * r1
// is at least 2^-29 for any non-zero a: it overflows or goes denormal only where the quotient does.
// Everything but the two multiplications depends on b alone, so a divisor shared by many elements - a
// row's sum, a per-channel scale, any loop invariant - costs two multiplications per element, where
// scaling both operands by their exponents cost five.  (The compiler flag that asks for a 2.5-ulp lowering
// of `/` is lost on the way through the optimiser for these kernels; spelling it out is what makes it stick.)
#ifdef THX_FAST_DIV
__device__ __forceinline__ float thx_fdiv(float a, float b) {
  const float mb = __builtin_amdgcn_frexp_mantf(b);
  const int eb = __builtin_amdgcn_frexp_expf(b);
  const int h = eb < -120 ? -120 : (eb > 120 ? 120 : eb);
  const float r1 = __builtin_ldexpf(__builtin_amdgcn_rcpf(mb), -h);
  const float f2 = __builtin_ldexpf(1.0f, h - eb);
  return (a * r1) * f2;
}
#else
__device__ __forceinline__ float thx_fdiv(float a, float b) { return a / b; }
#endif

// Square root in single precision as the generated per-element code spells it.  With THX_FAST_DIV: one
// v_sqrt_f32 (1 ulp); operands below 2^-96 are scaled by 2^32 first so that denormals keep their precision.
// The compiler's own lowering of sqrtf under the 2.5-ulp flag depends on the surrounding code (the
// permission is dropped where the optimiser vectorises the call, and the correctly rounded sequence comes
// out instead), so one expression compiled into two kernels, or into two loops of one kernel, could differ
// in the last bit - and a gradient of max, which compares the reduction's result with its recomputed
// operand for equality, would then miss the maximum.  Spelled out, every copy agrees.
#ifdef THX_FAST_DIV
__device__ __forceinline__ float thx_fsqrt(float x) {
  const bool small = x < 0x1.0p-96f;
  const float r = __builtin_amdgcn_sqrtf(small ? x * 0x1.0p+32f : x);
  return small ? r * 0x1.0p-16f : r;
}
#else
__device__ __forceinline__ float thx_fsqrt(float x) { return sqrtf(x); }
#endif

// Signed integer arithmetic in two's complement: a sum, difference, product or negation that leaves the
// range wraps, as NumPy's does and as the reference's compiled C does on its hosts.  Written through the
// unsigned type, because signed overflow is undefined in C++ and the compiler builds on that: abs(x) | 1
// "cannot" be negative, so a branch on its sign disappears and x % -(abs(y) | 1) comes out with the wrong
// sign for y = INT_MIN.  The operands take C's usual common type first, as in the reference's expressions;
// every type but int and long long computes as written.
template <class C> __device__ __forceinline__ C thx_wadd_(C a, C b) { return a + b; }
template <class C> __device__ __forceinline__ C thx_wsub_(C a, C b) { return a - b; }
template <class C> __device__ __forceinline__ C thx_wmul_(C a, C b) { return a * b; }
__device__ __forceinline__ int thx_wadd_(int a, int b) { return (int)((unsigned)a + (unsigned)b); }
__device__ __forceinline__ int thx_wsub_(int a, int b) { return (int)((unsigned)a - (unsigned)b); }
__device__ __forceinline__ int thx_wmul_(int a, int b) { return (int)((unsigned)a * (unsigned)b); }
__device__ __forceinline__ long long thx_wadd_(long long a, long long b) {
  return (long long)((unsigned long long)a + (unsigned long long)b);
}
__device__ __forceinline__ long long thx_wsub_(long long a, long long b) {
  return (long long)((unsigned long long)a - (unsigned long long)b);
}
__device__ __forceinline__ long long thx_wmul_(long long a, long long b) {
  return (long long)((unsigned long long)a * (unsigned long long)b);
}
template <class A, class B> __device__ __forceinline__ auto thx_wadd(A a, B b) -> decltype(a + b) {
  typedef decltype(a + b) C;
  return thx_wadd_((C)a, (C)b);
}
template <class A, class B> __device__ __forceinline__ auto thx_wsub(A a, B b) -> decltype(a - b) {
  typedef decltype(a - b) C;
  return thx_wsub_((C)a, (C)b);
}
template <class A, class B> __device__ __forceinline__ auto thx_wmul(A a, B b) -> decltype(a * b) {
  typedef decltype(a * b) C;
  return thx_wmul_((C)a, (C)b);
}
template <class A> __device__ __forceinline__ auto thx_wneg(A a) -> decltype(-a) {
  typedef decltype(-a) C;
  return thx_wsub_((C)0, (C)a);
}
template <class A> __device__ __forceinline__ auto thx_wabs(A a) -> decltype(-a) { return a < 0 ? thx_wneg(a) : a; }

// exp(x) in single precision.  In the 2.5-ulp build: one hardware exp2 of the rounded product
// x * log2(e); the rounding of the product is a relative error of up to |x| * 4e-8 in the result
// (3.8e-6 at the ends of the finite range, |x| = 88), overflow gives infinity and underflow zero as
// expf does.  3 instructions instead of 9.
#ifdef THX_FAST_DIV
__device__ __forceinline__ float thx_fexp(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f); }
#else
__device__ __forceinline__ float thx_fexp(float x) { return expf(x); }
#endif

// 1 / (1 + exp(-x)) for -88 <= x <= 15 (the caller applies the reference's saturation outside).
// In the 2.5-ulp build the exponential is one hardware exp2 of the rounded product x * log2(e),
// whose rounding is a relative error of up to |x| * 4e-8 in exp(-x); it reaches the result only
// where exp(-x) dominates it: below 8.5e-7 relative wherever the result exceeds 1e-6, 3.8e-6 at
// x = -88 (where the result is 1e-38).  The reciprocal is one hardware rcp: its argument lies in
// [1, 2e38], where rcp needs no rescaling.  8 instructions instead of 22.
#ifdef THX_FAST_DIV
__device__ __forceinline__ float thx_sigmoid_core(float x) {
  return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.44269504088896340736f));
}
#else
__device__ __forceinline__ float thx_sigmoid_core(float x) { return 1.0f / (1.0f + expf(-x)); }
#endif

// x / y in the type C gives the quotient, correctly rounded even when single-precision division
// is built in its 2.5-ulp form: a double quotient rounded to float is the correctly rounded float
// quotient (53 >= 2 * 24 + 2 bits).
// Two integers divide as integers (a signed integer beside a uint64 makes a float64 node whose text still
// divides its integer operands first).
template <class A, class B>
__device__ __forceinline__ auto thx_exact_div(A a, B b) -> decltype(a / b) {
  typedef decltype(a / b) R;
  if constexpr (R(1) / R(2) == R(0)) {
    return a / b;
  } else {
    return (R)((double)a / (double)b);
  }
}

// Digamma and trigamma (the reference ships its own C for both, theano/scalar/basic_scipy.py:
// 340-391, 430-470): arguments below 10 are moved up with psi(x) = psi(x + 1) - 1/x and
// psi'(x) = psi'(x + 1) + 1/x^2, negative ones first reflected to 1 - x, then the asymptotic
// series in 1/x^2 is summed in double precision.  Poles (0, -1, -2, ...) give NaN.
__device__ inline double thx_psi(double x) {
  double r = 0.0;
  if (x <= 0.0) {
    if (x == floor(x)) return NAN;
    r = -3.14159265358979323846 / tan(3.14159265358979323846 * x);
    x = 1.0 - x;
  }
  while (x < 10.0) {
    r -= 1.0 / x;
    x += 1.0;
  }
  const double f = 1.0 / (x * x);
  const double t = f * (1.0 / 12 - f * (1.0 / 120 - f * (1.0 / 252 - f * (1.0 / 240 - f * (1.0 / 132)))));
  return r + log(x) - 0.5 / x - t;
}
__device__ inline float thx_psi(float x) { return (float)thx_psi((double)x); }

__device__ inline double thx_trigamma(double x) {
  double r = 0.0, sign = 1.0;
  if (x <= 0.0) {
    if (x == floor(x)) return NAN;
    const double s = sin(3.14159265358979323846 * x);
    r = 9.86960440108935861883 / (s * s);
    sign = -1.0;
    x = 1.0 - x;
  }
  double acc = 0.0;
  while (x < 10.0) {
    acc += 1.0 / (x * x);
    x += 1.0;
  }
  const double f = 1.0 / (x * x);
  const double t = f * (1.0 / 6 - f * (1.0 / 30 - f * (1.0 / 42 - f * (1.0 / 30 - f * (5.0 / 66)))));
  return r + sign * (acc + 1.0 / x + 0.5 * f + t / x);
}
__device__ inline float thx_trigamma(float x) { return (float)thx_trigamma((double)x); }

// Modified Bessel functions of the first kind for any sign of the argument: the device library's
// cyl_bessel_i1 gives NaN below zero; I0 is even and I1 odd.
__device__ inline double thx_i0(double x) { return cyl_bessel_i0(fabs(x)); }
__device__ inline float thx_i0(float x) { return cyl_bessel_i0f(fabsf(x)); }
__device__ inline double thx_i1(double x) { return copysign(cyl_bessel_i1(fabs(x)), x); }
__device__ inline float thx_i1(float x) { return copysignf(cyl_bessel_i1f(fabsf(x)), x); }

// Regularized incomplete gamma functions P(k, x) and Q(k, x) = 1 - P (the reference ships C for
// them too, theano/scalar/c_code/gamma.c): the power series of P for x < k + 1, the continued
// fraction of Q (modified Lentz evaluation) beyond, each scaled by exp(-x + k ln x - lgamma(k));
// computed in double precision.  k <= 0 or x < 0 give NaN.
__device__ inline double thx_gamma_p_series(double k, double x) {
  double term = 1.0 / k, sum = term;
  for (int n = 1; n < 1000; ++n) {
    term *= x / (k + n);
    sum += term;
    if (fabs(term) < fabs(sum) * 1e-17) break;
  }
  return sum * exp(-x + k * log(x) - lgamma(k));
}
__device__ inline double thx_gamma_q_fraction(double k, double x) {
  const double tiny = 1e-300;
  double b = x + 1.0 - k, c = 1.0 / tiny, d = 1.0 / b, h = d;
  for (int i = 1; i < 1000; ++i) {
    const double an = -i * (i - k);
    b += 2.0;
    d = an * d + b;
    if (fabs(d) < tiny) d = tiny;
    c = b + an / c;
    if (fabs(c) < tiny) c = tiny;
    d = 1.0 / d;
    const double del = d * c;
    h *= del;
    if (fabs(del - 1.0) < 1e-16) break;
  }
  return h * exp(-x + k * log(x) - lgamma(k));
}
__device__ inline double thx_gammainc(double k, double x) {
  if (!(k > 0.0) || !(x >= 0.0)) return NAN;
  if (x == 0.0) return 0.0;
  if (isinf(x)) return 1.0;
  return x < k + 1.0 ? thx_gamma_p_series(k, x) : 1.0 - thx_gamma_q_fraction(k, x);
}
__device__ inline double thx_gammaincc(double k, double x) {
  if (!(k > 0.0) || !(x >= 0.0)) return NAN;
  if (x == 0.0) return 1.0;
  if (isinf(x)) return 0.0;
  return x < k + 1.0 ? 1.0 - thx_gamma_p_series(k, x) : thx_gamma_q_fraction(k, x);
}

namespace thx {

// How one operand is addressed along the vectorised (innermost) dimension.
enum { M_VEC = 0,      // unit stride: one wide load/store per thread
       M_BCAST = 1,    // zero stride: one element shared by the whole vector
       M_GATHER = 2,   // any other stride: one access per element
       M_IMM = 3,      // a single host value passed in the kernel arguments
       M_IOTA = 4 };   // no memory: the value is the element offset itself (a position index)

template <int B> struct AlignFor { enum { value = B >= 16 ? 16 : B }; };

// N consecutive elements, aligned so that a 16-byte pack is one dwordx4 access.
template <class T, int N>
struct __attribute__((aligned(AlignFor<sizeof(T) * N>::value))) Vec {
  T v[N];
};

// Raw B-byte accesses, optionally with the non-temporal hint (data that is
// touched once should not displace anything in L2).
typedef unsigned int thx_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int thx_u32x2 __attribute__((ext_vector_type(2)));

template <int B> struct RawOf;
template <> struct RawOf<16> { typedef thx_u32x4 type; };
template <> struct RawOf<8> { typedef thx_u32x2 type; };
template <> struct RawOf<4> { typedef unsigned int type; };
template <> struct RawOf<2> { typedef unsigned short type; };
template <> struct RawOf<1> { typedef unsigned char type; };

// The same accesses through pointers that are only aligned to A bytes (an element): rows of an odd length and views
// that start anywhere.  The compiler keeps them whole where the device reads and writes global memory at any
// alignment and splits them where it does not; measured 3 % slower than aligned accesses when streaming 256 MB.
template <int B, int A> struct RawUOf { typedef typename RawOf<B>::type type __attribute__((aligned(A))); };

template <class T, int N, bool NT, bool UA = false>
THX_DEV void load_vec(Vec<T, N>& r, const T* b) {
  constexpr int BYTES = sizeof(T) * N;
  constexpr int CH = BYTES >= 16 ? 16 : BYTES;  // bytes per access
  typedef typename RawOf<CH>::type Raw;
  Raw* dst = (Raw*)&r;
  if constexpr (UA && (int)sizeof(T) < CH) {
    typedef typename RawUOf<CH, (int)sizeof(T)>::type RawU;
    const RawU* src = (const RawU*)b;
#pragma unroll
    for (int c = 0; c < BYTES / CH; ++c) dst[c] = NT ? __builtin_nontemporal_load(src + c) : src[c];
  } else {
    const Raw* src = (const Raw*)b;
#pragma unroll
    for (int c = 0; c < BYTES / CH; ++c) dst[c] = NT ? __builtin_nontemporal_load(src + c) : src[c];
  }
}

template <class T, int N, bool NT, bool UA = false>
THX_DEV void store_vec(T* b, const Vec<T, N>& r) {
  constexpr int BYTES = sizeof(T) * N;
  constexpr int CH = BYTES >= 16 ? 16 : BYTES;
  typedef typename RawOf<CH>::type Raw;
  const Raw* src = (const Raw*)&r;
  if constexpr (UA && (int)sizeof(T) < CH) {
    typedef typename RawUOf<CH, (int)sizeof(T)>::type RawU;
    RawU* dst = (RawU*)b;
#pragma unroll
    for (int c = 0; c < BYTES / CH; ++c) {
      if (NT) __builtin_nontemporal_store(src[c], dst + c);
      else dst[c] = src[c];
    }
  } else {
    Raw* dst = (Raw*)b;
#pragma unroll
    for (int c = 0; c < BYTES / CH; ++c) {
      if (NT) __builtin_nontemporal_store(src[c], dst + c);
      else dst[c] = src[c];
    }
  }
}

// Sums over the V float16 elements of a vector, two elements per instruction (v_dot2_f32_f16: both products
// and both additions in float32, the products exact; float16 denormals count, measured): the sum of the
// elements, and the sum of the pairwise products of two vectors.
typedef _Float16 thx_f16x2 __attribute__((ext_vector_type(2)));

template <int V>
THX_DEV float half_dot(const Vec<thx_f16, V>& a, const Vec<thx_f16, V>& b) {
  static_assert(V % 2 == 0, "pairs of elements");
  const thx_f16x2* pa = (const thx_f16x2*)&a;
  const thx_f16x2* pb = (const thx_f16x2*)&b;
  float acc = 0.0f;
#pragma unroll
  for (int k = 0; k < V / 2; ++k) acc = __builtin_amdgcn_fdot2(pa[k], pb[k], acc, false);
  return acc;
}

template <int V>
THX_DEV float half_sum(const Vec<thx_f16, V>& a) {
  static_assert(V % 2 == 0, "pairs of elements");
  const thx_f16x2* pa = (const thx_f16x2*)&a;
  const thx_f16x2 ones = {(_Float16)1.0f, (_Float16)1.0f};
  float acc = 0.0f;
#pragma unroll
  for (int k = 0; k < V / 2; ++k) acc = __builtin_amdgcn_fdot2(pa[k], ones, acc, false);
  return acc;
}

// The sum of the V 8- or 16-bit integers of a vector, in 32 bits (16 elements cannot overflow them), four or two
// elements per instruction (v_dot4 / v_dot2 against ones).  Left to itself the compiler widens every element to the
// 64 bits of the accumulator first: 56 instructions per 16 bytes instead of 6.
typedef short thx_i16x2 __attribute__((ext_vector_type(2)));
typedef unsigned short thx_u16x2 __attribute__((ext_vector_type(2)));

template <int V, class T>
THX_DEV int packed_isum(const Vec<T, V>& a) {
  static_assert((V * sizeof(T)) % 4 == 0 && (sizeof(T) == 1 || sizeof(T) == 2), "whole 32-bit words of narrow integers");
  constexpr int W = V * (int)sizeof(T) / 4;
  const unsigned* w = (const unsigned*)&a;
  if constexpr (T(-1) < T(0)) {
    int acc = 0;
#pragma unroll
    for (int k = 0; k < W; ++k) {
      if constexpr (sizeof(T) == 1) {
        acc = __builtin_amdgcn_sdot4((int)w[k], 0x01010101, acc, false);
      } else {
        const thx_i16x2 ones = {1, 1};
        acc = __builtin_amdgcn_sdot2(*(const thx_i16x2*)&w[k], ones, acc, false);
      }
    }
    return acc;
  } else {
    unsigned acc = 0;
#pragma unroll
    for (int k = 0; k < W; ++k) {
      if constexpr (sizeof(T) == 1) {
        acc = __builtin_amdgcn_udot4(w[k], 0x01010101u, acc, false);
      } else {
        const thx_u16x2 ones = {1, 1};
        acc = __builtin_amdgcn_udot2(*(const thx_u16x2*)&w[k], ones, acc, false);
      }
    }
    return (int)acc;
  }
}

// Division by a run-time constant d >= 2 for dividends below 2^31:
// q = mulhi(n, m) >> s with m = ceil(2^(31+L)/d), s = L-1, L = ceil(log2 d).
struct FastDiv {
  unsigned m, s, d, pad;
};

THX_DEV void divmod(unsigned n, const FastDiv& f, unsigned& q, unsigned& r) {
  q = f.d == 1 ? n : (__umulhi(n, f.m) >> f.s);
  r = n - q * f.d;
}
THX_DEV void divmod(unsigned long long n, const FastDiv& f, unsigned long long& q,
                    unsigned long long& r) {
  q = n / f.d;
  r = n - q * f.d;
}

template <class IT> struct UnsignedOf;
template <> struct UnsignedOf<int> { typedef unsigned type; };
template <> struct UnsignedOf<long long> { typedef unsigned long long type; };

// ---- shuffles of every accumulator field type -----------------------------
THX_DEV int shfl_xor_t(int v, int m) { return __shfl_xor(v, m, THX_WAVE); }
THX_DEV unsigned shfl_xor_t(unsigned v, int m) { return (unsigned)__shfl_xor((int)v, m, THX_WAVE); }
THX_DEV float shfl_xor_t(float v, int m) { return __shfl_xor(v, m, THX_WAVE); }
THX_DEV double shfl_xor_t(double v, int m) { return __shfl_xor(v, m, THX_WAVE); }
THX_DEV long long shfl_xor_t(long long v, int m) { return __shfl_xor(v, m, THX_WAVE); }
THX_DEV unsigned long long shfl_xor_t(unsigned long long v, int m) {
  return (unsigned long long)__shfl_xor((long long)v, m, THX_WAVE);
}
THX_DEV unsigned char shfl_xor_t(unsigned char v, int m) { return (unsigned char)__shfl_xor((int)v, m, THX_WAVE); }
THX_DEV signed char shfl_xor_t(signed char v, int m) { return (signed char)__shfl_xor((int)v, m, THX_WAVE); }
THX_DEV short shfl_xor_t(short v, int m) { return (short)__shfl_xor((int)v, m, THX_WAVE); }
THX_DEV unsigned short shfl_xor_t(unsigned short v, int m) { return (unsigned short)__shfl_xor((int)v, m, THX_WAVE); }
THX_DEV _Float16 shfl_xor_t(_Float16 v, int m) { return (_Float16)__shfl_xor((float)v, m, THX_WAVE); }

// Butterfly over W lanes (W a power of two, <= 64): every lane ends with the
// combination of its W-lane group.
template <class R, int W>
THX_DEV typename R::Acc group_reduce(typename R::Acc a) {
#pragma unroll
  for (int m = W / 2; m >= 1; m >>= 1) {
    typename R::Acc b = R::shfl_xor(a, m);
    R::comb(a, b);
  }
  return a;
}

// Whole-block combine through LDS; `lds` holds NW accumulators. Result valid in
// every thread. Must be reached by all threads of the block.
template <class R, int NW>
THX_DEV typename R::Acc block_reduce(typename R::Acc a, typename R::Acc* lds) {
  a = group_reduce<R, THX_WAVE>(a);
  if (NW == 1) return a;
  const int lane = threadIdx.x & (THX_WAVE - 1), wave = threadIdx.x / THX_WAVE;
  __syncthreads();
  if (lane == 0) lds[wave] = a;
  __syncthreads();
  typename R::Acc r = lds[0];
#pragma unroll
  for (int w = 1; w < NW; ++w) R::comb(r, lds[w]);
  return r;
}

}  // namespace thx
