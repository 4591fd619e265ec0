// Host build of the device helpers in theano_amd/csrc/kernels/thx_special.h for the CPU tests: the
// header is plain C++ once the device qualifiers are defined away, so g++ and the host libm can run the
// same text that hipRTC compiles for the GPU.
#include <cmath>
#define __device__
#define __forceinline__ inline
#define THX_DEV inline
using namespace std;
namespace thx {
inline float shfl_xor_t(float v, int) { return v; }
inline double shfl_xor_t(double v, int) { return v; }
}
#include "thx_special.h"

extern "C" void host_jv(const double* v, const double* x, double* out, int n) {
  for (int i = 0; i < n; ++i) out[i] = thx_jv(v[i], x[i]);
}
extern "C" void host_iv(const double* v, const double* x, double* out, int n) {
  for (int i = 0; i < n; ++i) out[i] = thx_iv(v[i], x[i]);
}

template <class C>
static C apply(int which, C z, C w) {
  switch (which) {
    case 0: return thx_cexp(z);
    case 1: return thx_clog(z);
    case 2: return thx_csqrt(z);
    case 3: return thx_csin(z);
    case 4: return thx_ccos(z);
    case 5: return thx_ctan(z);
    case 6: return thx_csinh(z);
    case 7: return thx_ccosh(z);
    case 8: return thx_ctanh(z);
    case 9: return thx_cexpm1(z);
    case 10: return thx_clog1p(z);
    case 11: return z / w;
    case 12: return thx_cpow(z, w);
    case 13: return z * w;
    case 14: return thx_clog2(z);
    case 15: return thx_clog10(z);
    case 16: return thx_cconj(z);
    case 17: return C(thx_cabs(z), thx_cangle(z));
    default: return thx_cpolar(z.re, z.im);
  }
}
extern "C" void host_c128(int which, const double* z, const double* w, double* out, int n) {
  for (int i = 0; i < n; ++i) {
    const thx_c128 r = apply(which, thx_c128(z[2 * i], z[2 * i + 1]), thx_c128(w[2 * i], w[2 * i + 1]));
    out[2 * i] = r.re;
    out[2 * i + 1] = r.im;
  }
}
extern "C" void host_c64(int which, const float* z, const float* w, float* out, int n) {
  for (int i = 0; i < n; ++i) {
    const thx_c64 r = apply(which, thx_c64(z[2 * i], z[2 * i + 1]), thx_c64(w[2 * i], w[2 * i + 1]));
    out[2 * i] = r.re;
    out[2 * i + 1] = r.im;
  }
}
