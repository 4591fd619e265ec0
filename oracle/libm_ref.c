/* TEST INFRASTRUCTURE - not part of the product.
 *
 * The C expressions the reference's C backend emits for a few unary float ops, compiled as they
 * are and calling the host's libm (glibc here, as on the reference's own machines), so that the
 * NumPy restatements in oracle/scalar_ref.py can be checked against the real thing where NumPy's
 * own routine is not the same function (round) or not the same code (expf, log1pf).
 *
 *   op 0  RoundHalfAwayFromZero  "z = round(x);"                       theano/scalar/basic.py:2686
 *   op 1  Exp                    "z = exp((npy_float32)x);"             theano/scalar/basic.py:2950-2951
 *   op 2  ScalarSigmoid          thresholds -88 / 15 (f32), -709 / 19   theano/tensor/nnet/sigm.py:81-83
 *   op 3  ScalarSoftplus         thresholds -103 / 14 (f32), -745 / 16  theano/tensor/nnet/sigm.py:357-361
 *   op 4  Log1p, op 5 Expm1, op 6 Tanh, op 7 Sqrt, op 8 Log             theano/scalar/basic.py:2919-3200
 * With g++ and <math.h>, `exp(float)` resolves to the float overload, i.e. expf; the float entry
 * points below spell that out.
 */
#include <math.h>
#include <stdint.h>

int libm_unary_f32(int op, const float* x, float* z, int64_t n) {
  for (int64_t i = 0; i < n; ++i) {
    const float v = x[i];
    switch (op) {
      case 0: z[i] = roundf(v); break;
      case 1: z[i] = expf(v); break;
      case 2: z[i] = v < -88.0f ? 0.0 : v > 15.0f ? 1.0f : 1.0f / (1.0f + expf(-v)); break;
      case 3: z[i] = v < -103.0f ? 0.0 : v > 14.0f ? v : log1pf(expf(v)); break;
      case 4: z[i] = log1pf(v); break;
      case 5: z[i] = expm1f(v); break;
      case 6: z[i] = tanhf(v); break;
      case 7: z[i] = sqrtf(v); break;
      case 8: z[i] = logf(v); break;
      default: return 1;
    }
  }
  return 0;
}

int libm_unary_f64(int op, const double* x, double* z, int64_t n) {
  for (int64_t i = 0; i < n; ++i) {
    const double v = x[i];
    switch (op) {
      case 0: z[i] = round(v); break;
      case 1: z[i] = exp(v); break;
      case 2: z[i] = v < -709.0 ? 0.0 : v > 19.0 ? 1.0 : 1.0 / (1.0 + exp(-v)); break;
      case 3: z[i] = v < -745.0 ? 0.0 : v > 16.0 ? v : log1p(exp(v)); break;
      case 4: z[i] = log1p(v); break;
      case 5: z[i] = expm1(v); break;
      case 6: z[i] = tanh(v); break;
      case 7: z[i] = sqrt(v); break;
      case 8: z[i] = log(v); break;
      default: return 1;
    }
  }
  return 0;
}
